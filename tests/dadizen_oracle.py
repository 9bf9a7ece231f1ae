"""A plain, slow implementation of the Dadizen design, one function per mechanism.

Whole sequences, loops over positions and heads, no cache, no batching, float64 by default.  It
shares no code with localai_amd: the tests compare the framework's operators, model and engine
against it.  `W` is a dict name -> torch tensor (the checkpoint's names), `cfg` the parsed
config.json.
"""
import math

import torch


def gelu_tanh(z):
    return 0.5 * z * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (z + 0.044715 * z ** 3)))


def unit_rms(x, eps):
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def dyt(x, W, name):
    """Dynamic Tanh: an elementwise squashing norm with a scalar slope, a weight and a bias."""
    return torch.tanh(W[name + ".alpha"] * x) * W[name] + W[name + ".b"]


def rot_table(rot, n_pos, dtype=torch.float64):
    """(cos, sin) [n_pos, dims / 2] of a rotation spec {"base", "dims", "scaling"?}."""
    dims, base = int(rot["dims"]), float(rot["base"])
    half = dims // 2
    f = [base ** (-2.0 * i / dims) for i in range(half)]
    mag = 1.0
    sc = rot.get("scaling")
    if sc:
        factor, orig = float(sc["factor"]), float(sc["original"])

        def turn_dim(turns):
            return dims * math.log(orig / (2.0 * math.pi * turns)) / (2.0 * math.log(base))

        lo = max(math.floor(turn_dim(float(sc["fast"]))), 0)
        hi = min(math.ceil(turn_dim(float(sc["slow"]))), dims - 1)
        for i in range(half):
            ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
            f[i] = f[i] / factor * ramp + f[i] * (1.0 - ramp)
        mag = 0.1 * math.log(factor) + 1.0
    ang = torch.arange(n_pos, dtype=dtype)[:, None] * torch.tensor(f, dtype=dtype)[None, :]
    return torch.cos(ang) * mag, torch.sin(ang) * mag


def rotate(x, cos, sin, layout):
    """x [T, n, d] with the first 2 * cos.shape[1] dims of every head rotated; layout "half" pairs
    dim i with i + dims / 2, "interleaved" pairs 2i with 2i + 1."""
    half = cos.shape[1]
    out = x.clone()
    c, s = cos[:, None, :], sin[:, None, :]
    if layout == "half":
        u, v = x[..., :half], x[..., half:2 * half]
        out[..., :half] = u * c - v * s
        out[..., half:2 * half] = v * c + u * s
    else:
        u, v = x[..., 0:2 * half:2], x[..., 1:2 * half:2]
        out[..., 0:2 * half:2] = u * c - v * s
        out[..., 1:2 * half:2] = v * c + u * s
    return out


def retention(h, W, p, m, eps):
    """Decayed linear attention: per head S_t = decay S_(t-1) + k_t v_t^T, o_t = S_t^T q_t."""
    T = h.shape[0]
    H, dk, dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    q = (h @ W[p + "q"].T).view(T, H, dk)
    k = (h @ W[p + "k"].T).view(T, H, dk)
    v = (h @ W[p + "v"].T).view(T, H, dv)
    cos, sin = rot_table(m["rot"], T, h.dtype)
    q = rotate(q, cos, sin, "half")
    k = rotate(k, cos, sin, "half") * dk ** -0.5
    o = torch.zeros(T, H, dv, dtype=h.dtype)
    for hd in range(H):
        S = torch.zeros(dk, dv, dtype=h.dtype)
        for t in range(T):
            S = float(m["decay"][hd]) * S + torch.outer(k[t, hd], v[t, hd])
            o[t, hd] = S.T @ q[t, hd]
    o = unit_rms(o, eps).reshape(T, H * dv)
    g = h @ W[p + "g"].T
    return (o * (g * torch.sigmoid(g))) @ W[p + "o"].T


def softmax_rows(scores, visible):
    """scores [T, T], visible [T, T] bool -> probabilities, zero on invisible keys."""
    s = scores.masked_fill(~visible, float("-inf"))
    return torch.softmax(s, -1)


def attention(h, W, p, m):
    """Grouped-query softmax attention under a sliding window."""
    T = h.shape[0]
    H, G, dk, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = (h @ W[p + "q"].T).view(T, H, dk)
    k = (h @ W[p + "k"].T).view(T, G, dk)
    v = (h @ W[p + "v"].T).view(T, G, dv)
    cos, sin = rot_table(m["rot"], T, h.dtype)
    q, k = rotate(q, cos, sin, "interleaved"), rotate(k, cos, sin, "interleaved")
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    vis = (i - j >= 0) & (i - j < int(m["mask"]["size"]))
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for hd in range(H):
        g = hd // (H // G)
        pr = softmax_rows((q[:, hd] @ k[:, g].T) * float(m["scale"]), vis)
        out[:, hd] = pr @ v[:, g]
    return out.reshape(T, H * dv) @ W[p + "o"].T


def latent_attention(h, W, p, m, eps):
    """Queries, keys and values through low-rank latents; one rotated key part shared by all heads."""
    T = h.shape[0]
    H, dn, dr, dv, r = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["kv_rank"])
    cq = unit_rms(h @ W[p + "dq"].T, eps) * W[p + "dq.norm"]
    q = (cq @ W[p + "uq"].T).view(T, H, dn + dr)
    dkv = h @ W[p + "dkv"].T
    c = unit_rms(dkv[:, :r], eps) * W[p + "dkv.norm"]
    kr = dkv[:, r:].reshape(T, 1, dr)
    kn = (c @ W[p + "uk"].T).view(T, H, dn)
    v = (c @ W[p + "uv"].T).view(T, H, dv)
    cos, sin = rot_table(m["rot"], T, h.dtype)
    qr = rotate(q[..., dn:].contiguous(), cos, sin, "interleaved")
    kr = rotate(kr, cos, sin, "interleaved")[:, 0]
    i = torch.arange(T)[:, None]
    j = torch.arange(T)[None, :]
    vis = j <= i
    gate = torch.sigmoid(h @ W[p + "g"].T)
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for hd in range(H):
        s = (q[:, hd, :dn] @ kn[:, hd].T + qr[:, hd] @ kr.T) * float(m["scale"])
        out[:, hd] = (softmax_rows(s, vis) @ v[:, hd]) * gate[:, hd:hd + 1]
    return out.reshape(T, H * dv) @ W[p + "o"].T


def feed_forward(h, W, p, f):
    lim = float(f["limit"])
    g = torch.clamp(h @ W[p + "gate"].T, max=lim)
    u = torch.clamp(h @ W[p + "up"].T, -lim, lim)
    return (g * torch.sigmoid(1.702 * g) * (u + 1.0)) @ W[p + "down"].T


def token_side(x, tokens, W, i, dim, eps):
    """Per-layer token input: a gated second embedding, projected and unit-normed onto the stream."""
    e = W["side.embed"][tokens][:, i * dim:(i + 1) * dim]
    g = gelu_tanh(x @ W[f"l{i}.side.gate"].T) * e
    y = g @ W[f"l{i}.side.proj"].T
    return x + unit_rms(y, eps) * W[f"l{i}.side.norm"]


def layer(x, tokens, W, cfg, i):
    L = cfg["layers"][i]
    eps = float(cfg["norm"]["eps"])
    p = f"l{i}."
    h = dyt(x, W, p + "norm1")
    if L["type"] == "retention":
        y = retention(h, W, p + "mix.", L["mixer"], eps)
    elif L["type"] == "attention":
        y = attention(h, W, p + "mix.", L["mixer"])
    elif L["type"] == "latent_attention":
        y = latent_attention(h, W, p + "mix.", L["mixer"], eps)
    else:
        raise ValueError(L["type"])
    x = x + dyt(y, W, p + "norm1b")
    if L.get("mlp"):
        x = x + dyt(feed_forward(dyt(x, W, p + "norm2"), W, p + "mlp.", L["mlp"]), W, p + "norm2b")
    if cfg.get("token_side"):
        x = token_side(x, tokens, W, i, int(cfg["token_side"]["dim"]), eps)
    return x


def layer_runs(cfg):
    """[(layer index, pass number or -1)] in execution order."""
    n = len(cfg["layers"])
    lp = cfg.get("loop")
    if not lp:
        return [(i, -1) for i in range(n)]
    a, b, times = int(lp["start"]), int(lp["stop"]), int(lp["times"])
    return ([(i, -1) for i in range(a)] + [(i, t) for t in range(times) for i in range(a, b)]
            + [(i, -1) for i in range(b, n)])


def forward(tokens, W, cfg, dtype=torch.float64, layers_out=None):
    """Logits [T, vocab] of one whole sequence."""
    W = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in W.items()}
    tokens = torch.as_tensor(tokens, dtype=torch.long)
    x0 = W["embed"][tokens]
    x = x0
    lp = cfg.get("loop")
    for i, t in layer_runs(cfg):
        if t >= 0 and i == int(lp["start"]):
            x = torch.cat([x, x0], -1) @ W["loop.in"].T + W["loop.step"][t]
        x = layer(x, tokens, W, cfg, i)
        if layers_out is not None:
            layers_out.append(x.clone())
    logits = dyt(x, W, "final.norm") @ W["head"].T
    cap = float(cfg.get("logit_softcap") or 0.0)
    return cap * torch.tanh(logits / cap) if cap > 0 else logits
