"""Plain, slow fp32 implementation of the Suganex design: one function per mechanism, written from
its equations with loops over positions and heads.  The oracle of tests/test_suganex*.py; it
shares no code with localai_amd (no ops, no model class, no cache: every call sees whole sequences).

Weights are a dict name -> fp32 tensor under the checkpoint's names; cfg is the parsed config.json.
"""
import math

import torch


def rms_norm(x, w, eps):
    """x / sqrt(mean(x^2) + eps) * (1 + w): the weight is stored around zero."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps) * (1.0 + w)


def short_conv(u, w):
    """u [T, C], w [C, taps]: y[t] = sum_j w[:, j] * u[t - (taps - 1) + j], zeros before t = 0."""
    T, C = u.shape
    taps = w.shape[1]
    y = torch.zeros(T, C)
    for t in range(T):
        for j in range(taps):
            s = t - (taps - 1) + j
            if s >= 0:
                y[t] += w[:, j] * u[s]
    return y


def head_slopes(H):
    return [2.0 ** (-8.0 * (h + 1) / H) for h in range(H)]


def raw_score(qh, kh, scale, softcap, slope, dist):
    s = float(qh @ kh) * scale
    if softcap:
        s = softcap * math.tanh(s / softcap)
    return s - slope * dist


def visible(i, j, chunk):
    return j <= i and (not chunk or i // chunk == j // chunk)


def attention(q, k, v, gate_logit, talk, scale, softcap, chunk):
    """q [T, H, Dk], k [T, G, Dk], v [T, G, Dv], gate_logit [T, H], talk [H, H] -> [T, H * Dv]."""
    T, H, _ = q.shape
    G = k.shape[1]
    Dv = v.shape[2]
    rep = H // G
    slopes = head_slopes(H)
    out = torch.zeros(T, H, Dv)
    for i in range(T):
        js = [j for j in range(T) if visible(i, j, chunk)]
        s = torch.zeros(H, len(js))
        for g in range(H):
            for n, j in enumerate(js):
                s[g, n] = raw_score(q[i, g], k[j, g // rep], scale, softcap, slopes[g], i - j)
        s = talk @ s                                   # heads' scores mixed before the softmax
        p = torch.softmax(s, -1)
        for h in range(H):
            o = torch.zeros(Dv)
            for n, j in enumerate(js):
                o += p[h, n] * v[j, h // rep]
            out[i, h] = o * torch.sigmoid(gate_logit[i, h])
    return out.reshape(T, H * Dv)


def dense_ff(h, up, down):
    return torch.relu(h @ up.T) ** 2 @ down.T


def route(h, router, correction, top):
    """-> (chosen experts [T, top], their weights [T, top])."""
    s = torch.sigmoid(h @ router.T)
    choice = s + correction if correction is not None else s
    idx = torch.topk(choice, top, -1).indices
    w = s.gather(1, idx)
    return idx, w / (w.sum(-1, keepdim=True) + 1e-20)


def moe_ff(h, W, prefix, experts, top):
    idx, w = route(h, W[prefix + "router"], W.get(prefix + "correction"), top)
    y = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for n in range(top):
            e = int(idx[t, n])
            pe = f"{prefix}e{e}."
            a = W[pe + "gate"] @ h[t]
            y[t] += w[t, n] * (W[pe + "down"] @ (a * torch.sigmoid(a) * (W[pe + "up"] @ h[t])))
    return y


def forward(cfg, W, tokens, layers_out=None):
    """Logits [T, vocab] of one whole sequence."""
    eps = cfg["norm"]["eps"]
    x = W["embed"][torch.tensor(tokens)]
    T = len(tokens)
    v_first = None
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        H, G, Dk, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        h = rms_norm(x, W[p + "norm1"], eps)
        q, k, v = h @ W[p + "mix.q"].T, h @ W[p + "mix.k"].T, h @ W[p + "mix.v"].T
        if p + "mix.q.conv" in W:
            q, k, v = (short_conv(q, W[p + "mix.q.conv"]), short_conv(k, W[p + "mix.k.conv"]),
                       short_conv(v, W[p + "mix.v.conv"]))
        if m.get("v_mix"):
            if v_first is None:
                v_first = v
            else:
                lam = float(W[p + "mix.vmix"])
                v = (1 - lam) * v + lam * v_first
        a = attention(q.view(T, H, Dk), k.view(T, G, Dk), v.view(T, G, Dv), h @ W[p + "mix.g"].T, W[p + "mix.talk"],
                      m["scale"], m.get("softcap") or 0.0, (m.get("mask") or {}).get("size") or 0)
        x = x + a @ W[p + "mix.o"].T
        f = L.get("mlp")
        if f:
            h2 = rms_norm(x, W[p + "norm2"], eps)
            if f["kind"] == "dense":
                x = x + dense_ff(h2, W[p + "mlp.up"], W[p + "mlp.down"])
            else:
                x = x + moe_ff(h2, W, p + "mlp.", f["router"]["experts"], f["router"]["top"])
        if layers_out is not None:
            layers_out.append(x.clone())
    return rms_norm(x, W["final.norm"], eps) @ W["head"].T
