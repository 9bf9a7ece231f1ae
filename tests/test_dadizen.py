"""Dadizen through the framework (reader, model class, per-run KV pools, retention state slots,
native scheduler, schedule replay, generation) against the plain oracle of tests/dadizen_oracle.py.

Every test builds its own small random checkpoint.  The CPU runs use the operator layer's PyTorch
paths; the `gpu` runs put the same engine on the HIP kernels, in bf16 and in fp32.
"""
import json
import os

import numpy as np
import pytest
import torch

import dadizen_oracle as oracle
from localai_amd.engine.llm_engine import EngineConfig, LLMEngine
from localai_amd.engine.sampling_params import SamplingParams

DEVICES = ["cpu", pytest.param("cuda:0", marks=pytest.mark.gpu)]
MODES = [("cpu", "float32"), ("cpu", "bfloat16"),
         pytest.param("cuda:0", "float32", marks=pytest.mark.gpu), pytest.param("cuda:0", "bfloat16", marks=pytest.mark.gpu)]

YARN = {"factor": 4.0, "original": 32, "fast": 8.0, "slow": 1.0}      # stretched and unstretched frequencies


def rot(dims, base=10000.0, scaling=None):
    r = {"dims": dims, "base": base}
    if scaling:
        r["scaling"] = scaling
    return r


def attn(heads=4, kv=2, dim=16, vdim=8, window=12, dims=8, scale=0.25, scaling=YARN, base=10000.0):
    return {"type": "attention", "mixer": {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale,
                                           "mask": {"size": window}, "rot": rot(dims, base, scaling)}}


def latent(heads=3, dim=8, rot_dim=4, vdim=6, q_rank=12, kv_rank=10, scale=0.3, scaling=YARN, base=50000.0):
    return {"type": "latent_attention", "mixer": {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim,
                                                  "q_rank": q_rank, "kv_rank": kv_rank, "scale": scale,
                                                  "rot": rot(rot_dim, base, scaling)}}


def reten(heads=2, dim=8, vdim=12, decay=(0.9, 0.97), dims=8, base=1000.0):
    return {"type": "retention", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay),
                                           "rot": rot(dims, base)}}


def ff(layer, n=64, limit=1.25):
    return dict(layer, mlp={"kind": "dense", "ff": n, "limit": limit} if n else None)


# layer orders and sizes unlike one another: kv_heads 1 / = heads, key width = / != value width, the
# rotation over a part of a head or all of it, with and without frequency scaling, windows smaller and
# larger than a page and not dividing it, query rank != kv rank, loops at the start / in the middle /
# to the end, run 2 or 3 times, a mixer of every kind inside and outside the loop, layers without a
# feed-forward of every kind, decay 1 (nothing forgotten), no loop, no token side input, no soft cap
CONFIGS = {
    "small": {"vocab": 61, "width": 48, "norm": {"eps": 1e-5}, "token_side": {"dim": 6}, "logit_softcap": 20.0,
              "loop": {"start": 1, "stop": 3, "times": 2}, "layers": [
                  ff(attn()), ff(latent()), ff(reten(), 0), ff(attn(heads=2, kv=2, dim=8, vdim=8, window=20, dims=8))]},
    "varied": {"vocab": 83, "width": 40, "norm": {"eps": 1e-6}, "token_side": {"dim": 3}, "logit_softcap": 8.0,
               "loop": {"start": 0, "stop": 2, "times": 3}, "layers": [
                   ff(reten(heads=3, dim=12, vdim=4, decay=(1.0, 0.5, 0.99), dims=4), 24, 0.7),
                   ff(attn(heads=6, kv=1, dim=8, vdim=12, window=5, dims=2, scaling=None), 0),
                   ff(latent(heads=2, dim=4, rot_dim=8, vdim=10, q_rank=5, kv_rank=16, scaling=None), 0),
                   ff(attn(heads=3, kv=3, dim=10, vdim=6, window=33, dims=10, scale=0.2), 56, 4.0),
                   ff(reten(heads=1, dim=16, vdim=16, decay=(0.8,), dims=16), 32)]},
    "tail": {"vocab": 50, "width": 32, "norm": {"eps": 1e-5}, "token_side": {"dim": 8}, "logit_softcap": 16.0,
             "loop": {"start": 1, "stop": 3, "times": 2}, "layers": [
                 ff(latent(heads=4, dim=6, rot_dim=2, vdim=4, q_rank=8, kv_rank=6), 40),
                 ff(reten(heads=2, dim=6, vdim=10, decay=(0.95, 0.999), dims=6), 40),
                 ff(attn(heads=2, kv=1, dim=12, vdim=4, window=1000, dims=6), 40)]},
    "plain": {"vocab": 40, "width": 24, "norm": {"eps": 1e-5}, "layers": [
        ff(attn(heads=2, kv=2, dim=6, vdim=6, window=7, dims=6), 20), ff(reten(heads=2, dim=4, vdim=4, dims=4), 20),
        ff(latent(heads=2, dim=4, rot_dim=4, vdim=4, q_rank=6, kv_rank=6), 20)]},
    # sizes no vector load likes (width % 8 != 0, ff % 4 != 0, odd side width and ranks), three heads, a loop of one layer
    "odd": {"vocab": 51, "width": 36, "norm": {"eps": 1e-6}, "token_side": {"dim": 5}, "logit_softcap": 12.0,
            "loop": {"start": 2, "stop": 3, "times": 2}, "layers": [
                ff(attn(heads=3, kv=1, dim=10, vdim=7, window=9, dims=6, scale=0.3), 30),
                ff(reten(heads=3, dim=10, vdim=7, decay=(0.9, 0.95, 0.99), dims=10), 0),
                ff(latent(heads=3, dim=5, rot_dim=6, vdim=7, q_rank=9, kv_rank=11), 26, 2.0)]},
    # widths the GPU's specialised paths take: key width % 32 and value width % 16 (matrix-core
    # attention tiles, latent rows and cached rows % 32), GEMM depths % 256 (skinny GEMMs), retention rows over
    # several registers a lane
    "wide": {"vocab": 97, "width": 256, "norm": {"eps": 1e-6}, "token_side": {"dim": 16}, "logit_softcap": 25.0,
             "loop": {"start": 1, "stop": 4, "times": 2}, "layers": [
                 ff(attn(heads=4, kv=2, dim=64, vdim=32, window=40, dims=32, scale=0.125), 512),
                 ff(reten(heads=2, dim=128, vdim=64, decay=(0.97, 0.995), dims=64), 0),
                 ff(latent(heads=4, dim=32, rot_dim=32, vdim=32, q_rank=48, kv_rank=64, scale=0.125), 256),
                 ff(attn(heads=8, kv=2, dim=64, vdim=64, window=24, dims=32, scale=0.125), 256)]},   # decode rows: split-KV kernel
}


def make_weights(cfg, seed):
    g = torch.Generator().manual_seed(seed)
    D = cfg["width"]

    def rnd(*shape, s=1.0):
        return (torch.randn(*shape, generator=g) * s).to(torch.bfloat16)

    def lin(n, k):
        return rnd(n, k, s=k ** -0.5)

    W = {}

    def norm(name):
        W[name] = (1.0 + 0.2 * torch.randn(D, generator=g)).to(torch.bfloat16)
        W[name + ".b"] = rnd(D, s=0.1)
        W[name + ".alpha"] = torch.tensor(0.4 + 0.5 * float(torch.rand((), generator=g))).to(torch.bfloat16)

    W["embed"], W["head"] = rnd(cfg["vocab"], D), lin(cfg["vocab"], D)
    norm("final.norm")
    n = len(cfg["layers"])
    if cfg.get("token_side"):
        W["side.embed"] = rnd(cfg["vocab"], n * cfg["token_side"]["dim"])
    if cfg.get("loop"):
        W["loop.in"] = torch.cat([torch.eye(D) * 0.7, torch.eye(D) * 0.3], 1).to(torch.bfloat16) + rnd(D, 2 * D, s=0.1 * D ** -0.5)
        W["loop.step"] = rnd(cfg["loop"]["times"], D, s=0.3)
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        H, dk, dv = m["heads"], m["dim"], m["vdim"]
        norm(p + "norm1")
        norm(p + "norm1b")
        if L["type"] == "attention":
            G = m["kv_heads"]
            W[p + "mix.q"], W[p + "mix.k"], W[p + "mix.v"] = lin(H * dk, D) * 2, lin(G * dk, D) * 2, lin(G * dv, D)
        elif L["type"] == "retention":
            W[p + "mix.q"], W[p + "mix.k"] = lin(H * dk, D), lin(H * dk, D)
            W[p + "mix.v"], W[p + "mix.g"] = lin(H * dv, D), lin(H * dv, D)
        else:
            r, qr, dr = m["kv_rank"], m["q_rank"], m["rot_dim"]
            W[p + "mix.dq"], W[p + "mix.dq.norm"] = lin(qr, D), (1.0 + 0.2 * torch.randn(qr, generator=g)).to(torch.bfloat16)
            W[p + "mix.uq"] = lin(H * (dk + dr), qr) * 2
            W[p + "mix.dkv"], W[p + "mix.dkv.norm"] = lin(r + dr, D) * 2, (1.0 + 0.2 * torch.randn(r, generator=g)).to(torch.bfloat16)
            W[p + "mix.uk"], W[p + "mix.uv"], W[p + "mix.g"] = lin(H * dk, r), lin(H * dv, r), lin(H, D) * 2
        W[p + "mix.o"] = lin(D, H * dv)
        f = L["mlp"]
        if f:
            norm(p + "norm2")
            norm(p + "norm2b")
            W[p + "mlp.gate"], W[p + "mlp.up"] = lin(f["ff"], D) * 2, lin(f["ff"], D) * 2    # some beyond the clamp
            W[p + "mlp.down"] = lin(D, f["ff"])
        if cfg.get("token_side"):
            ds = cfg["token_side"]["dim"]
            W[p + "side.gate"], W[p + "side.proj"] = lin(ds, D), lin(D, ds)
            W[p + "side.norm"] = rnd(D, s=0.3)
    return W


def write_checkpoint(path, cfg, W):
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(dict(cfg, architecture="Dadizen"), f)
    save_file({k: v.contiguous() for k, v in W.items()}, os.path.join(path, "model.safetensors"))


_CKPT = {}


@pytest.fixture(scope="module")
def ckpt(tmp_path_factory):
    def get(name, seed=0):
        key = (name, seed)
        if key not in _CKPT:
            cfg = CONFIGS[name]
            W = make_weights(cfg, seed)
            path = str(tmp_path_factory.mktemp(f"dadizen_{name}_{seed}"))
            write_checkpoint(path, cfg, W)
            _CKPT[key] = (path, cfg, {k: v.float() for k, v in W.items()})
        return _CKPT[key]
    return get


def engine(path, device, dtype="float32", tokens=256, slots=4, bs=16, graphs=False):
    return LLMEngine(EngineConfig(model_path=path, device=device, context_size=tokens, max_num_seqs=slots,
                                  max_batched_tokens=tokens, block_size=bs, max_kv_tokens=tokens, kv_pool_exact=True,
                                  use_graphs=graphs, dtype=dtype, state_slots=slots, record_tokens=True))


def close(got, want, dtype):
    got, want = got.detach().float().cpu(), want.float()
    d = got - want
    d = d - d.mean(-1, keepdim=True)
    err = d.pow(2).mean(-1).sqrt() / want.std(-1).clamp_min(1e-6)
    if dtype == "float32":
        assert float(err.max()) < 2e-4, float(err.max())
    else:
        assert float(err.max()) < 0.12 and float(err.median()) < 0.03, (float(err.max()), float(err.median()))


def portions(n, sizes):
    out, i, k = [], 0, 0
    while i < n:
        s = min(sizes[k % len(sizes)], n - i)
        out.append(s)
        i += s
        k += 1
    return out


def replay_alone(eng, rid, toks, cuts):
    """Feed `toks` in the given portion sizes; logits of every position."""
    rows, i = [], 0
    for c in cuts:
        rows.append(eng.replay_step([(rid, toks[i:i + c], list(range(c)))], [rid] if i + c == len(toks) else []))
        i += c
    return torch.cat(rows, 0)


def rand_tokens(cfg, n, seed):
    return np.random.default_rng(seed).integers(0, cfg["vocab"], size=n).tolist()


def fwd(cfg, W, toks, layers_out=None):
    return oracle.forward(toks, W, cfg, layers_out=layers_out)


# --------------------------------------------------------------------------------------- whole prompts
@pytest.mark.parametrize("device,dtype", MODES)
@pytest.mark.parametrize("name", ["small", "varied", "tail", "plain", "odd", "wide"])
def test_whole_prompt_matches_oracle(ckpt, name, device, dtype):
    path, cfg, W = ckpt(name)
    toks = rand_tokens(cfg, 70, 1)            # several windows of most layers, pages of 16
    want = fwd(cfg, W, toks)
    eng = engine(path, device, dtype)
    close(replay_alone(eng, 1, toks, [len(toks)]), want, dtype)
    # the very first tokens: a one-token prompt, then two (zero state, a window with one key)
    close(replay_alone(eng, 2, toks[:1], [1]), fwd(cfg, W, toks[:1]), dtype)
    close(replay_alone(eng, 3, toks[:2], [2]), want[:2], dtype)


@pytest.mark.parametrize("device", DEVICES)
@pytest.mark.parametrize("name", ["varied", "tail"])
def test_residual_stream_after_every_layer_run(ckpt, name, device):
    path, cfg, W = ckpt(name)
    toks = rand_tokens(cfg, 23, 2)
    want = []
    fwd(cfg, W, toks, want)
    eng = engine(path, device, "float32")
    got = []
    from localai_amd.models.decoder import ForwardBatch
    eng.sched.add(1, toks, 0)
    plan = eng.sched.schedule_explicit([(1, len(toks))])
    fb = ForwardBatch(tokens=eng._dev(plan["p_tokens"]), pos=eng._dev(plan["p_pos"]), slots=eng._dev(plan["p_slots"]),
                      decode=False, block_tables=eng._dev(plan["p_bt"]), cu_q=eng._dev(plan["p_cu"]),
                      ctx_lens=eng._dev(plan["p_ctx"]), sslots=eng._dev(plan["p_sslot"]),
                      row_seq=eng._dev(np.zeros(len(toks), dtype=np.int32)))
    eng.model.forward(fb, eng.kv, layer_out=got)
    lp = cfg["loop"]
    assert len(got) == len(want) == len(cfg["layers"]) + (lp["stop"] - lp["start"]) * (lp["times"] - 1)
    for a, b in zip(got, want):
        assert float((a.cpu() - b).abs().max()) < 2e-4 * max(1.0, float(b.abs().max()))


# --------------------------------------------------------------------------------------- portions, decoding
@pytest.mark.parametrize("device,dtype", MODES)
@pytest.mark.parametrize("name", ["varied", "tail", "odd", "wide"])
def test_portions_and_token_by_token_decoding(ckpt, name, device, dtype):
    path, cfg, W = ckpt(name)
    toks = rand_tokens(cfg, 90, 3)
    want = fwd(cfg, W, toks)
    eng = engine(path, device, dtype)
    for rid, cuts in enumerate([portions(90, [2]), portions(90, [5, 2, 17, 3, 31]), portions(90, [64, 1, 1, 7]),
                                [40] + [1] * 50, [1] * 90], 1):
        close(replay_alone(eng, rid, toks, cuts), want, dtype)


@pytest.mark.parametrize("device,dtype", MODES)
def test_long_decoding_over_windows_and_pages(ckpt, device, dtype):
    path, cfg, W = ckpt("small")
    toks = rand_tokens(cfg, 150, 4)           # windows 12 and 20, pages of 16: 140 single tokens pass both often
    want = fwd(cfg, W, toks)
    eng = engine(path, device, dtype)
    close(replay_alone(eng, 1, toks, [10] + [1] * 140), want, dtype)


# --------------------------------------------------------------------------------------- batches, reuse
@pytest.mark.parametrize("device,dtype", MODES)
@pytest.mark.parametrize("name", ["varied", "wide"])
def test_mixed_batches_of_unequal_requests_with_page_and_slot_reuse(ckpt, name, device, dtype):
    """Four live requests at most in a pool of 160 tokens with 4 state slots, ten requests in all:
    portions of some beside single tokens of others, every finished request's pages and slot taken
    over by the next (whose retention state must start from zero, not from the leftovers).  Every
    position must equal the request run alone (the oracle)."""
    path, cfg, W = ckpt(name)
    rng = np.random.default_rng(5)
    lens = [33, 7, 48, 2, 21, 40, 1, 17, 30, 9]
    reqs = {i + 1: rand_tokens(cfg, n, 100 + i) for i, n in enumerate(lens)}
    want = {i: fwd(cfg, W, t) for i, t in reqs.items()}
    eng = engine(path, device, dtype, tokens=160, slots=4, bs=16)
    pending = list(reqs)
    live, at = [], {}
    got = {i: [] for i in reqs}
    while pending or live:
        while pending and len(live) < 4 and sum(-(-len(reqs[i]) // 16) * 16 for i in live + pending[:1]) <= 160:
            live.append(pending.pop(0))
            at[live[-1]] = 0
        entries = []
        for i in live:
            if rng.random() < 0.2 and len(live) > 1:
                continue                       # rests this step
            left = len(reqs[i]) - at[i]
            n = min(left, int(rng.choice([1, 1, 2, 3, 8, 19])))
            entries.append((i, reqs[i][at[i]:at[i] + n], list(range(n))))
        if not entries:
            continue
        end = [i for i, t, _ in entries if at[i] + len(t) == len(reqs[i])]
        lg = eng.replay_step(entries, end)
        o = 0
        for i, t, _ in entries:
            got[i].append(lg[o:o + len(t)])
            o += len(t)
            at[i] += len(t)
        for i in end:
            live.remove(i)
    assert eng.sched.num_free_state_slots == 4 and eng.sched.blocks().num_free == 10
    for i in reqs:
        close(torch.cat(got[i], 0), want[i], dtype)


@pytest.mark.parametrize("device", DEVICES)
def test_pools_follow_the_layer_runs(ckpt, device):
    """One pool entry per layer RUN: looped layers hold a cache per pass; latent layers one head of
    kv_rank + rot_dim columns and no value pages; retention layers no pages but fp32 state."""
    path, cfg, W = ckpt("small")
    eng = engine(path, device, "bfloat16", tokens=64, slots=2, bs=16)
    kv = eng.kv
    kinds = [cfg["layers"][i]["type"] for i, _ in oracle.layer_runs(cfg)]
    assert kinds == ["attention", "latent_attention", "retention", "latent_attention", "retention", "attention"]
    assert len(kv.k) == len(kinds) == len(kv.state)
    assert tuple(kv.k[0].shape[1:]) == (2, 16, 16) and tuple(kv.v[0].shape[1:]) == (2, 2, 8, 8)
    assert tuple(kv.k[1].shape[1:]) == (1, 16, 14) and kv.v[1] is None and kv.k[1].data_ptr() != kv.k[3].data_ptr()
    assert kv.k[2] is None and kv.state[2].dtype == torch.float32 and tuple(kv.state[2].shape) == (2, 2, 12, 8)
    assert kv.state[2].data_ptr() != kv.state[4].data_ptr() and kv.state[0] is None


# --------------------------------------------------------------------------------------- generation
@pytest.mark.parametrize("device,dtype,graphs,name", [
    ("cpu", "float32", False, "small"),
    pytest.param("cuda:0", "float32", False, "small", marks=pytest.mark.gpu),
    pytest.param("cuda:0", "bfloat16", True, "small", marks=pytest.mark.gpu),
    pytest.param("cuda:0", "float32", True, "varied", marks=pytest.mark.gpu),
    pytest.param("cuda:0", "bfloat16", True, "wide", marks=pytest.mark.gpu),
    pytest.param("cuda:0", "bfloat16", False, "wide", marks=pytest.mark.gpu)])
def test_greedy_generation_through_the_engine(ckpt, device, dtype, graphs, name):
    """engine.add_request / step: scheduler-planned chunked prefill, (graph-replayed multi-step)
    decode with the device sampler, several requests at once; every emitted token is the oracle's
    argmax at its position unless the oracle's top-2 margin is within rounding."""
    path, cfg, W = ckpt(name)
    eng = LLMEngine(EngineConfig(model_path=path, device=device, context_size=128, max_num_seqs=4,
                                 max_batched_tokens=24, block_size=16, use_graphs=graphs, dtype=dtype,
                                 record_tokens=True, decode_steps=4, decode_steps_wide=4))
    prompts = [rand_tokens(cfg, n, 200 + n) for n in (5, 30, 47)]
    done = {}
    for k, p in enumerate(prompts):
        def cb(ev, k=k):
            if ev.finished:
                done[k] = ev
        eng.add_request(p, SamplingParams(max_tokens=20, temperature=0.0, ignore_eos=True), cb)
    for _ in range(400):
        if len(done) == len(prompts):
            break
        eng.step()
    assert len(done) == len(prompts)
    margin_ok = 1e-3 if dtype == "float32" else 0.1
    for k, p in enumerate(prompts):
        gen = done[k].token_ids
        assert len(gen) == 20
        ref = fwd(cfg, W, p + gen[:-1])
        for j, t in enumerate(gen):
            row = ref[len(p) - 1 + j]
            top2 = torch.topk(row, 2).values
            assert t == int(row.argmax()) or float(top2[0] - top2[1]) <= margin_ok, (k, j)
    assert eng.sched.num_free_state_slots == 4


def test_registry_reader_and_configuration(ckpt):
    from localai_amd.models import model_class
    from localai_amd.models.dadizen import DadizenModel
    from localai_amd.models.hf_checkpoint import open_model
    path, cfg, W = ckpt("varied")
    r = open_model(path)
    assert r.architecture == "dadizen" and model_class(r.architecture) is DadizenModel
    m = DadizenModel(r, torch.device("cpu"), dtype=torch.float32)
    assert [x.kind for x in m.hp.mixers] == ["retention", "attention", "latent_attention", "attention", "retention"]
    assert m.hp.runs == [(0, 0), (1, 0), (0, 1), (1, 1), (0, 2), (1, 2), (2, -1), (3, -1), (4, -1)]
    assert m.hp.mixers[1].window == 5 and m.hp.mixers[1].rot.scaling is None and m.hp.mlps[1] is None
    assert m.hp.mixers[0].decay == (1.0, 0.5, 0.99) and m.hp.side_dim == 3 and m.hp.logit_softcap == 8.0
    bad = dict(cfg, layers=[dict(cfg["layers"][0], type="convolution")])
    with pytest.raises(ValueError):
        type(m.hp).from_config(bad)


def test_trace_runner_cli(ckpt, tmp_path):
    """The schedule replay program end to end on the CPU: two requests, a rest, a reused name."""
    import subprocess
    import sys
    path, cfg, W = ckpt("tail")
    a, b = rand_tokens(cfg, 20, 7), rand_tokens(cfg, 9, 8)
    steps = [{"step": 0, "entries": [{"id": "a", "tokens": a[:11], "want": [0, 10]}], "end": []},
             {"step": 1, "entries": [{"id": "a", "tokens": a[11:13], "want": []}, {"id": "b", "tokens": b, "want": [8]}],
              "end": ["b"]},
             {"step": 2, "entries": [{"id": "a", "tokens": a[13:], "want": [6]}, {"id": "b", "tokens": a[:3], "want": [2]}],
              "end": ["a", "b"]}]
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    out = tmp_path / "out"
    p = subprocess.run([sys.executable, os.path.join(root, "bin", "trace_run"), "--model", path, "--dtype", "float32",
                        "--out", str(out), "--max-tokens", "64", "--device", "cpu"],
                       input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, timeout=300)
    assert p.returncode == 0, p.stderr[-2000:]
    assert [l for l in p.stdout.splitlines() if l.startswith("done")] == ["done 0", "done 1", "done 2"]
    wa, wb = fwd(cfg, W, a), fwd(cfg, W, b)
    V = cfg["vocab"]
    g = [torch.from_numpy(np.fromfile(out / f"{k}.f32", dtype="<f4").reshape(-1, V)) for k in range(3)]
    close(g[0], wa[[0, 10]], "float32")
    close(g[1], wb[[8]], "float32")
    close(g[2], torch.stack([wa[19], wa[2]]), "float32")


def test_backend_service_loads_and_generates(ckpt, monkeypatch):
    """The gRPC backend servicer (what the gateway talks to): LoadModel on the checkpoint directory,
    Predict with a numeric prompt; greedy tokens follow the oracle."""
    import asyncio
    from localai_amd.grpc import backend_pb as pb
    from localai_amd.grpc.servicer import EngineServicer
    monkeypatch.setenv("LOCALAI_MAX_NUM_SEQS", "4")
    path, cfg, W = ckpt("plain")
    prompt = [3, 17, 5, 9, 30]

    async def run():
        sv = EngineServicer(device="cpu")
        r = await sv.LoadModel(pb.ModelOptions(ModelFile=path, ContextSize=64))
        assert r.success, r.message
        return await sv.Predict(pb.PredictOptions(Prompt=" ".join(str(t) for t in prompt), Tokens=5, Temperature=0.0,
                                                  IgnoreEOS=True))
    rep = asyncio.run(run())
    gen = [int(x) for x in rep.message.decode().strip("<>").split("><")]
    assert rep.tokens == 5 and rep.prompt_tokens == len(prompt) and len(gen) == 5
    ref = fwd(cfg, W, prompt + gen[:-1])
    for j, t in enumerate(gen):
        row = ref[len(prompt) - 1 + j]
        top2 = torch.topk(row, 2).values
        assert t == int(row.argmax()) or float(top2[0] - top2[1]) <= 0.1, j      # served in bf16 by default
