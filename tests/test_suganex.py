"""Suganex through the framework (reader, model class, paged KV pool, state slots, native scheduler,
schedule replay, generation) against the plain oracle of tests/suganex_oracle.py.

Every test builds its own small random checkpoint.  The CPU runs use the operator layer's PyTorch
paths; the `gpu` runs put the same engine on the HIP kernels, in bf16 and in fp32.
"""
import json
import math
import os

import numpy as np
import pytest
import torch

import suganex_oracle as oracle
from localai_amd.engine.llm_engine import EngineConfig, LLMEngine
from localai_amd.engine.sampling_params import SamplingParams

DEVICES = ["cpu", pytest.param("cuda:0", marks=pytest.mark.gpu)]


def mixer(heads=4, kv=2, dim=16, vdim=8, conv=3, chunk=12, scale=0.2, softcap=15.0, v_mix=True):
    m = {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "conv": conv, "scale": scale,
         "softcap": softcap, "v_mix": v_mix}
    if chunk:
        m["mask"] = {"size": chunk}
    return m


def dense(ff=64):
    return {"kind": "dense", "ff": ff}


def moe(ff=24, experts=5, top=2):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top}}


def layer(m, f):
    return {"type": "attention", "mixer": m, "mlp": f}


# layer orders and sizes unlike one another: kv_heads 1 / = heads, key width = / != value width,
# 2 / 3 / 4 taps, chunks that do not divide the page size, top 1 / 2 / 3, no feed-forward, v_mix
# starting at a later layer and skipping one
CONFIGS = {
    "small": {"vocab": 61, "width": 48, "norm": {"eps": 1e-5}, "layers": [
        layer(mixer(heads=4, kv=2, dim=16, vdim=8, conv=3, chunk=12), dense(64)),
        layer(mixer(heads=4, kv=2, dim=16, vdim=8, conv=3, chunk=12), moe(24, 5, 2)),
        layer(mixer(heads=4, kv=2, dim=16, vdim=8, conv=3, chunk=12), dense(64))]},
    "varied": {"vocab": 83, "width": 64, "norm": {"eps": 1e-6}, "layers": [
        layer(mixer(heads=2, kv=2, dim=24, vdim=24, conv=2, chunk=9, scale=0.15, softcap=8.0, v_mix=False), moe(16, 3, 1)),
        layer(mixer(heads=6, kv=1, dim=8, vdim=16, conv=4, chunk=40, scale=0.3, softcap=30.0), None),
        layer(mixer(heads=3, kv=3, dim=16, vdim=8, conv=3, chunk=33, scale=0.25, softcap=5.0, v_mix=False), dense(40)),
        layer(mixer(heads=6, kv=1, dim=8, vdim=16, conv=4, chunk=7, scale=0.3, softcap=30.0), moe(32, 6, 3)),
        layer(mixer(heads=6, kv=1, dim=8, vdim=16, conv=2, chunk=64, scale=0.2, softcap=12.0), dense(72))]},
    # sizes no vector load or fused kernel likes (width % 8 != 0, ff % 4 != 0), a one-tap convolution
    # (a per-channel scale), five taps, every expert chosen, no mask
    "odd": {"vocab": 51, "width": 36, "norm": {"eps": 1e-6}, "layers": [
        layer(mixer(heads=3, kv=1, dim=12, vdim=10, conv=5, chunk=11, scale=0.3, softcap=0.0), dense(30)),
        layer(mixer(heads=3, kv=3, dim=12, vdim=10, conv=1, chunk=0, scale=0.3, softcap=9.0, v_mix=False), moe(10, 3, 3))]},
    # widths the GPU's specialised paths take: key width % 32 and value width % 16 (matrix-core
    # attention tiles), GEMM depths % 256 (skinny / grouped expert GEMMs)
    "wide": {"vocab": 97, "width": 256, "norm": {"eps": 1e-6}, "layers": [
        layer(mixer(heads=4, kv=2, dim=32, vdim=16, conv=4, chunk=20, scale=0.18, softcap=25.0), moe(256, 4, 2)),
        layer(mixer(heads=8, kv=2, dim=64, vdim=32, conv=3, chunk=48, scale=0.125, softcap=0.0, v_mix=False), dense(512)),
        layer(mixer(heads=4, kv=2, dim=32, vdim=16, conv=2, chunk=20, scale=0.18, softcap=25.0), None)]},
}


def make_weights(cfg, seed):
    g = torch.Generator().manual_seed(seed)
    D = cfg["width"]

    def rnd(*shape, s=1.0):
        return (torch.randn(*shape, generator=g) * s).to(torch.bfloat16)

    W = {"embed": rnd(cfg["vocab"], D), "final.norm": rnd(D, s=0.1), "head": rnd(cfg["vocab"], D, s=D ** -0.5)}
    for i, L in enumerate(cfg["layers"]):
        p, m = f"l{i}.", L["mixer"]
        H, G, Dk, Dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
        W[p + "norm1"], W[p + "norm2"] = rnd(D, s=0.1), rnd(D, s=0.1)
        W[p + "mix.q"], W[p + "mix.k"] = rnd(H * Dk, D, s=D ** -0.5), rnd(G * Dk, D, s=D ** -0.5)
        W[p + "mix.v"], W[p + "mix.g"] = rnd(G * Dv, D, s=D ** -0.5), rnd(H, D, s=D ** -0.5)
        for n, c in (("q", H * Dk), ("k", G * Dk), ("v", G * Dv)):
            W[p + f"mix.{n}.conv"] = rnd(c, m["conv"], s=0.6)
        W[p + "mix.vmix"] = torch.tensor(0.3 + 0.1 * i).to(torch.bfloat16)
        W[p + "mix.talk"] = (torch.eye(H) + 0.3 * torch.randn(H, H, generator=g)).to(torch.bfloat16)
        W[p + "mix.o"] = rnd(D, H * Dv, s=(H * Dv) ** -0.5)
        f = L["mlp"]
        if f and f["kind"] == "dense":
            W[p + "mlp.up"], W[p + "mlp.down"] = rnd(f["ff"], D, s=D ** -0.5), rnd(D, f["ff"], s=f["ff"] ** -0.5)
        elif f:
            E, F = f["router"]["experts"], f["expert"]["ff"]
            W[p + "mlp.router"] = rnd(E, D, s=D ** -0.5)
            W[p + "mlp.correction"] = rnd(E, s=0.3)
            for e in range(E):
                W[p + f"mlp.e{e}.gate"], W[p + f"mlp.e{e}.up"] = rnd(F, D, s=D ** -0.5), rnd(F, D, s=D ** -0.5)
                W[p + f"mlp.e{e}.down"] = rnd(D, F, s=F ** -0.5)
    return W


def write_checkpoint(path, cfg, W):
    from safetensors.torch import save_file
    os.makedirs(path, exist_ok=True)
    with open(os.path.join(path, "config.json"), "w") as f:
        json.dump(dict(cfg, architecture="Suganex"), f)
    save_file({k: v.contiguous() for k, v in W.items()}, os.path.join(path, "model.safetensors"))


_CKPT = {}


@pytest.fixture(scope="module")
def ckpt(tmp_path_factory):
    def get(name, seed=0):
        key = (name, seed)
        if key not in _CKPT:
            cfg = CONFIGS[name]
            W = make_weights(cfg, seed)
            path = str(tmp_path_factory.mktemp(f"suganex_{name}_{seed}"))
            write_checkpoint(path, cfg, W)
            _CKPT[key] = (path, cfg, {k: v.float() for k, v in W.items()})
        return _CKPT[key]
    return get


def engine(path, device, dtype="float32", tokens=256, slots=4, bs=16, graphs=False):
    return LLMEngine(EngineConfig(model_path=path, device=device, context_size=tokens, max_num_seqs=slots,
                                  max_batched_tokens=tokens, block_size=bs, max_kv_tokens=tokens, kv_pool_exact=True,
                                  use_graphs=graphs, dtype=dtype, state_slots=slots, record_tokens=True))


def tol(dtype):
    return 2e-4 if dtype == "float32" else 6e-2


def close(got, want, dtype):
    got, want = got.detach().float().cpu(), want.float()
    d = (got - want)
    d = d - d.mean(-1, keepdim=True)
    err = d.pow(2).mean(-1).sqrt() / want.std(-1).clamp_min(1e-6)
    if dtype == "float32":
        assert float(err.max()) < tol(dtype), float(err.max())
    else:
        # bf16 rounding may flip a router's close call at a position or two (another expert: a
        # visibly different row); a wrong mechanism moves every row
        assert float((err < tol(dtype)).float().mean()) >= 0.97 and float(err.median()) < tol(dtype) / 4, \
            (float(err.max()), float(err.median()))


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


MODES = [("cpu", "float32"), ("cpu", "bfloat16"),
         pytest.param("cuda:0", "float32", marks=pytest.mark.gpu), pytest.param("cuda:0", "bfloat16", marks=pytest.mark.gpu)]


def rand_tokens(cfg, n, seed):
    return np.random.default_rng(seed).integers(0, cfg["vocab"], size=n).tolist()


# --------------------------------------------------------------------------------------- whole prompts
@pytest.mark.parametrize("device,dtype", MODES)
@pytest.mark.parametrize("name", ["small", "varied", "wide", "odd"])
def test_whole_prompt_matches_oracle(ckpt, name, device, dtype):
    path, cfg, W = ckpt(name)
    toks = rand_tokens(cfg, 70, 1)            # several chunks of every layer, pages of 16
    want = oracle.forward(cfg, W, toks)
    eng = engine(path, device, dtype)
    got = replay_alone(eng, 1, toks, [len(toks)])
    close(got, want, dtype)
    # the very first tokens: positions before the convolution has a full tail, one-token prompt
    got1 = replay_alone(eng, 2, toks[:1], [1])
    close(got1, oracle.forward(cfg, W, toks[:1]), dtype)


@pytest.mark.parametrize("device", DEVICES)
def test_residual_stream_after_every_layer(ckpt, device):
    path, cfg, W = ckpt("varied")
    toks = rand_tokens(cfg, 23, 2)
    want = []
    oracle.forward(cfg, W, toks, want)
    eng = engine(path, device, "float32")
    plan_rows = []
    # one forward through the engine's own batch construction, with the per-layer tap
    from localai_amd.models.decoder import ForwardBatch
    eng.sched.add(1, toks, 0)
    plan = eng.sched.schedule_explicit([(1, len(toks))])
    fb = ForwardBatch(tokens=eng._dev(plan["p_tokens"]), pos=eng._dev(plan["p_pos"]), slots=eng._dev(plan["p_slots"]),
                      decode=False, block_tables=eng._dev(plan["p_bt"]), cu_q=eng._dev(plan["p_cu"]),
                      ctx_lens=eng._dev(plan["p_ctx"]), sslots=eng._dev(plan["p_sslot"]),
                      row_seq=eng._dev(np.zeros(len(toks), dtype=np.int32)))
    eng.model.forward(fb, eng.kv, layer_out=plan_rows)
    assert len(plan_rows) == len(want)
    for a, b in zip(plan_rows, want):
        assert float((a.cpu() - b).abs().max()) < 2e-4 * max(1.0, float(b.abs().max()))


# --------------------------------------------------------------------------------------- portions, decoding
@pytest.mark.parametrize("device,dtype", MODES)
@pytest.mark.parametrize("name", ["varied", "wide", "odd"])
def test_portions_and_token_by_token_decoding(ckpt, name, device, dtype):
    path, cfg, W = ckpt(name)
    toks = rand_tokens(cfg, 90, 3)
    want = oracle.forward(cfg, W, toks)
    eng = engine(path, device, dtype)
    for rid, cuts in enumerate([portions(90, [2]), portions(90, [5, 2, 17, 3, 31]), portions(90, [64, 1, 1, 7]),
                                [40] + [1] * 50, [1] * 90], 1):
        close(replay_alone(eng, rid, toks, cuts), want, dtype)


@pytest.mark.parametrize("device,dtype", MODES)
def test_long_decoding_over_chunks_and_pages(ckpt, device, dtype):
    path, cfg, W = ckpt("small")
    toks = rand_tokens(cfg, 150, 4)           # chunk 12, pages of 16: 140 single tokens cross both many times
    want = oracle.forward(cfg, W, toks)
    eng = engine(path, device, dtype)
    close(replay_alone(eng, 1, toks, [10] + [1] * 140), want, dtype)


# --------------------------------------------------------------------------------------- batches, reuse
@pytest.mark.parametrize("device,dtype", MODES)
@pytest.mark.parametrize("name", ["varied", "wide"])
def test_mixed_batches_of_unequal_requests_with_page_and_slot_reuse(ckpt, name, device, dtype):
    """Four live requests at most in a pool of 160 tokens with 4 state slots, ten requests in all:
    portions of some beside single tokens of others, every finished request's pages and slot taken
    over by the next.  Every position must equal the request run alone (the oracle)."""
    path, cfg, W = ckpt(name)
    rng = np.random.default_rng(5)
    lens = [33, 7, 48, 2, 21, 40, 1, 17, 30, 9]
    reqs = {i + 1: rand_tokens(cfg, n, 100 + i) for i, n in enumerate(lens)}
    want = {i: oracle.forward(cfg, W, t) for i, t in reqs.items()}
    eng = engine(path, device, dtype, tokens=160, slots=4, bs=16)
    pending = list(reqs)
    live, at = [], {}
    got = {i: [] for i in reqs}
    slots_seen = set()
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
            slots_seen.add(i)
            got[i].append(lg[o:o + len(t)])
            o += len(t)
            at[i] += len(t)
        for i in end:
            live.remove(i)
    assert eng.sched.num_free_state_slots == 4 and eng.sched.blocks().num_free == 10
    for i in reqs:
        close(torch.cat(got[i], 0), want[i], dtype)


@pytest.mark.parametrize("device", DEVICES)
def test_replay_refuses_what_does_not_fit(ckpt, device):
    path, cfg, W = ckpt("small")
    eng = engine(path, device, "float32", tokens=64, slots=2, bs=16)
    eng.replay_step([(1, [1, 2, 3], []), (2, [4, 5], [])])
    with pytest.raises(RuntimeError):
        eng.replay_step([(3, [1], [0])])                    # no third state slot
    eng.replay_step([], [2])
    assert eng.replay_step([(3, [1], [0])]).shape == (1, cfg["vocab"])
    with pytest.raises(RuntimeError):
        eng.replay_step([(1, list(range(50)), [])])         # 3 + 50 tokens: 4 pages of 16, and request 3 holds one


# --------------------------------------------------------------------------------------- generation
@pytest.mark.parametrize("device,dtype,graphs,name", [
    ("cpu", "float32", False, "small"),
    pytest.param("cuda:0", "float32", False, "small", marks=pytest.mark.gpu),
    pytest.param("cuda:0", "bfloat16", True, "small", marks=pytest.mark.gpu),
    pytest.param("cuda:0", "float32", True, "small", marks=pytest.mark.gpu),
    # widths that put decode rows on the matrix-core tile kernel with key splits, inside the graphs
    pytest.param("cuda:0", "bfloat16", True, "wide", marks=pytest.mark.gpu),
    pytest.param("cuda:0", "bfloat16", False, "wide", marks=pytest.mark.gpu)])
def test_greedy_generation_through_the_engine(ckpt, device, dtype, graphs, name):
    """engine.generate: scheduler-planned chunked prefill, (graph-replayed multi-step) decode with
    the device sampler, several requests at once; every emitted token is the oracle's argmax at
    its position unless the oracle's top-2 margin is within rounding."""
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
    margin_ok = 1e-3 if dtype == "float32" else 0.08
    for k, p in enumerate(prompts):
        gen = done[k].token_ids
        assert len(gen) == 20
        ref = oracle.forward(cfg, W, p + gen[:-1])
        for j, t in enumerate(gen):
            row = ref[len(p) - 1 + j]
            top2 = torch.topk(row, 2).values
            assert t == int(row.argmax()) or float(top2[0] - top2[1]) <= margin_ok, (k, j)
    assert eng.sched.num_free_state_slots == 4


def test_text_prompts_are_token_ids(ckpt):
    path, cfg, W = ckpt("small")
    eng = engine(path, "cpu")
    assert eng.tokenize("3 17 <5>") == [3, 17, 5]
    res = eng.generate("3 17 5", SamplingParams(max_tokens=3, temperature=0.0, ignore_eos=True))
    assert res["completion_tokens"] == 3 and len(res["token_ids"]) == 3


def test_registry_and_reader(ckpt):
    from localai_amd.models import model_class
    from localai_amd.models.decoder import DecoderModel
    from localai_amd.models.hf_checkpoint import open_model
    from localai_amd.models.suganex import SuganexModel
    path, cfg, W = ckpt("varied")
    r = open_model(path)
    assert r.architecture == "suganex" and model_class(r.architecture) is SuganexModel
    assert model_class("llama") is DecoderModel
    m = SuganexModel(r, torch.device("cpu"), dtype=torch.float32)
    assert [x.kv_heads for x in m.hp.mixers] == [2, 1, 3, 1, 1] and m.hp.mlps[1] is None
    assert m.v_first_layer == 1 and m.layers[1].lam is None and m.layers[3].lam is not None


def test_bf16_only_families_refuse_float32(tiny_model_path):
    with pytest.raises(ValueError):
        LLMEngine(EngineConfig(model_path=tiny_model_path, device="cpu", context_size=64, max_num_seqs=2,
                               max_batched_tokens=64, dtype="float32"))


def test_trace_runner_cli(ckpt, tmp_path):
    """bin/trace_run end to end on the CPU: two requests, a rest, a reused name, logits files."""
    import subprocess
    import sys
    path, cfg, W = ckpt("small")
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
    wa, wb = oracle.forward(cfg, W, a), oracle.forward(cfg, W, b)
    V = cfg["vocab"]
    g0 = torch.from_numpy(np.fromfile(out / "0.f32", dtype="<f4").reshape(-1, V))
    g1 = torch.from_numpy(np.fromfile(out / "1.f32", dtype="<f4").reshape(-1, V))
    g2 = torch.from_numpy(np.fromfile(out / "2.f32", dtype="<f4").reshape(-1, V))
    close(g0, wa[[0, 10]], "float32")
    close(g1, wb[[8]], "float32")
    close(g2, torch.stack([wa[19], wa[2]]), "float32")
