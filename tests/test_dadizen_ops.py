"""The Dadizen mechanisms one by one -- operator layer (PyTorch CPU paths, HIP kernels under `gpu`)
and the model's mixers alone against the plain functions of tests/dadizen_oracle.py -- with inputs
made so that a fault shows: one (query, key) pair whose score towers over the rest, placed far
back, at a page border, just inside and just outside a window; state slots and pages holding
another sequence's leftovers; a decay of 1 that forgets nothing."""
import numpy as np
import pytest
import torch

import dadizen_oracle as oracle
from localai_amd import ops
from localai_amd.models.decoder import ForwardBatch

MODES = [("cpu", torch.float32), ("cpu", torch.bfloat16),
         pytest.param("cuda:0", torch.float32, marks=pytest.mark.gpu),
         pytest.param("cuda:0", torch.bfloat16, marks=pytest.mark.gpu)]


def i32(x, dev):
    return torch.tensor(np.asarray(x), dtype=torch.int32, device=dev)


def rel(got, want):
    want = want.float()
    return float((got.float().cpu() - want).abs().max() / want.abs().max().clamp_min(1e-6))


def tol(dtype):
    return 2e-5 if dtype == torch.float32 else 2e-2


def rounded(x, dtype):
    """Test inputs as the operator sees them: representable in its dtype."""
    return x.to(dtype).float()


# --------------------------------------------------------------------------------------- norms, gated units
@pytest.mark.parametrize("device,dtype", MODES)
@pytest.mark.parametrize("D", [40, 37])
def test_norm_chain_every_variant(device, dtype, D):
    g = torch.Generator().manual_seed(D)
    T = 7
    W = {}
    for n in ("a", "b"):
        W[n], W[n + ".b"], W[n + ".alpha"] = 1 + 0.3 * torch.randn(D, generator=g), torch.randn(D, generator=g), torch.tensor(0.3 if n == "a" else 1.7)
    dyt = lambda n: ("dyt", float(W[n + ".alpha"]), W[n].to(device), W[n + ".b"].to(device))  # noqa: E731
    res0 = torch.randn(T, D, generator=g) * 3
    br = rounded(torch.randn(T, D, generator=g) * 2, dtype)
    w = torch.randn(D, generator=g)
    vec = torch.randn(D, generator=g)
    # Dynamic Tanh on the branch, residual add, Dynamic Tanh for the next sublayer
    res = res0.clone().to(device)
    out = ops.norm_chain(res, br.to(device=device, dtype=dtype), dyt("a"), dyt("b"), out_dtype=dtype)
    want = res0 + oracle.dyt(br, W, "a")
    assert rel(res, want) < 1e-6 and rel(out, oracle.dyt(want, W, "b")) < tol(dtype)
    # unit norm with a plain weight on the branch; the stream itself handed on; fp32 split-K slabs
    res = res0.clone().to(device)
    slabs = torch.stack([br * 0.5, br * 0.25, br * 0.25]).to(device)
    out = ops.norm_chain(res, ops.Partial(slabs), ("rms", w.to(device), 1e-3), ("cast",), out_dtype=dtype)
    want = res0 + oracle.unit_rms(br, 1e-3) * w
    assert rel(res, want) < 1e-5 and rel(out, want) < tol(dtype)
    # the stream replaced by branch + vector (start of a loop pass)
    res = res0.clone().to(device)
    out = ops.norm_chain(res, br.to(device=device, dtype=dtype), None, dyt("a"), add_vec=vec.to(device), replace=True,
                         out_dtype=dtype)
    assert rel(res, br + vec) < 1e-6 and rel(out, oracle.dyt(br + vec, W, "a")) < tol(dtype)
    # nothing added: the first norm of a forward; no output: the stream only updated
    res = res0.clone().to(device)
    assert rel(ops.norm_chain(res, None, None, dyt("b"), out_dtype=dtype), oracle.dyt(res0, W, "b")) < tol(dtype)
    assert ops.norm_chain(res, br.to(device=device, dtype=dtype), dyt("b"), None) is None
    assert rel(res, res0 + oracle.dyt(br, W, "b")) < 1e-6


@pytest.mark.parametrize("device,dtype", MODES)
def test_clamped_gated_unit_beyond_both_limits(device, dtype):
    F, T = 11, 6
    g = torch.Generator().manual_seed(3)
    h = rounded(torch.randn(T, F, generator=g) * 3, dtype)       # |values| well beyond the limit 1.25
    eye = torch.eye(F)
    W = {"gate": eye, "up": -eye, "down": eye}
    want = oracle.feed_forward(h, W, "", {"limit": 1.25})
    src = torch.cat([h, -h], 1).to(device=device, dtype=dtype)
    assert rel(ops.glu_clamp(src, F, 1.25, out_dtype=dtype), want) < tol(dtype)
    assert rel(ops.glu_clamp(ops.Partial(src.float().unsqueeze(0)), F, 1.25, out_dtype=dtype), want) < tol(dtype)


@pytest.mark.parametrize("device,dtype", MODES)
def test_token_side_input_reads_its_layers_columns(device, dtype):
    g = torch.Generator().manual_seed(4)
    V, D, ds, n_layers, T = 13, 20, 5, 3, 9
    W = {"side.embed": rounded(torch.randn(V, n_layers * ds, generator=g), torch.bfloat16)}
    for i in range(n_layers):
        W[f"l{i}.side.gate"] = torch.randn(ds, D, generator=g) * D ** -0.5
        W[f"l{i}.side.proj"] = torch.randn(D, ds, generator=g)
        W[f"l{i}.side.norm"] = torch.randn(D, generator=g)
    x = torch.randn(T, D, generator=g)
    toks = torch.randint(0, V, (T,), generator=g)
    table = W["side.embed"].to(device=device, dtype=torch.bfloat16)
    for i in (0, 2):
        z = rounded(x @ W[f"l{i}.side.gate"].T, dtype)
        gt = ops.side_gate(z.to(device=device, dtype=dtype), i32(toks, device), table, i * ds, dtype)
        want_g = oracle.gelu_tanh(z) * W["side.embed"][toks][:, i * ds:(i + 1) * ds]
        assert rel(gt, want_g) < tol(dtype)
        y = rounded(want_g, dtype) @ W[f"l{i}.side.proj"].T
        res = x.clone().to(device)
        ops.norm_chain(res, y.to(device), ("rms", W[f"l{i}.side.norm"].to(device), 1e-5), None)
        assert rel(res, x + oracle.unit_rms(y, 1e-5) * W[f"l{i}.side.norm"]) < 1e-5


# --------------------------------------------------------------------------------------- rotations
@pytest.mark.parametrize("rot", [
    {"dims": 40, "base": 25000.0, "scaling": {"factor": 6.0, "original": 256, "fast": 24.0, "slow": 2.0}},
    {"dims": 8, "base": 100.0, "scaling": {"factor": 2.5, "original": 16, "fast": 4.0, "slow": 0.5}},   # lo / hi clamped
    {"dims": 6, "base": 500000.0, "scaling": {"factor": 8.0, "original": 4096, "fast": 1.0, "slow": 1.0}},  # hi - lo tiny
    {"dims": 10, "base": 1000.0}])
def test_rotation_frequencies_and_magnitude(rot):
    f, mag = ops.rot_freqs(rot["dims"], rot["base"], rot.get("scaling"))
    cos, sin = oracle.rot_table(rot, 50)
    ang = torch.arange(50, dtype=torch.float64)[:, None] * f.double()[None, :]
    assert float((torch.cos(ang) * mag - cos).abs().max()) < 1e-5 and float((torch.sin(ang) * mag - sin).abs().max()) < 1e-5


@pytest.mark.parametrize("device,dtype", MODES)
@pytest.mark.parametrize("interleaved,q_off,rot,Dq", [(True, 0, 6, 10), (True, 4, 6, 10), (False, 0, 8, 8), (False, 2, 4, 7)])
def test_rope_pages_rotates_a_span_and_appends(device, dtype, interleaved, q_off, rot, Dq):
    g = torch.Generator().manual_seed(rot + q_off)
    H, G, Dk, Dv, BS, T = 3, 2, max(rot, 6), 5, 8, 11
    spec = {"dims": rot, "base": 50.0, "scaling": {"factor": 3.0, "original": 8, "fast": 4.0, "slow": 1.0}}
    f, mag = ops.rot_freqs(rot, 50.0, spec["scaling"], device)
    pos = np.array([0, 1, 2, 3, 700, 701, 7, 8, 9, 15, 16])
    rows = rounded(torch.randn(T, H * Dq + G * Dk + G * Dv, generator=g), dtype)
    slots = np.array([8, 9, 10, 11, 31, 16, 0, 1, -1, 7, 24])       # page borders, one row not stored
    kc = torch.full((4, G, BS, Dk), 9.0, dtype=dtype, device=device)
    vc = torch.full((4, G, BS // 8, Dv, 8), 9.0, dtype=dtype, device=device)
    q = ops.rope_pages(rows.to(device=device, dtype=dtype), H, Dq, G, Dk, Dv, i32(pos, device), i32(slots, device), f, mag,
                       rot, q_off, interleaved, kc, vc)
    cos, sin = oracle.rot_table(spec, 702)
    lay = "interleaved" if interleaved else "half"
    qw = rows[:, :H * Dq].reshape(T, H, Dq).double()
    want_q = qw.clone()
    want_q[..., q_off:q_off + rot] = oracle.rotate(qw[..., q_off:q_off + rot].contiguous(), cos[pos], sin[pos], lay)
    want_k = oracle.rotate(rows[:, H * Dq:H * Dq + G * Dk].reshape(T, G, Dk).double(), cos[pos], sin[pos], lay)
    assert rel(q.view(T, H, Dq), want_q) < tol(dtype)
    for t, s in enumerate(slots):
        if s < 0:
            continue
        assert rel(kc[s // BS, :, s % BS], want_k[t]) < tol(dtype)
        assert rel(vc[s // BS, :, (s % BS) // 8, :, s % 8], rows[t, H * Dq + G * Dk:].reshape(G, Dv)) < 1e-6
    assert float(kc[1, :, 4].float().min()) == 9.0            # a place no row names is untouched
    # queries only
    q2 = ops.rope_pages(rows[:, :H * Dq].contiguous().to(device=device, dtype=dtype), H, Dq, 0, 0, 0, i32(pos, device),
                        None, f, mag, rot, q_off, interleaved)
    assert rel(q2.view(T, H, Dq), want_q) < tol(dtype)


@pytest.mark.parametrize("device,dtype", MODES)
def test_latent_rows_are_normed_rotated_and_stored_once(device, dtype):
    g = torch.Generator().manual_seed(6)
    rank, rot, BS, T = 9, 4, 8, 6
    f, mag = ops.rot_freqs(rot, 300.0, None, device)
    rows = rounded(torch.randn(T, rank + rot, generator=g) * 2, dtype)
    w = torch.randn(rank, generator=g)
    pos = np.array([0, 5, 6, 7, 8, 400])
    slots = np.array([3, 15, 16, 23, 8, -1])
    kc = torch.full((3, 1, BS, rank + rot), 9.0, dtype=dtype, device=device)
    ops.latent_kv(rows.to(device=device, dtype=dtype), rank, w.to(device), 1e-4, i32(pos, device), i32(slots, device), f, mag, kc)
    cos, sin = oracle.rot_table({"dims": rot, "base": 300.0}, 401)
    want_c = oracle.unit_rms(rows[:, :rank].double(), 1e-4) * w
    want_r = oracle.rotate(rows[:, rank:].reshape(T, 1, rot).double(), cos[pos], sin[pos], "interleaved")[:, 0]
    for t, s in enumerate(slots[:-1]):
        assert rel(kc[s // BS, 0, s % BS, :rank], want_c[t]) < tol(dtype)
        assert rel(kc[s // BS, 0, s % BS, rank:], want_r[t]) < tol(dtype)
    assert int((kc.float() == 9.0).sum()) == (3 * BS - 5) * (rank + rot)


# --------------------------------------------------------------------------------------- retention
@pytest.mark.parametrize("device,dtype", MODES)
@pytest.mark.parametrize("H,Dk,Dv,rot", [(2, 8, 12, 8), (3, 12, 5, 4), (1, 70, 40, 64), (2, 128, 16, 32)])
def test_retention_portions_state_slots_and_reuse(device, dtype, H, Dk, Dv, rot):
    g = torch.Generator().manual_seed(Dk)
    D = 24
    m = {"heads": H, "dim": Dk, "vdim": Dv, "decay": [1.0, 0.9, 0.99][:H], "rot": {"dims": rot, "base": 200.0}}
    W = {"q": torch.randn(H * Dk, D, generator=g) * D ** -0.5, "k": torch.randn(H * Dk, D, generator=g) * D ** -0.5,
         "v": torch.randn(H * Dv, D, generator=g) * D ** -0.5, "g": torch.randn(H * Dv, D, generator=g) * D ** -0.5,
         "o": torch.eye(H * Dv)}
    lens = {0: 37, 1: 6, 2: 19}
    h = {s: torch.randn(n, D, generator=g) for s, n in lens.items()}
    h[0][0] *= 8                              # a first token that towers: head 0 never forgets it
    proj = {s: rounded(torch.cat([h[s] @ W[n].T for n in "qkvg"], 1), dtype) for s in lens}
    # the oracle on the same rounded projections: identity projections of the stacked rows
    C = 2 * H * Dk + 2 * H * Dv
    eye = torch.eye(C)
    Wi = {"q": eye[:H * Dk], "k": eye[H * Dk:2 * H * Dk], "v": eye[2 * H * Dk:2 * H * Dk + H * Dv],
          "g": eye[2 * H * Dk + H * Dv:], "o": W["o"]}
    want = {s: oracle.retention(proj[s].double(), {k: v.double() for k, v in Wi.items()}, "", m, 1e-5) for s in lens}
    f, mag = ops.rot_freqs(rot, 200.0, None, device)
    # both slots hold another sequence's leftovers: a sequence starting at position 0 must not read them
    state = torch.full((2, H, Dv, Dk), 1e4, dtype=torch.float32, device=device)
    decay = torch.tensor(m["decay"], dtype=torch.float32, device=device)
    # steps of (sequence, start, rows): portions beside single rows; sequence 2 takes over sequence 1's slot
    steps = [[(0, 0, 1), (1, 0, 4)], [(0, 1, 1)], [(0, 2, 17), (1, 4, 1)], [(1, 5, 1), (0, 19, 2)], [(2, 0, 2), (0, 21, 1)],
             [(2, 2, 16), (0, 22, 15)], [(2, 18, 1)]]
    slot_of = {0: 0, 1: 1, 2: 1}
    got = {s: torch.zeros(n, H * Dv) for s, n in lens.items()}
    for st in steps:
        rows = torch.cat([proj[s][a:a + n] for s, a, n in st]).to(device=device, dtype=dtype)
        cu = np.concatenate([[0], np.cumsum([n for _, _, n in st])])
        pos = np.concatenate([np.arange(a, a + n) for _, a, n in st])
        out = ops.retention(rows, H, Dk, Dv, i32(pos, device), i32(cu, device), i32([slot_of[s] for s, _, _ in st], device),
                            state, decay, f, rot, 1e-5, mag)
        o = 0
        for s, a, n in st:
            got[s][a:a + n] = out[o:o + n].float().cpu()
            o += n
    for s in lens:
        assert rel(got[s], want[s]) < (1e-4 if dtype == torch.float32 else 3e-2), s


@pytest.mark.parametrize("device,dtype", MODES)
def test_retention_long_portions_in_segments(device, dtype):
    """A batch of more than a thousand rows (the GPU scans such portions in segments of 128 rows and
    joins the segment states): portion lengths that are no multiple of the segment, one shorter than
    a segment, a continuation from a live state, a slot with leftovers."""
    g = torch.Generator().manual_seed(9)
    H, Dk, Dv, rot = 2, 16, 24, 8
    m = {"heads": H, "dim": Dk, "vdim": Dv, "decay": [1.0, 0.98], "rot": {"dims": rot, "base": 100.0}}
    C = 2 * H * Dk + 2 * H * Dv
    lens = {0: 700 + 300, 1: 450, 2: 60}
    proj = {s: rounded(torch.randn(n, C, generator=g) * 0.5, dtype) for s, n in lens.items()}
    proj[0][0, 2 * H * Dk:2 * H * Dk + Dv] *= 20          # head 0 (decay 1) carries token 0 to the end
    eye = torch.eye(C).double()
    Wi = {"q": eye[:H * Dk], "k": eye[H * Dk:2 * H * Dk], "v": eye[2 * H * Dk:2 * H * Dk + H * Dv],
          "g": eye[2 * H * Dk + H * Dv:], "o": torch.eye(H * Dv).double()}
    want = {s: oracle.retention(proj[s].double(), Wi, "", m, 1e-5) for s in lens}
    f, mag = ops.rot_freqs(rot, 100.0, None, device)
    state = torch.full((3, H, Dv, Dk), -3e3, dtype=torch.float32, device=device)
    decay = torch.tensor(m["decay"], dtype=torch.float32, device=device)
    got = {s: torch.zeros(n, H * Dv) for s, n in lens.items()}
    for st in [[(0, 0, 700), (1, 0, 450), (2, 0, 60)], [(0, 700, 300)]]:      # 1210 rows, then 300 from the live state
        rows = torch.cat([proj[s][a:a + n] for s, a, n in st]).to(device=device, dtype=dtype)
        cu = np.concatenate([[0], np.cumsum([n for _, _, n in st])])
        pos = np.concatenate([np.arange(a, a + n) for _, a, n in st])
        out = ops.retention(rows, H, Dk, Dv, i32(pos, device), i32(cu, device), i32([s for s, _, _ in st], device), state,
                            decay, f, rot, 1e-5, mag)
        o = 0
        for s, a, n in st:
            got[s][a:a + n] = out[o:o + n].float().cpu()
            o += n
    for s in lens:
        assert rel(got[s], want[s]) < (2e-4 if dtype == torch.float32 else 3e-2), s


# --------------------------------------------------------------------------------------- windowed attention
def _attn_case(device, dtype, H, G, Dk, Dv, rot, window, BS, n, towers, tiles):
    """rope_pages + attn_mix over shuffled pages, prompt portion then single rows, against the oracle;
    towers = [(query position, key position)] whose score dwarfs every other."""
    g = torch.Generator().manual_seed(n + window)
    rng = np.random.default_rng(window)
    C = H * Dk + G * Dk + G * Dv
    rows = torch.randn(n, C, generator=g) * 0.5
    for p, (qi, kj) in enumerate(towers):                       # every pair on an unrotated dim of head 0 / kv head 0
        d = Dk - 1 - p % (Dk - rot)                             # (pairs sharing a dim lie out of each other's sight)
        rows[qi, d] = 24.0
        rows[kj, H * Dk + d] = 24.0
    rows = rounded(rows, dtype)
    eye = torch.eye(C).double()
    W = {"q": eye[:H * Dk], "k": eye[H * Dk:H * Dk + G * Dk], "v": eye[H * Dk + G * Dk:], "o": torch.eye(H * Dv).double()}
    spec = {"dims": rot, "base": 10000.0, "scaling": {"factor": 4.0, "original": 64, "fast": 16.0, "slow": 1.0}}
    m = {"heads": H, "kv_heads": G, "dim": Dk, "vdim": Dv, "scale": 0.2, "mask": {"size": window}, "rot": spec}
    want = oracle.attention(rows.double(), W, "", m)
    nb = -(-n // BS)
    table = rng.permutation(nb + 3)[:nb]
    slots = np.array([int(table[t // BS]) * BS + t % BS for t in range(n)])
    kc = torch.full((nb + 3, G, BS, Dk), 50.0, dtype=dtype, device=device)      # leftovers everywhere
    vc = torch.full((nb + 3, G, BS // 8, Dv, 8), 50.0, dtype=dtype, device=device)
    f, mag = ops.rot_freqs(rot, 10000.0, spec["scaling"], device)
    bt = i32([table], device)
    got = torch.zeros(n, H * Dv)
    cut = n - 20                                                 # a portion, then 20 single rows
    for a, b in [(0, cut)] + [(t, t + 1) for t in range(cut, n)]:
        pos = i32(np.arange(a, b), device)
        q = ops.rope_pages(rows[a:b].to(device=device, dtype=dtype), H, Dk, G, Dk, Dv, pos, i32(slots[a:b], device), f, mag,
                           rot, 0, True, kc, vc)
        kw = {}
        if tiles and device != "cpu":
            tl, tr = ops.attn_mix_tiles([b - a], device)
            kw = dict(tiles=tl, tile_rows=tr, cu_q=i32([0, b - a], device), key_splits=1 if b - a > 1 else 3)
        out = ops.attn_mix(q, kc, vc, i32(np.zeros(b - a), device), pos, bt, H, 0.2, window=window, **kw)
        got[a:b] = out.float().cpu()
    assert rel(got, want) < (1e-4 if dtype == torch.float32 else 3e-2)
    for qi, kj in towers:           # what the tower decides: head 0 is the towering key's value, or is not
        vj = rows[kj, H * Dk + G * Dk:H * Dk + G * Dk + Dv]
        seen = 0 <= qi - kj < window
        assert (float((got[qi, :Dv] - vj).abs().max()) < 0.05) == seen, (qi, kj)


@pytest.mark.parametrize("device,dtype", MODES)
def test_window_edges_in_prompts_and_decoding(device, dtype):
    # window 13, pages of 8, 60 rows (40 in the portion): keys just inside (i - 12) and just outside (i - 13),
    # for queries inside the portion (30) and decoded alone (50, 57); 57 - 12 = 45 decoded too, 50 - 12 = 38 in the portion
    _attn_case(device, dtype, H=4, G=2, Dk=10, Dv=6, rot=6, window=13, BS=8, n=60,
               towers=[(30, 18), (31, 18), (50, 38), (52, 39), (57, 45), (59, 46)], tiles=False)


@pytest.mark.parametrize("device,dtype", MODES)
def test_far_keys_and_page_borders_under_a_wide_window(device, dtype):
    # a window wider than the sequence: position 0 and the last slot of a page seen from hundreds of rows on
    _attn_case(device, dtype, H=2, G=1, Dk=8, Dv=8, rot=4, window=4096, BS=16, n=300,
               towers=[(270, 0), (285, 15), (290, 16), (299, 31)], tiles=False)


@pytest.mark.gpu
@pytest.mark.parametrize("window", [40, 33])
def test_window_edges_on_the_matrix_core_tiles(window):
    # widths the tile kernel takes (bf16, key width % 32, value width % 16): the same edges, portion rows on
    # 16-row tiles, single rows on one-row tiles split over the keys
    _attn_case("cuda:0", torch.bfloat16, H=4, G=2, Dk=64, Dv=32, rot=32, window=window, BS=16, n=120,
               towers=[(70, 70 - window + 1), (71, 71 - window), (110, 110 - window + 1), (115, 115 - window), (119, 99)],
               tiles=True)


# --------------------------------------------------------------------------------------- latent attention, alone
# (heads, dim, rot_dim, vdim, q_rank, kv_rank): small odd widths; widths the bf16 matrix-core kernel takes
# (cached row % 32, latent % 32) with more heads than one 16-row tile and a head count that fills no tile
LATENT_SHAPES = [(3, 6, 4, 5, 7, 12), (20, 16, 32, 8, 24, 96), (6, 32, 32, 16, 40, 64)]


@pytest.mark.parametrize("device,dtype", MODES)
@pytest.mark.parametrize("shape", LATENT_SHAPES)
def test_latent_attention_alone_with_a_far_key(device, dtype, shape, tmp_path):
    """The model's latent mixer on its own (one-layer checkpoint, crafted mixer input): the cached row
    is the only thing kept per token, the up-projections act on queries and outputs."""
    import test_dadizen as td
    from localai_amd.models.dadizen import DadizenModel
    from localai_amd.models.hf_checkpoint import open_model
    cfg = {"vocab": 20, "width": 24, "norm": {"eps": 1e-5}, "layers": [
        td.ff(td.latent(heads=shape[0], dim=shape[1], rot_dim=shape[2], vdim=shape[3], q_rank=shape[4], kv_rank=shape[5],
                        scale=0.25), 0)]}
    Wb = td.make_weights(cfg, 11)
    td.write_checkpoint(str(tmp_path), cfg, Wb)
    W = {k: v.float() for k, v in Wb.items()}
    model = DadizenModel(open_model(str(tmp_path)), torch.device(device), dtype=dtype)
    g = torch.Generator().manual_seed(12)
    n, BS = 200, 16
    h = torch.randn(n, 24, generator=g)
    h[3] *= 6                                  # a far key with a large latent: many later queries lean on it
    h = rounded(h, dtype)
    want = oracle.latent_attention(h.double(), {k: v.double() for k, v in W.items()}, "l0.mix.", cfg["layers"][0]["mixer"], 1e-5)
    nb = -(-n // BS)
    table = np.random.default_rng(1).permutation(nb + 2)[:nb]
    slots = np.array([int(table[t // BS]) * BS + t % BS for t in range(n)])
    kv = model.new_kv_cache(nb + 2, BS, 1)
    kv.k[0].fill_(30.0)
    got = torch.zeros(n, 24)
    L, m = model.layers[0], model.hp.mixers[0]
    for a, b in [(0, 2), (2, 150), (150, 153)] + [(t, t + 1) for t in range(153, n)]:
        pos = i32(np.arange(a, b), device)
        fb = ForwardBatch(tokens=pos, pos=pos, slots=i32(slots[a:b], device), decode=False, block_tables=i32([table], device))
        o = model._latent(L, m, h[a:b].to(device=device, dtype=dtype), fb, kv, 0, i32(np.zeros(b - a), device),
                          splits=3 if b - a == 1 else 1)     # single rows: keys dealt to three workgroups and merged
        got[a:b] = model._dense(ops.linear(o.contiguous(), L.wo)).float().cpu()
    assert rel(got, want) < (1e-4 if dtype == torch.float32 else 4e-2)
