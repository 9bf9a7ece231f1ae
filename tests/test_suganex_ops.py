"""The Suganex mechanisms one by one -- operator layer (PyTorch CPU paths, HIP kernels under `gpu`)
against the plain functions of tests/suganex_oracle.py -- with inputs made so that a fault shows:
a single (query, key) pair whose score towers over the rest, at a far key, at a page border, just
inside and just outside a chunk; state slots holding another sequence's leftovers."""
import numpy as np
import pytest
import torch

import suganex_oracle as oracle
from localai_amd import ops
from localai_amd.native import core

MODES = [("cpu", torch.float32), ("cpu", torch.bfloat16),
         pytest.param("cuda:0", torch.float32, marks=pytest.mark.gpu),
         pytest.param("cuda:0", torch.bfloat16, marks=pytest.mark.gpu)]


def i32(x, dev):
    return torch.tensor(np.asarray(x), dtype=torch.int32, device=dev)


def rel(got, want):
    return float((got.float().cpu() - want).abs().max() / want.abs().max().clamp_min(1e-6))


def paged(T, BS, rng, extra=3):
    """A shuffled block table for T tokens (+ spare pages) and every token's slot."""
    nb = -(-T // BS)
    table = rng.permutation(nb + extra)[:nb]
    slots = [int(table[t // BS]) * BS + t % BS for t in range(T)]
    return nb + extra, table, slots


# --------------------------------------------------------------------------------------- short convolution
@pytest.mark.parametrize("device,dtype", MODES)
@pytest.mark.parametrize("taps", [2, 4])
def test_shortconv_portions_state_and_value_mix(device, dtype, taps):
    rng = np.random.default_rng(taps)
    g = torch.Generator().manual_seed(taps)
    H, G, Dk, Dv, BS = 3, 1, 8, 5, 8
    Cq, Ck, Cv = H * Dk, G * Dk, G * Dv
    C = Cq + Ck + Cv
    lens = {0: 11, 1: 6}
    u = {s: torch.randn(n, C + 2, generator=g).to(dtype).float() for s, n in lens.items()}   # 2 spare columns (gate)
    w = torch.randn(C, taps, generator=g)
    vfirst = {s: torch.randn(n, Cv, generator=g) for s, n in lens.items()}
    lam = torch.tensor([0.37])
    want = {s: oracle.short_conv(u[s][:, :C], w) for s in lens}
    nblk, tab0, slots0 = paged(11, BS, rng)
    tab1 = [b for b in range(nblk + 2) if b not in set(tab0.tolist())][:2]
    slots = {0: slots0, 1: [tab1[t // BS] * BS + t % BS for t in range(6)]}
    kc = ops.kv_pages(nblk + 2, G, BS, Dk, dtype, device)
    vc = ops.v_pages(nblk + 2, G, BS, Dv, dtype, device)
    # both state slots hold another sequence's leftovers: nothing before position 0 may be read
    state = torch.full((2, taps - 1, C), 1e4, dtype=dtype, device=device)
    wd = w.to(device)
    # steps: (sequence, start, n) batched together; single rows run the fused one-row path
    steps = [[(0, 0, 1), (1, 0, 3)], [(0, 1, 1)], [(0, 2, 5), (1, 3, 1)], [(1, 4, 2), (0, 7, 2)], [(0, 9, 1)], [(0, 10, 1)]]
    q_got = {s: torch.zeros(n, Cq) for s, n in lens.items()}
    for st in steps:
        rows = torch.cat([u[s][a:a + n] for s, a, n in st]).to(device=device, dtype=dtype)
        row_seq = np.repeat(np.arange(len(st)), [n for _, _, n in st])
        cu = np.concatenate([[0], np.cumsum([n for _, _, n in st])])
        pos = np.concatenate([np.arange(a, a + n) for _, a, n in st])
        sl = np.concatenate([slots[s][a:a + n] for s, a, n in st])
        vin = torch.cat([vfirst[s][a:a + n] for s, a, n in st]).to(device)
        single = all(n == 1 for _, _, n in st)
        vout = torch.empty(len(pos), Cv, device=device)
        q = ops.shortconv_kv(rows, wd, Cq, Ck, Cv, i32(row_seq, device), i32(cu, device), i32(pos, device), i32(sl, device),
                             i32([s for s, _, _ in st], device), state, kc, vc, vfirst_in=vin, vfirst_out=vout,
                             lam=lam.to(device), single=single)
        o = 0
        for s, a, n in st:
            q_got[s][a:a + n] = q[o:o + n].float().cpu()
            assert rel(vout[o:o + n], want[s][a:a + n, Cq + Ck:]) < 1e-5   # the unmixed v, fp32
            o += n
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    for s, n in lens.items():
        assert rel(q_got[s], want[s][:, :Cq]) < tol
        sl = torch.tensor(slots[s])
        k = kc.cpu().float()[sl // BS, :, sl % BS].reshape(len(sl), Ck)
        v = vc.cpu().float()[sl // BS, :, (sl % BS) // 8, :, sl % 8].reshape(len(sl), Cv)
        assert rel(k, want[s][:, Cq:Cq + Ck]) < tol
        assert rel(v, (1 - 0.37) * want[s][:, Cq + Ck:] + 0.37 * vfirst[s]) < tol
    # the state ends as the last taps - 1 projected rows of each sequence
    assert rel(state[0], u[0][11 - (taps - 1):, :C]) < 1e-6
    assert rel(state[1], u[1][6 - (taps - 1):, :C]) < 1e-6


# --------------------------------------------------------------------------------------- attention
def _attn_case(device, dtype, T, H, G, Dk, Dv, BS, chunk, softcap, scale, boost, seed):
    """Random q / K / V with optional boosted (query, key) pairs, through pages; all T rows at once
    (a prompt) and the last rows again one by one (decoding reads the same pool)."""
    rng = np.random.default_rng(seed)
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(T, H, Dk, generator=g)
    k = torch.randn(T, G, Dk, generator=g)
    v = torch.randn(T, G, Dv, generator=g)
    for (i, j, h) in boost:                      # q_h(i) and k(j) share a large component: s(i, j) towers
        d = torch.zeros(Dk)
        d[(i + j) % Dk] = 6.0
        q[i, h] += d / scale ** 0.5
        k[j, h // (H // G)] += d / scale ** 0.5
    q, k, v = (t.to(dtype).float() for t in (q, k, v))
    gate = torch.randn(T, H, generator=g).to(dtype).float()
    talk = torch.eye(H) + 0.25 * torch.randn(H, H, generator=g)
    want = oracle.attention(q, k, v, gate, talk, scale, softcap, chunk)
    nblk, table, slots = paged(T, BS, rng)
    kc = ops.kv_pages(nblk, G, BS, Dk, dtype, device)
    vc = ops.v_pages(nblk, G, BS, Dv, dtype, device)
    sl = torch.tensor(slots)
    kc[sl // BS, :, sl % BS] = k.to(device=device, dtype=dtype)
    vc[sl // BS, :, (sl % BS) // 8, :, sl % 8] = v.to(device=device, dtype=dtype)
    bt = i32([table.tolist(), table.tolist()], device)
    qd = q.reshape(T, H * Dk).to(device=device, dtype=dtype)
    # the gate rides in a wider matrix, as it does beside the projections
    wide = torch.zeros(T, H + 5, dtype=dtype, device=device)
    wide[:, 3:3 + H] = gate.to(device=device, dtype=dtype)
    args = dict(H=H, scale=scale, softcap=softcap, slopes=ops.alibi_slopes(H, device), talk=talk.to(device), chunk=chunk)
    got = ops.attn_mix(qd, kc, vc, i32([1] * T, device), i32(range(T), device), bt, gate=wide[:, 3:3 + H], **args)
    tol = 2e-5 if dtype == torch.float32 else 3e-2
    assert rel(got, want) < tol
    tail = list(range(max(0, T - 9), T))
    got1 = ops.attn_mix(qd[tail].contiguous(), kc, vc, i32([0] * len(tail), device), i32(tail, device), bt,
                        gate=wide[tail][:, 3:3 + H], **args)
    assert rel(got1, want[tail]) < tol
    return want, v


@pytest.mark.parametrize("device,dtype", MODES)
def test_attention_far_key_and_page_borders(device, dtype):
    # one chunk of 512: the last query's towering key lies 290 back, others sit on page borders
    T, BS = 300, 16
    boost = [(299, 9, 3), (298, 15, 3), (297, 16, 2), (200, 31, 3), (150, 32, 0), (64, 63, 1)]
    want, v = _attn_case(device, dtype, T, 4, 2, 16, 8, BS, 512, 0.0, 0.25, boost, 11)
    # the towering pair decides its head's output before the head mix smears it: the row moves a lot
    assert float(want[299].abs().max()) > 0.05


@pytest.mark.parametrize("device,dtype", MODES)
@pytest.mark.parametrize("chunk", [7, 24])
def test_attention_chunk_edges(device, dtype, chunk):
    # towering keys at the first position of the query's chunk (seen) and one before it (not seen),
    # for queries at a chunk's first, second and last position
    T = 4 * chunk + 3
    boost = []
    for c in (1, 2, 3):
        a = c * chunk
        boost += [(a, a, 0), (a, a - 1, 1), (a + 1, a, 2), (a + 1, a - 1, 3), (a + chunk - 1, a, 1), (a + chunk - 1, a - 1, 0)]
    _attn_case(device, dtype, T, 4, 4, 8, 8, 8, chunk, 30.0, 0.35, boost, 12)


@pytest.mark.parametrize("device,dtype", MODES)
def test_attention_shapes_that_the_usual_model_hides(device, dtype):
    # one kv head for six query heads, value wider than key, odd widths (no vector loads), no chunk
    _attn_case(device, dtype, 41, 6, 1, 5, 11, 8, 0, 4.0, 0.5, [(40, 0, 5)], 13)
    # one head: the head mix is a scalar
    _attn_case(device, dtype, 20, 1, 1, 8, 8, 8, 6, 0.0, 0.3, [], 14)


@pytest.mark.gpu
@pytest.mark.parametrize("H,G,Dk,Dv,BS,chunk,softcap", [(4, 2, 64, 32, 16, 40, 20.0), (16, 4, 128, 128, 32, 100, 30.0),
                                                      (32, 8, 64, 64, 8, 24, 0.0), (3, 1, 32, 16, 16, 0, 10.0),
                                                      (6, 6, 32, 48, 16, 33, 15.0)])
def test_attention_tile_kernel_portions(H, G, Dk, Dv, BS, chunk, softcap):
    """The matrix-core kernel on prompt portions that start mid-sequence (not on a tile, page or
    chunk border) beside single decode rows in the same launch, two sequences of unequal length,
    towering keys at the chunk's edges; against the oracle over the whole sequences."""
    dev, dtype = "cuda:0", torch.bfloat16
    rng = np.random.default_rng(H)
    g = torch.Generator().manual_seed(H)
    lens, starts = [151, 77, 60], [37, 0, 59]          # portion = rows [start, len); the third is one decode row
    scale = Dk ** -0.5
    talk = torch.eye(H) + 0.25 * torch.randn(H, H, generator=g)
    nblk = sum(-(-n // BS) for n in lens) + 2
    perm = rng.permutation(nblk)
    kc, vc = ops.kv_pages(nblk, G, BS, Dk, dtype, dev), ops.v_pages(nblk, G, BS, Dv, dtype, dev)
    maxb = max(-(-n // BS) for n in lens)
    bt = np.zeros((3, maxb), dtype=np.int32)
    qs, gates, wants, o = [], [], [], 0
    for s, (n, a) in enumerate(zip(lens, starts)):
        q, k, v = torch.randn(n, H, Dk, generator=g), torch.randn(n, G, Dk, generator=g), torch.randn(n, G, Dv, generator=g)
        c = chunk or n
        for i in (a, a + 1, n - 1):                      # towering keys: first of the chunk, one before it
            i = min(i, n - 1)
            for j, h in (((i // c) * c, 0), ((i // c) * c - 1, H - 1)):
                if j >= 0:
                    d = torch.zeros(Dk)
                    d[(i + j) % Dk] = 5.0
                    q[i, h] += d / scale ** 0.5
                    k[j, h // (H // G)] += d / scale ** 0.5
        q, k, v = (t.to(dtype).float() for t in (q, k, v))
        gate = torch.randn(n, H, generator=g).to(dtype).float()
        wants.append(oracle.attention(q, k, v, gate, talk, scale, softcap, chunk)[a:])
        tab = perm[o:o + -(-n // BS)]
        o += len(tab)
        bt[s, :len(tab)] = tab
        sl = torch.tensor([int(tab[t // BS]) * BS + t % BS for t in range(n)])
        kc[sl // BS, :, sl % BS] = k.to(device=dev, dtype=dtype)
        vc[sl // BS, :, (sl % BS) // 8, :, sl % 8] = v.to(device=dev, dtype=dtype)
        qs.append(q[a:].reshape(n - a, H * Dk))
        gates.append(gate[a:])
    rows = [n - a for n, a in zip(lens, starts)]
    qd = torch.cat(qs).to(device=dev, dtype=dtype)
    gd = torch.cat(gates).to(device=dev, dtype=dtype)
    row_seq = i32(np.repeat(np.arange(3), rows), dev)
    pos = i32(np.concatenate([np.arange(a, n) for n, a in zip(lens, starts)]), dev)
    cu = i32(np.concatenate([[0], np.cumsum(rows)]), dev)
    tiles, tile_rows = ops.attn_mix_tiles(rows[:2], dev)
    assert tile_rows == rows[0] + rows[1]
    args = dict(H=H, scale=scale, softcap=softcap, slopes=ops.alibi_slopes(H, dev), talk=talk.to(dev), chunk=chunk, gate=gd)
    got = ops.attn_mix(qd, kc, vc, row_seq, pos, i32(bt, dev), tiles=tiles, tile_rows=tile_rows, cu_q=cu, **args)
    ref = ops.attn_mix(qd, kc, vc, row_seq, pos, i32(bt, dev), **args)          # the row kernel alone
    want = torch.cat(wants)
    assert rel(got, want) < 3e-2 and rel(ref, want) < 3e-2
    assert rel(got, ref.float().cpu()) < 2e-2
    # every tile's keys dealt to several workgroups and merged (how decode batches run), the lone
    # decode row included as a one-row tile
    tiles_all, n_all = ops.attn_mix_tiles(rows, dev)
    for splits in (2, 5):
        got2 = ops.attn_mix(qd, kc, vc, row_seq, pos, i32(bt, dev), tiles=tiles_all, tile_rows=n_all, cu_q=cu,
                            key_splits=splits, **args)
        assert rel(got2, want) < 3e-2 and rel(got2, ref.float().cpu()) < 2e-2


@pytest.mark.gpu
def test_attention_many_heads_wide_values():
    # the accumulator and LDS limits of the kernel: 32 heads x 128 value channels
    _attn_case("cuda:0", torch.bfloat16, 70, 32, 8, 64, 128, 16, 32, 20.0, 0.125, [(69, 40, 7)], 15)


# --------------------------------------------------------------------------------------- experts
@pytest.mark.parametrize("device,dtype", MODES)
def test_router_correction_moves_the_choice_not_the_weights(device, dtype):
    g = torch.Generator().manual_seed(3)
    T, D, E, top = 37, 40, 7, 3
    x = torch.randn(T, D, generator=g).to(dtype)
    router = torch.randn(E, D, generator=g) * D ** -0.5
    corr = torch.zeros(E)
    corr[4] = 10.0                       # expert 4 is always chosen, whatever its score
    corr[0] = -10.0                      # expert 0 never
    ids, wts = ops.router_sigmoid(x.to(device), router.to(device), corr.to(device), top, True)
    idx, w = oracle.route(x.float(), router, corr, top)
    ids, wts = ids.cpu().long(), wts.cpu().view(T, top)
    assert (ids == 4).any(-1).all() and not (ids == 0).any()
    assert torch.equal(ids.sort(-1).values, idx.sort(-1).values)
    order = ids.argsort(-1)
    assert rel(wts.gather(1, order), w.gather(1, idx.argsort(-1))) < 1e-5
    assert float((wts.sum(-1) - 1).abs().max()) < 1e-5
    # without the correction the choice follows the scores alone
    ids0, _ = ops.router_sigmoid(x.to(device), router.to(device), None, top, True)
    assert torch.equal(ids0.cpu().long().sort(-1).values, oracle.route(x.float(), router, None, top)[0].sort(-1).values)


@pytest.mark.parametrize("device,dtype", MODES)
def test_routed_experts_and_dense_ff(device, dtype):
    g = torch.Generator().manual_seed(4)
    T, D, E, F, top = 9, 24, 5, 12, 2
    W = {"router": torch.randn(E, D, generator=g) * D ** -0.5, "correction": torch.randn(E, generator=g) * 0.2}
    for e in range(E):
        W[f"e{e}.gate"] = (torch.randn(F, D, generator=g) * D ** -0.5).to(dtype).float()
        W[f"e{e}.up"] = (torch.randn(F, D, generator=g) * D ** -0.5).to(dtype).float()
        W[f"e{e}.down"] = (torch.randn(D, F, generator=g) * F ** -0.5).to(dtype).float()
    x = torch.randn(T, D, generator=g).to(dtype)
    want = oracle.moe_ff(x.float(), W, "", E, top)
    ids, wts = ops.router_sigmoid(x.to(device), W["router"].to(device), W["correction"].to(device), top, True)
    st = lambda n: torch.stack([W[f"e{e}.{n}"] for e in range(E)]).to(device=device, dtype=dtype).contiguous()  # noqa: E731
    got = ops.moe_pairs(x.to(device), st("gate"), st("up"), st("down"), ids, wts)
    assert rel(got, want) < (1e-5 if dtype == torch.float32 else 2e-2)
    # squared ReLU
    up = (torch.randn(16, D, generator=g) * D ** -0.5)
    h = ops.act(ops.Partial((x.float() @ up.T).unsqueeze(0).to(device)), 16, ops.ACT_RELU2)
    assert rel(h, torch.relu(x.float() @ up.T) ** 2) < 1e-2


# --------------------------------------------------------------------------------------- scheduler
def test_scheduler_state_slots_and_explicit_plans():
    s = core.Scheduler(6, 4, 8, 64, 64, False, 0, 2)         # 6 pages of 4, 2 state slots
    s.add(1, [1, 2, 3, 4, 5], 0)
    s.add(2, [6, 7], 0)
    s.add(3, [8], 0)
    p = s.schedule_explicit([(2, 2), (1, 3)])
    assert p["p_ids"].tolist() == [2, 1] and p["p_decode"].tolist() == [0, 0]
    assert sorted(p["p_sslot"].tolist()) == [0, 1] and s.num_free_state_slots == 0
    with pytest.raises(RuntimeError):
        s.schedule_explicit([(3, 1)])                        # no state slot left; nothing changes
    p = s.schedule_explicit([(1, 1)])
    assert p["p_decode"].tolist() == [1] and p["p_pos"].tolist() == [3]
    slot2 = s.state_slot(2)
    s.finish(2)
    p = s.schedule_explicit([(3, 1), (1, 1)])                # a first token is a portion, not a decode row
    assert p["p_ids"].tolist() == [3, 1] and p["p_decode"].tolist() == [0, 1]
    assert s.state_slot(3) == slot2                          # the freed slot is taken over
    with pytest.raises(ValueError):
        s.schedule_explicit([(1, 1)])                        # sequence 1 has no tokens left
    s.extend(1, [9, 9, 9, 9])
    assert s.schedule_explicit([(1, 4)])["p_pos"].tolist() == [5, 6, 7, 8]
    # the ordinary planner waits for a state slot instead of failing
    s.add(4, [1, 2], 4)
    plan = s.schedule(1, False)
    assert 4 not in plan["p_ids"].tolist() and s.num_waiting == 1
    s.finish(3)
    assert s.schedule(1, False)["p_ids"].tolist() == [4]
