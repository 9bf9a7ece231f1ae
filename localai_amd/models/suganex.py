"""Suganex: a decoder-only design described layer by layer in its config.json.

Every layer is pre-norm, x <- x + mixer(norm1 x), x <- x + ff(norm2 x) (ff optional), with RMS norms
whose weights are stored around zero (y = x / rms(x) * (1 + w)).  The one mixer kind, "attention":

  * grouped-query attention with separate key and value widths and NO rotation;
  * a depthwise causal convolution of `conv` taps over time on the projected q, k and v
    (ops.shortconv_kv): its tail, the last conv - 1 projected rows of a sequence, is per-sequence
    state kept in a slot pool beside the paged K/V;
  * scores: scale q.k -> softcap tanh -> minus slope_h * distance (slope_h = 2^(-8 (h + 1) / H))
    -> mixed across heads by a learned H x H matrix -> visible within the query's chunk of
    `mask.size` positions -> softmax (ops.attn_mix);
  * value mixing across layers: layers flagged v_mix blend their v with the v of the FIRST flagged
    layer, v <- (1 - lambda) v + lambda v_first, before it is cached;
  * one sigmoid output gate per head, read from the mixer input.

Feed-forwards: dense, down(relu(up x)^2), or a mixture of gated SiLU experts routed by sigmoid
scores with a selection-only correction and normalised weights (ops.router_sigmoid).

The model plugs into LLMEngine like DecoderModel: same ForwardBatch, the engine's paged KV pool
(per-layer K/V widths: KVCache.layered), the native scheduler's block tables and state slots.
Because its kernels take one query row per token, a prompt portion and a single decoded token are
the same kind of row: `mixed_batches` lets the engine run portions and decode rows of different
sequences in ONE forward.  Serving dtype bf16 (fp32 residual, norms, scores, routers, like the
framework's other models) or true fp32 end to end (dtype=torch.float32).
"""
from __future__ import annotations

import os
from dataclasses import dataclass, field
from typing import Dict, List, Optional

import numpy as np
import torch

from .. import ops
from ..gguf import dequantize
from .decoder import ForwardBatch, KVCache, TPInfo

# batches of at most this many tokens (and every captured decode graph) run the routed experts as
# pair GEMVs; larger ones group rows by expert for library GEMMs (one host read of the grouping)
MOE_PAIR_MAX_T = 32
# ... and from this many tokens on, where the grouped expert GEMM kernels apply (see _moe)
MOE_DENSE_MIN_T = 6144
# decode rows through the matrix-core tile kernel (one-row tiles, split over the keys) instead of the row kernel
DECODE_TILES = os.environ.get("LOCALAI_AMD_SUGANEX_DECODE_TILES", "1") == "1"


# ... with the keys of a row dealt to about this many workgroups per batch
DECODE_WGS = int(os.environ.get("LOCALAI_AMD_SUGANEX_DECODE_WGS", "512"))


def res_is_cuda(fb) -> bool:
    return fb.tokens.is_cuda


@dataclass
class MixerSpec:
    heads: int
    kv_heads: int
    dim: int            # query / key width per head
    vdim: int           # value width per head
    taps: int           # short convolution taps (1: none)
    scale: float
    softcap: float      # 0: none
    chunk: int          # chunked causal mask size (0: plain causal)
    window: int         # sliding window (0: none)
    v_mix: bool

    @property
    def Cq(self) -> int:
        return self.heads * self.dim

    @property
    def Ck(self) -> int:
        return self.kv_heads * self.dim

    @property
    def Cv(self) -> int:
        return self.kv_heads * self.vdim


@dataclass
class MlpSpec:
    kind: str           # "dense" | "moe"
    ff: int
    experts: int = 0
    top: int = 0


@dataclass
class SuganexHParams:
    n_vocab: int
    n_embd: int
    norm_eps: float
    mixers: List[MixerSpec] = field(default_factory=list)
    mlps: List[Optional[MlpSpec]] = field(default_factory=list)
    arch: str = "suganex"
    name: str = ""

    @property
    def n_layer(self) -> int:
        return len(self.mixers)

    @staticmethod
    def from_config(c: dict, name: str = "") -> "SuganexHParams":
        hp = SuganexHParams(n_vocab=int(c["vocab"]), n_embd=int(c["width"]), norm_eps=float(c["norm"]["eps"]),
                            name=name)
        for i, L in enumerate(c["layers"]):
            if L.get("type") != "attention":
                raise ValueError(f"layer {i}: unknown mixer type {L.get('type')!r}")
            m = L["mixer"]
            mask = m.get("mask") or {}
            hp.mixers.append(MixerSpec(
                heads=int(m["heads"]), kv_heads=int(m.get("kv_heads") or m["heads"]), dim=int(m["dim"]),
                vdim=int(m.get("vdim") or m["dim"]), taps=int(m.get("conv") or 1), scale=float(m["scale"]),
                softcap=float(m.get("softcap") or 0.0), chunk=int(mask.get("size") or 0),
                window=int(mask.get("window") or 0), v_mix=bool(m.get("v_mix"))))
            f = L.get("mlp")
            if not f:
                hp.mlps.append(None)
            elif f["kind"] == "dense":
                hp.mlps.append(MlpSpec("dense", int(f["ff"])))
            elif f["kind"] == "moe":
                hp.mlps.append(MlpSpec("moe", int(f["expert"]["ff"]), int(f["router"]["experts"]),
                                       int(f["router"]["top"])))
            else:
                raise ValueError(f"layer {i}: unknown feed-forward kind {f['kind']!r}")
        return hp


@dataclass
class _Layer:
    norm1: torch.Tensor
    qkvg: ops.QWeight                 # [Cq + Ck + Cv + H, D]: q | k | v | gate rows
    conv: torch.Tensor                # [Cq + Ck + Cv, taps] fp32
    conv_t: torch.Tensor              # the same tap-major, [taps, Cq + Ck + Cv]
    lam: Optional[torch.Tensor]       # [1] fp32 (v_mix layers after the first)
    talk: torch.Tensor                # [H, H] fp32
    slopes: torch.Tensor              # [H] fp32
    wo: ops.QWeight
    norm2: Optional[torch.Tensor] = None
    up: Optional[ops.QWeight] = None
    down: Optional[ops.QWeight] = None
    router: Optional[torch.Tensor] = None
    corr: Optional[torch.Tensor] = None
    wg: Optional[torch.Tensor] = None          # [E, F, D] stacked expert weights (activation dtype)
    wu: Optional[torch.Tensor] = None
    wd: Optional[torch.Tensor] = None          # [E, D, F]
    experts: Optional[list] = None             # [(gate QWeight, up QWeight, down QWeight)]
    moe_gu: Optional[object] = None            # ops.MoEWeights of the fused gate|up / down projections, where
    moe_down: Optional[object] = None          # the grouped expert GEMM kernels take the shape (bf16, K % 256 == 0)


class SuganexModel:
    # what this family launches from ops/csrc (ops.require_kernels: a first run compiles only these)
    kernel_sources = ("elementwise.hip", "shortconv.hip", "attention_mix.hip", "moe_dense.hip", "moe.hip",
                      "sampling.hip", "decode_loop.hip", "gemm_skinny.hip")
    stateful = True         # per-sequence convolution tails: state slots, no prefix-cache reuse
    mixed_batches = True    # prompt portions and decode rows of different sequences in one forward

    def __init__(self, reader, device: torch.device, tp: Optional[TPInfo] = None, max_pos: Optional[int] = None,
                 rope_overrides: Optional[dict] = None, lora=None, dtype: torch.dtype = torch.bfloat16):
        self.tp = tp or TPInfo()
        if self.tp.world > 1:
            raise ValueError("suganex: tensor parallelism is not implemented for this design")
        if lora is not None:
            raise ValueError("suganex: LoRA adapters are not supported")
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("suganex: serving dtype is bfloat16 or float32")
        self.device, self.dtype = device, dtype
        self.f32 = dtype == torch.float32
        self.hp = hp = SuganexHParams.from_config(reader.config, str(reader.kv.get("general.name", "")))
        self.max_pos = max_pos or 1 << 20
        self.vocab_local = hp.n_vocab
        T = reader.tensors
        D = hp.n_embd

        def raw(name):
            if name not in T:
                raise KeyError(f"suganex: missing tensor {name}")
            t = T[name]
            return torch.from_numpy(dequantize(t.data, t.ggml_type, t.shape).astype(np.float32).reshape(t.shape))

        def f32(name):
            return raw(name).to(device).contiguous()

        def qw(w: torch.Tensor) -> ops.QWeight:
            w = w.to(device)
            return ops.QWeight.from_f32(w) if self.f32 else ops.QWeight.from_float(w)

        self.tok_embd = ops.QWeight.from_float(raw("embed").to(device))     # bf16 table, exact: stored as bf16
        if tuple(raw("embed").shape) != (hp.n_vocab, D):
            raise ValueError("suganex: embed shape does not fit config vocab / width")
        self.layers: List[_Layer] = []
        self.v_first_layer = next((i for i, m in enumerate(hp.mixers) if m.v_mix), -1)
        if len({m.Cv for m in hp.mixers if m.v_mix}) > 1:
            raise ValueError("suganex: layers that mix values must share kv_heads * vdim")
        for i, (m, f) in enumerate(zip(hp.mixers, hp.mlps)):
            p = f"l{i}."
            H = m.heads
            if m.heads % m.kv_heads:
                raise ValueError(f"layer {i}: heads must be a multiple of kv_heads")
            wq, wk, wv, wg = raw(p + "mix.q"), raw(p + "mix.k"), raw(p + "mix.v"), raw(p + "mix.g")
            if (tuple(wq.shape), tuple(wk.shape), tuple(wv.shape), tuple(wg.shape)) != (
                    (m.Cq, D), (m.Ck, D), (m.Cv, D), (H, D)):
                raise ValueError(f"layer {i}: projection shapes do not fit the config")
            if m.taps > 1 or p + "mix.q.conv" in T:      # one tap is a per-channel scale
                conv = torch.cat([raw(p + "mix.q.conv"), raw(p + "mix.k.conv"), raw(p + "mix.v.conv")], 0)
            else:
                conv = torch.ones(m.Cq + m.Ck + m.Cv, 1)
            if conv.shape[1] != m.taps:
                raise ValueError(f"layer {i}: convolution taps do not fit the config")
            lam = None
            if m.v_mix and i != self.v_first_layer:
                lam = raw(p + "mix.vmix").reshape(1).to(device).contiguous()
            L = _Layer(norm1=(1.0 + f32(p + "norm1")), qkvg=qw(torch.cat([wq, wk, wv, wg], 0)),
                       conv=conv.to(device).contiguous(), conv_t=conv.t().contiguous().to(device), lam=lam, talk=f32(p + "mix.talk"),
                       slopes=ops.alibi_slopes(H, device), wo=qw(raw(p + "mix.o")))
            if f is not None:
                L.norm2 = 1.0 + f32(p + "norm2")
            if f is not None and f.kind == "dense":
                L.up, L.down = qw(raw(p + "mlp.up")), qw(raw(p + "mlp.down"))
            elif f is not None:
                L.router = f32(p + "mlp.router")
                L.corr = f32(p + "mlp.correction") if p + "mlp.correction" in T else None
                g = torch.stack([raw(p + f"mlp.e{e}.gate") for e in range(f.experts)])
                u = torch.stack([raw(p + f"mlp.e{e}.up") for e in range(f.experts)])
                d = torch.stack([raw(p + f"mlp.e{e}.down") for e in range(f.experts)])
                if tuple(g.shape) != (f.experts, f.ff, D) or tuple(d.shape) != (f.experts, D, f.ff):
                    raise ValueError(f"layer {i}: expert shapes do not fit the config")
                L.wg, L.wu, L.wd = (t.to(device=device, dtype=dtype).contiguous() for t in (g, u, d))
                L.experts = [(qw(L.wg[e]), qw(L.wu[e]), qw(L.wd[e])) for e in range(f.experts)]
                if not self.f32 and device.type == "cuda" and D % 256 == 0 and f.ff % 256 == 0:
                    # the framework's grouped expert GEMMs (one weight stream per active expert, device
                    # routing, no host sync) read [gate; up] fused per expert
                    gu = torch.cat([L.wg, L.wu], 1).contiguous()
                    L.moe_gu = ops.MoEWeights([ops.QWeight.from_float(gu[e]) for e in range(f.experts)])
                    L.moe_down = ops.MoEWeights([d_ for _, _, d_ in L.experts])
            self.layers.append(L)
        self.out_norm = 1.0 + f32("final.norm")
        self.output = qw(raw("head"))
        self._aranges: Dict[int, tuple] = {}

    # --------------------------------------------------------------------------- engine interface
    def kv_bytes_per_token(self) -> int:
        es = 4 if self.f32 else 2
        return sum((m.Ck + m.Cv) * es for m in self.hp.mixers)

    def new_kv_cache(self, num_blocks: int, block_size: int, state_slots: int = 0) -> KVCache:
        return KVCache.layered([(m.kv_heads, m.dim, m.vdim, (m.taps - 1, m.Cq + m.Ck + m.Cv)) for m in self.hp.mixers],
                               num_blocks, block_size, self.device, self.dtype, state_slots)

    def decode_workspace(self, Bp: int, ctx: int, block_size: int):
        return None

    def prefill_tiles(self, q_lens, device):
        """(16-row work tiles of the leading prompt portions for ops.attn_mix, rows they cover)."""
        if device.type != "cuda" or self.f32:
            return None, 0
        return ops.attn_mix_tiles(q_lens, device)

    def _single_rows(self, T: int):
        """(row -> sequence, row ranges, one-row work tiles) of a batch with one row per sequence."""
        a = self._aranges.get(T)
        if a is None:
            r = torch.arange(T + 1, dtype=torch.int32, device=self.device)
            tiles = torch.stack([r[:T], torch.zeros_like(r[:T])], 1).contiguous()
            a = self._aranges[T] = (r[:T].contiguous(), r, tiles)
        return a

    # --------------------------------------------------------------------------- forward
    def _dense(self, p: ops.Partial) -> torch.Tensor:
        """A projection's rows as one [T, N] matrix of the activation dtype."""
        if p.t.dim() == 2 and p.bias is None:
            return p.t if p.t.dtype == self.dtype else p.t.to(self.dtype)
        if p.t.dim() == 3 and p.t.shape[0] == 1 and p.bias is None:
            return p.t[0] if self.f32 else p.t[0].to(self.dtype)
        if p.t.is_cuda and p.N % 4:       # the slab-sum kernel moves 4 columns per thread
            return p.dense().to(self.dtype)
        return ops.reduce(p, dtype=self.dtype)

    def _norm(self, res: torch.Tensor, add, w: torch.Tensor) -> torch.Tensor:
        if res.is_cuda and res.shape[1] % 4:   # widths the fused kernel does not take: the same steps unfused
            if add is not None:
                res += add.dense()
            y = res * torch.rsqrt(res.pow(2).mean(-1, keepdim=True) + self.hp.norm_eps) * w
            return y if self.f32 else y.to(torch.bfloat16)
        if not self.f32:
            return ops.add_norm(res, add, w, None, self.hp.norm_eps, 0)
        y = torch.empty_like(res)
        ops.add_norm(res, add, w, None, self.hp.norm_eps, 0, out_f32=y)
        return y

    def _act(self, p: ops.Partial, F: int, mode: int) -> torch.Tensor:
        if not self.f32 and (F % 4 == 0 or not p.t.is_cuda):
            return ops.act(p, F, mode)
        x = self._dense(p).float()
        y = torch.relu(x).square() if mode == ops.ACT_RELU2 else torch.nn.functional.silu(x[:, :F]) * x[:, F:2 * F]
        return y.to(self.dtype)

    def _moe(self, L: _Layer, f: MlpSpec, xn: torch.Tensor) -> ops.Partial:
        T = xn.shape[0]
        ids, wts = ops.router_sigmoid(xn, L.router, L.corr, f.top, True)
        capturing = xn.is_cuda and torch.cuda.is_current_stream_capturing()
        if L.moe_gu is not None and (T < MOE_DENSE_MIN_T or capturing) and T > 2:
            # grouped expert GEMMs on the routed rows, as the Mixtral path: gate|up, SiLU gating, then
            # the down projection whose routing-weighted slabs the next add_norm sums
            order, off = ops.moe_route(ids, f.experts)
            gu = ops.moe_linear(xn, L.moe_gu, order, off, f.top, T)
            h = ops.act(gu, f.ff, ops.ACT_SWIGLU)
            return ops.moe_linear(h, L.moe_down, order, off, f.top, T, down=True, wts=wts)
        if T <= MOE_PAIR_MAX_T or capturing:
            return ops.Partial(ops.moe_pairs(xn, L.wg, L.wu, L.wd, ids, wts).unsqueeze(0))
        # rows grouped by expert (device), one host read of the group offsets, then per expert
        # gate|up and down as library GEMMs over its rows and a weighted scatter-add in fp32
        order, off = ops.moe_route(ids, f.experts)
        off_h = off.cpu().tolist()
        order_l = order.long()
        tok = order_l // f.top
        xs = xn.index_select(0, tok)
        wsel = wts.index_select(0, order_l)
        out = torch.zeros(T, self.hp.n_embd, dtype=torch.float32, device=xn.device)
        with ops.blas_tuning_paused():
            for e in range(f.experts):
                r0, r1 = off_h[e], off_h[e + 1]
                if r1 <= r0:
                    continue
                g, u, d = L.experts[e]
                h = self._act(ops.linear_multi(xs[r0:r1].contiguous(), [g, u]), f.ff, ops.ACT_SWIGLU)
                y = self._dense(ops.linear(h, d)).float()
                out.index_add_(0, tok[r0:r1], y * wsel[r0:r1].unsqueeze(1))
        return ops.Partial(out.unsqueeze(0))

    def _mlp(self, L: _Layer, f: MlpSpec, xn: torch.Tensor) -> ops.Partial:
        if f.kind == "moe":
            return self._moe(L, f, xn)
        h = self._act(ops.linear(xn, L.up), f.ff, ops.ACT_RELU2)
        return ops.linear(h, L.down)

    def forward(self, fb: ForwardBatch, kv: KVCache, attn_workspace=None, return_hidden: bool = False,
                local_logits: bool = False, layer_out: Optional[list] = None) -> torch.Tensor:
        """fp32 logits [R, V] of the rows fb.logits_idx selects (all rows when None).  Rows of one
        sequence are consecutive; fb.decode batches bring one row per sequence (fb.sslots per row),
        other batches fb.cu_q / fb.row_seq / fb.sslots per sequence.  layer_out: a list that
        receives the fp32 residual stream after every layer (diagnostics)."""
        hp = self.hp
        T = fb.tokens.shape[0]
        if kv.state is None or fb.sslots is None:
            raise ValueError("suganex: the batch needs state slots (engine built without a state pool?)")
        if fb.decode:
            row_seq, cu_q, tiles = self._single_rows(T)
            tile_rows = T if (DECODE_TILES and not self.f32 and res_is_cuda(fb)) else 0
            single = True
            splits_for = lambda m: max(1, min(32, DECODE_WGS // max(T, 1), -(-(m.chunk or fb.max_len or 1) // 32)))  # noqa: E731
        else:
            row_seq, cu_q, tiles, tile_rows = fb.row_seq, fb.cu_q, fb.tiles, fb.tile_rows
            if row_seq is None:
                raise ValueError("suganex: prompt batches need fb.row_seq")
            single = False
            splits_for = lambda m: 1  # noqa: E731
        if fb.tokens.is_cuda and hp.n_embd % 8:   # the embedding kernel reads 8 columns per thread
            res = self.tok_embd.materialize_bf16().index_select(0, fb.tokens.long()).float()
        else:
            res = ops.embed(fb.tokens, self.tok_embd)
        if not res.is_contiguous() or res.dtype != torch.float32:
            res = res.float().contiguous()
        vfirst = None
        xn = self._norm(res, None, self.layers[0].norm1)
        n = len(self.layers)
        for i, (L, m, f) in enumerate(zip(self.layers, hp.mixers, hp.mlps)):
            C = m.Cq + m.Ck + m.Cv
            proj = self._dense(ops.linear(xn, L.qkvg))
            vin = vout = lam = None
            if m.v_mix and i == self.v_first_layer:
                vfirst = vout = torch.empty(T, m.Cv, dtype=torch.float32, device=res.device)
            elif m.v_mix:
                vin, lam = vfirst, L.lam
            q = ops.shortconv_kv(proj, L.conv, m.Cq, m.Ck, m.Cv, row_seq, cu_q, fb.pos, fb.slots, fb.sslots,
                                 kv.state[i], kv.k[i], kv.v[i], vfirst_in=vin, vfirst_out=vout, lam=lam, single=single,
                                 w_t=L.conv_t)
            a = ops.attn_mix(q, kv.k[i], kv.v[i], row_seq, fb.pos, fb.block_tables, m.heads, m.scale, m.softcap,
                             L.slopes, L.talk, m.chunk, m.window, gate=proj[:, C:C + m.heads],
                             tiles=tiles, tile_rows=tile_rows, cu_q=cu_q, key_splits=splits_for(m))
            o = ops.linear(a, L.wo)
            nxt = self.layers[i + 1].norm1 if i + 1 < n else self.out_norm
            if f is not None:
                xn = self._norm(res, o, L.norm2)
                o = self._mlp(L, f, xn)
            xn = self._norm(res, o, nxt)
            if layer_out is not None:
                layer_out.append(res.clone())
        if return_hidden:
            return xn
        rows = xn if fb.logits_idx is None else xn.index_select(0, fb.logits_idx)
        lp = ops.linear(rows.contiguous(), self.output)
        return self._dense(lp).float() if not (lp.t.dim() == 3 and lp.t.shape[0] == 1) else lp.t[0]
