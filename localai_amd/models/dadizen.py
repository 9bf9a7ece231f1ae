"""Dadizen: a decoder-only design described layer by layer in its config.json.

A layer is post-normed on both sides of each sublayer, x <- x + n1b(mixer(n1 x)), x <- x +
n2b(ff(n2 x)) (ff optional), with Dynamic-Tanh norms tanh(alpha x) * w + b (ops.norm_chain), and
ends with a per-layer token input: a slice of a second embedding table, gated by gelu(Wg x),
projected, unit-normed and added (ops.side_gate).  A range of layers may run several times in a row
with the same weights (`loop`); every pass has its own cache / state, starts from W_in [x; x0] + a
per-pass vector, x0 being the embedding output.  Three mixers:

  * "attention": grouped-query softmax attention under a sliding window, interleaved rotary
    positions on the first rot.dims dims with YaRN frequency scaling (ops.rope_pages, ops.attn_mix);
  * "latent_attention": queries through a normed low-rank latent; keys and values from one normed
    latent row plus a rotated key part shared by all heads.  Only that row is cached (ops.latent_kv:
    a one-head pool whose rows are key and value at once); the per-head up-projections are applied
    to the query and to the attention output instead of to every cached token.  Causal, one sigmoid
    output gate per head;
  * "retention": linear attention with a fixed decay per head, rotate-half rotary positions, no
    softmax; its Dk x Dv state per head is per-sequence fp32 state in the scheduler's slot pool
    (ops.retention).

Feed-forward: clamped gated unit (ops.glu_clamp).  Output: the norm, the head, tanh soft cap.

The model plugs into LLMEngine like the other layer-list family: ForwardBatch, KVCache.layered (one
pool entry per layer RUN, so looped layers get a cache per pass), the native scheduler's block
tables and state slots; one query row per token, so prompt portions and decoded tokens of different
sequences share a forward (`mixed_batches`).  bf16 serving keeps the residual stream, norms,
rotations, scores, the recurrence and its inputs after projection in fp32; dtype=torch.float32
serves in true fp32 end to end.
"""
from __future__ import annotations

import os
from dataclasses import dataclass, field
from typing import Dict, List, Optional, Tuple

import numpy as np
import torch

from .. import ops
from ..gguf import dequantize
from .decoder import ForwardBatch, KVCache, TPInfo

# decode rows of softmax attention through the matrix-core tile kernel where the shape allows
DECODE_TILES = os.environ.get("LOCALAI_AMD_DADIZEN_DECODE_TILES", "1") == "1"
DECODE_WGS = int(os.environ.get("LOCALAI_AMD_DADIZEN_DECODE_WGS", "1024"))


@dataclass
class RotSpec:
    dims: int
    base: float
    scaling: Optional[dict] = None      # {"factor", "original", "fast", "slow"} (YaRN)


@dataclass
class MixSpec:
    kind: str                # "attention" | "latent_attention" | "retention"
    heads: int
    dim: int                 # query / key width per head (latent attention: the unrotated part)
    vdim: int
    rot: RotSpec
    kv_heads: int = 0        # attention
    scale: float = 1.0       # attention, latent attention
    window: int = 0          # attention: keys i - window < j <= i (0: all)
    rot_dim: int = 0         # latent attention: rotated query / key width
    q_rank: int = 0
    kv_rank: int = 0
    decay: Tuple[float, ...] = ()   # retention, per head


@dataclass
class FfSpec:
    ff: int
    limit: float


@dataclass
class DadizenHParams:
    n_vocab: int
    n_embd: int
    norm_eps: float
    mixers: List[MixSpec] = field(default_factory=list)
    mlps: List[Optional[FfSpec]] = field(default_factory=list)
    loop: Optional[Tuple[int, int, int]] = None     # (start, stop, times)
    side_dim: int = 0
    logit_softcap: float = 0.0
    arch: str = "dadizen"
    name: str = ""

    @property
    def n_layer(self) -> int:
        return len(self.mixers)

    @property
    def runs(self) -> List[Tuple[int, int]]:
        """(layer, pass) in execution order; pass -1 outside the loop."""
        n = self.n_layer
        if not self.loop:
            return [(i, -1) for i in range(n)]
        a, b, times = self.loop
        return ([(i, -1) for i in range(a)] + [(i, t) for t in range(times) for i in range(a, b)]
                + [(i, -1) for i in range(b, n)])

    @staticmethod
    def _rot(r: dict) -> RotSpec:
        return RotSpec(int(r["dims"]), float(r["base"]), dict(r["scaling"]) if r.get("scaling") else None)

    @staticmethod
    def from_config(c: dict, name: str = "") -> "DadizenHParams":
        hp = DadizenHParams(n_vocab=int(c["vocab"]), n_embd=int(c["width"]), norm_eps=float(c["norm"]["eps"]),
                            side_dim=int((c.get("token_side") or {}).get("dim") or 0),
                            logit_softcap=float(c.get("logit_softcap") or 0.0), name=name)
        for i, L in enumerate(c["layers"]):
            m, kind = L["mixer"], L.get("type")
            if kind == "attention":
                hp.mixers.append(MixSpec(kind, int(m["heads"]), int(m["dim"]), int(m.get("vdim") or m["dim"]),
                                         hp._rot(m["rot"]), kv_heads=int(m.get("kv_heads") or m["heads"]),
                                         scale=float(m["scale"]), window=int((m.get("mask") or {}).get("size") or 0)))
            elif kind == "latent_attention":
                hp.mixers.append(MixSpec(kind, int(m["heads"]), int(m["dim"]), int(m.get("vdim") or m["dim"]),
                                         hp._rot(m["rot"]), scale=float(m["scale"]), rot_dim=int(m["rot_dim"]),
                                         q_rank=int(m["q_rank"]), kv_rank=int(m["kv_rank"])))
            elif kind == "retention":
                hp.mixers.append(MixSpec(kind, int(m["heads"]), int(m["dim"]), int(m.get("vdim") or m["dim"]),
                                         hp._rot(m["rot"]), decay=tuple(float(d) for d in m["decay"])))
            else:
                raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
            f = L.get("mlp")
            if not f:
                hp.mlps.append(None)
            elif f.get("kind") == "dense":
                hp.mlps.append(FfSpec(int(f["ff"]), float(f["limit"])))
            else:
                raise ValueError(f"layer {i}: unknown feed-forward kind {f.get('kind')!r}")
        lp = c.get("loop")
        if lp and int(lp.get("times", 1)) >= 1 and int(lp["stop"]) > int(lp["start"]):
            hp.loop = (int(lp["start"]), int(lp["stop"]), int(lp["times"]))
            if not 0 <= hp.loop[0] < hp.loop[1] <= hp.n_layer:
                raise ValueError("loop: start / stop outside the layer list")
        return hp


@dataclass
class _Layer:
    norm1: tuple
    norm1b: tuple
    win: ops.QWeight                   # fused input projections of the mixer (see _load_mixer)
    wo: ops.QWeight
    freqs: torch.Tensor                # rotation frequencies fp32 [rot / 2]
    mag: float
    norm2: Optional[tuple] = None
    norm2b: Optional[tuple] = None
    gate_up: Optional[ops.QWeight] = None
    down: Optional[ops.QWeight] = None
    side_gate: Optional[ops.QWeight] = None
    side_proj: Optional[ops.QWeight] = None
    side_norm: Optional[torch.Tensor] = None
    decay: Optional[torch.Tensor] = None        # retention: fp32 [H]
    dq_norm: Optional[torch.Tensor] = None      # latent attention
    dkv_norm: Optional[torch.Tensor] = None
    uq: Optional[ops.QWeight] = None
    uk: Optional[torch.Tensor] = None           # [H, dim, kv_rank] activation dtype
    uv_t: Optional[torch.Tensor] = None         # [H, kv_rank, vdim]


class DadizenModel:
    # what this family launches from ops/csrc (ops.require_kernels: a first run compiles only these)
    kernel_sources = ("elementwise.hip", "norm_chain.hip", "rope_pages.hip", "retention.hip", "attention_mix.hip",
                      "attention.hip", "attention_latent.hip", "sampling.hip", "decode_loop.hip", "gemm_skinny.hip")
    stateful = True         # retention state per sequence: state slots, no prefix-cache reuse
    mixed_batches = True    # prompt portions and decode rows of different sequences in one forward

    def __init__(self, reader, device: torch.device, tp: Optional[TPInfo] = None, max_pos: Optional[int] = None,
                 rope_overrides: Optional[dict] = None, lora=None, dtype: torch.dtype = torch.bfloat16):
        self.tp = tp or TPInfo()
        if self.tp.world > 1:
            raise ValueError("dadizen: tensor parallelism is not implemented for this design")
        if lora is not None:
            raise ValueError("dadizen: LoRA adapters are not supported")
        if dtype not in (torch.bfloat16, torch.float32):
            raise ValueError("dadizen: serving dtype is bfloat16 or float32")
        self.device, self.dtype = device, dtype
        self.f32 = dtype == torch.float32
        self.hp = hp = DadizenHParams.from_config(reader.config, str(reader.kv.get("general.name", "")))
        self.max_pos = max_pos or 1 << 20
        self.vocab_local = hp.n_vocab
        self.T = reader.tensors
        D = hp.n_embd
        raw, f32, qw = self._raw, self._f32, self._qw
        emb = raw("embed")
        if tuple(emb.shape) != (hp.n_vocab, D):
            raise ValueError("dadizen: embed shape does not fit config vocab / width")
        self.tok_embd = ops.QWeight.from_float(emb.to(device))      # bf16 table, exact: stored as bf16
        self.side_table = None
        if hp.side_dim:
            st = raw("side.embed")
            if tuple(st.shape) != (hp.n_vocab, hp.n_layer * hp.side_dim):
                raise ValueError("dadizen: side.embed shape does not fit token_side.dim x layers")
            self.side_table = st.to(device=device, dtype=torch.bfloat16).contiguous()
        self.loop_in = self.loop_step = None
        if hp.loop:
            self.loop_in = qw(self._shaped("loop.in", (D, 2 * D)))
            self.loop_step = self._shaped("loop.step", (hp.loop[2], D)).to(device).contiguous()
        self.layers: List[_Layer] = []
        for i, (m, f) in enumerate(zip(hp.mixers, hp.mlps)):
            p = f"l{i}."
            L = self._load_mixer(p, m)
            L.norm1, L.norm1b = self._dyt(p + "norm1"), self._dyt(p + "norm1b")
            if f is not None:
                L.norm2, L.norm2b = self._dyt(p + "norm2"), self._dyt(p + "norm2b")
                L.gate_up = qw(torch.cat([self._shaped(p + "mlp.gate", (f.ff, D)), self._shaped(p + "mlp.up", (f.ff, D))], 0))
                L.down = qw(self._shaped(p + "mlp.down", (D, f.ff)))
            if hp.side_dim:
                L.side_gate = qw(self._shaped(p + "side.gate", (hp.side_dim, D)))
                L.side_proj = qw(self._shaped(p + "side.proj", (D, hp.side_dim)))
                L.side_norm = f32(p + "side.norm")
            self.layers.append(L)
        self.out_norm = self._dyt("final.norm")
        self.output = qw(self._shaped("head", (hp.n_vocab, D)))
        self._aranges: Dict[int, tuple] = {}
        self.T = None

    # --------------------------------------------------------------------------- loading
    def _raw(self, name: str) -> torch.Tensor:
        if name not in self.T:
            raise KeyError(f"dadizen: missing tensor {name}")
        t = self.T[name]
        return torch.from_numpy(dequantize(t.data, t.ggml_type, t.shape).astype(np.float32).reshape(t.shape))

    def _shaped(self, name: str, shape) -> torch.Tensor:
        w = self._raw(name)
        if tuple(w.shape) != tuple(shape):
            raise ValueError(f"dadizen: {name} is {tuple(w.shape)}, the config asks for {tuple(shape)}")
        return w

    def _f32(self, name: str) -> torch.Tensor:
        return self._raw(name).to(self.device).contiguous()

    def _qw(self, w: torch.Tensor) -> ops.QWeight:
        w = w.to(self.device)
        return ops.QWeight.from_f32(w) if self.f32 else ops.QWeight.from_float(w)

    def _dyt(self, name: str) -> tuple:
        return ("dyt", float(self._raw(name + ".alpha").reshape(-1)[0]), self._f32(name), self._f32(name + ".b"))

    def _load_mixer(self, p: str, m: MixSpec) -> _Layer:
        D, H = self.hp.n_embd, m.heads
        sh = self._shaped
        freqs, mag = ops.rot_freqs(m.rot.dims, m.rot.base, m.rot.scaling, self.device)
        if m.kind == "attention":
            if H % m.kv_heads:
                raise ValueError(f"{p}: heads must be a multiple of kv_heads")
            if m.rot.dims > m.dim or m.rot.dims % 2:
                raise ValueError(f"{p}: rot.dims must be even and at most dim")
            win = torch.cat([sh(p + "mix.q", (H * m.dim, D)), sh(p + "mix.k", (m.kv_heads * m.dim, D)),
                             sh(p + "mix.v", (m.kv_heads * m.vdim, D))], 0)
            return _Layer(None, None, self._qw(win), self._qw(sh(p + "mix.o", (D, H * m.vdim))), freqs, mag)
        if m.kind == "retention":
            if len(m.decay) != H or m.rot.dims > m.dim or m.rot.dims % 2:
                raise ValueError(f"{p}: decay per head, rot.dims even and at most dim")
            win = torch.cat([sh(p + "mix.q", (H * m.dim, D)), sh(p + "mix.k", (H * m.dim, D)),
                             sh(p + "mix.v", (H * m.vdim, D)), sh(p + "mix.g", (H * m.vdim, D))], 0)
            L = _Layer(None, None, self._qw(win), self._qw(sh(p + "mix.o", (D, H * m.vdim))), freqs, mag)
            L.decay = torch.tensor(m.decay, dtype=torch.float32, device=self.device)
            return L
        # latent attention: one fused down-projection [query latent | kv latent + rotated key | head gates]
        if m.rot.dims != m.rot_dim or m.rot_dim % 2:
            raise ValueError(f"{p}: rot.dims must equal rot_dim (even)")
        win = torch.cat([sh(p + "mix.dq", (m.q_rank, D)), sh(p + "mix.dkv", (m.kv_rank + m.rot_dim, D)),
                         sh(p + "mix.g", (H, D))], 0)
        L = _Layer(None, None, self._qw(win), self._qw(sh(p + "mix.o", (D, H * m.vdim))), freqs, mag)
        L.dq_norm, L.dkv_norm = self._f32(p + "mix.dq.norm"), self._f32(p + "mix.dkv.norm")
        L.uq = self._qw(sh(p + "mix.uq", (H * (m.dim + m.rot_dim), m.q_rank)))
        L.uk = sh(p + "mix.uk", (H * m.dim, m.kv_rank)).view(H, m.dim, m.kv_rank).to(self.device, self.dtype).contiguous()
        L.uv_t = (sh(p + "mix.uv", (H * m.vdim, m.kv_rank)).view(H, m.vdim, m.kv_rank).transpose(1, 2)
                  .to(self.device, self.dtype).contiguous())
        return L

    # --------------------------------------------------------------------------- engine interface
    def _run_specs(self):
        """KVCache.layered spec of every layer run."""
        out = []
        for i, _ in self.hp.runs:
            m = self.hp.mixers[i]
            if m.kind == "attention":
                out.append((m.kv_heads, m.dim, m.vdim, None))
            elif m.kind == "latent_attention":
                out.append((1, m.kv_rank + m.rot_dim, 0, None))
            else:
                out.append((0, 0, 0, (m.heads, m.vdim, m.dim), torch.float32))
        return out

    def kv_bytes_per_token(self) -> int:
        es = 4 if self.f32 else 2
        return max(es, sum(g * (dk + dv) * es for g, dk, dv, *_ in self._run_specs()))

    def new_kv_cache(self, num_blocks: int, block_size: int, state_slots: int = 0) -> KVCache:
        return KVCache.layered(self._run_specs(), num_blocks, block_size, self.device, self.dtype, state_slots)

    def decode_workspace(self, Bp: int, ctx: int, block_size: int):
        """Split-KV buffers of the decode attention kernel per (heads, kv heads, width) of the layers it serves."""
        out = {}
        for m in self.hp.mixers:
            if m.kind == "attention" and self._decode_kernel_ok(m, block_size):
                key = (m.heads, m.kv_heads, m.dim)
                if key not in out:
                    out[key] = ops.decode_workspace(Bp, m.heads, m.kv_heads, m.dim, ctx, self.device, block_size)
        return out or None

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
        """A projection's rows as one contiguous [T, N] matrix of the activation dtype."""
        t = p.t
        if p.bias is None and t.dim() == 3 and t.shape[0] == 1:
            t = t[0]
        elif p.bias is not None or t.dim() == 3:
            if t.is_cuda and p.N % 4 == 0:
                return ops.reduce(p, dtype=self.dtype)
            t = p.dense()
        return t if t.dtype == self.dtype else t.to(self.dtype)

    def _rms(self, x: torch.Tensor, w: torch.Tensor) -> torch.Tensor:
        """Rows of a projection slice divided by their root mean square, times w (fp32 inside)."""
        y = torch.empty(x.shape[0], x.shape[1], dtype=torch.float32, device=x.device)
        return ops.norm_chain(y, x.contiguous(), post=("rms", w, self.hp.norm_eps), pre=("cast",), replace=True,
                              out_dtype=self.dtype)

    def _decode_kernel_ok(self, m: MixSpec, block_size: int) -> bool:
        """Decode batches of this layer on the framework's split-KV decode attention kernel (the llama
        families'): bf16, equal key and value widths it is instantiated for; it takes the window."""
        return (not self.f32 and self.device.type == "cuda" and m.dim == m.vdim and m.dim in (64, 80, 96, 128, 192, 256)
                and m.heads // m.kv_heads <= 16 and block_size % 16 == 0 and (128 % block_size == 0 or block_size % 128 == 0)
                and ops._has("la_attn_decode"))

    def _attention(self, L: _Layer, m: MixSpec, xn, fb, kv, run, row_seq, cu_q, tiles, tile_rows, splits, ws=None):
        proj = self._dense(ops.linear(xn, L.win))
        q = ops.rope_pages(proj, m.heads, m.dim, m.kv_heads, m.dim, m.vdim, fb.pos, fb.slots, L.freqs, L.mag,
                           m.rot.dims, 0, True, kv.k[run], kv.v[run])
        if fb.decode and fb.seq_lens is not None and self._decode_kernel_ok(m, kv.block_size):
            T = q.shape[0]
            return ops.attn_decode(q.view(T, m.heads, m.dim), kv.k[run], kv.v[run], fb.block_tables, fb.seq_lens, m.scale,
                                   fb.max_len, workspace=ws, window=m.window).view(T, m.heads * m.vdim)
        return ops.attn_mix(q, kv.k[run], kv.v[run], row_seq, fb.pos, fb.block_tables, m.heads, m.scale,
                            window=m.window, tiles=tiles, tile_rows=tile_rows, cu_q=cu_q, key_splits=splits)

    def _latent(self, L: _Layer, m: MixSpec, xn, fb, kv, run, row_seq, splits: int = 1):
        T, H, r, dn, dr = xn.shape[0], m.heads, m.kv_rank, m.dim, m.rot_dim
        proj = self._dense(ops.linear(xn, L.win))                     # [T, q_rank | kv_rank + dr | H]
        cq = self._rms(proj[:, :m.q_rank], L.dq_norm)
        q = ops.rope_pages(self._dense(ops.linear(cq, L.uq)), H, dn + dr, 0, 0, 0, fb.pos, None, L.freqs, L.mag,
                           dr, dn, True).view(T, H, dn + dr)
        ops.latent_kv(proj[:, m.q_rank:m.q_rank + r + dr].contiguous(), r, L.dkv_norm, self.hp.norm_eps, fb.pos,
                      fb.slots, L.freqs, L.mag, kv.k[run])
        # the key up-projection moves to the query side: (W_uk c) . q = c . (W_uk^T q)
        qf = torch.empty(T, H, r + dr, dtype=self.dtype, device=xn.device)
        qf[:, :, :r] = torch.bmm(q[:, :, :dn].transpose(0, 1), L.uk).transpose(0, 1)
        qf[:, :, r:] = q[:, :, dn:]
        a = ops.attn_mix(qf.view(T, H * (r + dr)), kv.k[run], None, row_seq, fb.pos, fb.block_tables, H, m.scale,
                         gate=proj[:, m.q_rank + r + dr:], v_width=r, key_splits=splits)
        # ... and the value up-projection to the output side: sum_j p_j W_uv c_j = W_uv sum_j p_j c_j
        return torch.bmm(a.view(T, H, r).transpose(0, 1), L.uv_t).transpose(0, 1).reshape(T, H * m.vdim)

    def _retention(self, L: _Layer, m: MixSpec, xn, fb, kv, run, cu_q, sslots):
        proj = self._dense(ops.linear(xn, L.win))                     # [T, q | k | v | gate]
        return ops.retention(proj, m.heads, m.dim, m.vdim, fb.pos, cu_q, sslots, kv.state[run], L.decay, L.freqs,
                             m.rot.dims, self.hp.norm_eps, L.mag, max_rows=1 if fb.decode else fb.max_q)

    def forward(self, fb: ForwardBatch, kv: KVCache, attn_workspace=None, return_hidden: bool = False,
                local_logits: bool = False, layer_out: Optional[list] = None) -> torch.Tensor:
        """fp32 logits [R, V] of the rows fb.logits_idx selects (all rows when None).  Rows of one
        sequence are consecutive; fb.decode batches bring one row per sequence (fb.sslots per row),
        other batches fb.cu_q / fb.row_seq / fb.sslots per sequence.  layer_out: a list that
        receives the fp32 residual stream after every layer run (diagnostics)."""
        hp = self.hp
        T = fb.tokens.shape[0]
        if fb.sslots is None or (kv.state is None and any(m.kind == "retention" for m in hp.mixers)):
            raise ValueError("dadizen: the batch needs state slots (engine built without a state pool?)")
        if fb.decode:
            row_seq, cu_q, tiles = self._single_rows(T)
            tile_rows = T if (DECODE_TILES and not self.f32 and fb.tokens.is_cuda) else 0
            splits_for = lambda m: max(1, min(32, DECODE_WGS // max(T, 1), -(-(m.window or fb.max_len or 1) // 32)))  # noqa: E731
        else:
            row_seq, cu_q, tiles, tile_rows = fb.row_seq, fb.cu_q, fb.tiles, fb.tile_rows
            if row_seq is None:
                raise ValueError("dadizen: prompt batches need fb.row_seq")
            splits_for = lambda m: 1  # noqa: E731
        if fb.tokens.is_cuda and hp.n_embd % 8:   # the embedding kernel reads 8 columns per thread
            res = self.tok_embd.materialize_bf16().index_select(0, fb.tokens.long()).float()
        else:
            res = ops.embed(fb.tokens, self.tok_embd)
        if not res.is_contiguous() or res.dtype != torch.float32:
            res = res.float().contiguous()
        runs = hp.runs
        loop_at = hp.loop[0] if hp.loop else -1
        x0 = (res.clone() if self.f32 else res.to(self.dtype)) if hp.loop else None   # the embedding output (a bf16 table: exact)
        nc = lambda branch, post, pre, **kw: ops.norm_chain(res, branch, post, pre, out_dtype=self.dtype, **kw)  # noqa: E731

        def entry_norm(r: int):
            """What the boundary before run r hands on: the stream itself when a loop pass starts
            there (its input projection reads it), else the run's first norm."""
            if r >= len(runs):
                return self.out_norm
            i, t = runs[r]
            return ("cast",) if (t >= 0 and i == loop_at) else self.layers[i].norm1

        xn = nc(None, None, entry_norm(0))
        for r, (i, t) in enumerate(runs):
            L, m, f = self.layers[i], hp.mixers[i], hp.mlps[i]
            if t >= 0 and i == loop_at:
                y = ops.linear(torch.cat([xn, x0], 1), self.loop_in)
                xn = nc(y, None, L.norm1, add_vec=self.loop_step[t], replace=True)
            if m.kind == "attention":
                ws = attn_workspace.get((m.heads, m.kv_heads, m.dim)) if isinstance(attn_workspace, dict) else None
                a = self._attention(L, m, xn, fb, kv, r, row_seq, cu_q, tiles, tile_rows, splits_for(m), ws)
            elif m.kind == "latent_attention":
                a = self._latent(L, m, xn, fb, kv, r, row_seq, splits_for(m))
            else:
                a = self._retention(L, m, xn, fb, kv, r, cu_q, fb.sslots)
            o = ops.linear(a, L.wo)
            after = ("cast",) if L.side_gate is not None else entry_norm(r + 1)
            if f is not None:
                xn = nc(o, L.norm1b, L.norm2)
                h = ops.glu_clamp(ops.linear(xn, L.gate_up), f.ff, f.limit, out_dtype=self.dtype)
                xn = nc(ops.linear(h, L.down), L.norm2b, after)
            else:
                xn = nc(o, L.norm1b, after)
            if L.side_gate is not None:
                g = ops.side_gate(ops.linear(xn, L.side_gate), fb.tokens, self.side_table, i * hp.side_dim, self.dtype)
                xn = nc(ops.linear(g, L.side_proj), ("rms", L.side_norm, hp.norm_eps), entry_norm(r + 1))
            if layer_out is not None:
                layer_out.append(res.clone())
        if return_hidden:
            return xn
        rows = xn if fb.logits_idx is None else xn.index_select(0, fb.logits_idx)
        lp = ops.linear(rows.contiguous(), self.output)
        logits = lp.t[0] if (lp.t.dim() == 3 and lp.t.shape[0] == 1) else self._dense(lp).float()
        if hp.logit_softcap > 0:
            logits = torch.tanh(logits / hp.logit_softcap) * hp.logit_softcap
        return logits
