"""Layer-list decoders: every layer names its token mixer (windowed attention with a softmax
sink, the Mamba-2 recurrence, latent attention, rotary grouped-query attention or fixed-decay
linear attention) and an optional feed-forward; a span of layers may run several times with shared
weights.  ``Dunesun``, ``Kisutar`` and ``Bitonex`` are the designs served; mixers are registered by
name (``MIXERS``) and feed-forward families by the design's ``ffn`` trait (``_ffn_for``), with their
sizes and constants read from the layer's spec, so another layer-list design can reuse them in
another order.  What a design fixes (block form, norm form, positions, token shift, depth average,
gated residual, rotation layout) is models/config.DESIGN_TRAITS.

Bitonex, per layer (sequential block): ``x += m * mixer(h) * sigmoid(R1 h + b1)`` with
``h = norm1(x)``, then the same with the feed-forward, ``norm2``, ``R2`` and ``b2`` (gated
residual; ``m`` = ``residual_mult``; a norm's weight is one number).  The gate's projection rides
as extra rows of the sublayer's own input projection (one GEMM), and the gated sum is folded into
the next norm's launch (ops.hybrid.gated_add_norm).  Its mixers: grouped-query attention with rotary
positions on part of each head, a temperature per head and a sigmoid output gate; linear attention
with a fixed decay per head as an fp32 recurrence over per-sequence state slots; latent attention
without window or sink.  Logits are soft-capped.

Kisutar, per layer (sequential block): ``x += mixer(shift(norm1(x)))``, then ``x += ff(norm2(x))``.
``shift`` moves every row towards the previous token's (per-channel learned fractions; the last
row of a sequence is state, one [d] fp32 vector per layer run and sequence slot).  The input of
layer i + 1 is a learned combination of the embedding output and the results of layers 0 .. i
(ops.hybrid.depth_mix; the results live in one fp32 stack [layers + 2, T, d]).  Its mixer is
latent attention: queries through a normed low-rank bottleneck; keys and values expanded per head
from one normed latent per token plus one rotated key part shared by all heads - only those two
are cached, and the per-head expansions are moved to the query side (the unrotated query is
multiplied into the latent space, the attention runs over the latent pages as one shared
key/value head, and the result is expanded to the value size afterwards), so prompt chunks and
decoding use the same pages and kernels as windowed attention.  A layer may read another layer's
pages (``kv_from``) with its own expansions.

Dunesun, per layer (parallel block): ``h = norm(x); x += mixer(h) + ff(h)`` with one one-plus
RMSNorm feeding both branches.  The residual stream is fp32 whatever the activation dtype, and the
branch sums of layer i are folded into layer i+1's norm launch (ops.hybrid.add_norm), like the
fused add + RMSNorm of the Llama path.  Looped layers: pass t starts with ``x += loop.step[t]``
(and ``x += embedding output`` for t > 0), folded into the same launch.

State: an attention run owns paged K ``[blocks, 16, heads*dim]`` and V ``[blocks, heads, vdim, 16]``
(activation dtype); a
Mamba-2 run owns per-sequence slots - the fp32 state ``[slots, heads, N, P]`` and the last
taps-1 convolution inputs.  Every RUN (a looped layer counts once per pass) has its own.

Dense projections go to the BLAS library (``F.linear``); everything else is ops.hybrid.
"""
from __future__ import annotations

import hashlib
import math
from typing import Optional

import torch
import torch.nn.functional as F

from .. import ops as _ops
from ..ops import hybrid as hops
from ..parallel.state import ParallelState, get_state
from .config import DenseSpec, HybridConfig, LayerSpec, MoESpec
from .llama import AttnMeta

BLOCK = 16  # tokens per cache page (engine/runner.BLOCK_SIZE)


def _seed_for(name: str, seed: int) -> int:
    h = hashlib.blake2b(f"{seed}:{name}".encode(), digest_size=8).digest()
    return int.from_bytes(h, "little") & 0x7FFF_FFFF_FFFF_FFFF


class _Params:
    """Creates a model's tensors: seeded random values per checkpoint name, or the checkpoint's."""

    def __init__(self, device, dtype, seed: int, src=None, empty: bool = False):
        self.device, self.dtype, self.seed, self.src, self.empty = device, dtype, seed, src, empty
        self.used: set = set()

    def rows_of(self, name: str, default: int) -> int:
        """Rows of a tensor whose first size no config key gives (a low-rank bottleneck): the
        checkpoint's, or ``default`` for a random-init model."""
        return int(self.src.get(name).shape[0]) if self.src is not None else int(default)

    def get(self, name: str, shape: tuple, std: float = 0.02, mean: float = 0.0, small: bool = False) -> torch.Tensor:
        """``small``: a vector or table the kernels read as fp32, kept fp32 on the device."""
        dt = torch.float32 if small else self.dtype
        if self.src is not None:
            t = self.src.get(name)
            if tuple(t.shape) != tuple(shape):
                raise ValueError(f"{name}: checkpoint shape {tuple(t.shape)}, config says {tuple(shape)}")
            self.used.add(name)
            return t.to(self.device, dt).contiguous()
        if self.empty:
            return torch.empty(shape, dtype=dt, device=self.device)
        g = torch.Generator().manual_seed(_seed_for(name, self.seed))
        t = torch.randn(shape, generator=g) * std + mean
        return t.to(torch.bfloat16).to(self.device, dt).contiguous()  # values a bf16 checkpoint could hold


class WindowAttention:
    """Grouped-query attention with a whole-projection RMSNorm of q and of k, no positional
    rotation, a sliding window of ``mask.size`` keys (0 / absent: unbounded) and a softmax sink."""

    kind = "attention"

    def __init__(self, spec: LayerSpec, d: int, eps: float, p: _Params, prefix: str, traits: Optional[dict] = None,
                 tail: Optional[torch.Tensor] = None):
        m = spec.m
        self.H, self.G, self.dk, self.dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
        if self.H % self.G:
            raise ValueError(f"{prefix}: heads {self.H} not a multiple of kv_heads {self.G}")
        self.scale = float(m.get("scale", 1.0 / math.sqrt(self.dk)))
        self.window = int(m.get("mask.size", 0) or 0)
        self.sink = bool(m.get("sink", True))
        self.eps = eps
        self.fast = 1  # 0: the any-size attention kernels only (ops.hybrid mfma / vec switches; tests)
        nq, nk, nv = self.H * self.dk, self.G * self.dk, self.G * self.dv
        s = 1.0 / math.sqrt(d)
        self.wqkv = torch.cat([p.get(prefix + "q", (nq, d), s), p.get(prefix + "k", (nk, d), s),
                               p.get(prefix + "v", (nv, d), s)]).contiguous()
        self.qn = p.get(prefix + "q.norm", (nq,), 0.1, 1.0, small=True)
        self.kn = p.get(prefix + "k.norm", (nk,), 0.1, 1.0, small=True)
        self.wo = p.get(prefix + "o", (d, self.H * self.dv), 1.0 / math.sqrt(self.H * self.dv))

    def new_cache(self, num_blocks: int, num_slots: int, dtype, device) -> dict:
        return {"k": torch.zeros(num_blocks, BLOCK, self.G * self.dk, dtype=dtype, device=device),
                "v": torch.zeros(num_blocks, self.G, self.dv, BLOCK, dtype=dtype, device=device)}

    def cache_bytes(self, esize: int) -> tuple:
        """(bytes per page, bytes per state slot)."""
        return BLOCK * self.G * (self.dk + self.dv) * esize, 0

    def forward(self, h: torch.Tensor, meta: AttnMeta, cache: dict) -> torch.Tensor:
        H, G, dk, dv = self.H, self.G, self.dk, self.dv
        qkv = F.linear(h, self.wqkv)
        kc, vc = cache["k"], cache["v"]
        hops.qk_norm_cache(qkv, self.qn, self.kn, self.eps, H, G, dk, dv, kc, vc, meta.slot_mapping)
        args = (H, G, dk, dv, self.scale, self.window, self.sink)
        if not meta.is_prefill:
            o = hops.window_attention_decode(qkv, kc, vc, meta.block_tables, meta.seq_lens, *args, vec=bool(self.fast))
        else:
            nd = meta.num_decode
            o = hops.window_attention_prefill(qkv[nd:], kc, vc, meta.cu_seqlens, meta.ctx_start, meta.block_tables,
                                              *args, mfma=self.fast)
            if nd:  # a mixed step: the single decode tokens in front go through the decode kernel
                od = hops.window_attention_decode(qkv[:nd], kc, vc, meta.dec_block_tables, meta.dec_seq_lens, *args,
                                                  vec=bool(self.fast))
                o = torch.cat([od, o])
        return F.linear(o, self.wo)


class Mamba2Mixer:
    """Mamba-2 (state-space duality) mixer: in-projection [z | x | B | C | dt], short causal
    convolution + SiLU over x, B, C, the fp32 recurrence per head, gate then grouped RMSNorm, and
    the out-projection."""

    kind = "mamba2"
    stateful = True

    def __init__(self, spec: LayerSpec, d: int, eps: float, p: _Params, prefix: str, traits: Optional[dict] = None,
                 tail: Optional[torch.Tensor] = None):
        m = spec.m
        self.nh, self.P, self.N = int(m["heads"]), int(m["vdim"]), int(m["state"])
        self.G, self.taps, self.ng = int(m.get("groups", 1)), int(m["conv"]), int(m.get("norm_groups", 1))
        self.inner = self.nh * self.P
        self.C = self.inner + 2 * self.G * self.N
        if self.nh % self.G or self.inner % self.ng or self.taps < 1:
            raise ValueError(f"{prefix}: heads/groups/norm_groups/conv do not fit")
        self.eps = eps
        self.w_in = p.get(prefix + "in", (self.inner + self.C + self.nh, d), 1.0 / math.sqrt(d))
        self.conv_w = p.get(prefix + "conv", (self.C, self.taps), 0.4, small=True)
        self.conv_b = p.get(prefix + "conv.b", (self.C,), 0.1, small=True)
        self.dt_bias = p.get(prefix + "dt_bias", (self.nh,), 0.5, -1.0, small=True)
        self.a_log = p.get(prefix + "A_log", (self.nh,), 0.5, -0.5, small=True)
        self.d_skip = p.get(prefix + "D", (self.nh,), 0.3, 1.0, small=True)
        self.norm_w = p.get(prefix + "norm", (self.inner,), 0.1, 1.0, small=True)
        self.wo = p.get(prefix + "o", (d, self.inner), 1.0 / math.sqrt(self.inner))

    def new_cache(self, num_blocks: int, num_slots: int, dtype, device) -> dict:
        return {"conv": torch.zeros(num_slots, max(1, self.taps - 1), self.C, dtype=dtype, device=device),
                "ssm": torch.zeros(num_slots, self.nh, self.N, self.P, dtype=torch.float32, device=device)}

    def cache_bytes(self, esize: int) -> tuple:
        return 0, (self.taps - 1) * self.C * esize + self.nh * self.N * self.P * 4

    def forward(self, h: torch.Tensor, meta: AttnMeta, cache: dict) -> torch.Tensor:
        proj = F.linear(h, self.w_in)
        seg = (meta.seg_cu, meta.seg_ctx, meta.seg_slot)
        xbc = hops.conv_silu(proj, self.inner, self.C, self.conv_w, self.conv_b, cache["conv"], *seg)
        y = hops.ssm_scan(xbc, proj, self.inner + self.C, self.dt_bias, self.a_log, self.d_skip, cache["ssm"], *seg,
                          self.nh, self.P, self.N, self.G)
        g = hops.gated_group_norm(y, proj, 0, self.norm_w, self.eps, self.ng, h.dtype)
        return F.linear(g, self.wo)


def _fresh_pages(meta: AttnMeta, T: int, device) -> tuple:
    """Temporary pages for a step of whole prompts: (slot of every row, block tables [S, W], blocks),
    every segment starting on a page of its own.  Computed once per step (cached on ``meta``), on the
    device, from the segment offsets."""
    got = getattr(meta, "_fresh_pages", None)
    if got is None:
        cu = meta.cu_seqlens.long()
        S = cu.numel() - 1
        nblk = (cu[1:] - cu[:-1] + BLOCK - 1) // BLOCK
        first = torch.cumsum(nblk, 0) - nblk  # a segment's first temporary block
        rows = torch.arange(T, device=device)
        seg = torch.bucketize(rows, cu[1:], right=True).clamp(max=S - 1)
        slots = (first[seg] * BLOCK + rows - cu[:-1][seg]).to(torch.int32)
        nb = T // BLOCK + S
        W = meta.block_tables.shape[1]
        bt = (first[:, None] + torch.arange(W, device=device)[None, :]).clamp(max=nb - 1).to(torch.int32)
        got = meta._fresh_pages = (slots, bt.contiguous(), nb)
    return got


class LatentAttention:
    """Attention over a compressed key/value stream (one normed latent of ``kv_rank`` and one
    rotated key part of ``rot_dim`` per token, shared by all heads), rotary positions on the
    ``rot_dim`` part of queries and keys, a sliding window (``mask.size``; 0 / absent: none) and -
    where the design has one - a learned per-head sink.  The design's ``latent`` trait fixes the
    rotation layout (``rotary`` "half" / "pairs") and ``sink``.
    ``kv_from``: j - no key/value projection of its own; reads layer j's pages.
    ``tail``: extra rows [n, d] for the down-projection; forward leaves their outputs in ``tail_out``
    (a [T, n] view) - the block's residual gate rides in the mixer's first GEMM.

    Two forms of the same attention.  Over the cache the per-head expansions are moved to the query
    side (module docstring): every step can take it.  A step of whole prompts (every chunk starts at
    position 0, no decode rows beside them; bf16, head sizes of the matrix-core kernel) of at least
    ``EXPAND_MIN_ROWS`` rows instead expands this step's keys ``[W_uk c | shared part]`` and values
    ``W_uv c`` per head into temporary pages and runs windowed attention's kernel over them:
    ``dim + rot_dim + vdim`` multiply-adds per (query, key, head) instead of ``2 kv_rank + rot_dim``."""

    kind = "latent_attention"
    EXPAND_MIN_ROWS = 1024

    def __init__(self, spec: LayerSpec, d: int, eps: float, p: _Params, prefix: str, traits: Optional[dict] = None,
                 tail: Optional[torch.Tensor] = None):
        m = spec.m
        lt = (traits or {}).get("latent", {})
        self.pairs = lt.get("rotary", "half") == "pairs"
        self.sink = bool(lt.get("sink", True))
        self.H, self.dn, self.dr, self.dv = int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"])
        self.Q, self.R = int(m["q_rank"]), int(m["kv_rank"])
        self.scale = float(m.get("scale", 1.0 / math.sqrt(self.dn + self.dr)))
        self.window = int(m.get("mask.size", 0) or 0)
        self.base, self.rdims = float(m.get("rot.base", 10000.0)), int(m.get("rot.dims", self.dr))
        if self.rdims % 2 or self.rdims > self.dr:
            raise ValueError(f"{prefix}: rot.dims {self.rdims} must be even and at most rot_dim {self.dr}")
        self.kv_from = m.get("kv_from")
        self.kv_from = None if self.kv_from is None else int(self.kv_from)
        self.eps = eps
        self.fast = 1
        self.pitch = (self.R + self.dr + 31) // 32 * 32
        H, dn, dr, dv, Q, R = self.H, self.dn, self.dr, self.dv, self.Q, self.R
        wd = [p.get(prefix + "dq", (Q, d), 1.0 / math.sqrt(d))]
        self.kn = None
        if self.kv_from is None:
            wd.append(p.get(prefix + "dkv", (R + dr, d), 1.0 / math.sqrt(d)))
            self.kn = p.get(prefix + "dkv.norm", (R,), 0.1, 1.0, small=True)
        self.n_down = sum(w.shape[0] for w in wd)
        self.n_tail = 0 if tail is None else tail.shape[0]
        if tail is not None:
            wd.append(tail)
        self.tail_out = None
        self.w_down = torch.cat(wd).contiguous()  # [q_rank (+ kv_rank + rot_dim) (+ tail), d]: one launch
        self.qn = p.get(prefix + "dq.norm", (Q,), 0.1, 1.0, small=True)
        self.w_uq = p.get(prefix + "uq", (H * (dn + dr), Q), 1.0 / math.sqrt(Q))
        self.w_uk = p.get(prefix + "uk", (H * dn, R), 1.0 / math.sqrt(R))  # viewed [H, dn, R]
        self.w_uv = p.get(prefix + "uv", (H * dv, R), 1.0 / math.sqrt(R))  # viewed [H, dv, R]
        self.sinks = p.get(prefix + "sink", (H,), 1.0, small=True) if self.sink else None
        self.freq = hops.rotary_freq(self.base, self.rdims, p.device)
        self.wo = p.get(prefix + "o", (d, H * dv), 1.0 / math.sqrt(H * dv))

    def new_cache(self, num_blocks: int, num_slots: int, dtype, device) -> dict:
        if self.kv_from is not None:
            return {}
        # key rows [latent | rotated part], padded with zeros to the matrix-core kernel's multiple of 32
        return {"k": torch.zeros(num_blocks, BLOCK, self.pitch, dtype=dtype, device=device),
                "v": torch.zeros(num_blocks, 1, self.R, BLOCK, dtype=dtype, device=device)}

    def cache_bytes(self, esize: int) -> tuple:
        return (0 if self.kv_from is not None else BLOCK * (self.pitch + self.R) * esize), 0

    def forward(self, h: torch.Tensor, meta: AttnMeta, cache: dict) -> torch.Tensor:
        H, dn, dr, dv, Q, R = self.H, self.dn, self.dr, self.dv, self.Q, self.R
        T = h.shape[0]
        down = F.linear(h, self.w_down)
        if self.n_tail:
            self.tail_out = (down, self.n_down)
            down = down[:, :self.n_down]
        kc, vc = cache["k"], cache["v"]
        own = self.kv_from is None
        hops.latent_prep(down, Q, R, dr, self.qn, self.kn, self.eps, meta.positions, self.freq,
                         kc if own else None, vc if own else None, meta.slot_mapping if own else None, pairs=self.pairs)
        q = F.linear(down[:, :Q], self.w_uq)
        if self._expand_ok(h, meta):
            return self._forward_expanded(q, down, meta, kc)
        # the per-head key expansion moved to the query: q_lat[h] = q_unrotated[h] @ W_uk[h]  ([H, T, R])
        q_lat = torch.bmm(q.view(T, H, dn + dr)[:, :, :dn].transpose(0, 1), self.w_uk.view(H, dn, R))
        qa = hops.latent_queries(q, q_lat, H, dn, dr, meta.positions, self.freq, self.pitch, pairs=self.pairs)
        args = (H, self.scale, self.window, self.sinks)
        kw = dict(fast=self.fast, sink=self.sink)
        if not meta.is_prefill:
            o = hops.latent_attention(qa, kc, vc, meta.block_tables, *args, seq_lens=meta.seq_lens, **kw)
        else:
            nd = meta.num_decode
            o = hops.latent_attention(qa[nd:], kc, vc, meta.block_tables, *args, cu=meta.cu_seqlens, ctx=meta.ctx_start, **kw)
            if nd:
                od = hops.latent_attention(qa[:nd], kc, vc, meta.dec_block_tables, *args, seq_lens=meta.dec_seq_lens, **kw)
                o = torch.cat([od, o])
        # ... and the value expansion to the result: v[h] = o_lat[h] @ W_uv[h]^T, written head by head
        # into the rows the out-projection reads
        v = torch.empty(T, H, dv, dtype=h.dtype, device=h.device)
        torch.bmm(o.view(T, H, R).transpose(0, 1), self.w_uv.view(H, dv, R).transpose(1, 2), out=v.transpose(0, 1))
        return F.linear(v.view(T, H * dv), self.wo)

    def _expand_ok(self, h: torch.Tensor, meta: AttnMeta) -> bool:
        return (meta.is_prefill and meta.all_fresh and not meta.num_decode and h.is_cuda and h.dtype == torch.bfloat16
                and bool(self.fast) and h.shape[0] >= self.EXPAND_MIN_ROWS
                and (self.dn + self.dr) in (64, 128) and self.dv in (64, 128))

    def _forward_expanded(self, q: torch.Tensor, down: torch.Tensor, meta: AttnMeta, kc: torch.Tensor) -> torch.Tensor:
        """Whole prompts: per-head keys and values of this step's rows in temporary pages, windowed
        attention's matrix-core kernel over them.  ``q`` [T, H * (dim + rot_dim)] still unturned."""
        H, dn, dr, dv, Q, R = self.H, self.dn, self.dr, self.dv, self.Q, self.R
        T, D = q.shape[0], self.dn + self.dr
        if self.kv_from is None:  # latent_prep left the normed latent and the turned shared part in place
            c, kr = down[:, Q:Q + R], down[:, Q + R:Q + R + dr]
        else:  # the other layer's, as its pages hold them
            rows = kc.view(-1, kc.shape[2]).index_select(0, meta.slot_mapping[:T].long())
            c, kr = rows[:, :R], rows[:, R:R + dr]
        fused = torch.empty(T, 2 * H * D + H * dv, dtype=q.dtype, device=q.device)  # [q | k | v], head by head
        fused[:, :H * D] = q
        kx = fused[:, H * D:2 * H * D].view(T, H, D)
        kx[:, :, :dn] = F.linear(c, self.w_uk).view(T, H, dn)
        kx[:, :, dn:] = kr.unsqueeze(1)
        fused[:, 2 * H * D:] = F.linear(c, self.w_uv)
        slots, bt, nb = _fresh_pages(meta, T, q.device)
        kt = torch.zeros(nb, BLOCK, H * D, dtype=q.dtype, device=q.device)
        vt = torch.zeros(nb, H, dv, BLOCK, dtype=q.dtype, device=q.device)
        # the queries' rotated parts turn here; the shared key part was turned by latent_prep
        hops.rotary_cache(fused, H, H, D, dv, meta.positions, self.freq, self.pairs, None, kt, vt, slots, rot_off=dn, rot_k=False)
        o = hops.window_attention_prefill(fused, kt, vt, meta.cu_seqlens, meta.ctx_start, bt, H, H, D, dv, self.scale,
                                          self.window, self.sink, mfma=self.fast, sinks=self.sinks)
        return F.linear(o, self.wo)


class RotaryAttention:
    """Grouped-query softmax attention with rotary positions on the first ``rot.dims`` entries of every
    query / key head (frequencies ``rot.base^(-2i/dims)``, optionally rescaled for long contexts by
    ``rot.scaling`` {factor, low, high, original}, ops.hybrid.rotary_freq).  Causal; ``mask.size`` keys
    of sliding window where given (0 / absent: all).  Pages and attention kernels are windowed
    attention's.  What a design fixes comes as ``opts`` (absent: the first value):

    * ``rotary`` "half" (entry i turns with entry i + rot.dims / 2) / "pairs" (2i with 2i + 1);
    * ``temp`` True: a learned temperature per query head (``temp``: score = q.k * scale * temp[h]),
      folded into the query in the rotation pass;
    * ``gate`` True: a sigmoid output gate ``heads * sigmoid(G h)`` in front of the out-projection;
    * ``qk_norm`` None / "before" (every q and k head RMS-normed over ``dim`` with the weights ``q.norm`` /
      ``k.norm`` [dim], then turned) / "after" (turned, then divided by its root mean square, no weight);
    * ``sink`` False / True: a learned logit per query head (``sink``) joins the softmax denominator;
    * ``values`` "own" (``v`` projection) / "keys" (the values are the keys as projected, before norm
      and turn; no ``v`` tensor, vdim = dim).

    ``tail``: extra rows for the input projection (see LatentAttention).  ``forward(..., proj=)``: the
    input projection computed by the caller (this mixer's columns of a wider GEMM)."""

    kind = "rotary_attention"

    def __init__(self, spec: LayerSpec, d: int, eps: float, p: _Params, prefix: str, traits: Optional[dict] = None,
                 tail: Optional[torch.Tensor] = None, opts: Optional[dict] = None):
        m = spec.m
        o = opts or {}
        self.H, self.G, self.dk = int(m["heads"]), int(m["kv_heads"]), int(m["dim"])
        self.v_from_k = o.get("values", "own") == "keys"
        self.dv = self.dk if self.v_from_k else int(m["vdim"])
        if self.H % self.G:
            raise ValueError(f"{prefix}: heads {self.H} not a multiple of kv_heads {self.G}")
        self.scale = float(m.get("scale", 1.0 / math.sqrt(self.dk)))
        self.window = int(m.get("mask.size", 0) or 0)
        self.base, self.rdims = float(m.get("rot.base", 10000.0)), int(m.get("rot.dims", self.dk))
        if self.rdims % 2 or not 0 <= self.rdims <= self.dk:
            raise ValueError(f"{prefix}: rot.dims {self.rdims} must be even and at most dim {self.dk}")
        self.pairs = o.get("rotary", (traits or {}).get("attention_rotary", "half")) == "pairs"
        self.norm = {None: 0, "before": 1, "after": 2}[o.get("qk_norm")]
        self.has_temp, self.has_gate, self.sink = bool(o.get("temp", True)), bool(o.get("gate", True)), bool(o.get("sink", False))
        self.eps = eps
        self.fast = 1
        nq, nk, nv = self.H * self.dk, self.G * self.dk, (0 if self.v_from_k else self.G * self.dv)
        s = 1.0 / math.sqrt(d)
        ws = [p.get(prefix + "q", (nq, d), s), p.get(prefix + "k", (nk, d), s)]
        if not self.v_from_k:
            ws.append(p.get(prefix + "v", (nv, d), s))
        if self.has_gate:
            ws.append(p.get(prefix + "g", (self.H * self.dv, d), s))
        self.g_col = nq + nk + nv
        self.n_in = self.g_col + (self.H * self.dv if self.has_gate else 0)
        self.n_tail = 0 if tail is None else tail.shape[0]
        if tail is not None:
            ws.append(tail)
        self.tail_out = None
        self.w_in = torch.cat(ws).contiguous()  # [q | k (| v) (| gate) (| tail)]: one launch
        self.temp = p.get(prefix + "temp", (self.H,), 0.2, 1.0, small=True) if self.has_temp else None
        self.qn = p.get(prefix + "q.norm", (self.dk,), 0.1, 1.0, small=True) if self.norm == 1 else None
        self.kn = p.get(prefix + "k.norm", (self.dk,), 0.1, 1.0, small=True) if self.norm == 1 else None
        self.sinks = p.get(prefix + "sink", (self.H,), 1.0, small=True) if self.sink else None
        sc = {k[len("rot.scaling."):]: v for k, v in m.items() if k.startswith("rot.scaling.")}
        self.freq = hops.rotary_freq(self.base, self.rdims, p.device, scaling=sc or None)
        self.wo = p.get(prefix + "o", (d, self.H * self.dv), 1.0 / math.sqrt(self.H * self.dv))

    def new_cache(self, num_blocks: int, num_slots: int, dtype, device) -> dict:
        return {"k": torch.zeros(num_blocks, BLOCK, self.G * self.dk, dtype=dtype, device=device),
                "v": torch.zeros(num_blocks, self.G, self.dv, BLOCK, dtype=dtype, device=device)}

    def cache_bytes(self, esize: int) -> tuple:
        return BLOCK * self.G * (self.dk + self.dv) * esize, 0

    def forward(self, h: torch.Tensor, meta: AttnMeta, cache: dict, proj: Optional[torch.Tensor] = None) -> torch.Tensor:
        H, G, dk, dv = self.H, self.G, self.dk, self.dv
        if proj is None:
            proj = F.linear(h, self.w_in)
        if self.n_tail:
            self.tail_out = (proj, self.n_in)
        kc, vc = cache["k"], cache["v"]
        hops.rotary_cache(proj, H, G, dk, dv, meta.positions, self.freq, self.pairs, self.temp, kc, vc, meta.slot_mapping,
                          norm=self.norm, qw=self.qn, kw=self.kn, eps=self.eps, v_from_k=self.v_from_k)
        args = (H, G, dk, dv, self.scale, self.window, self.sink)
        if not meta.is_prefill:
            o = hops.window_attention_decode(proj, kc, vc, meta.block_tables, meta.seq_lens, *args, vec=bool(self.fast),
                                             sinks=self.sinks)
        else:
            nd = meta.num_decode
            o = hops.window_attention_prefill(proj[nd:], kc, vc, meta.cu_seqlens, meta.ctx_start, meta.block_tables,
                                              *args, mfma=self.fast, sinks=self.sinks)
            if nd:
                od = hops.window_attention_decode(proj[:nd], kc, vc, meta.dec_block_tables, meta.dec_seq_lens, *args,
                                                  vec=bool(self.fast), sinks=self.sinks)
                o = torch.cat([od, o])
        if self.has_gate:
            o = hops.sigmoid_gate(o, proj, self.g_col)
        return F.linear(o, self.wo)

    def export(self, p: str) -> dict:
        nq, nk = self.H * self.dk, self.G * self.dk
        out = {p + "q": self.w_in[:nq], p + "k": self.w_in[nq:nq + nk], p + "o": self.wo}
        if not self.v_from_k:
            out[p + "v"] = self.w_in[nq + nk:self.g_col]
        if self.has_gate:
            out[p + "g"] = self.w_in[self.g_col:self.n_in]
        for key, t in (("temp", self.temp), ("q.norm", self.qn), ("k.norm", self.kn), ("sink", self.sinks)):
            if t is not None:
                out[p + key] = t
        return out


class LightningMixer:
    """Linear attention with a fixed decay per head: ``q, k, v = silu(projections)``; per head
    ``S_t = decay[h] S_(t-1) + k_t v_t^T``, ``o_t = S_t^T q_t`` (no other scale); all heads' outputs
    are RMS-normed together (weight ``norm``), multiplied by ``sigmoid(G h)`` and projected.  The
    state [heads, dim, vdim] is fp32, one per sequence slot, carried from step to step; it is the
    recurrence of ops.hybrid.ssm_scan with a constant decay, step size 1 and no skip term.
    ``tail``: extra rows for the input projection (see LatentAttention)."""

    kind = "lightning"
    stateful = True

    def __init__(self, spec: LayerSpec, d: int, eps: float, p: _Params, prefix: str, traits: Optional[dict] = None,
                 tail: Optional[torch.Tensor] = None):
        m = spec.m
        self.H, self.dk, self.dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
        dec = m["decay"]
        dec = [float(dec)] * self.H if isinstance(dec, (int, float)) else [float(x) for x in dec]
        if len(dec) != self.H:
            raise ValueError(f"{prefix}: {len(dec)} decays for {self.H} heads")
        self.eps = eps
        H, dk, dv = self.H, self.dk, self.dv
        s = 1.0 / math.sqrt(d)
        # rows [v | k | q | gate (| tail)]: the recurrence reads x, B, C = v, k, q in that order
        ws = [p.get(prefix + "v", (H * dv, d), s), p.get(prefix + "k", (H * dk, d), s), p.get(prefix + "q", (H * dk, d), s),
              p.get(prefix + "g", (H * dv, d), s)]
        self.n_act = H * dv + 2 * H * dk
        self.n_in = self.n_act + H * dv
        self.n_tail = 0 if tail is None else tail.shape[0]
        if tail is not None:
            ws.append(tail)
        self.tail_out = None
        self.w_in = torch.cat(ws).contiguous()
        self.decay = torch.tensor(dec, dtype=torch.float32, device=p.device)
        self.norm_w = p.get(prefix + "norm", (H * dv,), 0.1, 1.0, small=True)
        self.wo = p.get(prefix + "o", (d, H * dv), 1.0 / math.sqrt(H * dv))

    def new_cache(self, num_blocks: int, num_slots: int, dtype, device) -> dict:
        return {"state": torch.zeros(num_slots, self.H, self.dk, self.dv, dtype=torch.float32, device=device)}

    def cache_bytes(self, esize: int) -> tuple:
        return 0, self.H * self.dk * self.dv * 4

    def forward(self, h: torch.Tensor, meta: AttnMeta, cache: dict) -> torch.Tensor:
        proj = F.linear(h, self.w_in)
        if self.n_tail:
            self.tail_out = (proj, self.n_in)
        vkq = hops.activation_cols(proj, 0, self.n_act, "silu")
        o = hops.linear_attention(vkq, self.decay, cache["state"], meta.seg_cu, meta.seg_ctx, meta.seg_slot,
                                  self.H, self.dk, self.dv)
        g = hops.gated_group_norm(o, proj, self.n_act, self.norm_w, self.eps, 1, h.dtype, after=True)
        return F.linear(g, self.wo)


def _low_rank(p: _Params, prefix: str, name1: str, name2: str, n_out: int, d: int, default: int) -> tuple:
    """A two-stage projection ``W2 (W1 h)`` whose inner size only the tensors give."""
    r = p.rows_of(prefix + name1, default)
    return p.get(prefix + name1, (r, d), 1.0 / math.sqrt(d)), p.get(prefix + name2, (n_out, r), 1.0 / math.sqrt(r))


class GatedDeltaMixer:
    """The delta rule with a decay per head and key channel.  ``q, k`` ([kv_heads, dim]) and ``v``
    ([heads, vdim]) pass a short causal convolution per channel (``q.conv`` ... [channels, conv taps], no
    bias) and SiLU; q and k are made unit vectors per head and q is scaled by ``dim^-1/2``;
    ``beta = sigmoid(W_b h)`` per head; decays ``g = exp(-exp(A_log[h]) softplus(W_a2 (W_a1 h) + dt_bias))``
    per head and key channel.  Per head (reading q / k head ``h // (heads / kv_heads)``):
    ``S <- diag(g) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q``.  Each head's o is RMS-normed
    over vdim (weight ``norm`` [vdim], shared by the heads) and multiplied by ``sigmoid(W_g2 (W_g1 h))``,
    then projected.  State per sequence slot: S (fp32) and the last taps - 1 convolution inputs.
    Everything behind the convolution is fp32 (ops.hybrid.decay_scan)."""

    kind = "gated_delta"
    stateful = True

    def __init__(self, spec: LayerSpec, d: int, eps: float, p: _Params, prefix: str, traits: Optional[dict] = None,
                 tail: Optional[torch.Tensor] = None, opts: Optional[dict] = None):
        m = spec.m
        self.H, self.dk, self.dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
        self.Gk, self.taps = int(m.get("kv_heads", self.H)), int(m["conv"])
        if self.H % self.Gk or self.taps < 1:
            raise ValueError(f"{prefix}: heads {self.H} / kv_heads {self.Gk} / conv {self.taps} do not fit")
        self.eps = eps
        H, Gk, dk, dv = self.H, self.Gk, self.dk, self.dv
        s = 1.0 / math.sqrt(d)
        self.C = 2 * Gk * dk + H * dv  # convolved channels [q | k | v]
        wa1, self.wa2 = _low_rank(p, prefix, "a1", "a2", H * dk, d, int(m.get("a_rank", 16)))
        wg1, self.wg2 = _low_rank(p, prefix, "g1", "g2", H * dv, d, int(m.get("g_rank", 16)))
        self.ra, self.rg = wa1.shape[0], wg1.shape[0]
        # rows [q | k | v | beta | a1 | g1]: everything that reads the mixer's input, one launch
        self.w_in = torch.cat([p.get(prefix + "q", (Gk * dk, d), s), p.get(prefix + "k", (Gk * dk, d), s),
                               p.get(prefix + "v", (H * dv, d), s), p.get(prefix + "b", (H, d), s), wa1, wg1]).contiguous()
        self.b_col, self.a_col, self.g_col = self.C, self.C + H, self.C + H + self.ra
        self.conv_w = torch.cat([p.get(prefix + "q.conv", (Gk * dk, self.taps), 0.4, small=True),
                                 p.get(prefix + "k.conv", (Gk * dk, self.taps), 0.4, small=True),
                                 p.get(prefix + "v.conv", (H * dv, self.taps), 0.4, small=True)]).contiguous()
        self.a_log = p.get(prefix + "A_log", (H,), 0.5, -0.5, small=True)
        self.dt_bias = p.get(prefix + "dt_bias", (H * dk,), 0.5, -1.0, small=True)
        self.norm_w = p.get(prefix + "norm", (dv,), 0.1, 1.0, small=True)
        self.norm_all = self.norm_w.repeat(H).contiguous()  # the norm kernel reads one weight per column
        self.wo = p.get(prefix + "o", (d, H * dv), 1.0 / math.sqrt(H * dv))

    def new_cache(self, num_blocks: int, num_slots: int, dtype, device) -> dict:
        return {"conv": torch.zeros(num_slots, max(1, self.taps - 1), self.C, dtype=dtype, device=device),
                "state": torch.zeros(num_slots, self.H, self.dv, self.dk, dtype=torch.float32, device=device)}

    def cache_bytes(self, esize: int) -> tuple:
        return 0, (self.taps - 1) * self.C * esize + self.H * self.dk * self.dv * 4

    def forward(self, h: torch.Tensor, meta: AttnMeta, cache: dict, proj: Optional[torch.Tensor] = None) -> torch.Tensor:
        H, Gk, dk, dv = self.H, self.Gk, self.dk, self.dv
        if proj is None:
            proj = F.linear(h, self.w_in)
        seg = (meta.seg_cu, meta.seg_ctx, meta.seg_slot)
        qkv = hops.conv_silu(proj, 0, self.C, self.conv_w, None, cache["conv"], *seg)
        z = F.linear(proj[:, self.a_col:self.a_col + self.ra], self.wa2)
        gate = F.linear(proj[:, self.g_col:self.g_col + self.rg], self.wg2)
        o = hops.decay_scan(qkv, 0, Gk * dk, 2 * Gk * dk, z, self.dt_bias, cache["state"], *seg, H, Gk, dk, dv,
                            dk ** -0.5, a_log=self.a_log, beta=proj, beta_col=self.b_col, unit=True)
        g = hops.gated_group_norm(o, gate, 0, self.norm_all, self.eps, H, h.dtype, after=True)
        return F.linear(g, self.wo)

    def export(self, p: str) -> dict:
        n = self.Gk * self.dk
        w, cw = self.w_in, self.conv_w
        return {p + "q": w[:n], p + "k": w[n:2 * n], p + "v": w[2 * n:self.C], p + "b": w[self.b_col:self.a_col],
                p + "a1": w[self.a_col:self.g_col], p + "g1": w[self.g_col:self.g_col + self.rg], p + "a2": self.wa2,
                p + "g2": self.wg2, p + "q.conv": cw[:n], p + "k.conv": cw[n:2 * n], p + "v.conv": cw[2 * n:],
                p + "A_log": self.a_log, p + "dt_bias": self.dt_bias, p + "norm": self.norm_w, p + "o": self.wo}


class GatedLinearMixer:
    """Linear attention with a decay per head and key channel: ``q = W_q h * dim^-1/2``, ``k``, ``v`` per
    head; ``alpha = sigmoid(W_a2 (W_a1 h) + a2.b)^(1 / tau)``; per head ``S <- diag(alpha) S + k v^T``,
    ``o = S^T q``.  Each head's o is RMS-normed over vdim (weight ``norm`` [vdim], shared by the heads);
    the concatenated heads are multiplied by ``silu(W_g h)`` and projected.  The state S is fp32, one
    per sequence slot (ops.hybrid.decay_scan)."""

    kind = "gated_linear"
    stateful = True

    def __init__(self, spec: LayerSpec, d: int, eps: float, p: _Params, prefix: str, traits: Optional[dict] = None,
                 tail: Optional[torch.Tensor] = None, opts: Optional[dict] = None):
        m = spec.m
        self.H, self.dk, self.dv, self.tau = int(m["heads"]), int(m["dim"]), int(m["vdim"]), float(m.get("tau", 1.0))
        self.eps = eps
        H, dk, dv = self.H, self.dk, self.dv
        s = 1.0 / math.sqrt(d)
        wa1, self.wa2 = _low_rank(p, prefix, "a1", "a2", H * dk, d, int(m.get("a_rank", 16)))
        self.ra = wa1.shape[0]
        # rows [q | k | v | gate | a1]
        self.w_in = torch.cat([p.get(prefix + "q", (H * dk, d), s), p.get(prefix + "k", (H * dk, d), s),
                               p.get(prefix + "v", (H * dv, d), s), p.get(prefix + "g", (H * dv, d), s), wa1]).contiguous()
        self.g_col = 2 * H * dk + H * dv
        self.a_col = self.g_col + H * dv
        self.a_bias = p.get(prefix + "a2.b", (H * dk,), 0.5, 3.0, small=True)
        self.norm_w = p.get(prefix + "norm", (dv,), 0.1, 1.0, small=True)
        self.norm_all = self.norm_w.repeat(H).contiguous()
        self.wo = p.get(prefix + "o", (d, H * dv), 1.0 / math.sqrt(H * dv))

    def new_cache(self, num_blocks: int, num_slots: int, dtype, device) -> dict:
        return {"state": torch.zeros(num_slots, self.H, self.dv, self.dk, dtype=torch.float32, device=device)}

    def cache_bytes(self, esize: int) -> tuple:
        return 0, self.H * self.dk * self.dv * 4

    def forward(self, h: torch.Tensor, meta: AttnMeta, cache: dict, proj: Optional[torch.Tensor] = None) -> torch.Tensor:
        H, dk, dv = self.H, self.dk, self.dv
        if proj is None:
            proj = F.linear(h, self.w_in)
        z = F.linear(proj[:, self.a_col:self.a_col + self.ra], self.wa2)
        o = hops.decay_scan(proj, 0, H * dk, 2 * H * dk, z, self.a_bias, cache["state"], meta.seg_cu, meta.seg_ctx,
                            meta.seg_slot, H, H, dk, dv, dk ** -0.5, tau=self.tau)
        g = hops.gated_group_norm(o, proj, self.g_col, self.norm_all, self.eps, H, h.dtype, after=True, gate="silu")
        return F.linear(g, self.wo)

    def export(self, p: str) -> dict:
        n, w = self.H * self.dk, self.w_in
        return {p + "q": w[:n], p + "k": w[n:2 * n], p + "v": w[2 * n:self.g_col], p + "g": w[self.g_col:self.a_col],
                p + "a1": w[self.a_col:self.a_col + self.ra], p + "a2": self.wa2, p + "a2.b": self.a_bias,
                p + "norm": self.norm_w, p + "o": self.wo}


class SideBySide:
    """Two mixers on the same normed input, added with fixed weights: ``left_scale * left(h) +
    right_scale * right(h)``.  Which two, and what the design fixes for each, is the design's
    ``composite`` trait for the layer's ``type``; their constants sit under ``mixer.left`` /
    ``mixer.right`` and their tensors under ``mix.left.`` / ``mix.right.``.  Both input projections run
    as ONE GEMM (each mixer then reads its own columns); forward returns the two results with their
    weights, and the sum happens in fp32 in the launch of the next norm (ops.hybrid.sum_norm)."""

    kind = "side_by_side"

    def __init__(self, spec: LayerSpec, d: int, eps: float, p: _Params, prefix: str, traits: Optional[dict] = None,
                 tail: Optional[torch.Tensor] = None, opts: Optional[dict] = None):
        comp = (traits or {}).get("composite", {}).get(spec.kind)
        if comp is None:
            raise ValueError(f"{prefix}: the design names no pair of mixers for layers of type {spec.kind!r}")
        m = spec.m
        self.subs = []
        for side in ("left", "right"):
            kind, o = comp[side]
            self.subs.append(MIXERS[kind](spec.sub(side, kind), d, eps, p, f"{prefix}{side}.", traits=traits, opts=o))
        self.scales = (float(m.get("left_scale", 1.0)), float(m.get("right_scale", 1.0)))
        self.stateful = any(getattr(x, "stateful", False) for x in self.subs)
        self.n_left = nl = self.subs[0].w_in.shape[0]
        n = nl + self.subs[1].w_in.shape[0]
        # rows padded with zeros to a multiple of 8: the kernels' 16-byte accesses need aligned row strides
        pad = [torch.zeros(-n % 8, d, dtype=self.subs[0].w_in.dtype, device=self.subs[0].w_in.device)] if n % 8 else []
        self.w_in = torch.cat([x.w_in for x in self.subs] + pad).contiguous()
        self.subs[0].w_in, self.subs[1].w_in = self.w_in[:nl], self.w_in[nl:n]

    @property
    def fast(self) -> int:
        return getattr(self.subs[0], "fast", 1)

    @fast.setter
    def fast(self, v: int) -> None:
        for x in self.subs:
            if hasattr(x, "fast"):
                x.fast = v

    def new_cache(self, num_blocks: int, num_slots: int, dtype, device) -> dict:
        return {"left": self.subs[0].new_cache(num_blocks, num_slots, dtype, device),
                "right": self.subs[1].new_cache(num_blocks, num_slots, dtype, device)}

    def cache_bytes(self, esize: int) -> tuple:
        a, b = (x.cache_bytes(esize) for x in self.subs)
        return a[0] + b[0], a[1] + b[1]

    def forward(self, h: torch.Tensor, meta: AttnMeta, cache: dict) -> tuple:
        proj = F.linear(h, self.w_in)
        yl = self.subs[0].forward(h, meta, cache["left"], proj=proj[:, :self.n_left])
        yr = self.subs[1].forward(h, meta, cache["right"], proj=proj[:, self.n_left:self.n_left + self.subs[1].w_in.shape[0]])
        return (yl, self.scales[0]), (yr, self.scales[1])

    def export(self, p: str) -> dict:
        return {**self.subs[0].export(p + "left."), **self.subs[1].export(p + "right.")}


MIXERS = {WindowAttention.kind: WindowAttention, Mamba2Mixer.kind: Mamba2Mixer, LatentAttention.kind: LatentAttention,
          RotaryAttention.kind: RotaryAttention, LightningMixer.kind: LightningMixer,
          GatedDeltaMixer.kind: GatedDeltaMixer, GatedLinearMixer.kind: GatedLinearMixer, SideBySide.kind: SideBySide}


class RoutedFFN:
    """Top-k routed SwiGLU experts (biased fp32 router, softmax over the chosen logits) plus an
    optional shared expert scaled by sigmoid of a per-token gate.  The gate's weight row rides as
    one more row of the router matrix, so router logits and gate come out of one launch."""

    def __init__(self, spec: MoESpec, d: int, p: _Params, prefix: str):
        self.E, self.K, self.ff, self.fs = spec.experts, spec.top, spec.ff, spec.shared_ff
        if not 1 <= self.K <= self.E:
            raise ValueError(f"{prefix}: top {self.K} of {self.E} experts")
        s, s2 = 1.0 / math.sqrt(d), 1.0 / math.sqrt(self.ff)
        # gate / up rows interleaved per 128 ([64 gate | 64 up]): the layout of the prefill tile GEMM's
        # SwiGLU epilogue, which large bf16 steps on the GPU use (ops.hybrid.moe_experts); ONE copy
        self.il = (p.device.type == "cuda" and p.dtype == torch.bfloat16 and self.ff % 128 == 0 and d % 128 == 0)
        pair = _ops.interleave_gate_up if self.il else (lambda w: w)
        self.w13 = torch.stack([pair(torch.cat([p.get(f"{prefix}e{e}.gate", (self.ff, d), s),
                                                p.get(f"{prefix}e{e}.up", (self.ff, d), s)])) for e in range(self.E)])
        self.w2 = torch.stack([p.get(f"{prefix}e{e}.down", (d, self.ff), s2) for e in range(self.E)])
        wr = p.get(prefix + "router", (self.E, d), 2 * s, small=True)
        self.bias = p.get(prefix + "router.b", (self.E,), 0.2, small=True)
        self.ws13 = self.ws2 = None
        if self.fs:
            self.ws13 = torch.cat([p.get(prefix + "shared.gate", (self.fs, d), s),
                                   p.get(prefix + "shared.up", (self.fs, d), s)]).contiguous()
            self.ws2 = p.get(prefix + "shared.down", (d, self.fs), 1.0 / math.sqrt(self.fs))
            wr = torch.cat([wr, p.get(prefix + "shared.sg", (1, d), s, small=True)])
        self.wr = wr.contiguous()

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        ids, wts, gate = hops.moe_router(h, self.wr, self.bias, self.E, self.K)
        shared = None
        if self.fs:
            shared = F.linear(hops.swiglu(F.linear(h, self.ws13)), self.ws2)
        return hops.moe_experts(h, ids, wts, self.w13, self.w2, shared, gate, il=self.il)


def _softplus(z: float) -> float:
    return z if z > 30.0 else math.log1p(math.exp(z))


class DenseFFN:
    """``down(xIELU(up h))``; the activation's two constants come from the two learned numbers of
    ``act`` (softplus of the first; one half plus softplus of the second), evaluated once at load."""

    def __init__(self, spec: DenseSpec, d: int, p: _Params, prefix: str):
        self.ff = spec.ff
        self.w_up = p.get(prefix + "up", (self.ff, d), 1.0 / math.sqrt(d))
        self.w_down = p.get(prefix + "down", (d, self.ff), 1.0 / math.sqrt(self.ff))
        self.act = p.get(prefix + "act", (2,), 0.5, small=True)
        a = self.act.float().cpu().tolist() if not p.empty else [0.0, 0.0]
        self.a_pos, self.a_neg = _softplus(a[0]), 0.5 + _softplus(a[1])

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        return F.linear(hops.activation(F.linear(h, self.w_up), "xielu", self.a_pos, self.a_neg), self.w_down)


class GatedDenseFFN:
    """``down(act(gate h) * (up h))`` with ``act`` the tanh GELU (or ``relu``, ``silu``): gate and up (and
    ``tail``: extra rows whose outputs forward leaves in ``tail_out``) in one projection, the gated unit
    in one launch."""

    def __init__(self, spec: DenseSpec, d: int, p: _Params, prefix: str, tail: Optional[torch.Tensor] = None,
                 act: str = "gelu_tanh"):
        self.ff, self.act = spec.ff, act
        s = 1.0 / math.sqrt(d)
        ws = [p.get(prefix + "gate", (self.ff, d), s), p.get(prefix + "up", (self.ff, d), s)]
        self.n_tail = 0 if tail is None else tail.shape[0]
        if tail is not None:
            ws.append(tail)
        self.tail_out = None
        self.w_in = torch.cat(ws).contiguous()
        self.w_down = p.get(prefix + "down", (d, self.ff), 1.0 / math.sqrt(self.ff))

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        proj = F.linear(h, self.w_in)
        if self.n_tail:
            self.tail_out = (proj, 2 * self.ff)
        return F.linear(hops.glu(proj, 0, self.ff, self.act), self.w_down)


class PlainRoutedFFN:
    """Top-k routed ungated experts ``down_e(gelu(up_e h))`` (erf GELU): fp32 router without bias,
    softmax over all experts, the chosen experts weighted by their probabilities as they are; plus
    an optional shared expert of the same form, added for every token."""

    def __init__(self, spec: MoESpec, d: int, p: _Params, prefix: str):
        self.E, self.K, self.ff, self.fs = spec.experts, spec.top, spec.ff, spec.shared_ff
        if not 1 <= self.K <= self.E:
            raise ValueError(f"{prefix}: top {self.K} of {self.E} experts")
        s, s2 = 1.0 / math.sqrt(d), 1.0 / math.sqrt(self.ff)
        self.il = False
        # large bf16 steps of such experts run on the Mixtral path's tile GEMM (ops.hybrid.moe_experts)
        self.tile = p.device.type == "cuda" and p.dtype == torch.bfloat16 and self.ff % 256 == 0 and d % 256 == 0
        self.w1 = torch.stack([p.get(f"{prefix}e{e}.up", (self.ff, d), s) for e in range(self.E)])
        self.w2 = torch.stack([p.get(f"{prefix}e{e}.down", (d, self.ff), s2) for e in range(self.E)])
        self.wr = p.get(prefix + "router", (self.E, d), 2 * s, small=True)
        self.ws1 = self.ws2 = None
        if self.fs:
            self.ws1 = p.get(prefix + "shared.up", (self.fs, d), s)
            self.ws2 = p.get(prefix + "shared.down", (d, self.fs), 1.0 / math.sqrt(self.fs))

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        ids, wts, _ = hops.moe_router(h, self.wr, None, self.E, self.K, over_all=True)
        shared = None
        if self.fs:
            shared = F.linear(hops.activation(F.linear(h, self.ws1), "gelu"), self.ws2)
        return hops.moe_experts(h, ids, wts, self.w1, self.w2, shared, None, act="gelu")


class GroupRoutedFFN:
    """Top-k routed gated experts with clamped pre-activations (``g = min(gate_e h, limit)``,
    ``u = clamp(up_e h, -limit, limit)``, ``down_e(g sigmoid(1.702 g) (u + 1))``).  The fp32 router
    scores every expert with a sigmoid; the experts form ``groups`` equal groups of neighbours, a
    group's score is the sum of its two best experts' and only experts of the ``keep_groups`` best groups
    can be chosen; the chosen scores are divided by their sum and multiplied by ``route_scale``."""

    def __init__(self, spec: MoESpec, d: int, p: _Params, prefix: str):
        self.E, self.K, self.ff = spec.experts, spec.top, spec.ff
        self.limit, self.groups, self.keep, self.route_scale = spec.limit, spec.groups, spec.keep_groups, spec.route_scale
        if not 1 <= self.K <= self.E or self.E % self.groups or not 1 <= self.keep <= self.groups:
            raise ValueError(f"{prefix}: top {self.K} of {self.E} experts in {self.groups} groups, {self.keep} kept")
        if self.K > self.keep * (self.E // self.groups):
            raise ValueError(f"{prefix}: top {self.K} exceeds the experts of {self.keep} groups")
        if self.limit <= 0:
            raise ValueError(f"{prefix}: experts of this form need a positive limit")
        s, s2 = 1.0 / math.sqrt(d), 1.0 / math.sqrt(self.ff)
        self.il = False
        # large bf16 steps run on the Mixtral path's tile GEMM (ops.hybrid.moe_experts)
        self.tile = p.device.type == "cuda" and p.dtype == torch.bfloat16 and self.ff % 128 == 0 and d % 256 == 0
        self.w13 = torch.stack([torch.cat([p.get(f"{prefix}e{e}.gate", (self.ff, d), s),
                                           p.get(f"{prefix}e{e}.up", (self.ff, d), s)]) for e in range(self.E)])
        self.w2 = torch.stack([p.get(f"{prefix}e{e}.down", (d, self.ff), s2) for e in range(self.E)])
        self.wr = p.get(prefix + "router", (self.E, d), 2 * s, small=True)

    def forward(self, h: torch.Tensor) -> torch.Tensor:
        ids, wts = hops.moe_router_grouped(h, self.wr, self.E, self.K, self.groups, self.keep, self.route_scale)
        return hops.moe_experts(h, ids, wts, self.w13, self.w2, None, None, act="clamped_swish", limit=self.limit,
                                tile=self.tile)


def _ffn_for(family: str, spec, d: int, p: _Params, prefix: str, tail: Optional[torch.Tensor] = None):
    """The feed-forward of a layer in a design's family (models/config.DESIGN_TRAITS ``ffn``)."""
    if spec is None:
        return None
    if family == "gated_gelu" and isinstance(spec, DenseSpec):
        return GatedDenseFFN(spec, d, p, prefix, tail)
    if family == "swiglu_topk" and isinstance(spec, MoESpec):
        return RoutedFFN(spec, d, p, prefix)
    if family == "relu_glu_grouped":
        return GatedDenseFFN(spec, d, p, prefix, tail, act="relu") if isinstance(spec, DenseSpec) else \
            GroupRoutedFFN(spec, d, p, prefix)
    if family == "plain_softmax":
        return DenseFFN(spec, d, p, prefix) if isinstance(spec, DenseSpec) else PlainRoutedFFN(spec, d, p, prefix)
    raise ValueError(f"{prefix}: no {type(spec).__name__} feed-forward in the {family!r} family")


class HybridLM:
    """The model class of layer-list configs (models/registry.py).  TP = 1."""

    def __init__(self, cfg: HybridConfig, device: torch.device | str = "cpu", dtype=torch.bfloat16, seed: int = 0,
                 pstate: Optional[ParallelState] = None, init: str = "random", weights=None):
        """``weights``: a models/checkpoint.SafetensorsDir to read the tensors from (names
        ``embed``, ``pos``, ``loop.step``, ``l<i>.norm1``, ``l<i>.mix.*``, ``l<i>.mlp.*``,
        ``final.norm``, ``head``); otherwise ``init`` "random" (seeded per name) or "empty"."""
        self.cfg = cfg
        self.device = torch.device(device)
        self.dtype = dtype
        self.seed = seed
        self.ps = pstate or get_state()
        if self.ps.tp_size != 1:
            raise ValueError(f"{cfg.name}: layer-list models run at tp=1")
        self.tp, self.rank = 1, 0
        d, V = cfg.d_model, cfg.vocab_size
        p = _Params(self.device, dtype, seed, src=weights, empty=init == "empty")
        tr = cfg.traits
        self.sequential = tr["block"] == "sequential"
        self.one_plus, self.shifted, self.depth_avg = tr["one_plus_norm"], tr["token_shift"], tr["depth_average"]
        self.scalar_norm, self.gated = bool(tr.get("scalar_norm")), bool(tr.get("gated_residual"))
        if (self.shifted or self.depth_avg or self.gated) and not self.sequential:
            raise ValueError(f"{cfg.name}: token shift, depth average and gated residual are built for sequential blocks")
        if self.gated and (self.shifted or self.depth_avg):
            raise ValueError(f"{cfg.name}: gated residual is not combined with token shift or depth average")
        if self.depth_avg and cfg.loop:
            raise ValueError(f"{cfg.name}: depth average over looped layers is not defined")
        self.center = tr.get("norm", "rms") == "layer"  # layer norm (weight, no bias) instead of RMSNorm
        self.composite = bool(tr.get("composite"))
        self.side_dim = cfg.side_dim
        # designs whose branches join the stream with weights, through a norm of their own or into a
        # layer norm take the summing forward (ops.hybrid.sum_norm)
        self.summed = self.center or self.composite or self.side_dim > 0
        if self.summed and (self.shifted or self.depth_avg or self.gated or not self.sequential):
            raise ValueError(f"{cfg.name}: layer norm, side-by-side mixers and per-layer token input are built for "
                             "plain sequential blocks")
        nm = 1.0 if not self.one_plus else 0.0  # plain norm weights sit around one
        self.embed = p.get("embed", (V, d), 0.5)
        self.pos = p.get("pos", (cfg.max_position, d), 0.1) if tr["learned_pos"] else None
        self.loop_step = p.get("loop.step", (cfg.loop[2], d), 0.1, small=True) if cfg.loop else None
        self.norms, self.norms2, self.mixers, self.ffns, self.shifts, self.dwa = [], [], [], [], [], []
        self.rg1, self.rg2 = [], []  # gated residual: (bias [d] fp32, weight rows kept for export), per sublayer
        names = dict(tr.get("mixers", {}))
        names.update({k: SideBySide.kind for k in tr.get("composite", {})})
        nshape = () if self.scalar_norm else (d,)
        # per-layer token input: layer i reads columns [i * side_dim, (i + 1) * side_dim) of a second table
        sd = self.side_dim
        self.side_embed = p.get("side.embed", (V, len(cfg.layers) * sd), 0.5) if sd else None
        self.side_gate, self.side_proj, self.side_norm = [], [], []

        def norm_w(name):  # one number per norm is kept as a [d] vector: the norm kernels read a vector
            w = p.get(name, nshape, 0.1, nm, small=True)
            return w.reshape(1).expand(d).contiguous() if self.scalar_norm else w

        def rgate(name):
            return p.get(name, (d, d), 1.0 / math.sqrt(d)), p.get(name + ".b", (d,), 0.5, small=True)

        for i, spec in enumerate(cfg.layers):
            kind = names.get(spec.kind, spec.kind)
            if kind not in MIXERS:
                raise ValueError(f"layer {i}: unknown mixer {spec.kind!r} (known: {sorted(MIXERS)})")
            self.norms.append(norm_w(f"l{i}.norm1"))
            g1 = rgate(f"l{i}.rg1") if self.gated else None
            self.mixers.append(MIXERS[kind](spec, d, cfg.norm_eps, p, f"l{i}.mix.", traits=tr,
                                            tail=g1[0] if g1 else None))
            g2 = rgate(f"l{i}.rg2") if self.gated and spec.mlp is not None else None
            self.ffns.append(_ffn_for(tr["ffn"], spec.mlp, d, p, f"l{i}.mlp.", tail=g2[0] if g2 else None)
                             if self.gated else _ffn_for(tr["ffn"], spec.mlp, d, p, f"l{i}.mlp."))
            self.rg1.append(self._gate_for(self.mixers[-1], g1))
            self.rg2.append(self._gate_for(self.ffns[-1], g2))
            self.norms2.append(norm_w(f"l{i}.norm2") if self.sequential and spec.mlp is not None else None)
            if sd:
                self.side_gate.append(p.get(f"l{i}.side.gate", (sd, d), 1.0 / math.sqrt(d)))
                self.side_proj.append(p.get(f"l{i}.side.proj", (d, sd), 1.0 / math.sqrt(sd)))
                self.side_norm.append(p.get(f"l{i}.side.norm", (d,), 0.1, 1.0, small=True))
            self.shifts.append(p.get(f"l{i}.shift", (d,), 0.25, 0.4, small=True) if self.shifted else None)
            # depth-average coefficients: random init leans on the newest result so the stream stays sane
            self.dwa.append(p.get(f"l{i}.dwa", (i + 2,), 0.3 / (i + 2), 1.0 / (i + 2), small=True)
                            if self.depth_avg else None)
        self.final_norm = norm_w("final.norm")
        self.head = p.get("head", (V, d), 1.0 / math.sqrt(d))
        self.runs = cfg.runs()
        # the run whose pages a run reads: its own, or the latest earlier run of the layer it names
        self.kv_run = []
        for r, (li, _, _) in enumerate(self.runs):
            src = getattr(self.mixers[li], "kv_from", None)
            if src is None:
                self.kv_run.append(r)
                continue
            if not 0 <= src < len(cfg.layers) or getattr(self.mixers[src], "kv_from", 0) is not None:
                raise ValueError(f"layer {li}: kv_from {src} is not a layer with key/value pages of its own")
            a, b = self.mixers[li], self.mixers[src]
            if (a.R, a.dr, a.base, a.rdims) != (b.R, b.dr, b.base, b.rdims):
                raise ValueError(f"layer {li}: kv_rank / rot_dim / rotation differ from layer {src}'s")
            prev = [q for q in range(r) if self.runs[q][0] == src]
            if not prev:
                raise ValueError(f"layer {li}: kv_from {src} has not run before it")
            self.kv_run.append(prev[-1])
        self.unused = sorted(set(weights.keys()) - p.used) if weights is not None else []
        self.has_state = self.shifted or any(getattr(m, "stateful", False) for m in self.mixers)
        # large steps of such layers run on the Mixtral path's tile GEMM (extension _k8sllm_ops)
        self.uses_tile_gemm = any(f is not None and (getattr(f, "il", False) or getattr(f, "tile", False))
                                  for f in self.ffns)
        self.layer_probe = None  # a list: forward() appends the residual stream after every run

    @staticmethod
    def _gate_for(sub, g: Optional[tuple]) -> Optional[dict]:
        """A sublayer's residual gate: its bias, and its weight rows where the sublayer's own input
        projection does not carry them (``tail``) - then the gate is a projection of its own."""
        if g is None:
            return None
        fused = getattr(sub, "n_tail", 0) > 0
        return {"b": g[1], "w": None if fused else g[0]}

    # ------------------------------------------------------------------ engine interface
    def overlap_ok(self) -> bool:
        return False

    def cache_bytes(self) -> tuple:
        """(bytes per cache page, bytes per state slot) summed over the layer runs."""
        es = torch.empty(0, dtype=self.dtype).element_size()
        per = [self.mixers[i].cache_bytes(es) for i, _, _ in self.runs]
        shift = 4 * self.cfg.d_model * len(self.runs) if self.shifted else 0
        return sum(a for a, _ in per), sum(b for _, b in per) + shift

    def new_cache(self, num_blocks: int, num_slots: int) -> list:
        """One cache per layer RUN (a looped layer has one per pass): the mixer's pages or state
        slots and, with token shift, the run's last normed row per sequence slot (``shift``)."""
        out = []
        for i, _, _ in self.runs:
            c = self.mixers[i].new_cache(num_blocks, num_slots, self.dtype, self.device)
            if self.shifted:
                c["shift"] = torch.zeros(num_slots, self.cfg.d_model, dtype=torch.float32, device=self.device)
            out.append(c)
        return out

    def resident_weight_bytes(self) -> int:
        n = 0
        for t in self._tensors():
            n += t.numel() * t.element_size()
        return n

    def num_local_params(self) -> int:
        return sum(t.numel() for t in self._tensors())

    def _tensors(self) -> list:
        ts = [self.embed, self.final_norm, self.head] + self.norms + self.side_gate + self.side_proj + self.side_norm
        ts += [t for t in [self.pos, self.loop_step, self.side_embed] + self.norms2 + self.shifts + self.dwa if t is not None]
        ts += [t for g in self.rg1 + self.rg2 if g is not None for t in g.values() if t is not None]
        subs = [x for m in self.mixers for x in getattr(m, "subs", ())]
        for o in self.mixers + subs + [f for f in self.ffns if f is not None]:
            ts += [v for v in vars(o).values() if isinstance(v, torch.Tensor)]
        seen, out = set(), []
        for t in ts:  # a nested mixer's input projection is a view of its parent's: counted once
            key = (t.untyped_storage().data_ptr(), t.storage_offset(), t.numel())
            if t._base is None and key not in seen:
                seen.add(key)
                out.append(t)
        return out

    # ------------------------------------------------------------------ forward
    def forward(self, ids: torch.Tensor, meta: AttnMeta, caches: list) -> torch.Tensor:
        """Logits [rows, vocab] (fp32) for the rows ``meta.logits_idx`` selects (all when None)."""
        c = self.cfg
        if self.sequential:
            return self._forward_sequential(ids, meta, caches)
        x0 = hops.embed_pos(ids, meta.positions, self.embed, self.pos, meta.dec_src, meta.dec_prev)
        x = x0.clone() if c.loop and c.loop[2] > 1 else x0
        pending: tuple = ()
        for r, (li, t, first) in enumerate(self.runs):
            adds, vec = pending, None
            if first:
                vec = self.loop_step[t]
                if t > 0:
                    adds = adds + (x0,)
            h = hops.add_norm(x, adds, vec, self.norms[li], c.norm_eps, True, self.dtype)
            ym = self.mixers[li].forward(h, meta, caches[r])
            ff = self.ffns[li]
            pending = (ym, ff.forward(h)) if ff is not None else (ym,)
            if self.layer_probe is not None:
                self.layer_probe.append(x + sum(a.float() for a in pending))
        if meta.logits_idx is not None:
            idx = meta.logits_idx
            x = x.index_select(0, idx)
            pending = tuple(a.index_select(0, idx) for a in pending)
        hf = hops.add_norm(x, pending, None, self.final_norm, c.norm_eps, True, self.dtype)
        return self._logits(hf)

    def _forward_sequential(self, ids: torch.Tensor, meta: AttnMeta, caches: list) -> torch.Tensor:
        """Pre-norm blocks with two norms.  Without depth average the stream is updated in place and
        a layer's feed-forward output is folded into the next layer's norm launch.  With it, entry
        n + 1 of the stack is layer n's working stream (its input, then += mixer, then += feed-forward
        = the layer's result) and depth_mix leaves the next layer's input in entry n + 2."""
        c = self.cfg
        T, d, L = ids.numel(), c.d_model, len(self.runs)
        seg = (meta.seg_cu, meta.seg_ctx, meta.seg_slot)
        if self.depth_avg:
            stack = torch.empty(L + 2, T, d, dtype=torch.float32, device=self.device)
            hops.embed_pos(ids, meta.positions, self.embed, self.pos, meta.dec_src, meta.dec_prev, out=stack[0])
            stack[1].copy_(stack[0])
            x = stack[1]
        else:
            x = hops.embed_pos(ids, meta.positions, self.embed, self.pos, meta.dec_src, meta.dec_prev,
                               scale=c.embed_scale)
        if self.gated:
            return self._forward_gated(x, meta, caches)
        if self.summed:
            return self._forward_summed(ids, x, meta, caches)
        pending: tuple = ()
        for r, (li, t, first) in enumerate(self.runs):
            if first and self.loop_step is not None:
                x += self.loop_step[t]
            if self.shifted:
                h = hops.norm_shift(x, pending, self.norms[li], c.norm_eps, self.one_plus, self.shifts[li],
                                    caches[r]["shift"], *seg, self.dtype, multi=meta.is_prefill)
            else:
                h = hops.add_norm(x, pending, None, self.norms[li], c.norm_eps, self.one_plus, self.dtype)
            pending = (self.mixers[li].forward(h, meta, caches[self.kv_run[r]]),)
            ff = self.ffns[li]
            if ff is not None:
                h2 = hops.add_norm(x, pending, None, self.norms2[li], c.norm_eps, self.one_plus, self.dtype)
                pending = (ff.forward(h2),)
            if self.depth_avg:
                x = hops.depth_mix(stack, r + 1, pending[0], self.dwa[li])
                pending = ()
            if self.layer_probe is not None:
                self.layer_probe.append(x + sum(a.float() for a in pending))
        if meta.logits_idx is not None:
            idx = meta.logits_idx
            x = x.index_select(0, idx)
            pending = tuple(a.index_select(0, idx) for a in pending)
        hf = hops.add_norm(x, pending, None, self.final_norm, c.norm_eps, self.one_plus, self.dtype)
        return self._logits(hf)

    def _forward_summed(self, ids: torch.Tensor, x: torch.Tensor, meta: AttnMeta, caches: list) -> torch.Tensor:
        """Sequential blocks whose branch results join the stream as weighted sums in the launch of
        the norm that follows (RMS or layer norm).  With a per-layer token input the layer ends with
        ``y = W_proj (gelu_tanh(W_gate x) * side_embed[token, layer's columns])`` of the finished stream
        x, joined as ``x += y / rms(y) * side.norm`` - in the next norm's launch too."""
        c = self.cfg
        eps, op, ctr, sd = c.norm_eps, self.one_plus, self.center, self.side_dim
        pend: tuple = ()  # (branch result, weight) pairs not yet in the stream
        normed = None  # (y, weight vector) of a branch that joins through its own RMS norm
        for r, (li, t, first) in enumerate(self.runs):
            if first and self.loop_step is not None:
                hops.sum_norm(x, pend, normed, None, eps, False, False, torch.float32)  # the stream, complete
                pend, normed = (), None
                x += self.loop_step[t]
            h = hops.sum_norm(x, pend, normed, self.norms[li], eps, ctr, op, self.dtype)
            y = self.mixers[li].forward(h, meta, caches[self.kv_run[r]])
            pend, normed = (y if isinstance(y, tuple) else ((y, 1.0),)), None
            ff = self.ffns[li]
            if ff is not None:
                h2 = hops.sum_norm(x, pend, None, self.norms2[li], eps, ctr, op, self.dtype)
                pend = ((ff.forward(h2), 1.0),)
            if sd:
                xs = hops.sum_norm(x, pend, None, None, eps, False, False, self.dtype)  # the finished stream
                pend = ()
                g = hops.gated_lookup(F.linear(xs, self.side_gate[li]), self.side_embed, ids, li * sd, meta.dec_src,
                                      meta.dec_prev)
                normed = (F.linear(g, self.side_proj[li]), self.side_norm[li])
            if self.layer_probe is not None:
                full = x + sum(a.float() * w for a, w in pend)
                if normed is not None:
                    yf = normed[0].float()
                    full = full + yf * torch.rsqrt(yf.pow(2).mean(-1, keepdim=True) + eps) * normed[1]
                self.layer_probe.append(full)
        if meta.logits_idx is not None:
            idx = meta.logits_idx
            x = x.index_select(0, idx)
            pend = tuple((a.index_select(0, idx), w) for a, w in pend)
            if normed is not None:
                normed = (normed[0].index_select(0, idx), normed[1])
        hf = hops.sum_norm(x, pend, normed, self.final_norm, eps, ctr, op, self.dtype)
        return self._logits(hf)

    def _logits(self, hf: torch.Tensor) -> torch.Tensor:
        c = self.cfg
        z = F.linear(hf, self.head).float()
        if c.logit_scale != 1.0:
            z = z * c.logit_scale
        if c.logit_softcap > 0:
            z = hops.softcap(z.contiguous(), c.logit_softcap)
        return z

    def _gate_of(self, sub, g: dict, h: torch.Tensor) -> tuple:
        """(projection, first column) holding a sublayer's residual-gate logits for this step."""
        if g["w"] is None:
            return sub.tail_out
        return F.linear(h, g["w"]), 0

    def _forward_gated(self, x: torch.Tensor, meta: AttnMeta, caches: list) -> torch.Tensor:
        """Sequential blocks with a gated residual: every sublayer's result y joins the stream as
        ``x += m * y * sigmoid(gate + b)``, folded into the launch of the norm that follows it."""
        c = self.cfg
        eps, op, mult = c.norm_eps, self.one_plus, c.residual_mult
        pend = None  # (y, projection holding the gate logits, their first column, bias)
        for r, (li, t, first) in enumerate(self.runs):
            if first and self.loop_step is not None:
                if pend is not None:
                    raise ValueError("looped layers with a gated residual are not built")
                x += self.loop_step[t]
            w1 = self.norms[li]
            h = hops.add_norm(x, (), None, w1, eps, op, self.dtype) if pend is None else \
                hops.gated_add_norm(x, pend[0], pend[1], pend[2], pend[3], mult, w1, eps, op, self.dtype)
            mx = self.mixers[li]
            y = mx.forward(h, meta, caches[self.kv_run[r]])
            pend = (y, *self._gate_of(mx, self.rg1[li], h), self.rg1[li]["b"])
            ff = self.ffns[li]
            if ff is not None:
                h2 = hops.gated_add_norm(x, pend[0], pend[1], pend[2], pend[3], mult, self.norms2[li], eps, op, self.dtype)
                y = ff.forward(h2)
                pend = (y, *self._gate_of(ff, self.rg2[li], h2), self.rg2[li]["b"])
            if self.layer_probe is not None:
                d = x.shape[1]
                g = pend[1][:, pend[2]:pend[2] + d].float() + pend[3].float()
                self.layer_probe.append(x + mult * pend[0].float() * torch.sigmoid(g))
        if meta.logits_idx is not None:
            idx, d = meta.logits_idx, x.shape[1]
            x = x.index_select(0, idx)
            if pend is not None:
                pend = (pend[0].index_select(0, idx), pend[1][:, pend[2]:pend[2] + d].index_select(0, idx), 0, pend[3])
        hf = hops.add_norm(x, (), None, self.final_norm, eps, op, self.dtype) if pend is None else \
            hops.gated_add_norm(x, pend[0], pend[1], pend[2], pend[3], mult, self.final_norm, eps, op, self.dtype)
        return self._logits(hf)


def state_dict(model: HybridLM) -> dict:
    """name -> tensor under the checkpoint's names (exporting a random-init model)."""
    one = (lambda w: w[0]) if model.scalar_norm else (lambda w: w)  # a one-number norm is kept as a vector
    out = {"embed": model.embed, "final.norm": one(model.final_norm), "head": model.head}
    if model.pos is not None:
        out["pos"] = model.pos
    if model.loop_step is not None:
        out["loop.step"] = model.loop_step
    if model.side_embed is not None:
        out["side.embed"] = model.side_embed
    for i, (n, m, f) in enumerate(zip(model.norms, model.mixers, model.ffns)):
        p = f"l{i}."
        out[p + "norm1"] = one(n)
        if model.side_dim:
            out.update({p + "side.gate": model.side_gate[i], p + "side.proj": model.side_proj[i],
                        p + "side.norm": model.side_norm[i]})
        if model.norms2[i] is not None:
            out[p + "norm2"] = one(model.norms2[i])
        for key, t in (("shift", model.shifts[i]), ("dwa", model.dwa[i])):
            if t is not None:
                out[p + key] = t
        for key, g, sub in (("rg1", model.rg1[i], m), ("rg2", model.rg2[i], f)):
            if g is not None:  # the gate's rows are the tail of the sublayer's input projection, or its own
                w_in = getattr(sub, "w_in", getattr(sub, "w_down", None))
                out[p + key] = g["w"] if g["w"] is not None else w_in[w_in.shape[0] - sub.n_tail:]
                out[p + key + ".b"] = g["b"]
        if isinstance(m, LatentAttention):
            out.update({p + "mix.dq": m.w_down[:m.Q], p + "mix.dq.norm": m.qn, p + "mix.uq": m.w_uq, p + "mix.uk": m.w_uk,
                        p + "mix.uv": m.w_uv, p + "mix.o": m.wo})
            if m.sinks is not None:
                out[p + "mix.sink"] = m.sinks
            if m.kv_from is None:
                out.update({p + "mix.dkv": m.w_down[m.Q:m.n_down], p + "mix.dkv.norm": m.kn})
        elif hasattr(m, "export"):
            out.update(m.export(p + "mix."))
        elif isinstance(m, LightningMixer):
            nv, nk = m.H * m.dv, m.H * m.dk
            out.update({p + "mix.v": m.w_in[:nv], p + "mix.k": m.w_in[nv:nv + nk], p + "mix.q": m.w_in[nv + nk:m.n_act],
                        p + "mix.g": m.w_in[m.n_act:m.n_in], p + "mix.norm": m.norm_w, p + "mix.o": m.wo})
        elif isinstance(m, WindowAttention):
            nq, nk = m.H * m.dk, m.G * m.dk
            out.update({p + "mix.q": m.wqkv[:nq], p + "mix.k": m.wqkv[nq:nq + nk], p + "mix.v": m.wqkv[nq + nk:],
                        p + "mix.q.norm": m.qn, p + "mix.k.norm": m.kn, p + "mix.o": m.wo})
        else:
            out.update({p + "mix.in": m.w_in, p + "mix.conv": m.conv_w, p + "mix.conv.b": m.conv_b,
                        p + "mix.dt_bias": m.dt_bias, p + "mix.A_log": m.a_log, p + "mix.D": m.d_skip,
                        p + "mix.norm": m.norm_w, p + "mix.o": m.wo})
        if isinstance(f, GatedDenseFFN):
            out.update({p + "mlp.gate": f.w_in[:f.ff], p + "mlp.up": f.w_in[f.ff:2 * f.ff], p + "mlp.down": f.w_down})
        elif isinstance(f, DenseFFN):
            out.update({p + "mlp.up": f.w_up, p + "mlp.down": f.w_down, p + "mlp.act": f.act})
        elif isinstance(f, GroupRoutedFFN):
            for e in range(f.E):
                out[f"{p}mlp.e{e}.gate"], out[f"{p}mlp.e{e}.up"] = f.w13[e, :f.ff], f.w13[e, f.ff:]
                out[f"{p}mlp.e{e}.down"] = f.w2[e]
            out[p + "mlp.router"] = f.wr
        elif isinstance(f, PlainRoutedFFN):
            for e in range(f.E):
                out[f"{p}mlp.e{e}.up"], out[f"{p}mlp.e{e}.down"] = f.w1[e], f.w2[e]
            out[p + "mlp.router"] = f.wr
            if f.fs:
                out.update({p + "mlp.shared.up": f.ws1, p + "mlp.shared.down": f.ws2})
        elif f is not None:
            for e in range(f.E):
                w13 = _ops.deinterleave_gate_up(f.w13[e]) if f.il else f.w13[e]
                out[f"{p}mlp.e{e}.gate"], out[f"{p}mlp.e{e}.up"] = w13[:f.ff], w13[f.ff:]
                out[f"{p}mlp.e{e}.down"] = f.w2[e]
            out[p + "mlp.router"], out[p + "mlp.router.b"] = f.wr[:f.E], f.bias
            if f.fs:
                out.update({p + "mlp.shared.gate": f.ws13[:f.fs], p + "mlp.shared.up": f.ws13[f.fs:],
                            p + "mlp.shared.down": f.ws2, p + "mlp.shared.sg": f.wr[f.E:]})
    return {k: v.detach().to("cpu", torch.bfloat16).contiguous() for k, v in out.items()}
