"""Operators of the layer-list (hybrid) decoders: fp32 residual stream with one-plus RMSNorm,
windowed attention with a softmax sink over a paged cache, the Mamba-2 recurrence with its short
convolution and per-sequence state slots, and routed experts with a biased fp32 router and a
gated shared expert; and, for the sequential-block designs, the token-shifted norm, the depth
average of layer results, latent (low-rank compressed) attention with rotary positions and learned
per-head sinks, and ungated experts with a softmax-over-all router; and the gated residual
(a sublayer's result times the sigmoid of a projection of its input, scaled, then the norm),
rotary grouped-query attention with per-head temperatures, the fixed-decay linear-attention
recurrence, gated linear units and the logit soft cap.

GPU tensors run the gfx950 kernels of ``_k8sllm_hybrid`` (``ops/csrc/hybrid``; built by
``python -m k8s_llm_monitor_amd.ops.build --only hybrid``) for bfloat16 and float32 activations
alike; CPU tensors run the torch forms below (the same arithmetic in fp32).  A GPU tensor never
falls back: without the extension the call raises.

Conventions.  ``T`` rows are the step's tokens, all sequences concatenated; a *segment* is one
sequence's rows of this step (a decode token is a segment of one row).  ``seg_cu`` [R+1] are the
segments' row offsets, ``seg_ctx`` [R] the tokens each sequence already holds in its cache /
state (0 = the sequence starts here, its state is taken as zero), ``seg_slot`` [R] its state slot
(< 0: a padding row, skipped).  Paged caches: keys ``[blocks, block_size, heads * dim]`` (a token's
keys contiguous), values ``[blocks, heads, vdim, block_size]`` (a value dim's tokens contiguous - the
direction the PV products read along).
"""
from __future__ import annotations

import importlib
import math
from typing import Optional

import torch
import torch.nn.functional as F

_EXT = None
_EXT_ERR: Optional[BaseException] = None


def native():
    """The compiled ``_k8sllm_hybrid`` module (raises with the build hint if unavailable)."""
    global _EXT, _EXT_ERR
    if _EXT is None and _EXT_ERR is None:
        try:
            _EXT = importlib.import_module("k8s_llm_monitor_amd.ops._k8sllm_hybrid")
        except BaseException as e:  # noqa: BLE001 - remembered, re-raised on GPU use
            _EXT_ERR = e
    if _EXT is None:
        raise RuntimeError("gfx950 kernels (_k8sllm_hybrid) are not built/loadable; run "
                           "`python -m k8s_llm_monitor_amd.ops.build --only hybrid` (cause: %r)" % (_EXT_ERR,))
    return _EXT


def native_available() -> bool:
    try:
        native()
        return True
    except RuntimeError:
        return False


def _silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


# ---------------------------------------------------------------- residual stream / norms

def embed_pos(ids: torch.Tensor, positions: torch.Tensor, embed: torch.Tensor, pos: Optional[torch.Tensor],
              src: Optional[torch.Tensor] = None, prev: Optional[torch.Tensor] = None,
              out: Optional[torch.Tensor] = None, scale: float = 1.0) -> torch.Tensor:
    """fp32 rows ``embed[id] * scale + pos[position]`` (``pos`` None: no learned positions).  ``src`` /
    ``prev`` (pipelined decode): row i takes token ``prev[src[i]]`` where ``src[i] >= 0``.
    ``out``: a contiguous fp32 [T, d] buffer to fill."""
    if not embed.is_cuda:
        if src is not None:
            ids = torch.where(src >= 0, prev.index_select(0, src.clamp(min=0).long()), ids)
        x = embed[ids.long()].float()
        if scale != 1.0:
            x = x * scale
        x = x + pos[positions.long()].float() if pos is not None else x
        if out is not None:
            out.copy_(x)
            return out
        return x
    if out is None:
        out = torch.empty(ids.numel(), embed.shape[1], dtype=torch.float32, device=embed.device)
    native().embed_pos(out, ids, positions, embed, pos, src, prev, float(scale))
    return out


def add_norm(residual: torch.Tensor, addends: tuple, vec: Optional[torch.Tensor], w: torch.Tensor, eps: float,
             one_plus: bool, out_dtype: torch.dtype) -> torch.Tensor:
    """``residual`` (fp32 [T, d], updated in place) += sum of ``addends`` ([T, d] each, any float
    dtype, at most three) + ``vec`` ([d], broadcast over the rows); returns the RMSNorm of the new
    residual times ``w`` (``one_plus``: times ``1 + w``) in ``out_dtype``.  The sum and the norm
    are fp32."""
    if not residual.is_cuda:
        for a in addends:
            residual += a.float()
        if vec is not None:
            residual += vec.float()
        y = residual * torch.rsqrt(residual.pow(2).mean(-1, keepdim=True) + eps)
        wf = w.float()
        return (y * (1.0 + wf if one_plus else wf)).to(out_dtype)
    assert len(addends) <= 3
    out = torch.empty(residual.shape, dtype=out_dtype, device=residual.device)
    a = list(addends) + [None] * (3 - len(addends))
    native().add_norm(out, residual, a[0], a[1], a[2], vec, w, float(eps), bool(one_plus))
    return out


def sum_norm(residual: torch.Tensor, addends: tuple, normed: Optional[tuple], w: Optional[torch.Tensor], eps: float,
             center: bool, one_plus: bool, out_dtype: torch.dtype) -> torch.Tensor:
    """``residual`` (fp32 [T, d], updated in place) += sum of ``scale * a`` over ``addends`` (at most
    two (a [T, d] of any float dtype, scale) pairs) + ``y / sqrt(mean(y^2) + eps) * wy`` for ``normed``
    = (y [T, d], wy [d] fp32) - a branch that joins the stream through an RMS norm of its own.  Returns
    the norm of the new residual times ``w`` (``one_plus``: ``1 + w``) in ``out_dtype``: ``center`` False
    the RMS norm, True the layer norm ``(x - mean) / sqrt(mean((x - mean)^2) + eps)``.  ``w`` None: no
    norm, the new residual itself in ``out_dtype``.  Sums and norms are fp32."""
    if not residual.is_cuda:
        for a, sc in addends:
            residual += a.float() * sc if sc != 1.0 else a.float()
        if normed is not None:
            y = normed[0].float()
            residual += y * torch.rsqrt(y.pow(2).mean(-1, keepdim=True) + eps) * normed[1].float()
        if w is None:
            return residual.to(out_dtype)
        x = residual - residual.mean(-1, keepdim=True) if center else residual
        h = x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)
        wf = w.float()
        return (h * (1.0 + wf if one_plus else wf)).to(out_dtype)
    assert len(addends) <= 2
    out = torch.empty(residual.shape, dtype=out_dtype, device=residual.device)
    a = list(addends) + [(None, 1.0)] * (2 - len(addends))
    yn, wy = normed if normed is not None else (None, None)
    native().sum_norm(out, residual, a[0][0], float(a[0][1]), a[1][0], float(a[1][1]), yn, wy, w, float(eps), bool(center),
                      bool(one_plus))
    return out


def gated_lookup(gate: torch.Tensor, table: torch.Tensor, ids: torch.Tensor, col: int,
                 src: Optional[torch.Tensor] = None, prev: Optional[torch.Tensor] = None) -> torch.Tensor:
    """``gelu_tanh(gate) * table[id, col : col + n]`` for ``gate`` [T, n]: a per-token table slice gated
    by a projection of the stream (fp32 arithmetic, result in the gate's dtype).  ``src`` / ``prev``: as
    in embed_pos."""
    n = gate.shape[1]
    if not gate.is_cuda:
        if src is not None:
            ids = torch.where(src >= 0, prev.index_select(0, src.clamp(min=0).long()), ids)
        e = table[ids.long(), col:col + n].float()
        return (F.gelu(gate.float(), approximate="tanh") * e).to(gate.dtype)
    out = torch.empty_like(gate)
    native().gated_lookup(out, gate, table, ids, int(col), src, prev)
    return out


def gated_add_norm(residual: torch.Tensor, y: torch.Tensor, proj: torch.Tensor, g_col: int, bias: torch.Tensor,
                   mult: float, w: torch.Tensor, eps: float, one_plus: bool, out_dtype: torch.dtype) -> torch.Tensor:
    """Gated residual: ``residual`` (fp32 [T, d], updated in place) += ``mult * y * sigmoid(g + bias)``
    with the gate logits ``g = proj[:, g_col : g_col + d]`` (a column range of a wider projection of
    the sublayer's input, activation dtype) and ``bias`` [d] fp32; returns the RMSNorm of the new
    residual times ``w`` (``one_plus``: ``1 + w``) in ``out_dtype``.  ``y`` [T, d]: any float dtype.
    Sigmoid, product, sum and norm are fp32."""
    d = residual.shape[1]
    if not residual.is_cuda:
        g = proj[:, g_col:g_col + d].float() + bias.float()
        residual += mult * y.float() * torch.sigmoid(g)
        h = residual * torch.rsqrt(residual.pow(2).mean(-1, keepdim=True) + eps)
        wf = w.float()
        return (h * (1.0 + wf if one_plus else wf)).to(out_dtype)
    out = torch.empty(residual.shape, dtype=out_dtype, device=residual.device)
    native().gated_add_norm(out, residual, y.contiguous(), proj, int(g_col), bias, float(mult), w, float(eps), bool(one_plus))
    return out


def norm_shift(residual: torch.Tensor, addends: tuple, w: torch.Tensor, eps: float, one_plus: bool,
               mu: torch.Tensor, state: torch.Tensor, seg_cu: torch.Tensor, seg_ctx: torch.Tensor,
               seg_slot: torch.Tensor, out_dtype: torch.dtype, advance: bool = True,
               multi: bool = True) -> torch.Tensor:
    """Token-shifted norm.  ``residual`` (fp32 [T, d], updated in place) += ``addends``; with
    ``h[t]`` the RMSNorm of row t times ``w`` (fp32), returns ``h[t] + (h[t-1] - h[t]) * mu`` in
    ``out_dtype``, where the row before a segment's first comes from ``state[slot]`` ([slots, d]
    fp32; zeros where seg_ctx is 0).  ``advance``: ``state[slot]`` then takes the segment's last
    ``h`` (unshifted).  GPU: the state of segments longer than one row is advanced by a second
    small launch, after every row has read the old state (``multi`` False: the caller knows every
    segment is one row, as in a decode step, and that launch is left out)."""
    if not residual.is_cuda:
        for a in addends:
            residual += a.float()
        h = residual * torch.rsqrt(residual.pow(2).mean(-1, keepdim=True) + eps)
        wf = w.float()
        h = h * (1.0 + wf if one_plus else wf)
        prev = torch.zeros_like(h)
        prev[1:] = h[:-1]
        cul = seg_cu.tolist()
        for s, (c0, slot) in enumerate(zip(seg_ctx.tolist(), seg_slot.tolist())):
            a, b = cul[s], cul[s + 1]
            if b <= a:
                continue
            prev[a] = state[slot] if (c0 > 0 and slot >= 0) else 0.0
            if advance and slot >= 0:
                state[slot] = h[b - 1]
        return (h + (prev - h) * mu.float()).to(out_dtype)
    for a in addends:  # a row also norms its predecessor, so the stream is complete before the launch
        residual += a
    out = torch.empty(residual.shape, dtype=out_dtype, device=residual.device)
    native().norm_shift(out, residual, w, float(eps), bool(one_plus), mu, state, seg_cu, seg_ctx, seg_slot,
                        bool(advance), bool(multi))
    return out


def depth_mix(stack: torch.Tensor, n: int, addend: Optional[torch.Tensor], coef: torch.Tensor) -> torch.Tensor:
    """Depth-weighted average.  ``stack`` [L, T, d] fp32 holds the embedding output and the layer
    results so far in entries 0 .. n (entry n is the newest, still missing ``addend``):
    ``stack[n] += addend``, then ``stack[n + 1] = sum_j coef[j] * stack[j]`` over j = 0 .. n
    (``coef`` [n + 1] fp32).  Returns ``stack[n + 1]``, the next layer's input."""
    if not stack.is_cuda:
        if addend is not None:
            stack[n] += addend.float()
        stack[n + 1] = torch.einsum("j,jtd->td", coef.float(), stack[: n + 1])
        return stack[n + 1]
    native().depth_mix(stack, int(n), addend, coef)
    return stack[n + 1]


ACTS = {"gelu": 0, "gelu_tanh": 1, "xielu": 2, "silu": 3, "relu": 4, "clamped_swish": 5}


def _act_torch(z: torch.Tensor, kind: str) -> torch.Tensor:
    if kind == "gelu":
        return F.gelu(z)
    if kind == "gelu_tanh":
        return F.gelu(z, approximate="tanh")
    if kind == "silu":
        return _silu(z)
    if kind == "relu":
        return torch.relu(z)
    raise ValueError(kind)


def _clamped_unit(g: torch.Tensor, u: torch.Tensor, limit: float) -> torch.Tensor:
    """Experts with clamped pre-activations: g <- min(g, limit), u <- clamp(u, -limit, limit);
    g * sigmoid(1.702 g) * (u + 1)."""
    g = g.clamp(max=limit)
    u = u.clamp(-limit, limit)
    return g * torch.sigmoid(1.702 * g) * (u + 1.0)


def activation(x: torch.Tensor, kind: str, a: float = 0.0, b: float = 0.0) -> torch.Tensor:
    """Elementwise on [T, f] rows, evaluated in fp32: ``gelu`` (erf form), ``gelu_tanh``, ``silu``, or
    ``xielu`` with the two positive constants ``a``, ``b``:  z > 0: a z^2 + z / 2;  z <= 0:
    b (exp(z) - 1 - z) + z / 2."""
    if not x.is_cuda:
        z = x.float()
        if kind == "xielu":
            y = torch.where(z > 0, a * z * z + 0.5 * z, b * (torch.expm1(z.clamp(max=0.0)) - z) + 0.5 * z)
        else:
            y = _act_torch(z, kind)
        return y.to(x.dtype)
    out = torch.empty_like(x)
    native().activation(out, x, ACTS[kind], float(a), float(b))
    return out


def activation_cols(proj: torch.Tensor, col: int, n: int, kind: str) -> torch.Tensor:
    """``act(proj[:, col : col + n])`` as a contiguous [T, n] tensor (``gelu``, ``gelu_tanh`` or
    ``silu``, evaluated in fp32): the activation of a column range of a wider projection."""
    if not proj.is_cuda:
        return _act_torch(proj[:, col:col + n].float(), kind).to(proj.dtype)
    out = torch.empty(proj.shape[0], n, dtype=proj.dtype, device=proj.device)
    native().activation_cols(out, proj, int(col), ACTS[kind])
    return out


def glu(proj: torch.Tensor, col: int, f: int, kind: str, limit: float = 0.0) -> torch.Tensor:
    """Gated linear unit ``act(proj[:, col : col + f]) * proj[:, col + f : col + 2 f]`` ([gate | up]
    columns of a possibly wider projection) with ``kind`` ``gelu_tanh``, ``silu`` or ``relu``, or
    ``clamped_swish``: with g = min(gate, limit) and u = clamp(up, -limit, limit),
    ``g * sigmoid(1.702 g) * (u + 1)``.  fp32 arithmetic, [T, f] in the activation dtype."""
    if not proj.is_cuda:
        g, u = proj[:, col:col + f].float(), proj[:, col + f:col + 2 * f].float()
        if kind == "clamped_swish":
            return _clamped_unit(g, u, limit).to(proj.dtype)
        return (_act_torch(g, kind) * u).to(proj.dtype)
    out = torch.empty(proj.shape[0], f, dtype=proj.dtype, device=proj.device)
    native().glu(out, proj, int(col), ACTS[kind], float(limit))
    return out


def sigmoid_gate(x: torch.Tensor, proj: torch.Tensor, col: int) -> torch.Tensor:
    """In place: ``x`` [T, n] *= sigmoid(proj[:, col : col + n]) (fp32 arithmetic)."""
    n = x.shape[1]
    if not x.is_cuda:
        x.copy_((x.float() * torch.sigmoid(proj[:, col:col + n].float())).to(x.dtype))
        return x
    native().sigmoid_gate(x, proj, int(col))
    return x


def softcap(logits: torch.Tensor, cap: float) -> torch.Tensor:
    """In place on fp32 logits: ``cap * tanh(logits / cap)``."""
    if not logits.is_cuda:
        return logits.copy_(cap * torch.tanh(logits / cap))
    native().softcap(logits, float(cap))
    return logits


# ---------------------------------------------------------------- windowed attention with a sink

def qk_norm_cache(qkv: torch.Tensor, qw: torch.Tensor, kw: torch.Tensor, eps: float, Hq: int, Hkv: int, dk: int,
                  dv: int, k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor],
                  slot_mapping: Optional[torch.Tensor]) -> None:
    """In place on the fused rows [T, Hq*dk | Hkv*dk | Hkv*dv]: q and k are each divided by the
    root mean square of their WHOLE projection (all heads together, fp32) and multiplied by
    ``qw`` / ``kw``; the normed k and v go to the paged cache at ``slot_mapping`` (< 0: not
    written)."""
    nq, nk = Hq * dk, Hkv * dk
    if not qkv.is_cuda:
        q, k = qkv[:, :nq].float(), qkv[:, nq:nq + nk].float()
        q = q * torch.rsqrt(q.pow(2).mean(-1, keepdim=True) + eps) * qw.float()
        k = k * torch.rsqrt(k.pow(2).mean(-1, keepdim=True) + eps) * kw.float()
        qkv[:, :nq] = q.to(qkv.dtype)
        qkv[:, nq:nq + nk] = k.to(qkv.dtype)
        if k_cache is not None:
            ok = slot_mapping >= 0
            s = slot_mapping[ok].long()
            k_cache.view(-1, nk)[s] = qkv[ok, nq:nq + nk]
            bs = k_cache.shape[1]
            v_cache.view(-1, Hkv * dv, bs)[s // bs, :, s % bs] = qkv[ok, nq + nk:]
        return
    native().qk_norm_cache(qkv, qw, kw, float(eps), Hq, Hkv, dk, dv, k_cache, v_cache, slot_mapping)


def rotary_cache(qkv: torch.Tensor, Hq: int, Hkv: int, dk: int, dv: int, positions: torch.Tensor, freq: torch.Tensor,
                 pairs: bool, q_scale: Optional[torch.Tensor], k_cache: Optional[torch.Tensor],
                 v_cache: Optional[torch.Tensor], slot_mapping: Optional[torch.Tensor], rot_off: int = 0,
                 rot_k: bool = True, norm: int = 0, qw: Optional[torch.Tensor] = None, kw: Optional[torch.Tensor] = None,
                 eps: float = 0.0, v_from_k: bool = False) -> None:
    """In place on the fused rows [T, Hq*dk | Hkv*dk | Hkv*dv | ...]: the first ``2 len(freq)`` entries
    of every query and key head turn by the angle ``position * freq[i]`` (fp32; ``pairs``: entry 2i
    with 2i + 1, else entry i with i + len(freq); rotary_freq); the rest of a head passes.  ``q_scale``
    [Hq] fp32 (optional): every query head is multiplied by its number in the same pass (a per-head
    temperature folded into the query).  Keys (turned) and values go to the paged cache at
    ``slot_mapping`` (< 0: not written).  ``rot_off``: the turning entries are ``rot_off .. rot_off +
    2 len(freq)`` of every head instead of the first; ``rot_k`` False: the keys are taken as they are
    (turned already) and only written to the pages.

    ``norm``: every query and key head is also RMS-normed over its ``dk`` entries (fp32, ``eps`` inside
    the root) - 1: BEFORE the turn, times ``qw`` / ``kw`` ([dk] fp32, shared by the heads); 2: AFTER the
    turn, no weight.  ``v_from_k``: there are no value columns; the values are the keys as projected
    (before norm and turn), ``dv == dk``."""
    nq, nk, nv = Hq * dk, Hkv * dk, Hkv * dv
    if not qkv.is_cuda:
        T = qkv.shape[0]

        def rms(x):
            return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + eps)

        def turn(x, w):
            x = x.clone()
            if norm == 1:
                x = rms(x) * w.float()
            x[..., rot_off:] = _rotate(x[..., rot_off:], positions, freq, pairs)
            return rms(x) if norm == 2 else x

        q = turn(qkv[:, :nq].float().view(T, Hq, dk), qw)
        if q_scale is not None:
            q = q * q_scale.float().view(1, Hq, 1)
        k_raw = qkv[:, nq:nq + nk].clone()
        k = qkv[:, nq:nq + nk].float().view(T, Hkv, dk)
        k = turn(k, kw) if rot_k else k
        qkv[:, :nq] = q.reshape(T, nq).to(qkv.dtype)
        qkv[:, nq:nq + nk] = k.reshape(T, nk).to(qkv.dtype)
        if k_cache is not None:
            ok = slot_mapping[:T] >= 0
            s = slot_mapping[:T][ok].long()
            k_cache.view(-1, nk)[s] = qkv[ok, nq:nq + nk]
            bs = k_cache.shape[1]
            v_cache.view(-1, nv, bs)[s // bs, :, s % bs] = k_raw[ok] if v_from_k else qkv[ok, nq + nk:nq + nk + nv]
        return
    if norm or v_from_k:
        native().rotary_norm_cache(qkv, Hq, Hkv, dk, dv, positions, freq, bool(pairs), int(norm), qw, kw, float(eps), q_scale,
                                   k_cache, v_cache, slot_mapping, bool(v_from_k))
        return
    native().rotary_cache(qkv, Hq, Hkv, dk, dv, positions, freq, bool(pairs), q_scale, k_cache, v_cache, slot_mapping,
                          int(rot_off), bool(rot_k))


def _attend(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, sink: bool,
            sinks: Optional[torch.Tensor] = None) -> torch.Tensor:
    """q [H, dk], k [n, G, dk], v [n, G, dv] (fp32) -> [H, dv].  ``sinks`` [H]: the sink's logit per
    head (absent: 0)."""
    H, G = q.shape[0], k.shape[1]
    kk = k.repeat_interleave(H // G, dim=1)
    vv = v.repeat_interleave(H // G, dim=1)
    s = torch.einsum("hd,nhd->hn", q, kk) * scale
    m = s.max(-1, keepdim=True).values
    z = sinks.float().view(H, 1) if sinks is not None else torch.zeros(H, 1)
    if sink:
        m = torch.maximum(m, z)
    e = torch.exp(s - m)
    den = e.sum(-1, keepdim=True) + (torch.exp(z - m) if sink else 0.0)
    return torch.einsum("hn,nhd->hd", e / den, vv)


def window_attention_prefill(qkv: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, cu: torch.Tensor,
                             ctx: torch.Tensor, block_tables: torch.Tensor, Hq: int, Hkv: int, dk: int, dv: int,
                             scale: float, window: int, sink: bool, mfma: int = 1,
                             sinks: Optional[torch.Tensor] = None) -> torch.Tensor:
    """Attention of the step's prompt chunks over the paged cache (which already holds their own
    keys): row r of segment s at position p = ctx[s] + r sees positions max(0, p - window + 1) .. p
    (``window`` 0: all of 0 .. p).  ``sink``: the softmax denominator has one more term that carries
    no value - exp(0), or exp(sinks[h]) for head h where ``sinks`` [Hq] fp32 is given (a learned,
    unscaled logit).  Scores and weights are fp32.  Returns [T, Hq*dv].  GPU, bf16, head sizes
    64 / 128: the matrix-core kernel, 16 query rows per wave or 32 in large steps (``mfma`` 0: the
    any-size wave-per-row kernel; 16 / 32 / 64: that many rows per wave)."""
    T = qkv.shape[0]
    if not qkv.is_cuda:
        out = torch.empty(T, Hq * dv, dtype=qkv.dtype)
        bs = k_cache.shape[1]
        cul, ctxl = cu.tolist(), ctx.tolist()
        for s in range(len(ctxl)):
            n_all = ctxl[s] + cul[s + 1] - cul[s]
            bt = block_tables[s, : (n_all + bs - 1) // bs].long()
            ks = k_cache[bt].reshape(-1, Hkv, dk)[:n_all].float()
            vs = v_cache[bt].permute(0, 3, 1, 2).reshape(-1, Hkv, dv)[:n_all].float()
            for r in range(cul[s], cul[s + 1]):
                p = ctxl[s] + r - cul[s]
                lo = max(0, p - window + 1) if window > 0 else 0
                o = _attend(qkv[r, : Hq * dk].float().view(Hq, dk), ks[lo:p + 1], vs[lo:p + 1], scale, sink, sinks)
                out[r] = o.reshape(-1).to(qkv.dtype)
        return out
    out = torch.empty(T, Hq * dv, dtype=qkv.dtype, device=qkv.device)
    native().window_attention_prefill(out, qkv, k_cache, v_cache, cu, ctx, block_tables, Hq, Hkv, dk, dv, float(scale),
                                      int(window), bool(sink), sinks, int(mfma))
    return out


def window_attention_decode(qkv: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor,
                            block_tables: torch.Tensor, seq_lens: torch.Tensor, Hq: int, Hkv: int, dk: int, dv: int,
                            scale: float, window: int, sink: bool, vec: bool = True,
                            sinks: Optional[torch.Tensor] = None) -> torch.Tensor:
    """One query per sequence (its newest token, already in the cache) over the last ``window``
    cached positions; ``seq_lens`` count that token (0: a padding row, output zero)."""
    B = qkv.shape[0]
    if not qkv.is_cuda:
        out = torch.zeros(B, Hq * dv, dtype=qkv.dtype)
        bs = k_cache.shape[1]
        for b, n in enumerate(seq_lens.tolist()):
            if n <= 0:
                continue
            lo = max(0, n - window) if window > 0 else 0
            bt = block_tables[b, : (n + bs - 1) // bs].long()
            ks = k_cache[bt].reshape(-1, Hkv, dk)[lo:n].float()
            vs = v_cache[bt].permute(0, 3, 1, 2).reshape(-1, Hkv, dv)[lo:n].float()
            out[b] = _attend(qkv[b, : Hq * dk].float().view(Hq, dk), ks, vs, scale, sink,
                             sinks).reshape(-1).to(qkv.dtype)
        return out
    out = torch.empty(B, Hq * dv, dtype=qkv.dtype, device=qkv.device)
    native().window_attention_decode(out, qkv, k_cache, v_cache, block_tables, seq_lens, Hq, Hkv, dk, dv, float(scale),
                                     int(window), bool(sink), sinks, bool(vec))
    return out


# ---------------------------------------------------------------- latent attention

def rotary_freq(base: float, dims: int, device=None, scaling: Optional[dict] = None) -> torch.Tensor:
    """The ``dims / 2`` rotation frequencies base^(-2i/dims) as fp32 (evaluated in float64).
    ``scaling`` {factor, low, high, original}: the long-context rescaling of Llama 3.1 - with the
    wavelength ``l = 2 pi / f``, a frequency stays where ``l < original / high``, becomes ``f / factor``
    where ``l > original / low``, and in between is ``(1 - s) f / factor + s f`` with
    ``s = (original / l - low) / (high - low)``."""
    f = torch.pow(torch.tensor(float(base), dtype=torch.float64), -2.0 * torch.arange(dims // 2, dtype=torch.float64) / dims)
    if scaling:
        fac, lo, hi, orig = (float(scaling[k]) for k in ("factor", "low", "high", "original"))
        lam = 2.0 * math.pi / f
        s = (orig / lam - lo) / (hi - lo) if hi != lo else torch.ones_like(f)
        mid = (1.0 - s) * f / fac + s * f
        f = torch.where(lam < orig / hi, f, torch.where(lam > orig / lo, f / fac, mid))
    return f.float().to(device) if device is not None else f.float()


def _rotate_half(v: torch.Tensor, pos: torch.Tensor, freq: torch.Tensor) -> torch.Tensor:
    """v [T, ..., n] fp32: with nf = len(freq), entries i and i + nf of the last axis (i < nf) turn by
    the angle pos * freq[i] (angles in fp32); entries from 2 nf on pass."""
    half = freq.numel()
    a = pos.float().view(-1, *([1] * (v.dim() - 1))) * freq.float()
    c, s = torch.cos(a), torch.sin(a)
    u, x = v[..., :half], v[..., half:2 * half]
    return torch.cat([u * c - x * s, x * c + u * s, v[..., 2 * half:]], -1)


def _rotate_pairs(v: torch.Tensor, pos: torch.Tensor, freq: torch.Tensor) -> torch.Tensor:
    """The same turn with entries 2i and 2i + 1 paired (i < len(freq))."""
    nf = freq.numel()
    a = pos[:v.shape[0]].float().view(-1, *([1] * (v.dim() - 1))) * freq.float()
    c, s = torch.cos(a), torch.sin(a)
    u, x = v[..., 0:2 * nf:2], v[..., 1:2 * nf:2]
    out = v.clone()
    out[..., 0:2 * nf:2] = u * c - x * s
    out[..., 1:2 * nf:2] = x * c + u * s
    return out


def _rotate(v: torch.Tensor, pos: torch.Tensor, freq: torch.Tensor, pairs: bool) -> torch.Tensor:
    return _rotate_pairs(v, pos, freq) if pairs else _rotate_half(v, pos[:v.shape[0]], freq)


def latent_prep(proj: torch.Tensor, q_rank: int, kv_rank: int, rot_dim: int, qw: torch.Tensor,
                kw: Optional[torch.Tensor], eps: float, positions: torch.Tensor, freq: torch.Tensor,
                k_cache: Optional[torch.Tensor], v_cache: Optional[torch.Tensor],
                slot_mapping: Optional[torch.Tensor], pairs: bool = False) -> None:
    """In place on the fused down-projections [T, q_rank | kv_rank | rot_dim] (or [T, q_rank] for a
    layer that reads another layer's cache): the query latent is RMS-normed (weight ``qw``); the
    key/value latent is RMS-normed (weight ``kw``) and the shared key part behind it is rotated by
    its position (``freq``: rotary_freq; ``pairs``: entries 2i and 2i + 1 turn together instead of i
    and i + len(freq)); both go to the pages at ``slot_mapping`` - the key page
    row is [latent | rotated part] (the page's rows may be wider: what lies behind is left as it is,
    zero), the value page holds the latent once more, dim-major."""
    T = proj.shape[0]
    if not proj.is_cuda:
        q = proj[:, :q_rank].float()
        proj[:, :q_rank] = (q * torch.rsqrt(q.pow(2).mean(-1, keepdim=True) + eps) * qw.float()).to(proj.dtype)
        if k_cache is None:
            return
        c = proj[:, q_rank:q_rank + kv_rank].float()
        c = (c * torch.rsqrt(c.pow(2).mean(-1, keepdim=True) + eps) * kw.float()).to(proj.dtype)
        kr = _rotate(proj[:, q_rank + kv_rank:q_rank + kv_rank + rot_dim].float(), positions, freq, pairs).to(proj.dtype)
        proj[:, q_rank:q_rank + kv_rank] = c
        proj[:, q_rank + kv_rank:q_rank + kv_rank + rot_dim] = kr
        ok = slot_mapping[:T] >= 0
        s = slot_mapping[:T][ok].long()
        bs = k_cache.shape[1]
        k_cache.view(-1, k_cache.shape[2])[s, :kv_rank + rot_dim] = proj[ok, q_rank:q_rank + kv_rank + rot_dim]
        v_cache.view(-1, kv_rank, bs)[s // bs, :, s % bs] = c[ok]
        return
    native().latent_prep(proj, int(q_rank), int(kv_rank), int(rot_dim), qw, kw, float(eps), positions, freq,
                         k_cache, v_cache, slot_mapping, bool(pairs))


def latent_queries(q: torch.Tensor, q_lat: torch.Tensor, H: int, dim: int, rot_dim: int, positions: torch.Tensor,
                   freq: torch.Tensor, pitch: int = 0, pairs: bool = False) -> torch.Tensor:
    """The queries against the latent cache: per head [q_lat | rotated part | zeros], [T, H * pitch]
    (``pitch`` 0: R + rot_dim, no padding; else the key pages' row width).
    ``q`` [T, H * (dim + rot_dim)] are the up-projected queries (their last ``rot_dim`` entries per
    head are rotated by the position) and ``q_lat`` [H, T, R] the unrotated parts already
    multiplied into the latent space."""
    T, R = q.shape[0], q_lat.shape[2]
    pitch = pitch or R + rot_dim
    if not q.is_cuda:
        qr = _rotate(q.view(T, H, dim + rot_dim)[..., dim:].float(), positions, freq, pairs).to(q.dtype)
        pad = torch.zeros(T, H, pitch - R - rot_dim, dtype=q.dtype)
        return torch.cat([q_lat.transpose(0, 1), qr, pad], -1).reshape(T, H * pitch)
    out = torch.empty(T, H * pitch, dtype=q.dtype, device=q.device)
    native().latent_queries(out, q, q_lat, int(H), int(dim), int(rot_dim), positions, freq, bool(pairs))
    return out


_NO_SINK: dict = {}


def _no_sink(H: int, device) -> torch.Tensor:
    key = (H, str(device))
    if key not in _NO_SINK:
        _NO_SINK[key] = torch.full((H,), -1.0e30, dtype=torch.float32, device=device)
    return _NO_SINK[key]


def latent_attention(qa: torch.Tensor, k_cache: torch.Tensor, v_cache: torch.Tensor, block_tables: torch.Tensor,
                     H: int, scale: float, window: int, sinks: Optional[torch.Tensor], cu: Optional[torch.Tensor] = None,
                     ctx: Optional[torch.Tensor] = None, seq_lens: Optional[torch.Tensor] = None, fast: int = 1,
                     split: int = 0, sink: bool = True) -> torch.Tensor:
    """Attention of ``qa`` [T, H * pitch] (latent_queries) over the latent pages: every head reads
    the one key stream ``k_cache`` [blocks, bs, pitch] and the one value stream ``v_cache`` [blocks, 1,
    kv_rank, bs]; sliding window and learned sinks as in window_attention_* (``sink`` False: an
    ordinary softmax, nothing but the keys in the denominator).  ``cu`` / ``ctx``: prompt
    chunks (rows of segment s at positions ctx[s] ..); else ``seq_lens``: one row per sequence, at its
    newest token.  Returns [T, H * kv_rank].  GPU, bf16, pitch a multiple of 32 up to 320 and kv_rank a
    multiple of 16 up to 256 (``fast``): the matrix-core kernel, 16 heads of one token per tile
    (``split`` 1 / 2: one wave per one / two tokens, 4 / 8: that many waves share a token's window,
    32 / 33: pages staged in LDS for eight / four tokens of a chunk at a time; 0: by the step's size -
    large steps' chunks take 33, few rows 8); other sizes and fp32:
    the any-size kernels with one shared key/value head."""
    T, pitch, dv = qa.shape[0], k_cache.shape[2], v_cache.shape[2]
    if not sink:
        sinks = None
    if qa.is_cuda and fast and qa.dtype == torch.bfloat16:
        out = torch.empty(T, H * dv, dtype=qa.dtype, device=qa.device)
        # the matrix-core kernels start every row from a sink term; without one that term gets a logit
        # so low that its weight exp(logit - max) is exactly zero in fp32
        sk = sinks if sink else _no_sink(H, qa.device)
        if native().latent_attention(out, qa, k_cache, v_cache, cu, ctx, seq_lens, block_tables, int(H), float(scale),
                                     int(window), sk, int(split)):
            return out
    args = (H, 1, pitch, dv, scale, window, bool(sink))
    if cu is not None:
        return window_attention_prefill(qa, k_cache, v_cache, cu, ctx, block_tables, *args, mfma=fast, sinks=sinks)
    return window_attention_decode(qa, k_cache, v_cache, block_tables, seq_lens, *args, vec=bool(fast), sinks=sinks)


# ---------------------------------------------------------------- Mamba-2

def conv_silu(proj: torch.Tensor, col0: int, C: int, conv_w: torch.Tensor, conv_b: Optional[torch.Tensor],
              conv_state: torch.Tensor, seg_cu: torch.Tensor, seg_ctx: torch.Tensor,
              seg_slot: torch.Tensor) -> torch.Tensor:
    """Causal per-channel convolution + SiLU over columns [col0, col0 + C) of ``proj`` [T, *];
    ``conv_w`` [C, taps] (the last tap multiplies the current token), ``conv_b`` [C] (None: no bias).  The taps - 1
    inputs before a segment come from ``conv_state`` [slots, taps - 1, C] (zeros where seg_ctx is
    0), which is then advanced to the segment's end."""
    T = proj.shape[0]
    taps = conv_w.shape[1]
    if not proj.is_cuda:
        out = torch.empty(T, C, dtype=proj.dtype)
        wt = conv_w.float().t()  # [taps, C]
        bf = conv_b.float() if conv_b is not None else torch.zeros(C)
        cul = seg_cu.tolist()
        for s, (c0, slot) in enumerate(zip(seg_ctx.tolist(), seg_slot.tolist())):
            a, b = cul[s], cul[s + 1]
            if slot < 0 or b <= a:
                continue
            x = proj[a:b, col0:col0 + C]
            hist = conv_state[slot, : taps - 1]
            if c0 <= 0:
                hist = torch.zeros_like(hist)
            full = torch.cat([hist.to(proj.dtype), x]).float()  # [taps - 1 + n, C]
            acc = bf.expand(b - a, C).clone()
            for j in range(taps):
                acc += full[j:j + b - a] * wt[j]
            out[a:b] = _silu(acc).to(proj.dtype)
            if taps > 1:
                conv_state[slot] = full[full.shape[0] - (taps - 1):].to(conv_state.dtype)
        return out
    out = torch.empty(T, C, dtype=proj.dtype, device=proj.device)
    native().conv_silu(out, proj, int(col0), conv_w, conv_b, conv_state, seg_cu, seg_ctx, seg_slot)
    return out


def ssm_scan(xbc: torch.Tensor, proj: Optional[torch.Tensor], dt_col: int, dt_bias: Optional[torch.Tensor],
             a_log: Optional[torch.Tensor], d_skip: Optional[torch.Tensor], state: torch.Tensor, seg_cu: torch.Tensor,
             seg_ctx: torch.Tensor, seg_slot: torch.Tensor, nh: int, P: int, N: int, G: int, mode: int = 0,
             decay: Optional[torch.Tensor] = None) -> torch.Tensor:
    """The selective state-space recurrence, fp32, token by token within each segment:

        dt = softplus(proj[t, dt_col + h] + dt_bias[h]);  S <- exp(-exp(a_log[h]) dt) S + dt B_t x_t^T
        y_t = S^T C_t + d_skip[h] x_t

    ``xbc`` [T, nh*P | G*N | G*N] holds x, B, C (head h reads group h // (nh / G)); ``state``
    [slots, nh, N, P] fp32 is read at the segment's start (zero where seg_ctx is 0) and written
    back at its end.  Returns y [T, nh*P] fp32.  GPU: two lane mappings of the same arithmetic,
    chosen by the step's mean segment length (``mode`` 1 / 2 forces the decode / the prompt one).

    ``decay`` [nh] fp32 (then ``proj``, ``dt_bias``, ``a_log``, ``d_skip`` are not read): the
    recurrence with a fixed decay per head, step size 1 and no skip term,
    ``S <- decay[h] S + B_t x_t^T;  y_t = S^T C_t`` - linear attention with B, C, x = k, q, v
    (linear_attention below)."""
    T = xbc.shape[0]
    if not xbc.is_cuda:
        y = torch.zeros(T, nh * P, dtype=torch.float32)
        fixed = decay is not None
        A = torch.exp(a_log.float()) if not fixed else None
        Dk = d_skip.float() if not fixed else torch.zeros(nh)
        cul = seg_cu.tolist()
        inner = nh * P
        for s, (c0, slot) in enumerate(zip(seg_ctx.tolist(), seg_slot.tolist())):
            a, b = cul[s], cul[s + 1]
            if slot < 0 or b <= a:
                continue
            S = state[slot].clone() if c0 > 0 else torch.zeros_like(state[slot])
            xs = xbc[a:b, :inner].float().view(-1, nh, P)
            Bs = xbc[a:b, inner:inner + G * N].float().view(-1, G, N).repeat_interleave(nh // G, dim=1)
            Cs = xbc[a:b, inner + G * N:].float().view(-1, G, N).repeat_interleave(nh // G, dim=1)
            if fixed:
                dt = torch.ones(b - a, nh)
                dec = decay.float().expand(b - a, nh)
            else:
                dt = F.softplus(proj[a:b, dt_col:dt_col + nh].float() + dt_bias.float(), threshold=30.0)
                dec = torch.exp(-A * dt)
            for t in range(b - a):
                S = dec[t, :, None, None] * S + dt[t, :, None, None] * Bs[t, :, :, None] * xs[t, :, None, :]
                y[a + t] = (torch.einsum("hnp,hn->hp", S, Cs[t]) + Dk[:, None] * xs[t]).reshape(-1)
            state[slot] = S
        return y
    y = torch.empty(T, nh * P, dtype=torch.float32, device=xbc.device)
    native().ssm_scan(y, xbc, proj, int(dt_col), dt_bias, a_log, d_skip, decay, state, seg_cu, seg_ctx, seg_slot, nh, P,
                      N, G, int(mode))
    return y


def linear_attention(vkq: torch.Tensor, decay: torch.Tensor, state: torch.Tensor, seg_cu: torch.Tensor,
                     seg_ctx: torch.Tensor, seg_slot: torch.Tensor, H: int, dk: int, dv: int, mode: int = 0,
                     col_tiles: int = 0) -> torch.Tensor:
    """Linear attention with a fixed decay per head, as a recurrence over each segment:

        S_t = decay[h] S_(t-1) + k_t v_t^T;   o_t = S_t^T q_t

    ``vkq`` [T, H*dv | H*dk | H*dk] holds v, k, q head by head (contiguous); ``state`` [slots, H, dk,
    dv] fp32 is read at a segment's start (zero where seg_ctx is 0) and written back at its end.
    Returns o [T, H*dv] fp32.  State, products and sums are fp32.

    GPU: the sequential scan (``ssm_scan`` with the decay table; ``mode`` 1 / 2 force its decode /
    prompt lane mapping), or - bf16 prompts (a mean of 32 rows per segment and more), ``dim`` a multiple
    of 32 up to 128, ``vdim`` a multiple of 16; ``mode`` 3 forces it, ``col_tiles`` 1 / 2 its value
    columns per workgroup (16 / 32; 0: 16) - chunks of 64 tokens on the matrix
    cores: q.k on the bf16 instruction, everything that holds scores or state on the fp32 one, only the
    state crossing chunks (the order of the fp32 sums then follows the chunk grid, which starts at the
    segment's first row)."""
    if vkq.is_cuda and vkq.dtype == torch.bfloat16 and (mode == 3 or (mode == 0 and vkq.shape[0] >= 32 * seg_ctx.numel())):
        y = torch.empty(vkq.shape[0], H * dv, dtype=torch.float32, device=vkq.device)
        if native().linear_attention_chunked(y, vkq, decay, state, seg_cu, seg_ctx, seg_slot, H, dk, dv, int(col_tiles)):
            return y
    return ssm_scan(vkq, None, 0, None, None, None, state, seg_cu, seg_ctx, seg_slot, H, dv, dk, H, mode if mode < 3 else 0, decay=decay)


def decay_scan(qkv: torch.Tensor, q_col: int, k_col: int, v_col: int, z: torch.Tensor, z_bias: torch.Tensor,
               state: torch.Tensor, seg_cu: torch.Tensor, seg_ctx: torch.Tensor, seg_slot: torch.Tensor, H: int, Gk: int,
               dk: int, dv: int, q_scale: float, a_log: Optional[torch.Tensor] = None, tau: float = 1.0,
               beta: Optional[torch.Tensor] = None, beta_col: int = 0, unit: bool = False, mode: int = 0) -> torch.Tensor:
    """Linear attention with a decay per head and key channel, optionally with the delta rule, as an
    fp32 recurrence over each segment.  Per head h (reading query / key head ``h // (H / Gk)``) and token:

        S <- diag(g_t) S                       g_t [dk]: this token's decays
        delta rule:   u = beta_t (v_t - S^T k_t);   S <- S + k_t u^T
        otherwise:                                  S <- S + k_t v_t^T
        o_t = S^T q_t

    ``qkv`` [T, *] holds q, k ([Gk*dk] each) and v ([H*dv]) from columns ``q_col``, ``k_col``, ``v_col``
    on; q is multiplied by ``q_scale``.  ``unit``: q and k heads are first made unit vectors,
    ``x / sqrt(sum(x^2) + 1e-6)``.  The decays come from ``z`` [T, H*dk] (a projection, activation dtype)
    and ``z_bias`` [H*dk] fp32:  ``a_log`` [H] given: ``g = exp(-exp(a_log[h]) softplus(z + z_bias))``;
    else ``g = sigmoid(z + z_bias)^(1 / tau)``.  ``beta`` [T, *] (given = the delta rule): column
    ``beta_col + h`` holds head h's logit, ``beta_t = sigmoid(logit)``.  ``state`` [slots, H, dv, dk] fp32
    (a value row's key channels contiguous) is read at a segment's start (zero where seg_ctx is 0) and
    written back at its end.  Returns o [T, H*dv] fp32.  Decays, unit norms, gates, state, products and
    sums are fp32.

    GPU: steps of prompts (a mean segment length of 32 rows or more) run as two launches - everything
    that does not depend on the state (decays, unit norms, k . q, beta) for all rows at once into an fp32
    workspace, then the recurrence over it; decode steps run as one launch.  ``mode`` 1 / 2 force the
    one-launch / two-launch form (tests)."""
    T = qkv.shape[0]
    if not qkv.is_cuda:
        o = torch.zeros(T, H * dv, dtype=torch.float32)
        rep = H // Gk
        cul = seg_cu.tolist()
        for s, (c0, slot) in enumerate(zip(seg_ctx.tolist(), seg_slot.tolist())):
            a, b = cul[s], cul[s + 1]
            if slot < 0 or b <= a:
                continue
            n = b - a
            q = qkv[a:b, q_col:q_col + Gk * dk].float().view(n, Gk, dk)
            k = qkv[a:b, k_col:k_col + Gk * dk].float().view(n, Gk, dk)
            v = qkv[a:b, v_col:v_col + H * dv].float().view(n, H, dv)
            if unit:
                q = q * torch.rsqrt(q.pow(2).sum(-1, keepdim=True) + 1e-6)
                k = k * torch.rsqrt(k.pow(2).sum(-1, keepdim=True) + 1e-6)
            q = (q * q_scale).repeat_interleave(rep, dim=1)
            k = k.repeat_interleave(rep, dim=1)
            zz = (z[a:b].float() + z_bias.float()).view(n, H, dk)
            if a_log is not None:
                g = torch.exp(-torch.exp(a_log.float()).view(1, H, 1) * F.softplus(zz, threshold=30.0))
            else:
                g = torch.exp(F.logsigmoid(zz) / tau)
            bt = torch.sigmoid(beta[a:b, beta_col:beta_col + H].float()) if beta is not None else None
            S = state[slot].clone() if c0 > 0 else torch.zeros_like(state[slot])  # [H, dv, dk]
            for t in range(n):
                S = S * g[t, :, None, :]
                if bt is not None:
                    u = bt[t, :, None] * (v[t] - torch.einsum("hpn,hn->hp", S, k[t]))
                else:
                    u = v[t]
                S = S + u[:, :, None] * k[t, :, None, :]
                o[a + t] = torch.einsum("hpn,hn->hp", S, q[t]).reshape(-1)
            state[slot] = S
        return o
    o = torch.empty(T, H * dv, dtype=torch.float32, device=qkv.device)
    ws = None
    if mode == 2 or (mode == 0 and T >= 32 * seg_slot.numel()):
        ws = torch.empty(T * (2 * Gk * dk + H * dk + Gk + H), dtype=torch.float32, device=qkv.device)
    native().decay_scan(o, qkv, int(q_col), int(k_col), int(v_col), z, z_bias, a_log, float(tau), beta, int(beta_col),
                        state, seg_cu, seg_ctx, seg_slot, int(H), int(Gk), int(dk), int(dv), float(q_scale), bool(unit), ws)
    return o


def gated_group_norm(y: torch.Tensor, proj: torch.Tensor, z_col: int, w: torch.Tensor, eps: float, groups: int,
                     out_dtype: torch.dtype, after: bool = False, gate: str = "sigmoid") -> torch.Tensor:
    """``y`` [T, n] fp32 times silu of the gate ``proj[:, z_col : z_col + n]``, then RMS-normed in
    ``groups`` equal parts (each by its own root mean square) times ``w`` [n].  ``after``: the norm
    first (of ``y`` as it is), then times ``w`` and the SIGMOID of the gate (``gate`` "silu": its SiLU)."""
    T, n = y.shape
    if not y.is_cuda:
        if after:
            g = y.view(T, groups, n // groups)
            g = g * torch.rsqrt(g.pow(2).mean(-1, keepdim=True) + eps)
            z = proj[:, z_col:z_col + n].float()
            return (g.reshape(T, n) * w.float() * (torch.sigmoid(z) if gate == "sigmoid" else _silu(z))).to(out_dtype)
        g = y * _silu(proj[:, z_col:z_col + n].float())
        g = g.view(T, groups, n // groups)
        g = g * torch.rsqrt(g.pow(2).mean(-1, keepdim=True) + eps)
        return (g.reshape(T, n) * w.float()).to(out_dtype)
    out = torch.empty(T, n, dtype=out_dtype, device=y.device)
    native().gated_group_norm(out, y, proj, int(z_col), w, float(eps), int(groups), (2 if gate == "silu" else 1) if after else 0)
    return out


# ---------------------------------------------------------------- routed experts

def moe_router(h: torch.Tensor, wr: torch.Tensor, bias: Optional[torch.Tensor], E: int, K: int,
               over_all: bool = False) -> tuple:
    """fp32 router: logits = ``wr[:E] h + bias[:E]`` (``bias`` None: none), the ``K`` largest are
    chosen and weighted by the softmax over the chosen logits only - or, ``over_all``, by their
    probabilities in the softmax over all E logits, as they are.  ``wr`` may hold one more row (E + 1 in all): then
    ``gate = sigmoid(wr[E] h)`` per token is returned too (the shared expert's gate).
    Returns (ids [T, K] int32, weights [T, K] fp32, gate [T] fp32 or None)."""
    T = h.shape[0]
    has_gate = wr.shape[0] == E + 1
    if not h.is_cuda:
        lg = h.float() @ wr.float().t()
        gate = torch.sigmoid(lg[:, E]) if has_gate else None
        z = lg[:, :E] + bias.float()[:E] if bias is not None else lg[:, :E]
        top, idx = torch.topk(z, K, dim=-1)
        if over_all:
            return idx.to(torch.int32), torch.softmax(z, -1).gather(1, idx), gate
        return idx.to(torch.int32), torch.softmax(top, -1), gate
    ids = torch.empty(T, K, dtype=torch.int32, device=h.device)
    wts = torch.empty(T, K, dtype=torch.float32, device=h.device)
    gate = torch.empty(T, dtype=torch.float32, device=h.device) if has_gate else None
    native().moe_router(ids, wts, gate, h, wr, bias, E, K, bool(over_all))
    return ids, wts, gate


def moe_router_grouped(h: torch.Tensor, wr: torch.Tensor, E: int, K: int, groups: int, keep: int,
                       scale: float) -> tuple:
    """fp32 router with sigmoid scores and a choice restricted to groups: ``s = sigmoid(wr h)``; the E
    experts form ``groups`` equal groups of neighbours, a group's score is the sum of its two largest
    scores (its one score where a group is one expert), and only experts of the ``keep`` best groups
    can be chosen; the ``K`` largest scores among those are taken (lowest index wins a tie) and
    weighted ``s / (sum of the chosen s + 1e-20) * scale``.  Returns (ids [T, K] int32, weights [T, K] fp32)."""
    T = h.shape[0]
    if not h.is_cuda:
        sc = torch.sigmoid(h.float() @ wr.float().t())
        masked = sc
        if groups > 1:
            per = E // groups
            gs = sc.view(T, groups, per).topk(min(2, per), dim=-1).values.sum(-1)
            best = gs.topk(keep, dim=-1).indices
            ok = torch.zeros(T, groups, dtype=torch.bool).scatter_(1, best, True)
            masked = torch.where(ok.repeat_interleave(per, dim=1), sc, torch.full_like(sc, -1.0))
        idx = masked.topk(K, dim=-1).indices
        w = sc.gather(1, idx)
        return idx.to(torch.int32), w / (w.sum(-1, keepdim=True) + 1e-20) * scale
    ids = torch.empty(T, K, dtype=torch.int32, device=h.device)
    wts = torch.empty(T, K, dtype=torch.float32, device=h.device)
    native().moe_router_grouped(ids, wts, h, wr, int(E), int(K), int(groups), int(keep), float(scale))
    return ids, wts


# expert-sorted rows from which the routed GEMMs of an interleaved (``il``) layer go to the
# framework's 256 x 256 prefill tile kernel (ops.moe_grouped_gemm) instead of the 16-row kernel
TILE_MIN_ROWS = 1024


def moe_experts(h: torch.Tensor, ids: torch.Tensor, wts: torch.Tensor, w13: torch.Tensor, w2: torch.Tensor,
                shared: Optional[torch.Tensor] = None, gate: Optional[torch.Tensor] = None, il: bool = False,
                mfma: bool = True, act: str = "swiglu", limit: float = 0.0, tile: bool = False) -> torch.Tensor:
    """Sum over each token's chosen experts of ``wts * down_e(silu(gate_e h) * up_e h)`` with
    ``w13`` [E, 2*ff, d] (gate rows then up rows; ``il``: interleaved per 128 rows as [64 gate |
    64 up], ops.interleave_gate_up) and ``w2`` [E, d, ff], plus ``gate * shared`` (the shared
    expert's output [T, d] and its per-token gate; ``gate`` None: 1).  ``act`` "gelu": ungated
    experts ``down_e(gelu(up_e h))`` with ``w13`` [E, ff, d].  ``act`` "clamped_swish": gated experts whose
    unit is ``g * sigmoid(1.702 g) * (u + 1)`` with g = min(gate_e h, limit), u = clamp(up_e h, -limit,
    limit).  fp32 [T, d].

    GPU: the (token, slot) pairs are counting-sorted by expert on the device and both projections
    run as ONE grouped launch each over the sorted rows (SwiGLU in the first epilogue); no host
    synchronisation.  bf16: matrix-core kernels - 16-row tiles with the rows gathered on load
    (decode, small steps), or from TILE_MIN_ROWS sorted rows of an ``il`` layer the prefill tile
    GEMM of the Mixtral path (ungated experts whose widths are multiples of 256 take it too, with
    the GELU as a launch between); fp32 (and K not a multiple of 32): the 64 x 64 fp32 tile kernel."""
    T, d = h.shape
    E, K = w13.shape[0], ids.shape[1]
    ff = w2.shape[2]
    if not h.is_cuda:
        out = torch.zeros(T, d, dtype=torch.float32)
        hf = h.float()
        for e in range(E):
            rows, slot = torch.nonzero(ids == e, as_tuple=True)
            if rows.numel():
                we = w13[e].float()
                if il:
                    we = we.view(ff // 64, 2, 64, d).permute(1, 0, 2, 3).reshape(2 * ff, d)
                gu = (hf[rows] @ we.t()).to(h.dtype).float()
                if act == "gelu":
                    a = F.gelu(gu).to(h.dtype).float()
                elif act == "clamped_swish":
                    a = _clamped_unit(gu[:, :ff], gu[:, ff:], limit).to(h.dtype).float()
                else:
                    a = (_silu(gu[:, :ff]) * gu[:, ff:]).to(h.dtype).float()
                out.index_add_(0, rows, (a @ w2[e].float().t()).to(h.dtype).float() * wts[rows, slot].unsqueeze(-1))
        if shared is not None:
            out += shared.float() * gate.unsqueeze(-1) if gate is not None else shared.float()
        return out
    ext = native()
    n = T * K
    offsets = torch.empty(E + 1, dtype=torch.int32, device=h.device)
    sorted_idx = torch.empty(n, dtype=torch.int32, device=h.device)
    inv_idx = torch.empty(n, dtype=torch.int32, device=h.device)
    ext.moe_align(ids, E, offsets, sorted_idx, inv_idx)
    code = {"swiglu": 1, "gelu": 2, "clamped_swish": 3}[act]
    if act == "gelu" and n >= TILE_MIN_ROWS and h.dtype == torch.bfloat16 and ff % 256 == 0 and d % 256 == 0:
        from .. import ops  # large steps of plain experts: the prefill tile GEMM twice, GELU between

        xs = ops.gather_rows(h, sorted_idx, K)
        a = activation(ops.moe_grouped_gemm(xs, w13, offsets, zero_fill=False), "gelu")
        ys = ops.moe_grouped_gemm(a, w2, offsets, zero_fill=False)
    elif act == "clamped_swish" and tile and n >= TILE_MIN_ROWS and h.dtype == torch.bfloat16:
        from .. import ops  # large steps: the prefill tile GEMM twice, the clamped unit as a launch between

        xs = ops.gather_rows(h, sorted_idx, K)
        a = glu(ops.moe_grouped_gemm(xs, w13, offsets, zero_fill=False), 0, ff, "clamped_swish", limit)
        ys = ops.moe_grouped_gemm(a, w2, offsets, zero_fill=False)
    elif il and n >= TILE_MIN_ROWS and h.dtype == torch.bfloat16:
        from .. import ops  # the Mixtral path's kernels (_k8sllm_ops)

        xs = ops.gather_rows(h, sorted_idx, K)
        a = ops.moe_grouped_gemm(xs, w13, offsets, swiglu=True, zero_fill=False)
        ys = ops.moe_grouped_gemm(a, w2, offsets, zero_fill=False)
    else:
        a = torch.empty(n, ff, dtype=h.dtype, device=h.device)
        ext.grouped_gemm(a, h, w13, offsets, sorted_idx, K, code, il, mfma, float(limit))
        ys = torch.empty(n, d, dtype=h.dtype, device=h.device)
        ext.grouped_gemm(ys, a, w2, offsets, None, 1, 0, False, mfma, 0.0)
    out = torch.empty(T, d, dtype=torch.float32, device=h.device)
    ext.moe_combine(out, ys, inv_idx, wts, shared, gate)
    return out


def swiglu(gu: torch.Tensor) -> torch.Tensor:
    """silu(gu[:, :f]) * gu[:, f:] for [T, 2f] rows ([gate | up])."""
    f = gu.shape[1] // 2
    if not gu.is_cuda:
        return (_silu(gu[:, :f].float()) * gu[:, f:].float()).to(gu.dtype)
    out = torch.empty(gu.shape[0], f, dtype=gu.dtype, device=gu.device)
    native().swiglu(out, gu)
    return out
