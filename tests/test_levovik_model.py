"""The Levovik layer-list design in the engine against the plain float64 oracle
(tests/levovik_oracle.py): each mechanism alone (the two softmax attentions - sinks, norms before or
after the rotation, keys as values, rescaled rotation frequencies -, the gated delta rule with its
short convolutions, gated linear attention, the weighted sum of two mixers, layer norm, the per-layer
token input, ReLU-gated dense layers, the group-limited router with clamped experts), prefill against
token-by-token decoding, prompt portions down to two tokens, unequal batches, pages and state slots
that are reused, tokens far away and at page borders, the causal edge, the first tokens, long
decoding, odd sizes and sizes of one, and greedy generation through the engine and the trace command.

Runs on the CPU (the ops' torch forms); the ``gpu`` tests at the end run the same comparisons
through the HIP kernels."""
import copy
import json
import subprocess
import sys

import numpy as np
import pytest
import torch

import levovik_oracle as O
from k8s_llm_monitor_amd.engine import EngineConfig, LLMEngine, SamplingParams
from k8s_llm_monitor_amd.models.config import get_config, hybrid_config_from_dict, hybrid_config_to_dict
from k8s_llm_monitor_amd.models.hybrid import state_dict
from k8s_llm_monitor_amd.models.registry import build_model, config_from_dir
from k8s_llm_monitor_amd.ops import hybrid as hops
from test_hybrid_model import ROOT, Rig, _save, close, toks


# ------------------------------------------------------------------ small configurations

def rot(dims=8, base=100.0, factor=4.0, original=32, low=1.0, high=4.0):
    """base 100 over 8 entries with original 32: one frequency kept, one blended, two slowed."""
    return {"dims": dims, "base": base, "scaling": {"factor": factor, "low": low, "high": high, "original": original}}


def att_a(heads=4, kv=2, dim=12, vdim=10, scale=0.3, **r):
    return {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale, "rot": rot(**r)}


def att_b(heads=4, kv=2, dim=12, scale=0.3, **r):
    return {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": dim, "scale": scale, "rot": rot(**r)}


def delta(heads=4, kv=2, dim=6, vdim=10, conv=3, a_rank=5, g_rank=7):
    return {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "conv": conv, "a_rank": a_rank, "g_rank": g_rank}


def gla(heads=3, dim=6, vdim=10, tau=4.0, a_rank=5):
    return {"heads": heads, "dim": dim, "vdim": vdim, "tau": tau, "a_rank": a_rank}


def par(left=None, right=None, ls=0.9, rs=1.3, mlp=None):
    return {"type": "parallel", "mixer": {"left": left or att_a(), "right": right or delta(), "left_scale": ls,
                                          "right_scale": rs}, "mlp": mlp}


def par2(left=None, right=None, ls=1.2, rs=0.7, mlp=None):
    return {"type": "parallel_2", "mixer": {"left": left or att_b(), "right": right or gla(), "left_scale": ls,
                                            "right_scale": rs}, "mlp": mlp}


def dense(ff=36):
    return {"kind": "dense", "ff": ff}


def moe(experts=6, top=2, ff=10, limit=1.0, groups=(3, 2), scale=1.5):
    r = {"experts": experts, "top": top, "scale": scale}
    if groups:
        r["groups"] = {"count": groups[0], "keep": groups[1]}
    return {"kind": "moe", "expert": {"ff": ff, "limit": limit}, "router": r}


def make_cfg(layers, width=40, vocab=61, eps=1e-5, embed=3.0, side=6, logit_scale=0.7):
    c = {"architecture": "Levovik", "vocab": vocab, "width": width, "layers": layers, "norm": {"eps": eps},
         "embedding": {"scale": embed}, "logit_scale": logit_scale}
    if side:
        c["token_side"] = {"dim": side}
    return c


FULL = make_cfg([par2(mlp=dense(28)), par(mlp=moe()), par2(att_b(6, 3, 8, 0.35, dims=8, base=50.0), gla(2, 10, 4, 16.0)),
                 par(att_a(3, 1, 16, 6, 0.25, dims=4), delta(2, 2, 8, 12, 4), 0.5, 1.0, mlp=moe(8, 3, 6, 0.8, (2, 1), 2.0)),
                 par2(mlp=moe(4, 1, 12, 2.0, None, 1.0))])


def rig_for(cfg, seed=0, w=None, **kw):
    return Rig(dict(cfg, max_positions=kw.pop("max_positions", 1024)), w=w if w is not None else O.random_weights(cfg, seed), **kw)


# ------------------------------------------------------------------ mechanisms alone

@pytest.mark.parametrize("layers,kw", [
    ([par()], {}), ([par(att_a(1, 1, 8, 8, 1.0, dims=8, base=10.0), delta(1, 1, 1, 1, 1, 1, 1))], {}),
    ([par(att_a(6, 1, 10, 4, dims=2), delta(6, 1, 4, 3, 5))], {}), ([par(att_a(3, 3, 6, 9, dims=0), delta(3, 3, 9, 5, 2))], {}),
    ([par2()], {}), ([par2(att_b(1, 1, 2, 1.0, dims=2), gla(1, 1, 1, 1.0, 1))], {}),
    ([par2(att_b(6, 2, 10, dims=6, factor=1.0), gla(4, 9, 5, 64.0))], {}), ([par2(att_b(2, 2, 6, dims=0))], {}),
    ([par(ls=0.0, rs=1.0)], {}), ([par2(ls=1.0, rs=0.0)], {}), ([par(mlp=dense())], {}), ([par2(mlp=dense(1))], {}),
    ([par(mlp=moe())], {}), ([par2(mlp=moe(6, 6, 4, 0.5, None))], {}), ([par(mlp=moe(6, 2, 8, 1.0, (6, 3)))], {}),
    ([par2(mlp=moe(8, 4, 8, 3.0, (2, 1)))], {}), ([par(mlp=moe(5, 1, 8, 1.0, (1, 1)))], {}),
    ([par(), par2()], dict(side=0, embed=1.0, logit_scale=1.0)), ([par2(mlp=dense())], dict(side=1)),
    ([par(att_a(original=4096, factor=16.0, low=2.0, high=8.0, base=1e6))], {})],
    ids=["sinks-delta", "ones", "mqa-two-rotating-five-taps", "no-rotation-own-keys", "keys-as-values-gla", "gla-ones",
         "factor-one-slow-decay", "b-no-rotation", "delta-only", "attention-b-only", "dense", "dense-ff1", "routed",
         "all-experts-no-groups", "groups-of-one", "top-is-a-whole-group", "one-group-top1", "no-side-no-scales",
         "side-of-one", "long-original"])
def test_single_mechanism_whole_prompt(layers, kw):
    cfg = make_cfg(layers, **kw)
    rig = rig_for(cfg, 3)
    t = toks(45, cfg["vocab"], 1)
    close(rig.run_cut("a", t, [45]), O.forward(cfg, rig.w, t))


def test_odd_sizes_everywhere():
    """Widths, ranks and head sizes that are multiples of nothing (rotated sizes stay even)."""
    cfg = make_cfg([par(att_a(5, 5, 7, 3, dims=6), delta(6, 3, 5, 7, 2, 3, 9), mlp=dense(11)),
                    par2(att_b(3, 1, 9, dims=2), gla(3, 5, 7, 3.0, 2), mlp=moe(9, 2, 5, 0.7, (3, 1))),
                    par(att_a(2, 1, 11, 13, dims=10), delta(1, 1, 13, 3, 6, 1, 2), mlp=moe(10, 4, 3, 1.3, (5, 2)))],
                   width=37, vocab=53, side=5)
    rig = rig_for(cfg, 31)
    t = toks(41, 53, 3)
    want = O.forward(cfg, rig.w, t)
    for cuts in ([41], [3, 2, 17], [1]):
        close(rig.run_cut("a", t, cuts), want)


def test_layer_outputs_match_oracle():
    rig = rig_for(FULL, 5)
    t = toks(19, FULL["vocab"], 3)
    rig.model.layer_probe = []
    rig.run_cut("a", t, [19])
    layers = O.layers_of(FULL, rig.w, t)
    assert len(rig.model.layer_probe) == layers.shape[0] == 5
    for got, want in zip(rig.model.layer_probe, layers):
        close(got, want)
    rig.model.layer_probe = None


def test_ops_against_oracle_functions():
    g = torch.Generator().manual_seed(1)
    # frequencies: kept, blended and slowed entries, and no rescaling
    for r in (rot(), rot(16, 3e5, 6.0, 384), rot(6, 10.0, 2.0, 8, 0.5, 3.0)):
        close(hops.rotary_freq(r["base"], r["dims"], scaling=r["scaling"]), O.scaled_frequencies(r), tol=1e-6)
    fr = O.scaled_frequencies(rot())
    plain = O.scaled_frequencies({"dims": 8, "base": 100.0})
    assert fr[0] == plain[0] and plain[1] / 4 < fr[1] < plain[1] and abs(float(fr[3] * 4 / plain[3]) - 1) < 1e-12
    # weighted sums into the stream, a branch through its own RMS norm, then the layer norm
    x, a, b, y = (torch.randn(5, 12, generator=g) for _ in range(4))
    w, wy = torch.rand(12, generator=g) + 0.5, torch.rand(12, generator=g)
    res = x.clone()
    h = hops.sum_norm(res, ((a, 0.7), (b, 1.3)), (y, wy), w, 1e-5, True, False, torch.float32)
    want = x.double() + 0.7 * a.double() + 1.3 * b.double() + O.rms(y.double(), 1e-5) * wy.double()
    close(res, want, tol=1e-6)
    close(h, O.layer_norm(want, w.double(), 1e-5), tol=1e-6)
    # the per-layer token input's gate
    table, ids = torch.randn(9, 20, generator=g), torch.tensor([3, 8, 0, 3, 1], dtype=torch.int32)
    gate = torch.randn(5, 4, generator=g) * 2
    close(hops.gated_lookup(gate, table, ids, 8), O.gelu_tanh(gate.double()) * table[ids.long(), 8:12].double(), tol=1e-6)
    # the router against the written-out choice; the clamped unit against an expert
    hh, wr = torch.randn(40, 16, generator=g), torch.randn(12, 16, generator=g)
    for top, groups in ((3, (2, 1)), (2, (4, 2)), (4, (12, 5)), (5, None), (1, (3, 3))):
        r = {"experts": 12, "top": top, "scale": 2.5}
        if groups:
            r["groups"] = {"count": groups[0], "keep": groups[1]}
        ids_w, wt_w = O.route(hh.double(), {"router": wr.double()}, "", r)
        ids_g, wt_g = hops.moe_router_grouped(hh, wr, 12, top, *(groups or (1, 1)), 2.5)
        order = ids_g.long().argsort(-1)
        order_w = ids_w.argsort(-1)
        assert torch.equal(ids_g.long().gather(1, order), ids_w.gather(1, order_w))
        close(wt_g.gather(1, order), wt_w.gather(1, order_w), tol=1e-6)
    z = torch.randn(6, 24, generator=g) * 2
    we = {"gate": torch.eye(8, dtype=torch.float64), "up": torch.eye(8, dtype=torch.float64), "down": torch.eye(8, dtype=torch.float64)}
    gu = torch.cat([z[:, 3:11], z[:, 11:19]], 1)
    wantu = O.expert(torch.zeros(1, 8, dtype=torch.float64), we, "", 1.1)  # shape check of the oracle's expert
    assert wantu.shape == (1, 8)
    gcl, ucl = z[:, 3:11].double().clamp(max=1.1), z[:, 11:19].double().clamp(-1.1, 1.1)
    close(hops.glu(z, 3, 8, "clamped_swish", 1.1), gcl * torch.sigmoid(1.702 * gcl) * (ucl + 1.0), tol=1e-6)
    close(hops.glu(z, 3, 8, "relu"), torch.relu(gu[:, :8].double()) * gu[:, 8:].double(), tol=1e-6)
    # norm before the turn with weights, and after it without; keys as values
    Hq, G, dk, T = 4, 2, 10, 7
    pos = torch.tensor([0, 1, 2, 50, 51, 400, 1000], dtype=torch.int32)
    f32 = hops.rotary_freq(100.0, 6, scaling=rot(6)["scaling"])
    f64 = O.scaled_frequencies(rot(6))
    qw, kw = torch.rand(dk, generator=g) + 0.5, torch.rand(dk, generator=g) + 0.5
    for norm, pairs, vk in ((1, True, True), (2, False, False)):
        dv = dk if vk else 6
        qkv = torch.randn(T, Hq * dk + G * dk + (0 if vk else G * dv), generator=g)
        q0, k0 = qkv[:, :Hq * dk].double().view(T, Hq, dk), qkv[:, Hq * dk:Hq * dk + G * dk].double().view(T, G, dk)
        kc, vc = torch.zeros(80, 16, G * dk), torch.zeros(80, G, dv, 16)
        slots = pos.clone()
        got = qkv.clone()
        hops.rotary_cache(got, Hq, G, dk, dv, pos, f32, pairs, None, kc, vc, slots, norm=norm, qw=qw, kw=kw, eps=1e-5, v_from_k=vk)
        for t in range(T):
            p = int(pos[t])
            if norm == 1:
                wq = O.rotate(O.rms(q0[t], 1e-5) * qw.double(), p, f64, True)
                wk = O.rotate(O.rms(k0[t], 1e-5) * kw.double(), p, f64, True)
            else:
                wq, wk = O.rms(O.rotate(q0[t], p, f64, False), 1e-5), O.rms(O.rotate(k0[t], p, f64, False), 1e-5)
            close(got[t, :Hq * dk].view(Hq, dk), wq, tol=1e-4)
            close(kc.view(-1, G, dk)[p], wk, tol=1e-4)
            wantv = k0[t] if vk else qkv[t, Hq * dk + G * dk:].double().view(G, dv)
            close(vc[p // 16, :, :, p % 16], wantv, tol=1e-6)


def _scan_inputs(g, n, H, Gk, dk, dv):
    qkv = torch.randn(n, 2 * Gk * dk + H * dv + H, generator=g)
    z = torch.randn(n, H * dk, generator=g)
    return qkv, z, torch.randn(H * dk, generator=g), torch.randn(H, generator=g) * 0.5 - 0.5


def _scan_want(qkv, z, zb, a_log, H, Gk, dk, dv, delta_rule, tau):
    """The recurrence written out in float64 for one sequence, no cache: rows [q | k | v | beta]."""
    n = qkv.shape[0]
    q, k = qkv[:, :Gk * dk].double().view(n, Gk, dk), qkv[:, Gk * dk:2 * Gk * dk].double().view(n, Gk, dk)
    v, bl = qkv[:, 2 * Gk * dk:2 * Gk * dk + H * dv].double().view(n, H, dv), qkv[:, 2 * Gk * dk + H * dv:].double()
    zz = (z.double() + zb.double()).view(n, H, dk)
    if delta_rule:
        q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6)
        k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
        dec = torch.exp(-torch.exp(a_log.double()).view(1, H, 1) * O.softplus(zz))
    else:
        dec = torch.sigmoid(zz) ** (1.0 / tau)
    out = torch.zeros(n, H, dv, dtype=torch.float64)
    for h in range(H):
        gq = h // (H // Gk)
        S = torch.zeros(dk, dv, dtype=torch.float64)
        for t in range(n):
            S = dec[t, h].view(dk, 1) * S
            u = torch.sigmoid(bl[t, h]) * (v[t, h] - S.T @ k[t, gq]) if delta_rule else v[t, h]
            S = S + torch.outer(k[t, gq], u)
            out[t, h] = S.T @ q[t, gq] * dk ** -0.5
    return out.reshape(n, H * dv)


@pytest.mark.parametrize("delta_rule", [True, False], ids=["delta", "plain"])
def test_decay_scan_state_across_segments(delta_rule):
    """The recurrence over three segments of one sequence equals one pass; the slot holds leftovers of
    an earlier sequence, which a sequence that starts must not see."""
    g = torch.Generator().manual_seed(2)
    H, Gk, dk, dv, n = 4, (2 if delta_rule else 4), 3, 5, 21
    qkv, z, zb, a_log = _scan_inputs(g, n, H, Gk, dk, dv)
    want = _scan_want(qkv, z, zb, a_log, H, Gk, dk, dv, delta_rule, 3.0)
    state = torch.randn(3, H, dv, dk, generator=g)
    i32 = lambda *a: torch.tensor(a, dtype=torch.int32)
    outs = []
    for a, b in ((0, 4), (4, 5), (5, 21)):
        rows = qkv[a:b].contiguous()
        kw = dict(a_log=a_log, beta=rows, beta_col=2 * Gk * dk + H * dv, unit=True) if delta_rule else dict(tau=3.0)
        outs.append(hops.decay_scan(rows, 0, Gk * dk, 2 * Gk * dk, z[a:b].contiguous(), zb, state, i32(0, b - a),
                                    i32(a), i32(1), H, Gk, dk, dv, dk ** -0.5, **kw))
    close(torch.cat(outs), want, tol=1e-5)


# ------------------------------------------------------------------ cuts, decoding, batches

def test_prefill_equals_token_by_token_and_portions():
    rig = rig_for(FULL, 6)
    t = toks(70, FULL["vocab"], 4)
    want = O.forward(FULL, rig.w, t)
    for cuts in ([70], [], [2, 2, 3, 16, 1, 31], [15, 17, 16, 2], [33, 2, 2, 2], [64]):
        close(rig.run_cut("a", t, cuts), want)


def test_first_tokens_and_single_token_prompt():
    """Shorter than the convolutions' taps: the zeros before the start."""
    rig = rig_for(FULL, 7)
    for n in (1, 2, 3):
        t = toks(n, FULL["vocab"], 10 + n)
        close(rig.run_cut("a", t, [n]), O.forward(FULL, rig.w, t))
        close(rig.run_cut("a", t, []), O.forward(FULL, rig.w, t))


def test_long_decoding_over_pages():
    rig = rig_for(FULL, 8)
    t = toks(150, FULL["vocab"], 5)
    close(rig.run_cut("a", t, [20]), O.forward(FULL, rig.w, t))  # 130 decode steps over 9 pages


def test_unequal_batch_equals_each_alone_and_reuse():
    """Four live requests with portions beside decode tokens; one ends and its pages and slot are
    taken by a new request whose logits must not see the old pages, the old recurrent state or the old
    convolution inputs."""
    rig = rig_for(FULL, 9, num_blocks=24)
    V = FULL["vocab"]
    T = {n: toks(k, V, s) for n, k, s in (("a", 50, 1), ("b", 21, 2), ("c", 3, 3), ("d", 37, 4), ("e", 44, 5))}
    want = {n: O.forward(FULL, rig.w, t) for n, t in T.items()}
    got = {n: [] for n in T}
    at = {n: 0 for n in T}

    def go(plan, end=()):
        entries = []
        for n, k in plan:
            entries.append((n, T[n][at[n]:at[n] + k]))
            at[n] += k
        for n, lg in rig.step(entries, end).items():
            got[n].append(lg)

    go([("a", 17), ("b", 2), ("c", 3)], end=["c"])
    go([("a", 1), ("b", 19), ("d", 30)], end=["b"])
    go([("a", 1), ("d", 1), ("e", 16)])  # e takes the freed slot and pages
    go([("a", 31), ("d", 2), ("e", 1)], end=["a"])
    go([("d", 1), ("e", 1)])
    go([("d", 3), ("e", 26)], end=["d", "e"])
    assert not rig.live
    for n in T:
        assert at[n] == len(T[n])
        close(torch.cat(got[n]), want[n])
    assert rig.blocks.num_free == 24 and len(rig.blocks._free_slots) == 4


# ------------------------------------------------------------------ faults made visible

def _spiked(cfg, seed, far, n, scale_up=()):
    """Weights and a prompt in which ONE position stands out: its token has a large embedding, and the
    named projections are scaled up, so that a token that is lost or seen too early moves the logits
    far beyond rounding."""
    w = O.random_weights(cfg, seed)
    t = toks(n, cfg["vocab"] - 1, seed)
    special = cfg["vocab"] - 1
    t[far] = special
    w["embed"] = w["embed"].clone()
    w["embed"][special] *= 6.0
    for name in scale_up:
        w[name] = w[name] * 4.0
    return w, t


ALONE = {"attention-a": (par(att_a(2, 1, 8, 8, dims=4), ls=1.0, rs=0.0), "l0.mix.left.v"),
         "attention-b": (par2(att_b(2, 1, 8, dims=4), ls=1.0, rs=0.0), "l0.mix.left.o"),
         "delta": (par(right=delta(2, 1, 6, 6, 3), ls=0.0, rs=1.0), "l0.mix.right.v"),
         "gla": (par2(right=gla(2, 6, 6, 8.0), ls=0.0, rs=1.0), "l0.mix.right.v")}


@pytest.mark.parametrize("name", list(ALONE))
def test_causal_edge(name):
    """The position of the spiked token is the first that sees it: the one before does not, in a whole
    prompt, in decoding, with the edge at a page border, and in two-token portions."""
    layer, vname = ALONE[name]
    cfg = make_cfg([layer], width=24, vocab=37, side=0)
    for far in (15, 16, 30):
        w, t = _spiked(cfg, 11, far, far + 6, (vname,))
        want = O.forward(cfg, w, t)
        t2 = list(t)
        t2[far] = 0
        moved = O.forward(cfg, w, t2)
        assert float((moved[far] - want[far]).abs().max()) > 1e-2 and float((moved[far + 5] - want[far + 5]).abs().max()) > 1e-3
        assert float((moved[far - 1] - want[far - 1]).abs().max()) < 1e-12
        for cuts in ([len(t)], [far], [far - 3, 7], [2] * (far // 2 + 2)):
            close(rig_for(cfg, w=w).run_cut("a", t, cuts), want, tol=1e-4)


def _beacon(cfg, seed, far, n):
    """The left attention of a one-layer model scores ONE key far above the rest for every later query:
    the embedding axes 0, 1, 2 are set so that, after the layer norm's centring, (axis 0 - axis 2) is
    the same positive number for every token and (axis 1 - axis 2) is zero except for the special token;
    the last entry of every query head (it does not turn) reads the first, that of the key the second."""
    w, t = _spiked(cfg, seed, far, n)
    m = cfg["layers"][0]["mixer"]["left"]
    H, G, dk, d = m["heads"], m["kv_heads"], m["dim"], cfg["width"]
    e = O.random_weights(cfg, seed)["embed"]
    e[:, 0], e[:, 1], e[:, 2] = 1.0, 0.0, 0.0
    e[cfg["vocab"] - 1, 1] = 4.0
    w["embed"] = e
    w["l0.norm1"] = torch.ones(d)
    eye = torch.eye(d)
    c = dk - 1
    for h in range(H):
        w["l0.mix.left.q"][h * dk + c] = 8.0 * (eye[0] - eye[2])
    for g in range(G):
        w["l0.mix.left.k"][g * dk + c] = 8.0 * (eye[1] - eye[2])
    return w, t


@pytest.mark.parametrize("kind", ["a", "b"])
def test_far_key_among_hundreds_attention(kind):
    """One key takes a large part of the softmax of every later query, 300 tokens on: whole, decoded,
    and with the prompt cut at and around page borders."""
    layer = par(att_a(2, 1, 8, 8, 1.0, dims=4, base=1e4), ls=1.0, rs=0.2) if kind == "a" else \
        par2(att_b(2, 1, 8, 1.0, dims=4, base=1e4), ls=1.0, rs=0.2)
    cfg = make_cfg([layer], width=24, vocab=37, side=0, embed=1.0)
    n, far = 330, 20
    w, t = _beacon(cfg, 13, far, n)
    want = O.forward(cfg, w, t)
    t2 = list(t)
    t2[far] = 0
    assert float((O.forward(cfg, w, t2)[n - 1] - want[n - 1]).abs().max()) > 0.1
    for cuts in ([n], [310], [100, 2, 64, 130], [far + 12]):
        close(rig_for(cfg, w=w, num_blocks=32).run_cut("a", t, cuts), want, tol=1e-4)


def _marked_state(cfg, seed, far, n):
    """Only the special token writes to key channel 0 of the right mixer (its key row reads embedding
    axis 1 minus axis 2, zero for every other token also after the layer norm's centring), every query
    reads that channel (axis 0 minus axis 2, the same for all tokens), and the decays are near one: the
    far token's value stays in the state for hundreds of tokens, and other tokens' writes do not touch it."""
    w, t = _spiked(cfg, seed, far, n)
    L = cfg["layers"][0]
    m = L["mixer"]["right"]
    d, dk, P = cfg["width"], m["dim"], "l0.mix.right."
    e = w["embed"]
    e[:, 0], e[:, 1], e[:, 2] = 1.0, 0.0, 0.0
    e[cfg["vocab"] - 1, 1] = 2.0
    w["l0.norm1"] = torch.ones(d)
    eye = torch.eye(d)
    for r in range(w[P + "q"].shape[0] // dk):
        w[P + "q"][r * dk] = 3.0 * (eye[0] - eye[2])
        w[P + "k"][r * dk] = 3.0 * (eye[1] - eye[2])
    w[P + "v"] = w[P + "v"] * 3.0
    if L["type"] == "parallel":
        w[P + "A_log"] = torch.full_like(w[P + "A_log"], -4.0)
        w[P + "dt_bias"] = torch.full_like(w[P + "dt_bias"], -4.0)
        w[P + "a2"] = w[P + "a2"] * 0.1
        for nme in ("q", "k", "v"):  # the current token's tap dominates
            w[P + nme + ".conv"][:, -1] = 1.5
    else:
        w[P + "a2.b"] = torch.full_like(w[P + "a2.b"], 6.0)
        w[P + "a2"] = w[P + "a2"] * 0.1
    return w, t


@pytest.mark.parametrize("kind", ["delta", "gla"])
def test_far_token_in_the_recurrent_state(kind):
    """A state lost at the start of a portion or of a decode step, or a slot mixed up, would show."""
    layer = par(right=delta(2, 1, 6, 6, 3), ls=0.1, rs=1.0) if kind == "delta" else par2(right=gla(2, 6, 6, 16.0), ls=0.1, rs=1.0)
    cfg = make_cfg([layer], width=24, vocab=37, side=0, embed=1.0)
    n, far = 330, 20
    w, t = _marked_state(cfg, 14, far, n)
    want = O.forward(cfg, w, t)
    t2 = list(t)
    t2[far] = 0
    assert float((O.forward(cfg, w, t2)[n - 1] - want[n - 1]).abs().max()) > 0.05
    for cuts in ([n], [310], [100, 2, 64, 130], [far + 12]):
        close(rig_for(cfg, w=w, num_blocks=32).run_cut("a", t, cuts), want, tol=1e-4)


def test_convolution_inputs_cross_portions():
    """A portion that starts right after the spiked token still convolves it: with the state's
    convolution inputs lost, the next taps - 1 positions would move."""
    cfg = make_cfg([par(right=delta(2, 2, 6, 6, 5), ls=0.0, rs=1.0)], width=24, vocab=37, side=0)
    far = 16
    w, t = _spiked(cfg, 12, far, far + 8, ("l0.mix.right.v.conv",))
    want = O.forward(cfg, w, t)
    for cuts in ([far + 1], [far + 1, 2, 2], [far, 1, 1, 2], [far + 3]):
        close(rig_for(cfg, w=w).run_cut("a", t, cuts), want, tol=1e-4)


def test_every_constant_matters_and_is_read():
    """Sinks, norm weights, branch weights, the embedding scale, the token input, the experts' limit,
    the router's groups and scale: the oracle moves when one is changed, and the engine follows it."""
    cfg = make_cfg([par(att_a(3, 1, 8, 6, dims=4), mlp=moe(8, 2, 6, 0.6, (4, 1), 2.0)), par2(att_b(2, 1, 8, dims=4), mlp=dense(12))],
                   width=24, vocab=37)
    w = O.random_weights(cfg, 16)
    w["l0.mix.left.sink"] = torch.tensor([3.0, -2.0, 0.5])
    t = toks(14, 37, 6)
    want = O.forward(cfg, w, t)
    for name, other in (("l0.mix.left.sink", torch.full((3,), -30.0)), ("l1.mix.left.q.norm", torch.ones(8)),
                        ("l1.mix.left.k.norm", torch.ones(8)), ("l0.side.norm", torch.zeros(24)), ("l1.mix.right.a2.b", torch.zeros(18)),
                        ("l0.mix.right.dt_bias", torch.zeros(24)), ("l0.mix.right.b", torch.zeros(4, 24))):
        w0 = dict(w)
        w0[name] = other
        assert float((O.forward(cfg, w0, t) - want).abs().max()) > 1e-3, name
    variants = []
    for path, val in ((("layers", 0, "mixer", "left_scale"), 1.0), (("layers", 1, "mixer", "right_scale"), 1.0),
                      (("embedding", "scale"), 1.0), (("layers", 0, "mlp", "expert", "limit"), 5.0),
                      (("layers", 0, "mlp", "router", "groups", "keep"), 4), (("layers", 0, "mlp", "router", "scale"), 1.0),
                      (("layers", 1, "mixer", "right", "tau"), 1.0), (("layers", 0, "mixer", "left", "rot", "scaling", "factor"), 1.0),
                      (("layers", 1, "mixer", "left", "scale"), 1.0), (("logit_scale",), 1.0), (("norm", "eps"), 0.1)):
        c2 = copy.deepcopy(cfg)
        node = c2
        for k in path[:-1]:
            node = node[k]
        node[path[-1]] = val
        assert float((O.forward(c2, w, t) - want).abs().max()) > 1e-3, path
        variants.append(c2)
    for c in [cfg] + variants:
        ref = O.forward(c, w, t)
        for cuts in ([14], [3, 2]):
            close(rig_for(c, w=w).run_cut("a", t, cuts), ref, tol=1e-4)


def test_rotation_counts_from_zero_on_any_pages():
    """Positions count from 0 in every sequence whatever pages and slots it gets: the same prompt
    run second, on other pages, gives the same logits; large positions keep their accuracy."""
    cfg = make_cfg([par(att_a(2, 2, 12, 8, 0.4, dims=12, base=20.0, original=16)), par2(att_b(2, 1, 12, 0.4, dims=8, base=20.0, original=64))],
                   width=24, vocab=37)
    rig = rig_for(cfg, 15, num_blocks=48)
    t = toks(420, 37, 9)
    want = O.forward(cfg, rig.w, t)
    rig.step([("z", toks(90, 37, 1))])  # holds the first pages and slot 0
    close(rig.run_cut("a", t, [200, 3, 200]), want, tol=5e-4)


# ------------------------------------------------------------------ engine entry points

def test_greedy_generation_through_engine(tmp_path):
    w = O.random_weights(FULL, 21)
    d = _save(tmp_path, FULL, w)
    assert config_from_dir(d).arch == "levovik"
    eng = LLMEngine(EngineConfig(model=str(d), weights=str(d), max_num_seqs=3, max_model_len=256, num_blocks=40,
                                 dtype="float32", max_prefill_tokens=16, mixed_prefill_tokens=8), device="cpu")
    prompts = [toks(n, FULL["vocab"], 30 + n) for n in (4, 29, 18, 40)]  # 4 requests over 3 slots: one waits
    seqs = eng.generate(prompts, SamplingParams(max_tokens=10, temperature=0.0, ignore_eos=True))
    for p, s in zip(prompts, seqs):
        assert s.output_ids == O.greedy(FULL, w, p, 10)
    st = eng.stats()
    assert st["mixed_steps"] > 0 and st["kv_blocks_free"] == st["kv_blocks_total"]


def test_preset_round_trip_and_registry():
    c = get_config("levovik-tiny")
    assert hybrid_config_from_dict(hybrid_config_to_dict(c), c.name) == c
    m = build_model(c, device="cpu", dtype=torch.float32)
    w = state_dict(m)
    assert w["l1.mix.right.a1"].shape == (12, c.d_model) and w["l3.mix.right.g1"].shape[0] == 16 and "l2.norm2" not in w
    assert "l0.mix.left.v" not in w and w["side.embed"].shape == (c.vocab_size, 4 * c.side_dim)
    cfg = hybrid_config_to_dict(c)
    eng = LLMEngine(EngineConfig(model="levovik-tiny", max_num_seqs=2, max_model_len=128, num_blocks=16,
                                 dtype="float32"), device="cpu")
    p = toks(11, c.vocab_size, 1)
    s = eng.generate([p], SamplingParams(max_tokens=6, temperature=0.0, ignore_eos=True))[0]
    assert s.output_ids == O.greedy(cfg, w, p, 6)


def test_config_errors_are_loud():
    with pytest.raises(ValueError):
        rig_for(make_cfg([par(att_a(4, 3))]), 1)
    with pytest.raises(ValueError):
        rig_for(make_cfg([par(right=delta(4, 3))]), 1, w=O.random_weights(make_cfg([par()]), 1))
    with pytest.raises(ValueError):
        rig_for(make_cfg([par(mlp=moe(6, 3, 4, 1.0, (3, 1)))]), 1, w=O.random_weights(make_cfg([par(mlp=moe(6, 2, 4))]), 1))
    with pytest.raises(ValueError):
        rig_for(make_cfg([par(mlp=moe(6, 2, 4, 1.0, (4, 1)))]), 1, w=O.random_weights(make_cfg([par(mlp=moe(6, 2, 4))]), 1))
    bad = make_cfg([par()])
    bad["layers"][0]["type"] = "parallel_3"
    with pytest.raises(ValueError):
        rig_for(bad, 1, w=O.random_weights(make_cfg([par()]), 1))


def test_trace_command_replays_steps(tmp_path):
    """The command-line replayer: portions, a mixed step, a decode-only step, ends and reuse."""
    w = O.random_weights(FULL, 22)
    d = _save(tmp_path, FULL, w)
    V = FULL["vocab"]
    A, B = toks(23, V, 1), toks(9, V, 2)
    steps = [{"step": 0, "entries": [{"id": "x", "tokens": A[:20], "want": [0, 19]}], "end": []},
             {"step": 1, "entries": [{"id": "y", "tokens": B[:8], "want": [7]}, {"id": "x", "tokens": A[20:21], "want": [0]}],
              "end": []},
             {"step": 2, "entries": [{"id": "x", "tokens": A[21:22], "want": []}, {"id": "y", "tokens": B[8:], "want": [0]}],
              "end": ["y"]},
             {"step": 3, "entries": [{"id": "x", "tokens": A[22:], "want": [0]}], "end": ["x"]}]
    out = tmp_path / "o"
    r = subprocess.run([sys.executable, "-m", "k8s_llm_monitor_amd.cmd.trace_run", "--model", str(d), "--dtype", "float32",
                        "--out", str(out), "--max-tokens", "64", "--device", "cpu"],
                       input="\n".join(json.dumps(s) for s in steps) + "\n", capture_output=True, text=True, cwd=ROOT)
    assert r.returncode == 0, r.stderr[-2000:]
    assert [ln for ln in r.stdout.splitlines() if ln.startswith("done")] == [f"done {i}" for i in range(4)]
    wa, wb = O.forward(FULL, w, A), O.forward(FULL, w, B)

    def rd(i):
        return torch.from_numpy(np.fromfile(out / f"{i}.f32", dtype="<f4").reshape(-1, V).copy())

    close(rd(0), wa[[0, 19]])
    close(rd(1), torch.stack([wb[7], wa[20]]))  # entry order, not the engine's row order
    close(rd(2), wb[8:9])
    close(rd(3), wa[22:23])


# ------------------------------------------------------------------ the same through the HIP kernels

def _row_err(got, want):
    scale = float(want.pow(2).mean().sqrt())
    return (got.double() - want).pow(2).mean(-1).sqrt() / scale


def _bf16_ref_err(cfg, w, t, want, **kw):
    """What bf16 rounding alone costs on this model and prompt: the torch forms on the CPU, in bf16,
    against the oracle (row errors over the logits' scale)."""
    return _row_err(rig_for(cfg, w=w, dtype=torch.bfloat16, **kw).run_cut("a", t, [len(t)]), want)


def _bf16_close(got, want, ref_err):
    """A bf16 run through the kernels is about as close to the oracle as the bf16 torch forms are: the
    median and the 80th percentile of the row errors within 3 x theirs.  Both carry rounding noise of the
    same size but not the same noise, and a sharply peaked softmax or a slowly decaying state downstream
    amplifies one realisation two times more than another (measured on these configurations, in either
    direction); a router decision that is a near tie falls either way in both.  A wrong state, page or
    edge moves most rows by ten times the rounding level and more; the sharp comparisons are the fp32 ones."""
    e = _row_err(got, want)
    for q in (0.5, 0.8):
        a, b = float(e.quantile(q)), float(ref_err.quantile(q))
        assert a <= 3.0 * b + 2e-3, f"quantile {q}: {a:.3e} against {b:.3e} of the bf16 torch forms"


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gpu_cuts_and_batches_match_oracle(dtype):
    rig = rig_for(FULL, 6, device="cuda", dtype=dtype)
    t = toks(70, FULL["vocab"], 4)
    u = toks(40, FULL["vocab"], 8)
    want, wu = O.forward(FULL, rig.w, t), O.forward(FULL, rig.w, u)
    if dtype == torch.float32:
        cmp = lambda got, ref, which: close(got, ref)
    else:
        errs = {"t": _bf16_ref_err(FULL, rig.w, t, want), "u": _bf16_ref_err(FULL, rig.w, u, wu)}
        cmp = lambda got, ref, which: _bf16_close(got, ref, errs[which])
    for cuts in ([70], [2, 2, 3, 16, 1, 31], [33, 2, 2, 2], []):
        cmp(rig.run_cut("a", t, cuts), want, "t")
    a = rig.step([("a", t[:30]), ("b", u[:5])])
    b = rig.step([("a", t[30:31]), ("b", u[5:])], end=["b"])
    c = rig.step([("a", t[31:])], end=["a"])
    cmp(torch.cat([a["a"], b["a"], c["a"]]), want, "t")
    cmp(torch.cat([a["b"], b["b"]]), wu, "u")


@pytest.mark.gpu
def test_gpu_layers_and_mechanisms_fp32():
    rig = rig_for(FULL, 5, device="cuda", dtype=torch.float32)
    t = toks(19, FULL["vocab"], 3)
    rig.model.layer_probe = []
    rig.run_cut("a", t, [19])
    for got, want in zip(rig.model.layer_probe, O.layers_of(FULL, rig.w, t)):
        close(got.cpu(), want)
    rig.model.layer_probe = None
    for layers in ([par(att_a(1, 1, 8, 8, 1.0, dims=8, base=10.0), delta(1, 1, 1, 1, 1, 1, 1))],
                   [par(att_a(6, 1, 10, 4, dims=2), delta(6, 1, 4, 3, 5))], [par(att_a(3, 3, 6, 9, dims=0), delta(3, 3, 9, 5, 2))],
                   [par2(att_b(1, 1, 2, 1.0, dims=2), gla(1, 1, 1, 1.0, 1))], [par2(att_b(6, 2, 10, dims=6, factor=1.0), gla(4, 9, 5, 64.0))],
                   [par2(mlp=moe(6, 6, 4, 0.5, None))], [par(mlp=moe(6, 2, 8, 1.0, (6, 3)))], [par2(mlp=moe(8, 4, 8, 3.0, (2, 1)))],
                   [par(mlp=dense(1))]):
        cfg = make_cfg(layers)
        r2 = rig_for(cfg, 3, device="cuda", dtype=torch.float32)
        u = toks(45, cfg["vocab"], 1)
        close(r2.run_cut("a", u, [20, 2]), O.forward(cfg, r2.w, u))


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gpu_odd_sizes(dtype):
    cfg = make_cfg([par(att_a(5, 5, 7, 3, dims=6), delta(6, 3, 5, 7, 2, 3, 9), mlp=dense(11)),
                    par2(att_b(3, 1, 9, dims=2), gla(3, 5, 7, 3.0, 2), mlp=moe(9, 2, 5, 0.7, (3, 1))),
                    par(att_a(2, 1, 11, 13, dims=10), delta(1, 1, 13, 3, 6, 1, 2), mlp=moe(10, 4, 3, 1.3, (5, 2)))],
                   width=37, vocab=53, side=5)
    rig = rig_for(cfg, 31, device="cuda", dtype=dtype)
    t = toks(41, 53, 3)
    want = O.forward(cfg, rig.w, t)
    ref = _bf16_ref_err(cfg, rig.w, t, want) if dtype == torch.bfloat16 else None
    for cuts in ([41], [3, 2, 17]):
        got = rig.run_cut("a", t, cuts)
        close(got, want) if dtype == torch.float32 else _bf16_close(got, want, ref)


BIG = make_cfg([par2(att_b(8, 2, 64, 0.125, dims=64, base=5e5, original=64), gla(4, 64, 32, 12.0, 16), mlp=dense(192)),
                par(att_a(4, 2, 128, 128, 0.09, dims=32, base=1e6, factor=8.0, original=64), delta(4, 2, 32, 64, 4, 16, 24),
                    mlp=moe(8, 2, 64, 1.25, (4, 2), 1.75)),
                par2(att_b(4, 4, 128, 0.09, dims=128, base=1e4, original=128), gla(2, 128, 64, 8.0, 8), mlp=moe(4, 2, 128, 1.0, None)),
                par(att_a(8, 1, 64, 64, 0.125, dims=64, base=1e4, original=256), delta(2, 2, 128, 128, 4, 8, 8))],
               width=128, vocab=211, side=16)


@pytest.mark.gpu
def test_gpu_matrix_core_sizes_bf16():
    """Head sizes of 64 / 128 take the matrix-core attention kernels and the vector decode kernels; long
    enough for several pages per wave and several tiles of the scan."""
    rig = rig_for(BIG, 6, device="cuda", dtype=torch.bfloat16, num_blocks=48)
    t = toks(150, BIG["vocab"], 4)
    want = O.forward(BIG, rig.w, t)
    ref = _bf16_ref_err(BIG, rig.w, t, want, num_blocks=48)
    for cuts in ([150], [2, 2, 3, 16, 1, 31], [100]):
        _bf16_close(rig.run_cut("a", t, cuts), want, ref)
    r32 = rig_for(BIG, 6, device="cuda", dtype=torch.float32, num_blocks=48)
    close(r32.run_cut("a", t, [70, 3]), want)


@pytest.mark.gpu
def test_gpu_long_prompt_fp32_and_bf16():
    """700 tokens (44 pages, 44 tiles of the scan), whole and cut so that the second portion and the
    decoded tokens read the caches and the states."""
    cfg = make_cfg(BIG["layers"][:2], width=128, vocab=211, side=16)
    t = toks(700, cfg["vocab"], 4)
    w = O.random_weights(cfg, 7)
    want = O.forward(cfg, w, t)
    r32 = rig_for(cfg, w=w, device="cuda", dtype=torch.float32, num_blocks=96)
    close(r32.run_cut("a", t, [700]), want)
    close(r32.run_cut("a", t, [513, 180]), want)
    rig = rig_for(cfg, w=w, device="cuda", dtype=torch.bfloat16, num_blocks=96)
    _bf16_close(rig.run_cut("a", t, [600, 95]), want, _bf16_ref_err(cfg, w, t, want, num_blocks=96))


@pytest.mark.gpu
def test_gpu_far_tokens_and_causal_edge():
    n, far = 330, 20
    for kind in ("a", "b"):
        layer = par(att_a(2, 1, 8, 8, 1.0, dims=4, base=1e4), ls=1.0, rs=0.2) if kind == "a" else \
            par2(att_b(2, 1, 8, 1.0, dims=4, base=1e4), ls=1.0, rs=0.2)
        cfg = make_cfg([layer], width=24, vocab=37, side=0, embed=1.0)
        w, t = _beacon(cfg, 13, far, n)
        want = O.forward(cfg, w, t)
        for cuts in ([n], [310], [100, 2, 64, 130]):
            close(rig_for(cfg, w=w, num_blocks=32, device="cuda").run_cut("a", t, cuts), want, tol=1e-4)
    for kind in ("delta", "gla"):
        layer = par(right=delta(2, 1, 6, 6, 3), ls=0.1, rs=1.0) if kind == "delta" else par2(right=gla(2, 6, 6, 16.0), ls=0.1, rs=1.0)
        cfg = make_cfg([layer], width=24, vocab=37, side=0, embed=1.0)
        w, t = _marked_state(cfg, 14, far, n)
        want = O.forward(cfg, w, t)
        for cuts in ([n], [310], [100, 2, 64, 130]):
            close(rig_for(cfg, w=w, num_blocks=32, device="cuda").run_cut("a", t, cuts), want, tol=1e-4)
    for name, (layer, vname) in ALONE.items():
        cfg = make_cfg([layer], width=24, vocab=37, side=0)
        w, t = _spiked(cfg, 11, 16, 22, (vname,))
        want = O.forward(cfg, w, t)
        for cuts in ([22], [16], [2] * 10):
            close(rig_for(cfg, w=w, device="cuda").run_cut("a", t, cuts), want, tol=1e-4)


@pytest.mark.gpu
def test_gpu_unequal_batch_and_reuse_fp32():
    rig = rig_for(FULL, 9, num_blocks=24, device="cuda")
    V = FULL["vocab"]
    T = {n: toks(k, V, s) for n, k, s in (("a", 50, 1), ("b", 21, 2), ("c", 3, 3), ("d", 37, 4), ("e", 44, 5))}
    want = {n: O.forward(FULL, rig.w, t) for n, t in T.items()}
    got, at = {n: [] for n in T}, {n: 0 for n in T}
    for plan, end in (([("a", 17), ("b", 2), ("c", 3)], ["c"]), ([("a", 1), ("b", 19), ("d", 30)], ["b"]),
                      ([("a", 1), ("d", 1), ("e", 16)], []), ([("a", 31), ("d", 2), ("e", 1)], ["a"]), ([("d", 1), ("e", 1)], []),
                      ([("d", 3), ("e", 26)], ["d", "e"])):
        entries = []
        for n, k in plan:
            entries.append((n, T[n][at[n]:at[n] + k]))
            at[n] += k
        for n, lg in rig.step(entries, end).items():
            got[n].append(lg)
    for n in T:
        close(torch.cat(got[n]), want[n])


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gpu_new_ops_match_their_torch_forms(dtype):
    g = torch.Generator().manual_seed(3)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    dev = "cuda"

    def both(fn, *args, **kw):
        """fn on CPU copies and on GPU copies of the tensor arguments; returns (cpu, gpu, cpu args, gpu args)."""
        ca = [a.clone() if isinstance(a, torch.Tensor) else a for a in args]
        ga = [a.to(dev) if isinstance(a, torch.Tensor) else a for a in args]
        ck = {k: v.clone() if isinstance(v, torch.Tensor) else v for k, v in kw.items()}
        gk = {k: v.to(dev) if isinstance(v, torch.Tensor) else v for k, v in kw.items()}
        return fn(*ca, **ck), fn(*ga, **gk), ca, ga

    for T, n in ((5, 24), (3, 7), (2, 1), (4, 520)):
        x, a, b, y = torch.randn(T, n, generator=g), torch.randn(T, n, generator=g).to(dtype), torch.randn(T, n, generator=g), \
            torch.randn(T, n, generator=g).to(dtype)
        w, wy = torch.rand(n, generator=g) + 0.5, torch.rand(n, generator=g)
        for center, wn, normed, adds in ((True, w, (y, wy), ((a, 0.7), (b, 1.3))), (False, w, None, ((a, 1.0),)),
                                         (True, None, (y, wy), ()), (True, w, None, ())):
            def run(x_, *ts):
                ts = list(ts)
                ad = tuple((ts.pop(0), s) for _, s in adds)
                nr = (ts.pop(0), ts.pop(0)) if normed is not None else None
                return hops.sum_norm(x_, ad, nr, ts.pop(0) if wn is not None else None, 1e-5, center, False, dtype)
            flat = [t_ for t_, _ in adds] + (list(normed) if normed is not None else []) + ([wn] if wn is not None else [])
            c, u, ca, ga = both(run, x, *flat)
            close(u.cpu().float(), c.double(), tol=tol)
            close(ga[0].cpu(), ca[0].double(), tol=1e-5)
        table = torch.randn(9, n + 5, generator=g).to(dtype)
        ids = torch.tensor([3, 8, 0, 3, 1][:T], dtype=torch.int32)
        gate = (torch.randn(T, n, generator=g) * 2).to(dtype)
        c, u, _, _ = both(hops.gated_lookup, gate, table, ids, 5)
        close(u.cpu().float(), c.double(), tol=tol)
    # a norm per head, then the gate: groups of a wave's width and less, more, and beyond the wave kernel
    for T, groups, gs in ((5, 4, 32), (3, 3, 7), (4, 2, 128), (2, 2, 200), (3, 2, 300), (2, 16, 64), (2, 1, 48)):
        n = groups * gs
        yy, zz = torch.randn(T, n, generator=g) * 3, (torch.randn(T, n + 9, generator=g) * 2).to(dtype)
        ww = torch.rand(n, generator=g) + 0.5
        for gate in ("sigmoid", "silu"):
            c, u, _, _ = both(hops.gated_group_norm, yy, zz, 9, ww, 1e-5, groups, dtype, True, gate)
            close(u.cpu().float(), c.double(), tol=tol)
    z = (torch.randn(6, 40, generator=g) * 2).to(dtype)
    for col, f in ((8, 16), (3, 7)):
        for kind, lim in (("relu", 0.0), ("clamped_swish", 1.1)):
            c, u, _, _ = both(hops.glu, z, col, f, kind, lim)
            close(u.cpu().float(), c.double(), tol=tol)
    if dtype == torch.float32:
        for E, d, cases in ((12, 24, ((3, (2, 1)), (2, (4, 2)), (4, (12, 5)), (5, (1, 1)), (1, (3, 3)), (12, (1, 1)))),
                            (8, 21, ((2, (2, 1)), (8, (1, 1)))), (6, 40, ((3, (3, 2)),)), (24, 16, ((4, (4, 2)), (6, (8, 3)))),
                            (16, 2056, ((4, (4, 2)),))):
            hh, wr = torch.randn(70, d, generator=g), torch.randn(E, d, generator=g) * d ** -0.5
            for top, groups in cases:
                (ic, wc), (ig, wg), _, _ = both(hops.moe_router_grouped, hh, wr, E, top, *groups, 2.5)
                oc, og = ic.long().argsort(-1), ig.cpu().long().argsort(-1)
                assert torch.equal(ic.long().gather(1, oc), ig.cpu().long().gather(1, og))
                close(wg.cpu().gather(1, og), wc.gather(1, oc).double(), tol=1e-5)
    # norm + rotation + page writes, both orders and layouts, rotating part smaller than the head
    for Hq, G, dk, dv, rd in ((4, 2, 12, 6, 8), (6, 1, 64, 64, 64), (6, 2, 128, 128, 32), (3, 3, 7, 5, 4)):
        T = 9
        pos = torch.tensor([0, 1, 2, 3, 500, 501, 17, 18, 19], dtype=torch.int32)
        slots = torch.tensor([0, 1, 2, 3, 40, 41, -1, 16, 17], dtype=torch.int32)
        qw, kw = torch.rand(dk, generator=g) + 0.5, torch.rand(dk, generator=g) + 0.5
        for norm, pairs, vk in ((1, True, True), (2, False, False), (1, False, False), (2, True, True)):
            dvv = dk if vk else dv
            qkv = torch.randn(T, Hq * dk + G * dk + (0 if vk else G * dvv) + 8, generator=g).to(dtype)
            kc, vc = torch.zeros(4, 16, G * dk, dtype=dtype), torch.zeros(4, G, dvv, 16, dtype=dtype)
            _, _, ca, ga = both(hops.rotary_cache, qkv, Hq, G, dk, dvv, pos, hops.rotary_freq(100.0, rd), pairs, None, kc, vc, slots,
                                norm=norm, qw=qw, kw=kw, eps=1e-5, v_from_k=vk)
            for i in (0, 10, 11):
                close(ga[i].cpu().float(), ca[i].double(), tol=tol)


@pytest.mark.gpu
@pytest.mark.parametrize("H,Gk,dk,dv", [(2, 2, 32, 32), (4, 2, 48, 32), (3, 1, 64, 96), (2, 2, 128, 128), (1, 1, 200, 40), (6, 3, 5, 7),
                                        (2, 1, 16, 8), (1, 1, 1, 1), (2, 2, 256, 16), (2, 1, 12, 70), (3, 3, 36, 130), (2, 2, 100, 9)])
@pytest.mark.parametrize("delta_rule", [True, False], ids=["delta", "plain"])
def test_gpu_decay_scan_matches_the_recurrence(H, Gk, dk, dv, delta_rule):
    """The scan kernel against the float64 recurrence and the torch form: segments shorter than, equal
    to and longer than its 16- and 32-token tiles, some continuing from their slots, one padding segment, a slot
    with leftovers that a starting sequence must not see; outputs and the states left in the slots."""
    g = torch.Generator().manual_seed(5)
    if not delta_rule:
        Gk = H
    lens = [1, 15, 16, 17, 100, 7, 33, 32, 31]
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    ctx = torch.tensor([0, 5, 0, 64, 0, 3, 9, 0, 2], dtype=torch.int32)
    slot = torch.tensor([0, 1, 2, 3, 4, -1, 5, 7, 6], dtype=torch.int32)
    T = int(cu[-1])
    qkv, z, zb, a_log = _scan_inputs(g, T, H, Gk, dk, dv)
    st = torch.randn(8, H, dv, dk, generator=g) * 0.3
    kw = dict(a_log=a_log, beta=qkv, beta_col=2 * Gk * dk + H * dv, unit=True) if delta_rule else dict(tau=3.0)
    args = (0, Gk * dk, 2 * Gk * dk)
    want_state = st.clone()
    want = hops.decay_scan(qkv, *args, z, zb, want_state, cu, ctx, slot, H, Gk, dk, dv, dk ** -0.5, **kw)
    gk = {k: (v.to("cuda") if isinstance(v, torch.Tensor) else v) for k, v in kw.items()}
    a, b = int(cu[4]), int(cu[5])  # the 100-token segment starts from zero: the written-out recurrence
    alone = _scan_want(qkv[a:b], z[a:b], zb, a_log, H, Gk, dk, dv, delta_rule, 3.0)
    for mode in (1, 2):  # the one-launch form and the two-launch form for prompts
        got_state = st.to("cuda")
        got = hops.decay_scan(qkv.to("cuda"), *args, z.to("cuda"), zb.to("cuda"), got_state, cu.to("cuda"), ctx.to("cuda"),
                              slot.to("cuda"), H, Gk, dk, dv, dk ** -0.5, mode=mode, **gk)
        close(got.cpu(), want.double(), tol=2e-5)
        close(got_state.cpu(), want_state.double(), tol=2e-5)
        close(got[a:b].cpu(), alone, tol=2e-5)


@pytest.mark.gpu
def test_gpu_greedy_generation_with_graphs():
    eng = LLMEngine(EngineConfig(model="levovik-tiny", max_num_seqs=4, max_model_len=256, num_blocks=64,
                                 dtype="float32", max_prefill_tokens=32, mixed_prefill_tokens=16), device="cuda")
    eng.warmup()  # decode steps replay from captured hipGraphs
    cfg, w = hybrid_config_to_dict(eng.model_cfg), {k: v.cpu() for k, v in state_dict(eng.model).items()}
    prompts = [toks(n, 352, 40 + n) for n in (5, 37, 21)]
    seqs = eng.generate(prompts, SamplingParams(max_tokens=12, temperature=0.0, ignore_eos=True))
    assert eng.stats()["graph_buckets"]
    for p, s in zip(prompts, seqs):
        assert s.output_ids == O.greedy(cfg, w, p, 12)
