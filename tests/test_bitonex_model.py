"""The Bitonex layer-list design in the engine against the plain float64 oracle
(tests/bitonex_oracle.py): each mechanism alone (rotary grouped-query attention with head
temperatures and output gate, fixed-decay linear attention with its state, latent attention with
paired rotation and shared pages, the gated feed-forward, the gated residual with one-number norms,
the logit soft cap), prefill against token-by-token decoding, prompt portions down to two tokens,
unequal batches, pages and state slots that are reused, keys far away and at page borders, the
causal edge, the first tokens, long decoding, odd sizes and sizes of one, and greedy generation
through the engine and the trace command.

Runs on the CPU (the ops' torch forms); the ``gpu`` tests at the end run the same comparisons
through the HIP kernels."""
import json
import subprocess
import sys

import numpy as np
import pytest
import torch

import bitonex_oracle as O
from k8s_llm_monitor_amd.engine import EngineConfig, LLMEngine, SamplingParams
from k8s_llm_monitor_amd.models.config import get_config, hybrid_config_from_dict, hybrid_config_to_dict
from k8s_llm_monitor_amd.models.hybrid import state_dict
from k8s_llm_monitor_amd.models.registry import build_model, config_from_dir
from k8s_llm_monitor_amd.ops import hybrid as hops
from test_hybrid_model import ROOT, Rig, _save, close, close_most, toks


# ------------------------------------------------------------------ small configurations

def att(heads=4, kv=2, dim=12, vdim=10, rot=8, base=100.0, scale=0.3, mlp=None):
    return {"type": "attention", "mixer": {"heads": heads, "kv_heads": kv, "dim": dim, "vdim": vdim, "scale": scale,
                                           "rot": {"base": base, "dims": rot}}, "mlp": mlp}


def lin(heads=3, dim=6, vdim=10, decay=(0.5, 0.9, 0.995), mlp=None):
    return {"type": "lightning", "mixer": {"heads": heads, "dim": dim, "vdim": vdim, "decay": list(decay)}, "mlp": mlp}


def lat(heads=3, dim=12, rot=8, vdim=10, q_rank=20, kv_rank=24, scale=0.25, base=100.0, kv_from=None, mlp=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank, "scale": scale,
         "rot": {"base": base, "dims": rot}}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": m, "mlp": mlp}


def dense(ff=36):
    return {"kind": "dense", "ff": ff}


def make_cfg(layers, width=40, vocab=61, eps=1e-6, mult=0.45, cap=15.0):
    return {"architecture": "Bitonex", "vocab": vocab, "width": width, "layers": layers, "norm": {"eps": eps},
            "residual_mult": mult, "logit_softcap": cap, "max_positions": 1024}


FULL = make_cfg([lin(mlp=dense(28)), att(mlp=dense()), lat(mlp=None), att(6, 3, 8, 14, 8, 50.0, 0.35, mlp=dense(20)),
                 lat(2, 8, 8, 6, 12, 24, 0.3, kv_from=2, mlp=dense(24)), lin(2, 10, 4, (0.8, 0.99))])


def rig_for(cfg, seed=0, w=None, **kw):
    return Rig(cfg, w=w if w is not None else O.random_weights(cfg, seed), **kw)


# ------------------------------------------------------------------ mechanisms alone

@pytest.mark.parametrize("layers", [
    [att()], [att(1, 1, 8, 8, 8, 10.0, 1.0)], [att(6, 1, 10, 4, 2)], [att(3, 3, 6, 9, 0)], [lin()], [lin(1, 1, 1, (0.7,))],
    [lin(4, 9, 5, (1.0, 0.0, 0.31, 0.999))], [lat()], [lat(1, 8, 2, 8, 8, 8, 1.0)], [lat(4, 4, 16, 20, 9, 40, 0.2)],
    [lat(), lat(2, 8, 8, 8, 8, 24, 0.2, kv_from=0)], [att(mlp=dense())], [lin(mlp=dense(1))], [lat(mlp=dense(7))]],
    ids=["attention", "attention-ones-full-rotation", "attention-mqa-two-rotating", "attention-no-rotation", "lightning",
         "lightning-ones", "lightning-decays-one-and-zero", "latent", "latent-ones", "latent-wide-rotation", "shared-pages",
         "attention-ff", "lightning-ff1", "latent-ff"])
def test_single_mechanism_whole_prompt(layers):
    cfg = make_cfg(layers)
    rig = rig_for(cfg, 3)
    t = toks(45, cfg["vocab"], 1)
    close(rig.run_cut("a", t, [45]), O.forward(cfg, rig.w, t))


def test_odd_sizes_everywhere():
    """Widths, ranks and head sizes that are multiples of nothing (rotated sizes stay even)."""
    cfg = make_cfg([att(5, 5, 7, 3, 6, mlp=dense(11)), lin(3, 5, 7, (0.3, 0.6, 0.9), mlp=dense(5)),
                    lat(3, 5, 2, 3, 9, 7, 0.4, mlp=dense(13)), lat(5, 3, 2, 7, 5, 7, 0.3, kv_from=2), att(3, 1, 9, 5, 2)],
                   width=37, vocab=53, mult=1.0, cap=4.0)
    rig = rig_for(cfg, 31)
    t = toks(41, 53, 3)
    want = O.forward(cfg, rig.w, t)
    for cuts in ([41], [3, 2, 17], [1]):
        close(rig.run_cut("a", t, cuts), want)


def test_models_without_pages_or_without_state():
    """Only recurrent layers (no layer owns pages), and no recurrent layer (no state slots)."""
    for layers in ([lin(mlp=dense(9)), lin(2, 4, 6, (0.6, 0.8))], [lat(mlp=dense(9)), att(), lat(2, 8, 8, 6, 12, 24, 0.3, kv_from=0)]):
        cfg = make_cfg(layers)
        rig = rig_for(cfg, 4)
        assert (rig.runner.num_state_slots > 0) == (layers[0]["type"] == "lightning")
        t, u = toks(37, cfg["vocab"], 2), toks(20, cfg["vocab"], 3)
        want, wu = O.forward(cfg, rig.w, t), O.forward(cfg, rig.w, u)
        close(rig.run_cut("a", t, [18, 2]), want)
        a = rig.step([("a", t[:30]), ("b", u[:5])])
        b = rig.step([("a", t[30:31]), ("b", u[5:])], end=["b"])
        c = rig.step([("a", t[31:])], end=["a"])
        close(torch.cat([a["a"], b["a"], c["a"]]), want)
        close(torch.cat([a["b"], b["b"]]), wu)


def _force_expanded(monkeypatch):
    """Latent attention takes its expanded form (per-head keys and values in temporary pages) for
    every step of whole prompts, whatever the sizes and the dtype."""
    from k8s_llm_monitor_amd.models.hybrid import LatentAttention

    calls = []
    real = LatentAttention._forward_expanded
    monkeypatch.setattr(LatentAttention, "_forward_expanded", lambda self, *a: calls.append(1) or real(self, *a))
    monkeypatch.setattr(LatentAttention, "_expand_ok",
                        lambda self, h, meta: meta.is_prefill and meta.all_fresh and not meta.num_decode)
    return calls


def test_latent_expanded_form_equals_the_oracle(monkeypatch):
    """The expanded form in 32-bit, any sizes: unequal whole prompts in one step (every segment on
    temporary pages of its own), a layer reading another layer's latent, then portions and decoding
    over the latent cache those steps left."""
    calls = _force_expanded(monkeypatch)
    cfg = make_cfg([lat(3, 5, 6, 3, 9, 7, 0.4, mlp=dense(13)), att(), lat(5, 3, 6, 7, 5, 7, 0.3, kv_from=0), lat(mlp=dense(8))])
    rig = rig_for(cfg, 12)
    t, u, v = toks(50, cfg["vocab"], 4), toks(17, cfg["vocab"], 5), toks(33, cfg["vocab"], 6)
    want = {n: O.forward(cfg, rig.w, x) for n, x in (("a", t), ("b", u), ("c", v))}
    a = rig.step([("a", t[:40]), ("b", u[:16]), ("c", v[:33])], end=["c"])
    assert len(calls) == 3
    b = rig.step([("a", t[40:41]), ("b", u[16:])], end=["b"])
    c = rig.step([("a", t[41:])], end=["a"])
    assert len(calls) == 3
    close(torch.cat([a["a"], b["a"], c["a"]]), want["a"])
    close(torch.cat([a["b"], b["b"]]), want["b"])
    close(a["c"], want["c"])


def test_layer_outputs_match_oracle():
    rig = rig_for(FULL, 5)
    t = toks(19, FULL["vocab"], 3)
    rig.model.layer_probe = []
    rig.run_cut("a", t, [19])
    _, layers = O.forward(FULL, rig.w, t, return_layers=True)
    assert len(rig.model.layer_probe) == layers.shape[0] == 6
    for got, want in zip(rig.model.layer_probe, layers):
        close(got, want)
    rig.model.layer_probe = None


def test_ops_against_oracle_functions():
    g = torch.Generator().manual_seed(1)
    z = torch.randn(3, 40, generator=g) * 3
    close(hops.activation(z, "silu"), O.silu(z.double()), tol=1e-6)
    close(hops.activation_cols(z, 8, 16, "silu"), O.silu(z[:, 8:24].double()), tol=1e-6)
    close(hops.glu(z, 4, 12, "gelu_tanh"), O.gelu_tanh(z[:, 4:16].double()) * z[:, 16:28].double(), tol=1e-6)
    x = torch.randn(3, 10, generator=g)
    close(hops.sigmoid_gate(x.clone(), z, 30), x.double() * O.sigmoid(z[:, 30:].double()), tol=1e-6)
    close(hops.softcap(z.clone() * 10, 7.0), 7.0 * torch.tanh(z.double() * 10 / 7.0), tol=1e-6)
    # gated residual + norm: the gate's logits are a column range of a wider projection
    r, y, b, w = torch.randn(3, 12, generator=g), torch.randn(3, 12, generator=g), torch.randn(12, generator=g), torch.rand(12, generator=g)
    res = r.clone()
    h = hops.gated_add_norm(res, y, z, 5, b, 0.3, w, 1e-5, False, torch.float32)
    want = r.double() + 0.3 * y.double() * O.sigmoid(z[:, 5:17].double() + b.double())
    close(res, want, tol=1e-6)
    close(h, O.rms(want, 1e-5) * w.double(), tol=1e-6)
    # both rotation layouts, with entries that pass
    v = torch.randn(7, 2, 10, generator=g)
    pos = torch.tensor([0, 1, 2, 50, 51, 400, 1000], dtype=torch.int32)

    def at_positions(fn):  # the oracle turns positions 0 .. n-1: pick the rows
        full = torch.zeros(1001, 2, 10, dtype=torch.float64)
        full[pos.long()] = v.double()
        return fn(full, 6, 50.0)[pos.long()]

    close(hops._rotate(v, pos, hops.rotary_freq(50.0, 6), False), at_positions(O.turn_half), tol=1e-5)
    close(hops._rotate(v, pos, hops.rotary_freq(50.0, 6), True), at_positions(O.turn_pairs), tol=1e-5)
    # norm first, then the sigmoid gate
    yy, ww = torch.randn(3, 10, generator=g), torch.rand(10, generator=g)
    close(hops.gated_group_norm(yy, z, 2, ww, 1e-5, 1, torch.float32, after=True),
          O.rms(yy.double(), 1e-5) * ww.double() * O.sigmoid(z[:, 2:12].double()), tol=1e-6)


def test_linear_attention_state_across_segments():
    """The recurrence over two segments of one sequence equals one pass; a fresh sequence in a used
    slot starts from zero."""
    g = torch.Generator().manual_seed(2)
    H, dk, dv, n = 2, 3, 5, 9
    vkq = torch.randn(n, H * dv + 2 * H * dk, generator=g)
    decay = torch.tensor([0.6, 0.95])
    v, k, q = vkq[:, :H * dv].double().view(n, H, dv), vkq[:, H * dv:H * dv + H * dk].double().view(n, H, dk), \
        vkq[:, H * dv + H * dk:].double().view(n, H, dk)
    want = torch.zeros(n, H, dv, dtype=torch.float64)
    for h in range(H):
        S = torch.zeros(dk, dv, dtype=torch.float64)
        for t in range(n):
            S = float(decay[h]) * S + torch.outer(k[t, h], v[t, h])
            want[t, h] = S.T @ q[t, h]
    state = torch.randn(3, H, dk, dv, generator=g)  # slots hold leftovers of earlier sequences
    i32 = lambda *a: torch.tensor(a, dtype=torch.int32)
    a = hops.linear_attention(vkq[:4].contiguous(), decay, state, i32(0, 4), i32(0), i32(1), H, dk, dv)
    b = hops.linear_attention(vkq[4:].contiguous(), decay, state, i32(0, 5), i32(4), i32(1), H, dk, dv)
    close(torch.cat([a, b]).view(n, H, dv), want, tol=1e-5)


# ------------------------------------------------------------------ cuts, decoding, batches

def test_prefill_equals_token_by_token_and_portions():
    rig = rig_for(FULL, 6)
    t = toks(70, FULL["vocab"], 4)
    want = O.forward(FULL, rig.w, t)
    for cuts in ([70], [], [2, 2, 3, 16, 1, 31], [15, 17, 16, 2], [33, 2, 2, 2], [64]):
        close(rig.run_cut("a", t, cuts), want)


def test_first_tokens_and_single_token_prompt():
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
    taken by a new request whose logits must not see the old pages or the old recurrent state."""
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
    named value projections are scaled up, so that a key that is lost or seen too early moves the
    logits far beyond rounding."""
    w = O.random_weights(cfg, seed)
    t = toks(n, cfg["vocab"] - 1, seed)
    special = cfg["vocab"] - 1
    t[far] = special
    w["embed"] = w["embed"].clone()
    w["embed"][special] *= 6.0
    for name in scale_up:
        w[name] = w[name] * 4.0
    return w, t


@pytest.mark.parametrize("layer,vname", [(att(2, 1, 8, 8, 4), "l0.mix.v"), (lat(2, 8, 4, 8, 8, 12, 0.5), "l0.mix.uv"),
                                        (lin(2, 6, 6, (0.9, 0.99)), "l0.mix.v")], ids=["attention", "latent", "lightning"])
def test_causal_edge(layer, vname):
    """The position of the spiked token is the first that sees it: the one before does not, in a whole
    prompt, in decoding, with the edge at a page border, and in two-token portions."""
    cfg = make_cfg([layer], width=24, vocab=37)
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


def _beacon_attention(cfg, seed, far, n):
    """One attention layer whose every query scores ONE key far above the rest: every token's
    embedding has the same component on axis 0 (it becomes a constant in an entry of the query that
    does not turn) and only the special token has one on axis 1 (it becomes that entry of its key)."""
    w, t = _spiked(cfg, seed, far, n)
    m = cfg["layers"][0]["mixer"]
    H, G, dk, d = m["heads"], m["kv_heads"], m["dim"], cfg["width"]
    e = O.random_weights(cfg, seed)["embed"]
    e[:, 0], e[:, 1] = 2.0, 0.0
    e[cfg["vocab"] - 1, 1] = 4.0
    w["embed"] = e
    w["l0.norm1"] = torch.tensor(1.0)
    c = dk - 1  # beyond rot.dims: passes unchanged
    for h in range(H):
        w["l0.mix.q"][h * dk + c] = 1.5 * torch.eye(d)[0]
    for g in range(G):
        w["l0.mix.k"][g * dk + c] = 1.5 * torch.eye(d)[1]
    w["l0.mix.temp"] = torch.ones(H)
    return w, t


def test_far_key_among_hundreds_attention():
    """One key takes most of the softmax of every later query, 300 tokens on: whole, decoded, and with
    the prompt cut at and around page borders."""
    cfg = make_cfg([att(2, 1, 8, 8, 4, 1e4, 1.0)], width=24, vocab=37)
    n, far = 330, 20
    w, t = _beacon_attention(cfg, 13, far, n)
    want = O.forward(cfg, w, t)
    t2 = list(t)
    t2[far] = 0
    assert float((O.forward(cfg, w, t2)[n - 1] - want[n - 1]).abs().max()) > 0.3
    for cuts in ([n], [310], [100, 2, 64, 130], [far + 12]):
        close(rig_for(cfg, w=w, num_blocks=32).run_cut("a", t, cuts), want, tol=1e-4)


def _marked_linear(cfg, seed, far, n):
    """Only the special token has a component on axis 1 of its embedding, and the key and value
    projections of the linear attention layer amplify that axis: its outer product dominates the state
    of the slowly decaying head for hundreds of tokens."""
    w, t = _spiked(cfg, seed, far, n)
    e = O.random_weights(cfg, seed)["embed"]
    e[:, 1] = 0.0
    e[cfg["vocab"] - 1, 1] = 6.0
    w["embed"] = e
    w["l0.norm1"] = torch.tensor(1.0)
    w["l0.mix.v"][:, 1] = 6.0
    w["l0.mix.k"][:, 1] = 3.0
    return w, t


def test_far_token_in_the_linear_attention_state():
    """A head with a decay near one still carries a token from 300 positions back; a state lost at the
    start of a portion or of a decode step would show."""
    cfg = make_cfg([lin(2, 6, 6, (0.5, 0.999))], width=24, vocab=37)
    n, far = 330, 20
    w, t = _marked_linear(cfg, 14, far, n)
    want = O.forward(cfg, w, t)
    t2 = list(t)
    t2[far] = 0
    assert float((O.forward(cfg, w, t2)[n - 1] - want[n - 1]).abs().max()) > 0.1
    for cuts in ([n], [310], [100, 2, 64, 130], [far + 12]):
        close(rig_for(cfg, w=w, num_blocks=32).run_cut("a", t, cuts), want, tol=1e-4)


def test_far_key_in_shared_latent_pages():
    """Layer 1 reads layer 0's latent pages; the spiked token 300 back is seen through both."""
    cfg = make_cfg([lat(2, 8, 4, 8, 8, 12, 0.5, 1e4), lat(3, 6, 4, 6, 10, 12, 0.4, 1e4, kv_from=0)], width=24, vocab=37)
    n, far = 325, 18
    w, t = _spiked(cfg, 15, far, n, ("l0.mix.uv", "l1.mix.uv"))
    want = O.forward(cfg, w, t)
    t2 = list(t)
    t2[far] = 0
    assert float((O.forward(cfg, w, t2)[n - 1] - want[n - 1]).abs().max()) > 1e-3
    for cuts in ([n], [305], [100, 2, 64, 130]):
        close(rig_for(cfg, w=w, num_blocks=32).run_cut("a", t, cuts), want, tol=1e-4)


def test_head_temperatures_output_gate_and_residual_gate_matter():
    cfg = make_cfg([att(3, 1, 8, 6, 4, mlp=dense(12))], width=24, vocab=37)
    w = O.random_weights(cfg, 16)
    w["l0.mix.temp"] = torch.tensor([3.0, 0.125, 1.0])
    w["l0.rg1.b"] = torch.linspace(-4.0, 4.0, 24)
    t = toks(14, 37, 6)
    want = O.forward(cfg, w, t)
    for name, other in (("l0.mix.temp", torch.ones(3)), ("l0.mix.g", torch.zeros_like(w["l0.mix.g"])),
                        ("l0.rg1.b", torch.zeros(24)), ("l0.rg2", torch.zeros_like(w["l0.rg2"]))):
        w0 = dict(w)
        w0[name] = other
        assert float((O.forward(cfg, w0, t) - want).abs().max()) > 1e-2, name
    for cuts in ([14], [3], [2, 2, 2]):
        close(rig_for(cfg, w=w).run_cut("a", t, cuts), want, tol=1e-4)


def test_norm_numbers_multiplier_and_cap():
    """One-number norm weights far from one, a multiplier above one, logits deep in the cap."""
    cfg = make_cfg([att(mlp=dense()), lin()], mult=1.7, cap=2.5)
    w = O.random_weights(cfg, 17)
    w["l0.norm1"], w["l0.norm2"], w["l1.norm1"], w["final.norm"] = (torch.tensor(v) for v in (0.25, 3.0, -1.5, 2.0))
    w["head"] = w["head"] * 4.0
    t = toks(23, cfg["vocab"], 2)
    want = O.forward(cfg, w, t)
    assert float(want.abs().max()) > 2.4
    for cuts in ([23], [5, 2]):
        close(rig_for(cfg, w=w).run_cut("a", t, cuts), want, tol=1e-4)
    nocap = dict(cfg, logit_softcap=0.0)
    close(rig_for(nocap, w=w).run_cut("a", t, [23]), O.forward(nocap, w, t), tol=1e-4)


def test_rotation_counts_from_zero_on_any_pages():
    """Positions count from 0 in every sequence whatever pages and slots it gets: the same prompt
    run second, on other pages, gives the same logits; large positions keep their accuracy."""
    cfg = make_cfg([att(2, 2, 12, 8, 12, 20.0, 0.4), lat(2, 4, 12, 8, 8, 12, 0.6, 20.0)], width=24, vocab=37)
    rig = rig_for(cfg, 15, num_blocks=48)
    t = toks(420, 37, 9)
    want = O.forward(cfg, rig.w, t)
    rig.step([("z", toks(90, 37, 1))])  # holds the first pages and slot 0
    close(rig.run_cut("a", t, [200, 3, 200]), want, tol=5e-4)


# ------------------------------------------------------------------ engine entry points

def test_greedy_generation_through_engine(tmp_path):
    w = O.random_weights(FULL, 21)
    d = _save(tmp_path, FULL, w)
    assert config_from_dir(d).arch == "bitonex"
    eng = LLMEngine(EngineConfig(model=str(d), weights=str(d), max_num_seqs=3, max_model_len=256, num_blocks=40,
                                 dtype="float32", max_prefill_tokens=16, mixed_prefill_tokens=8), device="cpu")
    prompts = [toks(n, FULL["vocab"], 30 + n) for n in (4, 29, 18, 40)]  # 4 requests over 3 slots: one waits
    seqs = eng.generate(prompts, SamplingParams(max_tokens=10, temperature=0.0, ignore_eos=True))
    for p, s in zip(prompts, seqs):
        assert s.output_ids == O.greedy(FULL, w, p, 10)
    st = eng.stats()
    assert st["mixed_steps"] > 0 and st["kv_blocks_free"] == st["kv_blocks_total"]


def test_preset_round_trip_and_registry():
    c = get_config("bitonex-tiny")
    assert hybrid_config_from_dict(hybrid_config_to_dict(c), c.name) == c
    m = build_model(c, device="cpu", dtype=torch.float32)
    w = state_dict(m)
    assert w["l0.norm1"].shape == () and w["l0.rg1"].shape == (c.d_model, c.d_model) and "l2.rg2" not in w
    cfg = hybrid_config_to_dict(c)
    eng = LLMEngine(EngineConfig(model="bitonex-tiny", max_num_seqs=2, max_model_len=128, num_blocks=16,
                                 dtype="float32"), device="cpu")
    p = toks(11, c.vocab_size, 1)
    s = eng.generate([p], SamplingParams(max_tokens=6, temperature=0.0, ignore_eos=True))[0]
    assert s.output_ids == O.greedy(cfg, w, p, 6)


def test_config_errors_are_loud():
    with pytest.raises(ValueError):
        rig_for(make_cfg([lat(), lat(kv_from=0, kv_rank=16)]), 1)
    with pytest.raises(ValueError):
        rig_for(make_cfg([lat(kv_from=1), lat()]), 1)
    bad = make_cfg([lin()])
    bad["layers"][0]["mixer"]["decay"] = [0.5]
    with pytest.raises(ValueError):
        rig_for(bad, 1, w=O.random_weights(make_cfg([lin()]), 1))
    with pytest.raises(ValueError):
        rig_for(make_cfg([att(4, 3)]), 1)


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

@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gpu_cuts_and_batches_match_oracle(dtype):
    cmp = close if dtype == torch.float32 else (lambda g, w: close_most(g, w, 0.05, frac=1.0))
    rig = rig_for(FULL, 6, device="cuda", dtype=dtype)
    t = toks(70, FULL["vocab"], 4)
    want = O.forward(FULL, rig.w, t)
    for cuts in ([70], [2, 2, 3, 16, 1, 31], [33, 2, 2, 2], []):
        cmp(rig.run_cut("a", t, cuts), want)
    u = toks(40, FULL["vocab"], 8)
    wu = O.forward(FULL, rig.w, u)
    a = rig.step([("a", t[:30]), ("b", u[:5])])
    b = rig.step([("a", t[30:31]), ("b", u[5:])], end=["b"])
    c = rig.step([("a", t[31:])], end=["a"])
    cmp(torch.cat([a["a"], b["a"], c["a"]]), want)
    cmp(torch.cat([a["b"], b["b"]]), wu)


@pytest.mark.gpu
def test_gpu_layers_and_mechanisms_fp32():
    rig = rig_for(FULL, 5, device="cuda", dtype=torch.float32)
    t = toks(19, FULL["vocab"], 3)
    rig.model.layer_probe = []
    rig.run_cut("a", t, [19])
    _, layers = O.forward(FULL, rig.w, t, return_layers=True)
    for got, want in zip(rig.model.layer_probe, layers):
        close(got.cpu(), want)
    rig.model.layer_probe = None
    for layers in ([att(1, 1, 8, 8, 8, 10.0, 1.0)], [att(6, 1, 10, 4, 2)], [att(3, 3, 6, 9, 0)], [lin(1, 1, 1, (0.7,))],
                   [lin(4, 9, 5, (1.0, 0.0, 0.31, 0.999), mlp=dense(1))], [lat(1, 8, 2, 8, 8, 8, 1.0)],
                   [lat(), lat(8, 8, 8, 8, 8, 24, 0.2, kv_from=0)]):
        cfg = make_cfg(layers)
        r2 = rig_for(cfg, 3, device="cuda", dtype=torch.float32)
        u = toks(45, cfg["vocab"], 1)
        close(r2.run_cut("a", u, [20, 2]), O.forward(cfg, r2.w, u))


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gpu_odd_sizes(dtype):
    cfg = make_cfg([att(5, 5, 7, 3, 6, mlp=dense(11)), lin(3, 5, 7, (0.3, 0.6, 0.9), mlp=dense(5)),
                    lat(3, 5, 2, 3, 9, 7, 0.4, mlp=dense(13)), lat(5, 3, 2, 7, 5, 7, 0.3, kv_from=2), att(3, 1, 9, 5, 2)],
                   width=37, vocab=53, mult=1.0, cap=4.0)
    rig = rig_for(cfg, 31, device="cuda", dtype=dtype)
    t = toks(41, 53, 3)
    want = O.forward(cfg, rig.w, t)
    for cuts in ([41], [3, 2, 17]):
        got = rig.run_cut("a", t, cuts)
        close(got, want) if dtype == torch.float32 else close_most(got, want, 0.06, frac=1.0)


@pytest.mark.gpu
def test_gpu_matrix_core_sizes_bf16():
    """Head sizes of 64 / 128 and latent widths that are multiples of 32 / 16 take the matrix-core
    attention kernels and the vector decode kernels; long enough for several pages per wave."""
    cfg = make_cfg([att(8, 2, 64, 128, 32, 1e4, 0.125, mlp=dense(96)), lin(4, 64, 32, (0.9, 0.95, 0.99, 0.999)),
                    lat(4, 32, 32, 48, 48, 64, 0.12, 1e4, mlp=dense(64)), att(4, 4, 128, 64, 128, 1e4, 0.09),
                    lat(8, 16, 32, 32, 40, 64, 0.15, 1e4, kv_from=2), lin(2, 128, 64, (0.97, 0.999), mlp=dense(128))],
                   width=128, vocab=211, mult=0.35)
    rig = rig_for(cfg, 6, device="cuda", dtype=torch.bfloat16, num_blocks=48)
    t = toks(150, cfg["vocab"], 4)
    want = O.forward(cfg, rig.w, t)
    for cuts in ([150], [2, 2, 3, 16, 1, 31], [100]):
        close_most(rig.run_cut("a", t, cuts), want, 0.05, frac=1.0)
    r32 = rig_for(cfg, 6, device="cuda", dtype=torch.float32, num_blocks=48)
    close(r32.run_cut("a", t, [70, 3]), want)


@pytest.mark.gpu
def test_gpu_latent_whole_prompts_take_the_expanded_form(monkeypatch):
    """A step of whole prompts runs latent attention with per-head keys and values in temporary pages
    (unequal prompts in one step: every segment on pages of its own; a layer reading another layer's
    latent); portions and decoding go over the latent cache.  Both forms against the oracle and
    against each other."""
    from k8s_llm_monitor_amd.models.hybrid import LatentAttention

    cfg = make_cfg([lat(4, 32, 32, 64, 48, 64, 0.12, 1e4, mlp=dense(64)), att(4, 2, 64, 64, 32, 1e4, 0.125),
                    lat(2, 96, 32, 128, 40, 64, 0.09, 1e4, kv_from=0, mlp=dense(48))], width=128, vocab=211, mult=0.35)
    w = O.random_weights(cfg, 9)
    t, u = toks(150, cfg["vocab"], 4), toks(70, cfg["vocab"], 5)
    want, wu = O.forward(cfg, w, t), O.forward(cfg, w, u)
    calls = []
    real = LatentAttention._forward_expanded
    monkeypatch.setattr(LatentAttention, "_forward_expanded", lambda self, *a: calls.append(1) or real(self, *a))

    def run(min_rows):
        monkeypatch.setattr(LatentAttention, "EXPAND_MIN_ROWS", min_rows)
        rig = rig_for(cfg, w=w, device="cuda", dtype=torch.bfloat16, num_blocks=48)
        a = rig.step([("a", t[:140]), ("b", u[:64])])  # whole prompts, unequal, one step
        b = rig.step([("a", t[140:141]), ("b", u[64:])], end=["b"])  # a decode row beside a portion
        c = rig.step([("a", t[141:])], end=["a"])
        return torch.cat([a["a"], b["a"], c["a"]]), torch.cat([a["b"], b["b"]])

    ga, gb = run(32)
    assert len(calls) == 2  # both latent layers, the first step only
    ha, hb = run(1 << 30)
    assert len(calls) == 2
    for got, ref in ((ga, want), (gb, wu), (ha, want), (hb, wu)):
        close_most(got, ref, 0.05, frac=1.0)
    close_most(ga, ha.double(), 0.02, frac=1.0)
    close_most(gb, hb.double(), 0.02, frac=1.0)


@pytest.mark.gpu
def test_gpu_long_prompt_on_the_matrix_core_paths():
    """1300 tokens (81 pages, 21 chunks of the linear attention kernel, more than 1024 keys per query)
    at matrix-core sizes in bf16: the whole prompt in one step (latent attention in its expanded
    form), and cut so that the second portion and the decoded tokens read the caches."""
    cfg = make_cfg([att(4, 2, 128, 128, 64, 1e5, 0.09, mlp=dense(96)), lin(2, 64, 64, (0.95, 0.999)),
                    lat(4, 96, 32, 128, 48, 64, 0.09, 1e4, mlp=dense(64)), lat(2, 32, 32, 64, 40, 64, 0.12, 1e4, kv_from=2)],
                   width=128, vocab=211, mult=0.35)
    cfg["max_positions"] = 2048
    rig = rig_for(cfg, 7, device="cuda", dtype=torch.bfloat16, num_blocks=96)
    t = toks(1300, cfg["vocab"], 4)
    want = O.forward(cfg, rig.w, t)
    close_most(rig.run_cut("a", t, [1300]), want, 0.05, frac=1.0)
    close_most(rig.run_cut("a", t, [1100, 190]), want, 0.05, frac=1.0)


@pytest.mark.gpu
def test_gpu_latent_expanded_form_fp32(monkeypatch):
    calls = _force_expanded(monkeypatch)
    cfg = make_cfg([lat(3, 5, 6, 3, 9, 7, 0.4, mlp=dense(13)), att(), lat(5, 3, 6, 7, 5, 7, 0.3, kv_from=0),
                    lat(2, 32, 32, 64, 24, 32, 0.2)])
    rig = rig_for(cfg, 12, device="cuda", dtype=torch.float32)
    t, u = toks(50, cfg["vocab"], 4), toks(17, cfg["vocab"], 5)
    wt, wu = O.forward(cfg, rig.w, t), O.forward(cfg, rig.w, u)
    a = rig.step([("a", t[:40]), ("b", u[:16])])
    b = rig.step([("a", t[40:41]), ("b", u[16:])], end=["b"])
    c = rig.step([("a", t[41:])], end=["a"])
    assert len(calls) == 3
    close(torch.cat([a["a"], b["a"], c["a"]]), wt)
    close(torch.cat([a["b"], b["b"]]), wu)


@pytest.mark.gpu
def test_gpu_far_keys_and_causal_edge():
    cfg = make_cfg([att(2, 1, 8, 8, 4, 1e4, 1.0)], width=24, vocab=37)
    n, far = 330, 20
    w, t = _beacon_attention(cfg, 13, far, n)
    want = O.forward(cfg, w, t)
    for cuts in ([n], [310], [100, 2, 64, 130]):
        close(rig_for(cfg, w=w, num_blocks=32, device="cuda").run_cut("a", t, cuts), want, tol=1e-4)
    cfg = make_cfg([lin(2, 6, 6, (0.5, 0.999))], width=24, vocab=37)
    w, t = _marked_linear(cfg, 14, far, n)
    want = O.forward(cfg, w, t)
    for cuts in ([n], [310], [100, 2, 64, 130]):
        close(rig_for(cfg, w=w, num_blocks=32, device="cuda").run_cut("a", t, cuts), want, tol=1e-4)
    for layer, vname in ((att(2, 1, 8, 8, 4), "l0.mix.v"), (lat(2, 8, 4, 8, 8, 12, 0.5), "l0.mix.uv")):
        cfg = make_cfg([layer], width=24, vocab=37)
        w, t = _spiked(cfg, 11, 16, 22, (vname,))
        want = O.forward(cfg, w, t)
        for cuts in ([22], [16], [2] * 10):
            close(rig_for(cfg, w=w, device="cuda").run_cut("a", t, cuts), want, tol=1e-4)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gpu_new_ops_match_their_torch_forms(dtype):
    g = torch.Generator().manual_seed(3)
    tol = 1e-5 if dtype == torch.float32 else 2e-2
    dev = "cuda"

    def both(fn, *args):
        """fn on CPU copies and on GPU copies of the tensor arguments; returns (cpu, gpu, cpu args, gpu args)."""
        ca = [a.clone() if isinstance(a, torch.Tensor) else a for a in args]
        ga = [a.to(dev) if isinstance(a, torch.Tensor) else a for a in args]
        return fn(*ca), fn(*ga), ca, ga

    for T, n, col, wide in ((5, 24, 8, 64), (3, 7, 3, 20)):  # aligned (8-wide accesses) and not
        z = (torch.randn(T, wide, generator=g) * 2).to(dtype)
        for kind in ("silu", "gelu_tanh"):
            c, u, _, _ = both(hops.activation_cols, z, col, n, kind)
            close(u.cpu().float(), c.double(), tol=tol)
            c, u, _, _ = both(hops.glu, z, col, n // 2 * 2 // 2, kind)
            close(u.cpu().float(), c.double(), tol=tol)
        x = torch.randn(T, n, generator=g).to(dtype)
        c, u, _, _ = both(hops.sigmoid_gate, x, z, col)
        close(u.cpu().float(), c.double(), tol=tol)
        r, y = torch.randn(T, n, generator=g), torch.randn(T, n, generator=g).to(dtype)
        b, w = torch.randn(n, generator=g), torch.rand(n, generator=g) + 0.5
        c, u, ca, ga = both(hops.gated_add_norm, r, y, z, col, b, 0.3, w, 1e-5, False, dtype)
        close(u.cpu().float(), c.double(), tol=tol)
        close(ga[0].cpu(), ca[0].double(), tol=1e-5 if dtype == torch.float32 else 1e-2)
        yy = torch.randn(T, n, generator=g)
        c, u, _, _ = both(hops.gated_group_norm, yy, z, col, w, 1e-5, 1, dtype, True)
        close(u.cpu().float(), c.double(), tol=tol)
    lg = torch.randn(4, 50, generator=g) * 20
    c, u, _, _ = both(hops.softcap, lg, 9.0)
    close(u.cpu(), c.double(), tol=1e-6)
    # rotation + temperatures + page writes, both layouts, rotating part smaller than the head
    Hq, G, dk, dv, T = 4, 2, 12, 6, 9
    for pairs in (False, True):
        qkv = torch.randn(T, Hq * dk + G * dk + G * dv + 5, generator=g).to(dtype)
        pos = torch.tensor([0, 1, 2, 3, 500, 501, 17, 18, 19], dtype=torch.int32)
        slots = torch.tensor([0, 1, 2, 3, 40, 41, -1, 16, 17], dtype=torch.int32)
        kc, vc = torch.zeros(4, 16, G * dk, dtype=dtype), torch.zeros(4, G, dv, 16, dtype=dtype)
        _, _, ca, ga = both(hops.rotary_cache, qkv, Hq, G, dk, dv, pos, hops.rotary_freq(100.0, 8), pairs,
                            torch.tensor([1.0, 0.5, 2.0, 1.5]), kc, vc, slots)
        for i in (0, 9, 10):
            close(ga[i].cpu().float(), ca[i].double(), tol=tol)
    # the fixed-decay recurrence, decode-shaped and prompt-shaped launches
    H, dk, dv = 3, 16, 24
    vkq = torch.randn(70, H * dv + 2 * H * dk, generator=g).to(dtype)
    decay = torch.tensor([0.5, 0.9, 0.999])
    st = torch.randn(4, H, dk, dv, generator=g)
    i32 = lambda *a: torch.tensor(a, dtype=torch.int32)
    for cu, ctx, slot in ((i32(0, 66, 67, 70), i32(0, 5, 9), i32(2, 0, 3)), (i32(0, 1, 2, 3), i32(7, 0, 3), i32(1, 2, 0))):
        nrow = int(cu[-1])
        for mode in (0, 1, 2):
            c, u, ca, ga = both(hops.linear_attention, vkq[:nrow].contiguous(), decay, st, cu, ctx, slot, H, dk, dv, mode)
            close(u.cpu(), c.double(), tol=1e-4)
            close(ga[2].cpu(), ca[2].double(), tol=1e-4)


@pytest.mark.gpu
@pytest.mark.parametrize("H,dk,dv,tiles", [(2, 32, 32, 0), (3, 64, 96, 2), (1, 96, 32, 1), (2, 128, 128, 1), (4, 128, 64, 2),
                                           (3, 96, 48, 0), (2, 32, 16, 1)])
def test_gpu_chunked_linear_attention_matches_the_recurrence(H, dk, dv, tiles):
    """The matrix-core form (chunks of 64 tokens) against the token-by-token torch form: segments
    shorter than, equal to and longer than a chunk, one continuing from its slot, one padding
    segment, decays of 0, 1 and between; outputs and the states left in the slots."""
    g = torch.Generator().manual_seed(5)
    lens = [1, 63, 64, 65, 200, 7, 130]
    cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
    ctx = torch.tensor([0, 5, 0, 64, 0, 3, 9], dtype=torch.int32)
    slot = torch.tensor([0, 1, 2, 3, 4, -1, 5], dtype=torch.int32)
    T = int(cu[-1])
    vkq = (torch.randn(T, H * dv + 2 * H * dk, generator=g) * 0.7).to(torch.bfloat16)
    decay = torch.tensor(([0.9, 1.0, 0.0, 0.999] * 2)[:H])
    st = torch.randn(6, H, dk, dv, generator=g)
    want_state = st.clone()
    want = hops.linear_attention(vkq, decay, want_state, cu, ctx, slot, H, dk, dv)
    got_state = st.to("cuda")
    got = hops.linear_attention(vkq.to("cuda"), decay.to("cuda"), got_state, cu.to("cuda"), ctx.to("cuda"), slot.to("cuda"),
                                H, dk, dv, mode=3, col_tiles=tiles)
    close(got.cpu(), want.double(), tol=2e-5)
    close(got_state.cpu(), want_state.double(), tol=2e-5)
    scan_state = st.to("cuda")
    scan = hops.linear_attention(vkq.to("cuda"), decay.to("cuda"), scan_state, cu.to("cuda"), ctx.to("cuda"), slot.to("cuda"),
                                 H, dk, dv, mode=2)
    close(got.cpu(), scan.cpu().double(), tol=2e-5)


@pytest.mark.gpu
def test_gpu_greedy_generation_with_graphs():
    eng = LLMEngine(EngineConfig(model="bitonex-tiny", max_num_seqs=4, max_model_len=256, num_blocks=64,
                                 dtype="float32", max_prefill_tokens=32, mixed_prefill_tokens=16), device="cuda")
    eng.warmup()  # decode steps replay from captured hipGraphs
    cfg, w = hybrid_config_to_dict(eng.model_cfg), state_dict(eng.model)
    prompts = [toks(n, 310, 40 + n) for n in (5, 37, 21)]
    seqs = eng.generate(prompts, SamplingParams(max_tokens=12, temperature=0.0, ignore_eos=True))
    assert eng.stats()["graph_buckets"]
    for p, s in zip(prompts, seqs):
        assert s.output_ids == O.greedy(cfg, w, p, 12)
