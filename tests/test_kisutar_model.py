"""The Kisutar layer-list design in the engine against the plain float64 oracle
(tests/kisutar_oracle.py): each mechanism alone (latent attention with its rotation, window and
learned sinks, shared key/value pages, the token shift, the depth average, the xIELU dense layer,
the softmax-over-all router with plain experts), prefill against token-by-token decoding, prompt
portions down to two tokens, unequal batches, pages and state slots that are reused, keys far away
and at window and page edges, the first tokens, long decoding, odd sizes and sizes of one, and
greedy generation through the engine and the trace command.

Runs on the CPU (the ops' torch forms); the ``gpu`` tests at the end run the same comparisons
through the HIP kernels."""
import json
import math
import subprocess
import sys

import pytest
import torch

import kisutar_oracle as O
from k8s_llm_monitor_amd.engine import EngineConfig, LLMEngine, SamplingParams
from k8s_llm_monitor_amd.models.config import get_config, hybrid_config_from_dict, hybrid_config_to_dict
from k8s_llm_monitor_amd.models.hybrid import state_dict
from k8s_llm_monitor_amd.models.registry import build_model, config_from_dir
from k8s_llm_monitor_amd.ops import hybrid as hops
from test_hybrid_model import ROOT, Rig, _save, close, close_most, toks


# ------------------------------------------------------------------ small configurations

def lat(heads=3, dim=12, rot=8, vdim=10, q_rank=20, kv_rank=24, window=7, scale=0.25, base=100.0, kv_from=None,
        rot_dims=None, mlp=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
         "mask": {"size": window}, "scale": scale, "rot": {"base": base, "dims": rot if rot_dims is None else rot_dims}}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return {"type": "latent_attention", "mixer": m, "mlp": mlp}


def dense(ff=36):
    return {"kind": "dense", "ff": ff}


def moe(experts=5, top=2, ff=20, shared=28):
    return {"kind": "moe", "expert": {"ff": ff}, "router": {"experts": experts, "top": top},
            "shared": {"ff": shared} if shared else None}


def make_cfg(layers, width=40, vocab=61, eps=1e-6):
    return {"architecture": "Kisutar", "vocab": vocab, "width": width, "layers": layers, "norm": {"eps": eps},
            "max_positions": 1024}


FULL = make_cfg([lat(mlp=dense()), lat(2, 8, 4, 6, 12, 16, 19, 0.3, mlp=moe()), lat(4, 6, 4, 8, 10, 16, 5, 0.2, kv_from=1),
                 lat(2, 10, 4, 12, 16, 16, 33, 0.22, kv_from=1, mlp=moe(4, 1, 12, 0)), lat(1, 16, 6, 4, 8, 12, 3, 0.3, mlp=dense(20))])


def rig_for(cfg, seed=0, w=None, **kw):
    return Rig(cfg, w=w if w is not None else O.random_weights(cfg, seed), **kw)


# ------------------------------------------------------------------ mechanisms alone

@pytest.mark.parametrize("layers", [
    [lat()], [lat(1, 8, 2, 8, 8, 8, 1, 1.0)], [lat(4, 4, 16, 20, 9, 40, 100, 0.2)], [lat(2, 6, 8, 4, 6, 10, 9, 0.3, rot_dims=4)],
    [lat(), lat(2, 8, 8, 8, 8, 24, 4, 0.2, kv_from=0)], [lat(mlp=dense())], [lat(mlp=dense(1))], [lat(mlp=moe())],
    [lat(mlp=moe(3, 3, 8, 0))], [lat(mlp=moe(9, 1, 4, 4))], [lat(mlp=moe(1, 1, 6, 0))]],
    ids=["latent", "latent-ones", "latent-wide-window", "latent-partial-rotation", "shared-pages", "dense", "dense-ff1",
         "moe-shared", "moe-all-experts", "moe-top1", "moe-one-expert"])
def test_single_mechanism_whole_prompt(layers):
    cfg = make_cfg(layers)
    rig = rig_for(cfg, 3)
    t = toks(45, cfg["vocab"], 1)
    close(rig.run_cut("a", t, [45]), O.forward(cfg, rig.w, t))


def test_odd_sizes_everywhere():
    """Widths, ranks and head sizes that are multiples of nothing (rotated sizes stay even)."""
    cfg = make_cfg([lat(3, 5, 2, 3, 9, 7, 6, 0.4, mlp=dense(11)), lat(5, 3, 2, 7, 5, 7, 11, 0.3, kv_from=0, mlp=moe(3, 2, 5, 9)),
                    lat(1, 7, 4, 5, 3, 13, 4, 0.5, mlp=moe(7, 2, 3, 0))], width=37, vocab=53)
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
    _, layers = O.forward(FULL, rig.w, t, return_layers=True)
    assert len(rig.model.layer_probe) == layers.shape[0] == 5
    for got, want in zip(rig.model.layer_probe, layers):
        close(got, want)
    rig.model.layer_probe = None


def test_token_shift_fractions_zero_one_and_between():
    """Fractions of exactly 0 (no shift) and 1 (the mixer reads only the previous token) and the
    state across portions: the oracle shifts whole sequences at once."""
    cfg = make_cfg([lat(mlp=dense()), lat(2, 8, 4, 6, 12, 16, 6, 0.3)])
    t = toks(31, cfg["vocab"], 2)
    for mode in ("zero", "one", "mixed"):
        w = O.random_weights(cfg, 4)
        for i in range(2):
            mu = w[f"l{i}.shift"]
            w[f"l{i}.shift"] = {"zero": torch.zeros_like(mu), "one": torch.ones_like(mu), "mixed": mu}[mode]
        want = O.forward(cfg, w, t)
        for cuts in ([31], [], [2, 2, 9, 1, 1, 16], [17, 2]):
            close(rig_for(cfg, w=w).run_cut("a", t, cuts), want)


def test_depth_average_uses_every_earlier_result():
    """Coefficients that single out one earlier result (the embedding output, or layer 0's) show
    whether the stack keeps the results before averaging."""
    cfg = make_cfg([lat(mlp=dense()), lat(mlp=None), lat(mlp=moe())])
    t = toks(14, cfg["vocab"], 7)
    for pick in (0, 1, 2):
        w = O.random_weights(cfg, 8)
        w["l2.dwa"] = torch.zeros(4)
        w["l2.dwa"][pick] = 1.0
        w["l1.dwa"] = torch.tensor([0.5, -0.25, 1.5])
        close(rig_for(cfg, w=w).run_cut("a", t, [5, 9]), O.forward(cfg, w, t))


def test_ops_against_oracle_functions():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(9, 20, generator=g)
    # activation
    z = torch.randn(50, generator=g) * 3
    for a, b in ((0.3, 0.7), (1.2, 0.5)):
        want = torch.where(z.double() > 0, a * z.double() ** 2 + 0.5 * z.double(),
                           b * (torch.expm1(z.double().clamp(max=0)) - z.double()) + 0.5 * z.double())
        close(hops.activation(z.view(1, -1), "xielu", a, b)[0], want, tol=1e-6)
    close(hops.activation(z.view(1, -1), "gelu")[0], O.gelu_erf(z.double()), tol=1e-6)
    p, q = torch.tensor(0.4, dtype=torch.float64), torch.tensor(-0.9, dtype=torch.float64)
    close(hops.activation(z.view(1, -1), "xielu", float(O.softplus(p)), 0.5 + float(O.softplus(q)))[0],
          O.xielu(z.double(), p, q), tol=1e-6)
    # norm + shift over two segments, one continuing from its state slot
    w, mu = torch.rand(20, generator=g) + 0.5, torch.rand(20, generator=g)
    full = O.token_shift(O.rms_norm(x.double(), w.double(), 1e-6), mu.double())
    state = torch.zeros(3, 20)
    cu, ctx, slot = (torch.tensor(v, dtype=torch.int32) for v in ([0, 4], [0], [2]))
    a = hops.norm_shift(x[:4].clone(), (), w, 1e-6, False, mu, state, cu, ctx, slot, torch.float32)
    cu, ctx = torch.tensor([0, 5], dtype=torch.int32), torch.tensor([4], dtype=torch.int32)
    b = hops.norm_shift(x[4:].clone(), (), w, 1e-6, False, mu, state, cu, ctx, slot, torch.float32)
    close(torch.cat([a, b]), full, tol=1e-6)
    assert float(state[0].abs().max()) == 0.0 and float(state[2].abs().max()) > 0.0
    # depth mix
    stack = torch.randn(5, 6, 8, generator=g)
    add = torch.randn(6, 8, generator=g)
    coef = torch.tensor([0.2, -1.0, 0.7])
    ref = stack.double().clone()
    ref[2] += add.double()
    want = sum(coef[j].double() * ref[j] for j in range(3))
    out = hops.depth_mix(stack, 2, add, coef)
    close(out, want, tol=1e-6)
    close(stack[2], ref[2], tol=1e-6)
    # rotation: pairs (i, i + dims/2) of the first dims entries
    v = torch.randn(7, 2, 10, generator=g)
    pos = torch.tensor([0, 1, 2, 50, 51, 400, 1000], dtype=torch.int32)
    got = hops._rotate_half(v, pos, hops.rotary_freq(50.0, 6))
    close(got, O.rotate(v.double(), pos, 50.0, 6), tol=1e-5)
    # router: probabilities over all experts, not renormalised
    h = torch.randn(5, 12, generator=g)
    wr = torch.randn(6, 12, generator=g)
    ids, wts, _ = hops.moe_router(h, wr, None, 6, 2, over_all=True)
    s = torch.softmax(h.double() @ wr.double().T, -1)
    assert ids.tolist() == torch.topk(s, 2).indices.tolist()
    close(wts, torch.topk(s, 2).values, tol=1e-6)
    assert float(wts.sum(-1).max()) < 1.0


# ------------------------------------------------------------------ cuts, decoding, batches

def test_prefill_equals_token_by_token_and_portions():
    rig = rig_for(FULL, 6)
    t = toks(70, FULL["vocab"], 4)
    want = O.forward(FULL, rig.w, t)
    for cuts in ([70], [], [2, 2, 3, 16, 1, 31], [15, 17, 16, 2], [33, 2, 2, 2], [64]):
        close(rig.run_cut("a", t, cuts), want)


def test_whole_prompts_in_the_expanded_form(monkeypatch):
    """Latent attention's other form - this step's keys and values expanded per head into temporary
    pages, windowed attention over them - with windows, learned sinks and shared pages: unequal whole
    prompts in one step, then portions and decoding over the latent cache those steps left."""
    from k8s_llm_monitor_amd.models.hybrid import LatentAttention

    calls = []
    real = LatentAttention._forward_expanded
    monkeypatch.setattr(LatentAttention, "_forward_expanded", lambda self, *a: calls.append(1) or real(self, *a))
    monkeypatch.setattr(LatentAttention, "_expand_ok",
                        lambda self, h, meta: meta.is_prefill and meta.all_fresh and not meta.num_decode)
    rig = rig_for(FULL, 6)
    V = FULL["vocab"]
    t, u = toks(60, V, 4), toks(21, V, 5)
    wt, wu = O.forward(FULL, rig.w, t), O.forward(FULL, rig.w, u)
    a = rig.step([("a", t[:45]), ("b", u[:20])])
    assert len(calls) == 5
    b = rig.step([("a", t[45:46]), ("b", u[20:])], end=["b"])
    c = rig.step([("a", t[46:])], end=["a"])
    assert len(calls) == 5
    close(torch.cat([a["a"], b["a"], c["a"]]), wt)
    close(torch.cat([a["b"], b["b"]]), wu)


def test_first_tokens_and_single_token_prompt():
    rig = rig_for(FULL, 7)
    for n in (1, 2, 3):
        t = toks(n, FULL["vocab"], 10 + n)
        close(rig.run_cut("a", t, [n]), O.forward(FULL, rig.w, t))
        close(rig.run_cut("a", t, []), O.forward(FULL, rig.w, t))


def test_long_decoding_past_windows_and_pages():
    rig = rig_for(FULL, 8)
    t = toks(150, FULL["vocab"], 5)
    close(rig.run_cut("a", t, [20]), O.forward(FULL, rig.w, t))  # 130 decode steps over 9 pages


def test_unequal_batch_equals_each_alone_and_reuse():
    """Four live requests with portions beside decode tokens; one ends and its pages and slot are
    taken by a new request whose logits must not see the old pages or the old shift state."""
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


# ------------------------------------------------------------------ edges made visible

def _spiked(cfg, seed, far_pos, n, layers=(0,)):
    """Weights and a prompt in which ONE position dominates: its token has a huge embedding and the
    value expansions are scaled up, so a window off by one changes the logits far beyond rounding.
    The token shift is switched off: it would carry the token into the next position's keys."""
    w = O.random_weights(cfg, seed)
    t = toks(n, cfg["vocab"] - 1, seed)
    special = cfg["vocab"] - 1
    t[far_pos] = special
    w["embed"] = w["embed"].clone()
    w["embed"][special] *= 6.0
    for i in range(len(cfg["layers"])):
        w[f"l{i}.shift"] = torch.zeros_like(w[f"l{i}.shift"])
    for i in layers:
        w[f"l{i}.mix.uv"] = w[f"l{i}.mix.uv"] * 4.0
    return w, t


def _check_edge(cfg, w, t, far, win):
    want = O.forward(cfg, w, t)
    t2 = list(t)
    t2[far] = 0
    moved = O.forward(cfg, w, t2)
    # the oracle itself distinguishes the two sides clearly (otherwise the test shows nothing)
    assert float((moved[far + win - 1] - want[far + win - 1]).abs().max()) > 1e-2
    assert float((moved[far + win] - want[far + win]).abs().max()) < 1e-9
    return want


@pytest.mark.parametrize("win", [1, 2, 5, 16, 17, 33])
def test_window_edge_in_and_out(win):
    """The query at distance win-1 from the spiked key sees it, at distance win it does not; in a
    whole prompt, in decoding, with the key on the page before, and in two-token portions."""
    cfg = make_cfg([lat(2, 8, 4, 8, 8, 12, win, 0.5)], width=24, vocab=37)
    far = 30
    w, t = _spiked(cfg, 11, far, far + win + 4)
    want = _check_edge(cfg, w, t, far, win)
    for cuts in ([len(t)], [far + 1], [far - 3, 7], [2] * ((far + win) // 2)):
        close(rig_for(cfg, w=w).run_cut("a", t, cuts), want, tol=1e-4)


@pytest.mark.parametrize("wins", [(3, 21), (20, 6)])
def test_window_edge_of_a_layer_reading_another_layers_pages(wins):
    """Layer 1 reads layer 0's pages with a window of its own: its edge is where the logits stop
    depending on the spiked token when it is the wider one, and layer 0's otherwise."""
    a, b = wins
    cfg = make_cfg([lat(2, 8, 4, 8, 8, 12, a, 0.5), lat(3, 6, 4, 6, 10, 12, b, 0.4, kv_from=0)], width=24, vocab=37)
    far, win = 19, max(a, b)
    w, t = _spiked(cfg, 12, far, far + win + 5, layers=(0, 1))
    want = _check_edge(cfg, w, t, far, win)
    for cuts in ([len(t)], [far + 2], [far + win - 1], [2] * ((far + win) // 2)):
        close(rig_for(cfg, w=w).run_cut("a", t, cuts), want, tol=1e-4)


def _beacon(cfg, seed, far, n):
    """One layer whose every query scores ONE key far above the rest: every token's embedding has
    the same component on axis 0 (it becomes a constant in the query's slowest-turning rotated
    entry) and only the special token has one on axis 1 (it becomes that entry of its key)."""
    w, t = _spiked(cfg, seed, far, n)
    m = cfg["layers"][0]["mixer"]
    H, dn, dr, R, d = m["heads"], m["dim"], m["rot_dim"], m["kv_rank"], cfg["width"]
    half = m["rot"]["dims"] // 2
    lo, hi = half - 1, 2 * half - 1  # the pair with the lowest frequency
    special = cfg["vocab"] - 1
    e = O.random_weights(cfg, seed)["embed"]
    e[:, 0], e[:, 1] = 2.0, 0.0
    e[special, 1] = 4.0
    w["embed"] = e
    w["l0.norm1"][:2] = 1.0
    w["l0.mix.dq"][0] = torch.eye(d)[0]
    w["l0.mix.dq.norm"][0] = 1.0
    for h in range(H):
        w["l0.mix.uq"][h * (dn + dr) + dn + lo] = 1.25 * torch.eye(m["q_rank"])[0]
        w["l0.mix.uq"][h * (dn + dr) + dn + hi] = 0.0
    w["l0.mix.dkv"][R + lo] = 1.25 * torch.eye(d)[1]
    w["l0.mix.dkv"][R + hi] = 0.0
    return w, t


def test_far_key_among_hundreds():
    """One key 299 tokens back, just inside a window of 300, takes most of the softmax of the query
    that still sees it; the next query does not see it.  Whole, decoded, and across page borders."""
    cfg = make_cfg([lat(2, 8, 4, 8, 8, 12, 300, 1.0, base=1e6)], width=24, vocab=37)
    n, far = 330, 20
    w, t = _beacon(cfg, 13, far, n)
    want = O.forward(cfg, w, t)
    t2 = list(t)
    t2[far] = 0
    moved = O.forward(cfg, w, t2)
    assert float((moved[far + 299] - want[far + 299]).abs().max()) > 0.3
    assert float((moved[far + 300] - want[far + 300]).abs().max()) < 1e-9
    for cuts in ([n], [310], [100, 2, 64, 130], [far + 295]):
        close(rig_for(cfg, w=w, num_blocks=32).run_cut("a", t, cuts), want, tol=1e-4)


def test_sinks_matter_per_head():
    """Large and small learned sink logits: a head whose sink is large attends to almost nothing.
    Leaving the sinks out, or using one value for all heads, would change the logits."""
    cfg = make_cfg([lat(3, 8, 4, 8, 8, 12, 4, 0.05)], width=24, vocab=37)
    w = O.random_weights(cfg, 14)
    w["l0.mix.sink"] = torch.tensor([4.0, -3.0, 0.5])
    t = toks(12, 37, 6)
    want = O.forward(cfg, w, t)
    w0 = dict(w)
    w0["l0.mix.sink"] = torch.zeros(3)
    assert float((O.forward(cfg, w0, t) - want).abs().max()) > 1e-2
    for cuts in ([12], [3]):
        close(rig_for(cfg, w=w).run_cut("a", t, cuts), want, tol=1e-4)


def test_rotation_depends_on_distance_only_and_counts_from_zero():
    """Positions count from 0 in every sequence whatever pages and slots it gets: the same prompt
    run second, on other pages, gives the same logits; large positions keep their accuracy."""
    cfg = make_cfg([lat(2, 4, 12, 8, 8, 12, 50, 0.6, base=20.0)], width=24, vocab=37)
    rig = rig_for(cfg, 15, num_blocks=48)
    t = toks(420, 37, 9)
    want = O.forward(cfg, rig.w, t)
    rig.step([("z", toks(90, 37, 1))])  # holds the first pages and slot 0
    close(rig.run_cut("a", t, [200, 3, 200]), want, tol=5e-4)


# ------------------------------------------------------------------ engine entry points

def test_greedy_generation_through_engine(tmp_path):
    w = O.random_weights(FULL, 21)
    d = _save(tmp_path, FULL, w)
    assert config_from_dir(d).arch == "kisutar"
    eng = LLMEngine(EngineConfig(model=str(d), weights=str(d), max_num_seqs=3, max_model_len=256, num_blocks=40,
                                 dtype="float32", max_prefill_tokens=16, mixed_prefill_tokens=8), device="cpu")
    prompts = [toks(n, FULL["vocab"], 30 + n) for n in (4, 29, 18, 40)]  # 4 requests over 3 slots: one waits
    seqs = eng.generate(prompts, SamplingParams(max_tokens=10, temperature=0.0, ignore_eos=True))
    for p, s in zip(prompts, seqs):
        assert s.output_ids == O.greedy(FULL, w, p, 10)
    st = eng.stats()
    assert st["mixed_steps"] > 0 and st["kv_blocks_free"] == st["kv_blocks_total"]


def test_preset_round_trip_and_registry():
    c = get_config("kisutar-tiny")
    assert hybrid_config_from_dict(hybrid_config_to_dict(c), c.name) == c
    m = build_model(c, device="cpu", dtype=torch.float32)
    w = state_dict(m)
    cfg = hybrid_config_to_dict(c)
    eng = LLMEngine(EngineConfig(model="kisutar-tiny", max_num_seqs=2, max_model_len=128, num_blocks=16,
                                 dtype="float32"), device="cpu")
    p = toks(11, c.vocab_size, 1)
    s = eng.generate([p], SamplingParams(max_tokens=6, temperature=0.0, ignore_eos=True))[0]
    assert s.output_ids == O.greedy(cfg, w, p, 6)


def test_config_errors_are_loud():
    bad = make_cfg([lat(), lat(kv_from=0, kv_rank=16)])
    with pytest.raises(ValueError):
        rig_for(bad, 1)
    with pytest.raises(ValueError):
        rig_for(make_cfg([lat(kv_from=1), lat()]), 1)
    with pytest.raises(ValueError):
        hybrid_config_from_dict(make_cfg([lat(mlp={"kind": "conv"})]), "x")


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
    import numpy as np

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
    cmp = close if dtype == torch.float32 else (lambda g, w: close_most(g, w, 0.05))
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
    for layers in ([lat(1, 8, 2, 8, 8, 8, 1, 1.0)], [lat(2, 6, 8, 4, 6, 10, 9, 0.3, rot_dims=4, mlp=dense(1))],
                   [lat(mlp=moe(1, 1, 6, 0))], [lat(mlp=moe(9, 1, 4, 4)), lat(8, 8, 8, 8, 8, 24, 40, 0.2, kv_from=0)]):
        cfg = make_cfg(layers)
        r2 = rig_for(cfg, 3, device="cuda", dtype=torch.float32)
        u = toks(45, cfg["vocab"], 1)
        close(r2.run_cut("a", u, [20, 2]), O.forward(cfg, r2.w, u))


@pytest.mark.gpu
@pytest.mark.parametrize("win", [1, 16, 17, 33])
def test_gpu_window_edges_and_sinks(win):
    cfg = make_cfg([lat(2, 8, 4, 8, 8, 12, win, 0.5)], width=24, vocab=37)
    far = 30
    w, t = _spiked(cfg, 11, far, far + win + 4)
    w["l0.mix.sink"] = torch.tensor([2.5, -2.0])
    want = _check_edge(cfg, w, t, far, win)
    for cuts in ([len(t)], [far + 1], [2] * ((far + win) // 2)):
        close(rig_for(cfg, w=w, device="cuda").run_cut("a", t, cuts), want, tol=1e-4)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_gpu_odd_and_large_sizes(dtype):
    """Sizes that are multiples of nothing, and a latent wider than the vector and matrix-core
    kernels take (the any-size kernels)."""
    odd = make_cfg([lat(3, 5, 2, 3, 9, 7, 6, 0.4, mlp=dense(11)), lat(5, 3, 2, 7, 5, 7, 11, 0.3, kv_from=0, mlp=moe(3, 2, 5, 9)),
                    lat(1, 7, 4, 5, 3, 13, 4, 0.5, mlp=moe(7, 2, 3, 0))], width=37, vocab=53)
    wide = make_cfg([lat(2, 8, 8, 8, 16, 328, 20, 0.3, mlp=dense(24))], width=48, vocab=53)
    for cfg in (odd, wide):
        rig = rig_for(cfg, 31, device="cuda", dtype=dtype)
        t = toks(41, 53, 3)
        want = O.forward(cfg, rig.w, t)
        for cuts in ([41], [3, 2, 17]):
            got = rig.run_cut("a", t, cuts)
            close(got, want) if dtype == torch.float32 else close_most(got, want, 0.06, frac=0.85)


@pytest.mark.gpu
def test_gpu_far_key_among_hundreds():
    cfg = make_cfg([lat(2, 8, 4, 8, 8, 12, 300, 1.0, base=1e6)], width=24, vocab=37)
    n, far = 330, 20
    w, t = _beacon(cfg, 13, far, n)
    want = O.forward(cfg, w, t)
    for cuts in ([n], [310], [100, 2, 64, 130]):
        close(rig_for(cfg, w=w, num_blocks=32, device="cuda").run_cut("a", t, cuts), want, tol=1e-4)


@pytest.mark.gpu
def test_gpu_bf16_dense_only_is_within_rounding():
    """Without routed experts nothing is discrete: bf16 stays close on every row; eight heads and
    a latent width that is a multiple of eight take the vector decode kernel."""
    cfg = make_cfg([lat(8, 16, 8, 16, 24, 40, 30, 0.2, mlp=dense(64)), lat(4, 16, 8, 8, 16, 40, 12, 0.2, kv_from=0),
                    lat(2, 24, 16, 16, 16, 48, 100, 0.15, mlp=dense(48))], width=64, vocab=97)
    rig = rig_for(cfg, 6, device="cuda", dtype=torch.bfloat16)
    t = toks(130, cfg["vocab"], 4)
    want = O.forward(cfg, rig.w, t)
    for cuts in ([130], [2, 2, 3, 16, 1, 31], [90]):
        close_most(rig.run_cut("a", t, cuts), want, 0.05, frac=1.0)


@pytest.mark.gpu
def test_gpu_greedy_generation_with_graphs():
    eng = LLMEngine(EngineConfig(model="kisutar-tiny", max_num_seqs=4, max_model_len=256, num_blocks=64,
                                 dtype="float32", max_prefill_tokens=32, mixed_prefill_tokens=16), device="cuda")
    eng.warmup()  # decode steps replay from captured hipGraphs
    cfg, w = hybrid_config_to_dict(eng.model_cfg), state_dict(eng.model)
    prompts = [toks(n, 380, 40 + n) for n in (5, 37, 21)]
    seqs = eng.generate(prompts, SamplingParams(max_tokens=12, temperature=0.0, ignore_eos=True))
    assert eng.stats()["graph_buckets"]
    for p, s in zip(prompts, seqs):
        assert s.output_ids == O.greedy(cfg, w, p, 12)
