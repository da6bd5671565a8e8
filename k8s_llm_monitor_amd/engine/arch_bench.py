"""Prefill and decode throughput of a layer-list design beside the closest existing model at equal
layer sizes, random weights, one GPU (``python bench.py --mode arch [--arch-design NAME]``):
Dunesun beside a Mixtral-style model (attention + routed experts in every layer); Kisutar beside
an all-attention Dunesun model (windowed attention with sinks, fp32 residual stream, routed experts
with a shared expert in every layer - the same kernels family); Bitonex (rotary attention, linear
attention and latent attention layers in turn, dense gated feed-forward) beside a Dunesun model of
attention and Mamba-2 layers with the same heads, head sizes, recurrent state size and feed-forward
width (one expert, so every token takes it); Levovik (softmax attention beside gated linear attention
or the gated delta rule in every layer, routed clamped experts) beside a Dunesun model that has one
attention layer with the same experts and one Mamba-2 layer of equal state size for every Levovik
layer.  Both models run through the same
ModelRunner step functions the engine uses: one prefill step of ``seqs`` whole prompts, then decode
steps of ``batch`` sequences (hipGraph replay where the model's decode is captured)."""
from __future__ import annotations

import json
import time

import torch

from ..models.config import DenseSpec, HybridConfig, LayerSpec, ModelConfig, MoESpec
from ..models.registry import build_model
from .block_manager import BlockManager
from .runner import ModelRunner, RunnerConfig
from .sequence import SamplingParams, Sequence

# (name, width, heads, kv heads, head dim, experts, top, expert ff, layers)
SIZES = {
    "s": ("d1024", 1024, 8, 2, 128, 8, 2, 1024, 4),
    "m": ("d2048", 2048, 16, 4, 128, 8, 2, 2048, 4),
    "l": ("d4096", 4096, 32, 8, 128, 8, 2, 3584, 2),
}


def _pair(size: str, window: int) -> tuple:
    name, d, H, G, D, E, K, ff, L = SIZES[size]
    att = LayerSpec("attention", tuple(sorted({"heads": H, "kv_heads": G, "dim": D, "vdim": D, "mask.size": window,
                                               "scale": D ** -0.5}.items())), MoESpec(E, K, ff, 0))
    ssm = LayerSpec("mamba2", tuple(sorted({"heads": 2 * d // 64, "vdim": 64, "state": 128, "groups": 1, "conv": 4,
                                            "norm_groups": 1}.items())), MoESpec(E, K, ff, 0))
    hy = HybridConfig(name=f"dunesun-{name}", arch="dunesun", vocab_size=32000, d_model=d,
                      layers=tuple(att if i % 2 == 0 else ssm for i in range(L)), max_position=8192)
    ref = ModelConfig(name=f"mixtral-{name}", arch="llama", vocab_size=32000, d_model=d, n_layers=L, n_heads=H,
                      n_kv_heads=G, head_dim=D, ffn_dim=ff, max_position=8192, rope_theta=1e6, n_experts=E,
                      top_k_experts=K, bos_id=1, eos_ids=(2,))
    return hy, ref


# Kisutar: (name, width, heads, unrotated dim, rotated dim, value dim, q rank, kv rank, experts, top, expert ff,
#           shared ff, dense ff, layers); the reference gets the same width, heads, head size dim + rot, experts
KISUTAR_SIZES = {
    "s": ("d1024", 1024, 8, 96, 32, 128, 384, 128, 8, 2, 1024, 1024, 4096, 4),
    "m": ("d2048", 2048, 16, 96, 32, 128, 768, 256, 8, 2, 2048, 2048, 8192, 4),
    "l": ("d4096", 4096, 32, 96, 32, 128, 1536, 256, 8, 2, 3584, 3584, 14336, 2),
}


def _kisutar_pair(size: str, window: int) -> tuple:
    """Kisutar (dense and routed layers alternating, the second half of the layers reading the pages
    of the last layer before them that has its own) and an all-attention Dunesun model of equal
    width, heads, head size and experts."""
    name, d, H, dn, dr, dv, Q, R, E, K, ff, fs, fd, L = KISUTAR_SIZES[size]
    own = max(1, L // 2)

    def lat(i):
        m = {"heads": H, "dim": dn, "rot_dim": dr, "vdim": dv, "q_rank": Q, "kv_rank": R, "mask.size": window,
             "scale": (dn + dr) ** -0.5, "rot.base": 10000.0, "rot.dims": dr}
        if i >= own:
            m["kv_from"] = own - 1
        return LayerSpec("latent_attention", tuple(sorted(m.items())), DenseSpec(fd) if i % 2 == 0 else MoESpec(E, K, ff, fs))

    new = HybridConfig(name=f"kisutar-{name}", arch="kisutar", vocab_size=32000, d_model=d,
                       layers=tuple(lat(i) for i in range(L)), max_position=8192, norm_eps=1e-6)
    D = dn + dr
    att = LayerSpec("attention", tuple(sorted({"heads": H, "kv_heads": max(1, H // 4), "dim": D, "vdim": D, "mask.size": window,
                                               "scale": D ** -0.5}.items())), MoESpec(E, K, ff, fs))
    ref = HybridConfig(name=f"dunesun-attn-{name}", arch="dunesun", vocab_size=32000, d_model=d,
                       layers=tuple(att for _ in range(L)), max_position=8192)
    return new, ref


# Bitonex: (name, width, heads, kv heads, head dim, rotating dims, latent unrotated dim, rotated dim, q rank, kv rank,
#           ff, layers); layers take attention, linear attention, latent attention in turn
BITONEX_SIZES = {
    "s": ("d1024", 1024, 8, 2, 128, 64, 96, 32, 384, 128, 2816, 6),
    "m": ("d2048", 2048, 16, 4, 128, 64, 96, 32, 768, 256, 5632, 6),
    "l": ("d4096", 4096, 32, 8, 128, 64, 96, 32, 1536, 256, 11008, 3),
}


def _bitonex_pair(size: str, window: int) -> tuple:
    """Bitonex (the second latent layer reads the first one's pages) and a Dunesun model whose layers
    are attention, Mamba-2 (as many state entries per token as the linear attention layer), attention,
    each with ONE expert of the dense layers' width."""
    name, d, H, G, D, rd, dn, dr, Q, R, ff, L = BITONEX_SIZES[size]
    pair = lambda m: tuple(sorted(m.items()))
    decay = tuple(1.0 - 2.0 ** (-3 - 5 * h / max(1, H - 1)) for h in range(H))
    first_latent = 2

    def layer(i):
        if i % 3 == 0:
            return LayerSpec("attention", pair({"heads": H, "kv_heads": G, "dim": D, "vdim": D, "scale": D ** -0.5,
                                                "rot.dims": rd, "rot.base": 1e6}), DenseSpec(ff))
        if i % 3 == 1:
            return LayerSpec("lightning", pair({"heads": H, "dim": D, "vdim": D, "decay": decay}), DenseSpec(ff))
        m = {"heads": H, "dim": dn, "rot_dim": dr, "vdim": D, "q_rank": Q, "kv_rank": R, "scale": (dn + dr) ** -0.5,
             "rot.base": 1e4, "rot.dims": dr}
        if i > first_latent:
            m["kv_from"] = first_latent
        return LayerSpec("latent_attention", pair(m), DenseSpec(ff))

    new = HybridConfig(name=f"bitonex-{name}", arch="bitonex", vocab_size=32000, d_model=d,
                       layers=tuple(layer(i) for i in range(L)), max_position=8192, norm_eps=1e-6, residual_mult=0.5,
                       logit_softcap=30.0)
    one = MoESpec(1, 1, ff, 0)
    # Bitonex attends to the whole prefix: so does the reference (no window, whatever ``window`` says)
    att = LayerSpec("attention", pair({"heads": H, "kv_heads": G, "dim": D, "vdim": D, "mask.size": 0,
                                       "scale": D ** -0.5}), one)
    ssm = LayerSpec("mamba2", pair({"heads": H * D // 64, "vdim": 64, "state": D, "groups": 1, "conv": 4,
                                    "norm_groups": 1}), one)
    ref = HybridConfig(name=f"dunesun-hybrid-{name}", arch="dunesun", vocab_size=32000, d_model=d,
                       layers=tuple(ssm if i % 3 == 1 else att for i in range(L)), max_position=8192)
    return new, ref


# Levovik: (name, width, heads, kv heads, head dim, rotating dims, recurrent heads, key dim, value dim, low rank,
#           experts, top, expert ff, dense ff, token-input dim, layers)
LEVOVIK_SIZES = {
    "s": ("d1024", 1024, 8, 2, 128, 64, 8, 128, 128, 64, 8, 2, 1024, 2816, 128, 4),
    "m": ("d2048", 2048, 16, 4, 128, 64, 16, 128, 128, 64, 8, 2, 2048, 5632, 256, 4),
    "l": ("d4096", 4096, 32, 8, 128, 64, 32, 128, 128, 128, 8, 2, 3584, 11008, 256, 2),
}


def _levovik_pair(size: str, window: int) -> tuple:
    """Levovik (gated-linear and delta-rule layers in turn, the first feed-forward dense, the others
    routed in four groups) and a Dunesun model with, for every Levovik layer, an attention layer over the
    whole prefix with the same experts and a Mamba-2 layer with as many state entries per token."""
    name, d, H, G, D, rd, Hr, dk, dv, rank, E, K, ff, fd, side, L = LEVOVIK_SIZES[size]
    flat = lambda m: tuple(sorted(m.items()))
    rot = {"rot.dims": rd, "rot.base": 5e5, "rot.scaling.factor": 8.0, "rot.scaling.low": 1.0, "rot.scaling.high": 4.0,
           "rot.scaling.original": 8192}

    def layer(i):
        left = {"heads": H, "kv_heads": G, "dim": D, "vdim": D, "scale": D ** -0.5, **rot}
        if i % 2 == 0:
            kind, right = "parallel_2", {"heads": Hr, "dim": dk, "vdim": dv, "tau": 8.0, "a_rank": rank}
        else:
            kind, right = "parallel", {"heads": Hr, "kv_heads": max(1, Hr // 2), "dim": dk, "vdim": dv, "conv": 4, "a_rank": rank,
                                       "g_rank": rank}
        m = {"left_scale": 1.0, "right_scale": 1.0}
        m.update({"left." + k: v for k, v in left.items()})
        m.update({"right." + k: v for k, v in right.items()})
        mlp = DenseSpec(fd) if i == 0 else MoESpec(E, K, ff, 0, limit=7.0, groups=4, keep_groups=2, route_scale=1.5)
        return LayerSpec(kind, flat(m), mlp)

    new = HybridConfig(name=f"levovik-{name}", arch="levovik", vocab_size=32000, d_model=d,
                       layers=tuple(layer(i) for i in range(L)), max_position=8192, norm_eps=1e-5, logit_scale=0.7,
                       embed_scale=float(d) ** 0.5, side_dim=side)
    att = lambda mlp: LayerSpec("attention", flat({"heads": H, "kv_heads": G, "dim": D, "vdim": D, "mask.size": 0,
                                                   "scale": D ** -0.5}), mlp)
    ssm = LayerSpec("mamba2", flat({"heads": Hr * dv // 64, "vdim": 64, "state": dk, "groups": 1, "conv": 4,
                                    "norm_groups": 1}), None)
    ref_layers = []
    for i in range(L):
        ref_layers += [att(MoESpec(1, 1, fd, 0) if i == 0 else MoESpec(E, K, ff, 0)), ssm]
    ref = HybridConfig(name=f"dunesun-pairs-{name}", arch="dunesun", vocab_size=32000, d_model=d, layers=tuple(ref_layers),
                       max_position=8192)
    return new, ref


PAIRS = {"dunesun": _pair, "kisutar": _kisutar_pair, "bitonex": _bitonex_pair, "levovik": _levovik_pair}


def _measure(cfg, seqs: int, prompt: int, batch: int, steps: int, warmup: int, graphs: bool) -> dict:
    dev = torch.device("cuda:0")
    model = build_model(cfg, device=dev, dtype=torch.bfloat16)
    nseq = max(seqs, batch)
    nb = nseq * ((prompt + steps + warmup + 64) // 16 + 2)
    runner = ModelRunner(model, RunnerConfig(max_num_seqs=nseq, max_model_len=prompt + 256, num_blocks=nb,
                                             use_graphs=graphs))
    blocks = BlockManager(nb, prefix_caching=False, state_slots=runner.num_state_slots)
    g = torch.Generator().manual_seed(0)
    par = SamplingParams(temperature=0.0, ignore_eos=True)

    def fresh(n):
        qs = [Sequence(prompt_ids=torch.randint(3, 30000, (prompt,), generator=g).tolist(), params=par) for _ in range(n)]
        for q in qs:
            assert blocks.allocate(q)
            q.chunk = prompt
        return qs

    def timed(fn, k):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(k):
            fn()
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) / k

    out = {"model": cfg.name, "params_m": round(model.num_local_params() / 1e6, 1)}
    with torch.no_grad():
        qs = fresh(seqs)

        def pf():
            for q in qs:
                q.num_computed = 0
            runner.prefill(qs)

        timed(pf, warmup)
        t = timed(pf, steps)
        out["prefill_ms"] = round(t * 1e3, 3)
        out["prefill_tok_s"] = round(seqs * prompt / t, 1)
        for q in qs:
            blocks.free(q)
        qs = fresh(batch)
        toks = runner.prefill(qs)
        for q, tk in zip(qs, toks):
            q.num_computed, q.chunk, q.prefilled = prompt, 0, True
            q.output_ids.append(int(tk))
        if graphs:
            runner.capture_graphs([runner.bucket_for(batch)])

        def dec():
            for q in qs:
                assert blocks.ensure_slot(q)
            for q, tk in zip(qs, runner.decode(qs)):
                q.output_ids.append(int(tk))

        timed(dec, warmup)
        t = timed(dec, steps)
        out["decode_ms"] = round(t * 1e3, 3)
        out["decode_tok_s"] = round(batch / t, 1)
    del runner, model
    torch.cuda.empty_cache()
    return out


def run(a) -> None:
    """``a``: bench.py's parsed arguments (arch_sizes, arch_prompt, arch_seqs, batch, steps, warmup)."""
    rows = []
    for size in a.arch_sizes.split(","):
        hy, ref = PAIRS[getattr(a, "arch_design", "dunesun")](size, a.arch_window)
        for cfg in ((hy, ref) if a.arch_which == "both" else ((hy,) if a.arch_which == "new" else (ref,))):
            r = _measure(cfg, a.arch_seqs, a.arch_prompt, a.batch, a.steps, a.warmup, not a.no_graphs)
            r["size"] = size
            rows.append(r)
            print(json.dumps(r), flush=True)
    line = {"metric": "arch_compare_tokens_per_s", "unit": "tokens/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
            "dtype": "bf16", "data": "synthetic", "higher_is_better": True,
            "config": {"design": getattr(a, "arch_design", "dunesun"), "prompt": a.arch_prompt, "prefill_seqs": a.arch_seqs, "decode_batch": a.batch,
                       "window": a.arch_window}, "rows": rows}
    print(json.dumps(line), flush=True)
    if a.out:
        with open(a.out, "w") as f:
            f.write(json.dumps(line) + "\n")
