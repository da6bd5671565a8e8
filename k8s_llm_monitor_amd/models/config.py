"""Model architecture presets for the in-process diagnostic LLM.

The reference never runs a model: its ``llm:`` block names a remote OpenAI model
(``internal/config/config.go:141-145``, provider ``openai``, model ``gpt-4``).  BASELINE.json's
configs name the architectures this framework serves instead; their public hyper-parameters are
recorded in SURVEY.md §2.12.  Weights are random-initialised (no checkpoints on the GPU box), so a
preset is all that is needed to build a model of the right shape.
"""
from __future__ import annotations

import dataclasses
from dataclasses import dataclass, field
from typing import Optional


@dataclass(frozen=True)
class ModelConfig:
    name: str
    arch: str  # "llama" (Llama-3 / Mixtral) or "gpt2"
    vocab_size: int
    d_model: int
    n_layers: int
    n_heads: int
    n_kv_heads: int
    head_dim: int
    ffn_dim: int
    max_position: int = 8192
    rope_theta: float = 500000.0
    rope_scaling: Optional[dict] = None
    norm_eps: float = 1e-5
    n_experts: int = 0  # > 0: mixture-of-experts MLP (Mixtral)
    top_k_experts: int = 2
    tie_embeddings: bool = False
    bos_id: int = 128000
    eos_ids: tuple = (128001, 128009)
    extra: dict = field(default_factory=dict)

    @property
    def is_moe(self) -> bool:
        return self.n_experts > 0

    @property
    def q_dim(self) -> int:
        return self.n_heads * self.head_dim

    @property
    def kv_dim(self) -> int:
        return self.n_kv_heads * self.head_dim

    def num_params(self) -> int:
        d, f, L = self.d_model, self.ffn_dim, self.n_layers
        attn = d * (self.q_dim + 2 * self.kv_dim) + self.q_dim * d
        mlp = 3 * d * f * (self.n_experts if self.is_moe else 1) + (d * self.n_experts if self.is_moe else 0)
        if self.arch == "gpt2":
            mlp = 2 * d * f
        emb = self.vocab_size * d * (1 if self.tie_embeddings else 2)
        return L * (attn + mlp) + emb

    def vocab_size_padded(self, tp: int = 1) -> int:
        """Vocab rounded up to a multiple of 64*tp (vocab-parallel shards stay wave-aligned)."""
        m = 64 * tp
        return (self.vocab_size + m - 1) // m * m

    def kv_bytes_per_token(self, dtype_bytes: int = 2) -> int:
        return 2 * self.n_layers * self.kv_dim * dtype_bytes

    def replace(self, **kw) -> "ModelConfig":
        return dataclasses.replace(self, **kw)


PRESETS: dict[str, ModelConfig] = {}


def _reg(c: ModelConfig) -> ModelConfig:
    PRESETS[c.name] = c
    return c


# BASELINE.json config 1: CPU plumbing model.
GPT2_SMALL = _reg(ModelConfig(
    name="gpt2-small", arch="gpt2", vocab_size=50257, d_model=768, n_layers=12, n_heads=12, n_kv_heads=12,
    head_dim=64, ffn_dim=3072, max_position=1024, norm_eps=1e-5, tie_embeddings=True, bos_id=50256,
    eos_ids=(50256,)))

# BASELINE.json configs 2-3: the headline model.
LLAMA3_8B = _reg(ModelConfig(
    name="llama-3-8b", arch="llama", vocab_size=128256, d_model=4096, n_layers=32, n_heads=32, n_kv_heads=8,
    head_dim=128, ffn_dim=14336, max_position=8192, rope_theta=500000.0))

# BASELINE.json config 4: root-cause model, TP=8.
LLAMA3_70B = _reg(ModelConfig(
    name="llama-3-70b", arch="llama", vocab_size=128256, d_model=8192, n_layers=80, n_heads=64, n_kv_heads=8,
    head_dim=128, ffn_dim=28672, max_position=8192, rope_theta=500000.0))

# BASELINE.json config 5: anomaly-detection MoE model.
MIXTRAL_8X7B = _reg(ModelConfig(
    name="mixtral-8x7b", arch="llama", vocab_size=32000, d_model=4096, n_layers=32, n_heads=32, n_kv_heads=8,
    head_dim=128, ffn_dim=14336, max_position=32768, rope_theta=1e6, n_experts=8, top_k_experts=2,
    bos_id=1, eos_ids=(2,)))

# Small shapes with the same structure, for CPU tests and GPU smoke runs.
LLAMA_TINY = _reg(ModelConfig(
    name="llama-tiny", arch="llama", vocab_size=512, d_model=256, n_layers=2, n_heads=4, n_kv_heads=2,
    head_dim=64, ffn_dim=512, max_position=1024, rope_theta=10000.0, bos_id=1, eos_ids=(2,)))

LLAMA_TINY128 = _reg(ModelConfig(
    name="llama-tiny-d128", arch="llama", vocab_size=1024, d_model=512, n_layers=2, n_heads=8, n_kv_heads=2,
    head_dim=128, ffn_dim=1024, max_position=2048, rope_theta=500000.0, bos_id=1, eos_ids=(2,)))

MIXTRAL_TINY_D128 = _reg(ModelConfig(  # head_dim 128: the HIP attention kernels' shape, for GPU tests
    name="mixtral-tiny-d128", arch="llama", vocab_size=1024, d_model=512, n_layers=2, n_heads=8, n_kv_heads=2,
    head_dim=128, ffn_dim=1024, max_position=2048, rope_theta=1000000.0, n_experts=4, top_k_experts=2,
    bos_id=1, eos_ids=(2,)))

MIXTRAL_TINY = _reg(ModelConfig(
    name="mixtral-tiny", arch="llama", vocab_size=512, d_model=256, n_layers=2, n_heads=4, n_kv_heads=2,
    head_dim=64, ffn_dim=256, max_position=1024, rope_theta=10000.0, n_experts=4, top_k_experts=2,
    bos_id=1, eos_ids=(2,)))

MIXTRAL_TINY_E8 = _reg(ModelConfig(  # 8 query heads, 8 experts: TP / EP 8 parity tests on CPU
    name="mixtral-tiny-e8", arch="llama", vocab_size=512, d_model=256, n_layers=2, n_heads=8, n_kv_heads=2,
    head_dim=32, ffn_dim=256, max_position=1024, rope_theta=10000.0, n_experts=8, top_k_experts=2,
    bos_id=1, eos_ids=(2,)))

GPT2_TINY = _reg(ModelConfig(
    name="gpt2-tiny", arch="gpt2", vocab_size=512, d_model=128, n_layers=2, n_heads=2, n_kv_heads=2,
    head_dim=64, ffn_dim=512, max_position=512, tie_embeddings=True, bos_id=0, eos_ids=(0,)))

_ALIASES = {
    "gpt2": "gpt2-small", "gpt-2": "gpt2-small", "llama3-8b": "llama-3-8b", "meta-llama-3-8b": "llama-3-8b",
    "llama-3.1-8b": "llama-3-8b", "llama3-70b": "llama-3-70b", "mixtral": "mixtral-8x7b",
    "mixtral-8x7b-v0.1": "mixtral-8x7b",
}


def get_config(name: str) -> ModelConfig:
    key = name.strip().lower()
    key = _ALIASES.get(key, key)
    if key not in PRESETS:
        raise KeyError(f"unknown model preset {name!r}; known: {sorted(PRESETS)}")
    return PRESETS[key]


# ----------------------------------------------------------------------------- layer-list models

@dataclass(frozen=True)
class MoESpec:
    """Routed feed-forward: ``experts`` experts of width ``ff`` of which each token takes ``top``,
    plus an optional shared expert of width ``shared_ff`` (0 = none).  How the router weighs the
    chosen experts, the experts' form and the shared expert's gate belong to the design
    (DESIGN_TRAITS ``ffn``).  Designs whose experts clamp their pre-activations read ``limit``;
    designs whose router chooses within the best of ``groups`` equal groups of neighbouring experts
    read ``groups`` / ``keep_groups`` (1 group: no restriction) and scale the chosen weights by
    ``route_scale``."""

    experts: int
    top: int
    ff: int
    shared_ff: int = 0
    limit: float = 0.0
    groups: int = 1
    keep_groups: int = 1
    route_scale: float = 1.0


@dataclass(frozen=True)
class DenseSpec:
    """Dense feed-forward of width ``ff`` (up-projection, activation, down-projection; gated in
    designs whose ``ffn`` trait says so)."""

    ff: int


@dataclass(frozen=True)
class LayerSpec:
    """One decoder layer of a :class:`HybridConfig`: a token mixer (``kind`` names an entry of
    models/hybrid.py MIXERS, ``mixer`` holds that mixer's sizes and constants as sorted
    (key, value) pairs so the spec stays hashable) and an optional feed-forward."""

    kind: str
    mixer: tuple
    mlp: Optional[object] = None  # MoESpec, DenseSpec or None

    @property
    def m(self) -> dict:
        return dict(self.mixer)

    def sub(self, prefix: str, kind: str) -> "LayerSpec":
        """The spec of a mixer nested in this one: the constants under ``prefix.`` (a composite
        mixer's ``left`` / ``right``), without the prefix, as a layer of ``kind``."""
        n = len(prefix) + 1
        return LayerSpec(kind, tuple((k[n:], v) for k, v in self.mixer if k.startswith(prefix + ".")))


@dataclass(frozen=True)
class HybridConfig:
    """A decoder given as an explicit list of layers (attention and recurrent mixers may
    alternate in any order), optionally with a span of layers that runs several times with shared
    weights.  ``arch`` selects the model class (models/registry.py)."""

    name: str
    arch: str
    vocab_size: int
    d_model: int
    layers: tuple  # of LayerSpec
    max_position: int = 2048
    norm_eps: float = 1e-5
    logit_scale: float = 1.0
    residual_mult: float = 1.0  # every sublayer's result is scaled by this before it joins the stream
    logit_softcap: float = 0.0  # > 0: logits <- cap * tanh(logits / cap)
    embed_scale: float = 1.0  # the token embedding is multiplied by this
    side_dim: int = 0  # > 0: every layer also reads its own slice of a second token table (``side.embed``)
    loop: Optional[tuple] = None  # (start, stop, times): layers start .. stop-1 run `times` times
    bos_id: int = 1
    eos_ids: tuple = (2,)
    extra: dict = field(default_factory=dict)

    @property
    def n_layers(self) -> int:
        return len(self.layers)

    @property
    def is_moe(self) -> bool:
        return any(isinstance(s.mlp, MoESpec) for s in self.layers)

    @property
    def traits(self) -> dict:
        return DESIGN_TRAITS[self.arch]

    def runs(self) -> list:
        """Execution order as (layer index, pass number or -1, first layer of its pass)."""
        n = len(self.layers)
        if not self.loop:
            return [(i, -1, False) for i in range(n)]
        a, b, times = self.loop
        out = [(i, -1, False) for i in range(a)]
        for t in range(times):
            out += [(i, t, i == a) for i in range(a, b)]
        return out + [(i, -1, False) for i in range(b, n)]

    def replace(self, **kw) -> "HybridConfig":
        return dataclasses.replace(self, **kw)


# What a layer-list design fixes for all of its models (sizes and per-layer constants come from
# the model's config.json):
#   block          "parallel": one norm feeds mixer and feed-forward, both added to the stream;
#                  "sequential": x += mixer(norm1(x)), then x += ff(norm2(x))
#   one_plus_norm  RMSNorm weights are stored around zero and applied as 1 + w
#   learned_pos    a table of absolute positions is added to the token embedding
#   token_shift    what a mixer reads is moved towards the previous token's (per-channel weights
#                  ``l<i>.shift``); the previous token's rows are per-sequence state
#   depth_average  the input of layer i + 1 is a learned combination (``l<i>.dwa``) of the embedding
#                  output and the results of layers 0 .. i
#   ffn            the feed-forward family: "swiglu_topk" (gated experts, biased router, softmax over
#                  the chosen logits, sigmoid-gated shared expert), "plain_softmax" (ungated
#                  experts with erf-GELU, softmax over all logits and the chosen probabilities
#                  used as they are, ungated shared expert, dense layers with xIELU) or "gated_gelu"
#                  (dense layers down(gelu_tanh(gate h) * up h))
#   max_position   positions a model accepts when its config.json does not say
# and, where present (absent = the first value):
#   scalar_norm    False / True: a block or final norm's weight is one number for all coordinates
#   gated_residual False / True: every sublayer's result is multiplied elementwise by
#                  sigmoid(W h + b) of the sublayer's input (``l<i>.rg1`` / ``.rg2`` and ``.b``)
#   mixers         config ``type`` -> entry of models/hybrid.py MIXERS where the design's mixer of that
#                  name is not the entry of the same name
#   latent         what the design fixes for latent attention: ``rotary`` "half" (entry i turns with
#                  i + n/2) / "pairs" (2i with 2i + 1), ``sink`` True (a learned logit per head in the
#                  softmax denominator) / False
#   norm           "rms" / "layer": block and final norms are RMSNorms, or layer norms with a weight
#                  and no bias ((x - mean) / sqrt(variance + eps) * w)
#   composite      config ``type`` -> {"left": (MIXERS entry, options), "right": (MIXERS entry, options)}:
#                  a layer of that type runs two mixers side by side on the same normed input (their
#                  constants under ``mixer.left`` / ``mixer.right``, tensors under ``mix.left.`` /
#                  ``mix.right.``) and adds ``left_scale * left + right_scale * right``.  The options
#                  are what the design fixes for that mixer (models/hybrid.py documents each mixer's)
DESIGN_TRAITS = {
    "dunesun": dict(block="parallel", one_plus_norm=True, learned_pos=True, token_shift=False,
                    depth_average=False, ffn="swiglu_topk", max_position=2048),
    "kisutar": dict(block="sequential", one_plus_norm=False, learned_pos=False, token_shift=True,
                    depth_average=True, ffn="plain_softmax", max_position=1 << 17),
    "bitonex": dict(block="sequential", one_plus_norm=False, learned_pos=False, token_shift=False,
                    depth_average=False, ffn="gated_gelu", max_position=1 << 17, scalar_norm=True,
                    gated_residual=True, mixers={"attention": "rotary_attention"},
                    latent=dict(rotary="pairs", sink=False)),
    "levovik": dict(block="sequential", one_plus_norm=False, learned_pos=False, token_shift=False,
                    depth_average=False, ffn="relu_glu_grouped", max_position=1 << 17, norm="layer",
                    composite={
                        "parallel": dict(
                            left=("rotary_attention", dict(rotary="half", qk_norm="after", sink=True, temp=False, gate=False)),
                            right=("gated_delta", {})),
                        "parallel_2": dict(
                            left=("rotary_attention", dict(rotary="pairs", qk_norm="before", values="keys", temp=False,
                                                           gate=False)),
                            right=("gated_linear", {}))}),
}


def _flat(d: dict, prefix: str = "") -> list:
    out = []
    for k, v in d.items():
        if isinstance(v, dict):
            out += _flat(v, prefix + k + ".")
        else:  # a list (one number per head) becomes a tuple: the spec stays hashable
            out.append((prefix + k, tuple(v) if isinstance(v, list) else v))
    return out


def hybrid_config_from_dict(c: dict, name: Optional[str] = None) -> HybridConfig:
    """A :class:`HybridConfig` from a layer-list ``config.json``: ``architecture``, ``vocab``,
    ``width``, ``max_positions``, ``norm.eps``, ``logit_scale``, ``logit_softcap``, ``residual_mult``,
    ``embedding.scale``, ``token_side.dim``, ``loop`` {start, stop, times} and
    ``layers`` [{type, mixer {...}, mlp {kind: moe, expert.ff, expert.limit, router.experts, router.top,
    router.scale, router.groups {count, keep}, shared.ff} | {kind: dense, ff} | null}].  Nested mixer keys are flattened with dots (``mask.size``)."""
    arch = str(c["architecture"]).lower()
    if arch not in DESIGN_TRAITS:
        raise ValueError(f"unknown architecture {c['architecture']!r} (known: {sorted(DESIGN_TRAITS)})")
    layers = []
    for spec in c["layers"]:
        ml = spec.get("mlp")
        moe = None
        if ml is not None:
            kind = ml.get("kind", "moe")
            if kind == "moe":
                sh = ml.get("shared")
                rt = ml["router"]
                gr = rt.get("groups") or {}
                moe = MoESpec(experts=int(rt["experts"]), top=int(rt["top"]),
                              ff=int(ml["expert"]["ff"]), shared_ff=int(sh["ff"]) if sh else 0,
                              limit=float(ml["expert"].get("limit", 0.0)), groups=int(gr.get("count", 1)),
                              keep_groups=int(gr.get("keep", gr.get("count", 1))), route_scale=float(rt.get("scale", 1.0)))
            elif kind == "dense":
                moe = DenseSpec(ff=int(ml["ff"]))
            else:
                raise ValueError(f"unsupported feed-forward kind {kind!r}")
        layers.append(LayerSpec(kind=spec["type"], mixer=tuple(sorted(_flat(spec.get("mixer") or {}))), mlp=moe))
    lp = c.get("loop")
    loop = (int(lp["start"]), int(lp["stop"]), int(lp["times"])) if lp else None
    if loop and not (0 <= loop[0] < loop[1] <= len(layers) and loop[2] >= 1):
        raise ValueError(f"bad loop {lp!r} for {len(layers)} layers")
    V = int(c["vocab"])
    return HybridConfig(name=name or arch, arch=arch, vocab_size=V, d_model=int(c["width"]),
                        layers=tuple(layers),
                        max_position=int(c.get("max_positions", DESIGN_TRAITS[arch]["max_position"])),
                        norm_eps=float(c["norm"]["eps"]), logit_scale=float(c.get("logit_scale", 1.0)),
                        residual_mult=float(c.get("residual_mult", 1.0)),
                        logit_softcap=float(c.get("logit_softcap") or 0.0), loop=loop,
                        embed_scale=float((c.get("embedding") or {}).get("scale", 1.0)),
                        side_dim=int((c.get("token_side") or {}).get("dim", 0)),
                        bos_id=int(c.get("bos_id", min(1, V - 1))), eos_ids=tuple(c.get("eos_ids", (min(2, V - 1),))))


def hybrid_config_to_dict(c: HybridConfig) -> dict:
    """The inverse of :func:`hybrid_config_from_dict`."""
    def nest(pairs):
        out: dict = {}
        for k, v in pairs:
            cur = out
            parts = k.split(".")
            for p in parts[:-1]:
                cur = cur.setdefault(p, {})
            cur[parts[-1]] = list(v) if isinstance(v, tuple) else v
        return out

    layers = []
    for s in c.layers:
        ml = None
        if isinstance(s.mlp, DenseSpec):
            ml = {"kind": "dense", "ff": s.mlp.ff}
        elif s.mlp is not None:
            ml = {"kind": "moe", "expert": {"ff": s.mlp.ff}, "router": {"experts": s.mlp.experts, "top": s.mlp.top},
                  "shared": {"ff": s.mlp.shared_ff} if s.mlp.shared_ff else None}
            if s.mlp.limit:
                ml["expert"]["limit"] = s.mlp.limit
            if s.mlp.groups > 1:
                ml["router"]["groups"] = {"count": s.mlp.groups, "keep": s.mlp.keep_groups}
            if s.mlp.route_scale != 1.0:
                ml["router"]["scale"] = s.mlp.route_scale
        layers.append({"type": s.kind, "mixer": nest(s.mixer), "mlp": ml})
    d = {"architecture": c.arch.capitalize(), "vocab": c.vocab_size, "width": c.d_model, "layers": layers,
         "max_positions": c.max_position, "norm": {"eps": c.norm_eps}, "logit_scale": c.logit_scale,
         "bos_id": c.bos_id, "eos_ids": list(c.eos_ids)}
    if c.residual_mult != 1.0:
        d["residual_mult"] = c.residual_mult
    if c.logit_softcap:
        d["logit_softcap"] = c.logit_softcap
    if c.embed_scale != 1.0:
        d["embedding"] = {"scale": c.embed_scale}
    if c.side_dim:
        d["token_side"] = {"dim": c.side_dim}
    if c.loop:
        d["loop"] = {"start": c.loop[0], "stop": c.loop[1], "times": c.loop[2]}
    return d


def _attn(heads, kv_heads, dim, vdim, window, scale):
    return LayerSpec("attention", tuple(sorted({"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
                                                "mask.size": window, "scale": scale}.items())))


def _ssm(heads, vdim, state, groups, conv, norm_groups):
    return LayerSpec("mamba2", tuple(sorted({"heads": heads, "vdim": vdim, "state": state, "groups": groups,
                                             "conv": conv, "norm_groups": norm_groups}.items())))


def _latent(heads, dim, rot_dim, vdim, q_rank, kv_rank, window, scale, base=10000.0, kv_from=None):
    m = {"heads": heads, "dim": dim, "rot_dim": rot_dim, "vdim": vdim, "q_rank": q_rank, "kv_rank": kv_rank,
         "mask.size": window, "scale": scale, "rot.base": base, "rot.dims": rot_dim}
    if kv_from is not None:
        m["kv_from"] = kv_from
    return LayerSpec("latent_attention", tuple(sorted(m.items())))


def _rot_attn(heads, kv_heads, dim, vdim, rot_dims, base, scale):
    return LayerSpec("attention", tuple(sorted({"heads": heads, "kv_heads": kv_heads, "dim": dim, "vdim": vdim,
                                                "rot.dims": rot_dims, "rot.base": base, "scale": scale}.items())))


def _lightning(heads, dim, vdim, decay):
    return LayerSpec("lightning", tuple(sorted({"heads": heads, "dim": dim, "vdim": vdim, "decay": tuple(decay)}.items())))


def _with_mlp(s: LayerSpec, m) -> LayerSpec:
    return dataclasses.replace(s, mlp=m)


# Small Dunesun-design model for CPU tests and GPU smoke runs (random weights): recurrent and
# windowed-attention layers interleaved, layers 1..2 looped twice.
DUNESUN_TINY = _reg(HybridConfig(
    name="dunesun-tiny", arch="dunesun", vocab_size=512, d_model=128,
    layers=(_with_mlp(_ssm(4, 32, 16, 2, 4, 2), MoESpec(4, 2, 64, 96)),
            _with_mlp(_attn(4, 2, 32, 16, 24, 0.2), MoESpec(4, 2, 64, 0)),
            _with_mlp(_ssm(2, 64, 32, 1, 3, 1), None),
            _with_mlp(_attn(2, 2, 64, 64, 8, 0.125), MoESpec(6, 3, 32, 64))),
    max_position=1024, loop=(1, 3, 2), logit_scale=1.5, bos_id=1, eos_ids=(2,)))

# Small Kisutar-design model for CPU tests and GPU smoke runs (random weights): latent attention in
# every layer, the last two reading layer 1's compressed keys, dense / routed / no feed-forward.
KISUTAR_TINY = _reg(HybridConfig(
    name="kisutar-tiny", arch="kisutar", vocab_size=384, d_model=96,
    layers=(_with_mlp(_latent(4, 24, 8, 16, 40, 32, 20, 0.18), DenseSpec(160)),
            _with_mlp(_latent(2, 32, 16, 24, 48, 40, 12, 0.15), MoESpec(6, 2, 48, 64)),
            _with_mlp(_latent(4, 16, 16, 32, 32, 40, 28, 0.2, kv_from=1), None),
            _with_mlp(_latent(2, 24, 16, 24, 24, 40, 9, 0.17, kv_from=1), MoESpec(4, 3, 32, 0))),
    max_position=4096, norm_eps=1e-6, bos_id=1, eos_ids=(2,)))

# Small Bitonex-design model for CPU tests and GPU smoke runs (random weights): rotary grouped-query
# attention, fixed-decay linear attention and latent attention, the last layer reading layer 1's latent.
BITONEX_TINY = _reg(HybridConfig(
    name="bitonex-tiny", arch="bitonex", vocab_size=320, d_model=80,
    layers=(_with_mlp(_rot_attn(4, 2, 24, 16, 12, 10000.0, 0.21), DenseSpec(112)),
            _with_mlp(_latent(3, 16, 8, 24, 40, 24, 0, 0.2, base=5000.0), DenseSpec(96)),
            _with_mlp(_lightning(2, 24, 40, (0.9, 0.97)), None),
            _with_mlp(_latent(2, 24, 8, 16, 32, 24, 0, 0.18, base=5000.0, kv_from=1), DenseSpec(64))),
    max_position=4096, norm_eps=1e-6, residual_mult=0.4, logit_softcap=20.0, bos_id=1, eos_ids=(2,)))


def _pair(kind, left: dict, right: dict, left_scale: float, right_scale: float) -> LayerSpec:
    """A layer of two mixers side by side (DESIGN_TRAITS ``composite``): nested constants flattened with dots."""
    m = {"left_scale": left_scale, "right_scale": right_scale}
    m.update(_flat({"left": left, "right": right}))
    return LayerSpec(kind, tuple(sorted(m.items())))


def _rot(dims, base, factor, original, low=1.0, high=4.0) -> dict:
    return {"dims": dims, "base": base, "scaling": {"factor": factor, "low": low, "high": high, "original": original}}


# Small Levovik-design model for CPU tests and GPU smoke runs (random weights): softmax attention beside
# gated linear attention (``parallel_2``) and beside the gated delta rule (``parallel``), a dense, two
# routed and one absent feed-forward, a per-layer token input.
LEVOVIK_TINY = _reg(HybridConfig(
    name="levovik-tiny", arch="levovik", vocab_size=352, d_model=96,
    layers=(_with_mlp(_pair("parallel_2", dict(heads=4, kv_heads=2, dim=16, scale=0.25, rot=_rot(8, 10000.0, 4.0, 64)),
                            dict(heads=2, dim=24, vdim=16, tau=8.0, a_rank=8), 0.7, 1.2), DenseSpec(144)),
            _with_mlp(_pair("parallel", dict(heads=3, kv_heads=1, dim=32, vdim=24, scale=0.18, rot=_rot(16, 50000.0, 8.0, 64)),
                            dict(heads=4, kv_heads=2, dim=16, vdim=24, conv=3, a_rank=12, g_rank=8), 0.9, 0.6),
                      MoESpec(8, 2, 40, limit=1.25, groups=4, keep_groups=2, route_scale=1.5)),
            _with_mlp(_pair("parallel_2", dict(heads=2, kv_heads=2, dim=32, scale=0.2, rot=_rot(32, 10000.0, 2.0, 128)),
                            dict(heads=3, dim=8, vdim=32, tau=4.0), 1.0, 1.0), None),
            _with_mlp(_pair("parallel", dict(heads=4, kv_heads=4, dim=16, vdim=16, scale=0.25, rot=_rot(4, 1000.0, 4.0, 32)),
                            dict(heads=2, kv_heads=2, dim=24, vdim=8, conv=4), 0.8, 0.5),
                      MoESpec(6, 3, 24, limit=2.0, groups=2, keep_groups=1, route_scale=2.5))),
    max_position=1 << 17, norm_eps=1e-5, logit_scale=0.6, embed_scale=9.0, side_dim=12, bos_id=1, eos_ids=(2,)))
