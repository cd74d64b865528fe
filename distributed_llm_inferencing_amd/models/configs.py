"""Architecture registry: every model family the framework serves.

The reference loads arbitrary HF checkpoints through ``AutoModelForCausalLM``
(``worker/app.py:121``); offline we define the architectures ourselves from the
public HF ``config.json`` values and random-init them.

Names accepted by ``get_config`` are case-insensitive and include the HF hub ids
the reference UI would send (``gpt2``, ``meta-llama/Meta-Llama-3-8B`` ...).
"""
from __future__ import annotations

from dataclasses import asdict, dataclass, replace
from typing import Optional


@dataclass(frozen=True)
class LayerSpec:
    """One layer of a hybrid (layer-list) design: which sequence mixer it has, the mixer's
    sizes and constants, and its feed-forward width (0 = none).

    kinds: ``attention`` (windowed softmax attention, values = the un-normed keys, linear
    distance bias, head mixing, output gate), ``hgrn2`` (gated linear recurrence with a
    [dim, vdim] state per head), ``latent_attention`` (keys / values expanded from a cached
    low-rank latent plus one shared rotated key) and ``talk_attention`` (biased q / k / v
    projections, unit-RMS queries and keys, scores mixed across heads before the softmax,
    attention inside blocks of ``chunk`` positions, optionally the cache of layer ``kv_from``)
    and ``gla`` (gated linear attention: a [dim, vdim] state per head with independent keys and
    a per-channel decay sigmoid(z)^(1/tau), z from a low-rank projection of width ``decay_rank``;
    per-head RMS norm, SiLU output gate). ``latent_attention`` options: ``q_rank`` > 0 sends
    the queries through an RMS-normed latent of that width, ``head_gate`` multiplies each
    head's output by one sigmoid gate, ``rot_half`` pairs rotated dimension i with i +
    rot_dims/2 instead of (2i, 2i+1), and ``kv_from`` reads another layer's cached latent.

    feed-forward kinds (``ff_kind``): ``gated_gelu`` (down(gelu(gate) * up)), ``gelu``
    (down(gelu(up))) and ``moe`` (``experts`` gated-SiLU experts of width ``ff`` plus
    ``identity`` pass-through experts, ``top`` per token chosen by softmax score + a learned
    correction and weighted by the un-renormalised score, and a shared expert of width
    ``shared_ff`` behind a per-token sigmoid gate) and ``gated_silu`` (down(silu(gate) * up)).
    A mixture with ``router`` = ``logit_topk`` picks the ``top`` largest biased logits and
    weighs them by the softmax over the chosen ones; ``expert_act`` = ``gelu_erf`` makes the
    experts (and the shared one, then ungated) down(gelu(up)) with the exact GELU."""
    kind: str
    heads: int
    dim: int
    vdim: int
    kv_heads: int = 0
    window: int = 0
    scale: float = 1.0
    rot_dim: int = 0          # latent attention: rotated query/key dims per head
    kv_rank: int = 0          # latent attention: width of the cached latent
    rot_dims: int = 0         # how many of the rot_dim dims actually rotate
    rot_base: float = 10000.0
    ff: int = 0
    chunk: int = 0            # > 0: position i sees j only when i // chunk == j // chunk
    kv_from: int = -1         # >= 0: keys / values are those of that layer (no own projections)
    shift: bool = False       # the mixer reads h + (h_prev - h) * mu (token shift)
    ff_kind: str = "gated_gelu"
    experts: int = 0
    identity: int = 0
    top: int = 0
    shared_ff: int = 0
    router: str = "score"     # "score" (softmax score + correction) | "logit_topk"
    expert_act: str = "silu_mul"   # "silu_mul" (gated) | "gelu_erf" (ungated)
    q_rank: int = 0           # latent attention: width of the query latent (0: none)
    head_gate: bool = False   # latent attention: one sigmoid output gate per head
    rot_half: bool = False    # rotation pairs (i, i + rot_dims/2) instead of (2i, 2i+1)
    tau: float = 1.0          # gla: the decay is sigmoid(z)^(1/tau)
    decay_rank: int = 0       # gla: inner width of the decay's two-step projection
    decays: tuple = ()        # lightning: the state's decay per head
    rot_scaling: tuple = ()   # sink_attention: YaRN (factor, original, fast, slow) or ()
    gate_cap: float = 0.0     # mlstm: soft cap of the gate pre-activations
    left: Optional["LayerSpec"] = None     # parallel: the attention side
    right: Optional["LayerSpec"] = None    # parallel: the recurrent side
    left_scale: float = 1.0
    right_scale: float = 1.0
    router_groups: int = 1    # group_score router: equal groups of neighbouring experts
    router_keep: int = 1      # ... of which the best this many may be chosen from
    router_scale: float = 1.0     # ... and the chosen scores are multiplied by this
    act_limit: float = 0.0    # clamp_swish experts: the clamp

    @property
    def has_state(self) -> bool:
        """The layer keeps something per sequence besides cache rows: a recurrent state, or
        the previous token's mixer input."""
        return self.kind in ("hgrn2", "gla", "lightning", "parallel", "mlstm") or self.shift

    @classmethod
    def from_dict(cls, d: dict) -> "LayerSpec":
        kw = dict(d)
        for side in ("left", "right"):
            if isinstance(kw.get(side), dict):
                kw[side] = cls.from_dict(kw[side])
        for k in ("decays", "rot_scaling"):
            if k in kw:
                kw[k] = tuple(kw[k] or ())
        return cls(**kw)


@dataclass(frozen=True)
class ModelConfig:
    name: str
    arch: str                 # "llama" (llama / mixtral family), "gpt2", or a hybrid
                              # (layer-list) design: "buborax", "pulunex", "risutar",
                              # "lapunex"
    hidden_size: int
    num_layers: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    intermediate_size: int
    vocab_size: int
    max_position: int = 8192
    rope_theta: float = 500000.0
    norm_eps: float = 1e-5
    num_experts: int = 0      # 0 -> dense MLP
    top_k_experts: int = 2
    tie_embeddings: bool = False
    bos_token_id: int = 1
    eos_token_id: int = 2
    # HF ``rope_scaling`` as sorted (key, value) pairs: () = none; rope_type "llama3"
    # (Llama-3.1 / 3.2 checkpoints: low-frequency inv_freq rescaled) or "linear"
    rope_scaling: tuple = ()
    # hybrid designs (arch "buborax"): the layer list, the shared-weight loop
    # (start, stop, times) or (), grouped-norm group count and the residual multiplier
    layer_specs: tuple = ()
    loop: tuple = ()
    norm_groups: int = 1
    residual_mult: float = 1.0
    embed_scale: float = 1.0      # the embedding row is multiplied by this
    logit_scale: float = 1.0      # the LM head's output is multiplied by this
    learned_pos: bool = False     # a learned vector per position is added to the embedding
    scalar_norm: bool = False     # every norm's weight is one number (checkpoint layout)
    # post-norm layers (arch "risutar"): x = LayerNorm(postln_alpha * x + sublayer(x)) with
    # weight and bias, the sublayers reading x itself; False = pre-norm residual layers
    post_norm: bool = False
    postln_alpha: float = 1.0
    # hashed bigram embedding (buckets, mul_prev, mul_cur): row (prev * mul_prev + cur *
    # mul_cur) mod buckets of a second table is added, row ``buckets`` for a first token
    bigram: tuple = ()
    # per-layer token input: width of each layer's slice of a second embedding table
    side_dim: int = 0
    # hyper-connections: this many copies of the residual stream (0: one plain stream); each
    # sublayer reads a learned combination of them and writes back through a learned mix
    streams: int = 0
    # norm weights are stored as offsets from this value (1.0: weights around zero)
    norm_offset: float = 0.0
    # a loop pass starts with x = W_in [x ; x0] + step[pass]; False: passes follow each other
    # with nothing in between
    loop_entry: bool = True

    @property
    def is_hybrid(self) -> bool:
        return bool(self.layer_specs)

    def layer_runs(self) -> list:
        """Execution order of a hybrid design: (layer index, pass number or -1, first of its
        pass). Layers [start, stop) of ``loop`` run ``times`` times in a row; each run owns a
        cache or state of its own."""
        n = len(self.layer_specs)
        if not self.loop:
            return [(i, -1, False) for i in range(n)]
        start, stop, times = self.loop
        runs = [(i, -1, False) for i in range(start)]
        for t in range(times):
            runs += [(i, t, i == start and self.loop_entry) for i in range(start, stop)]
        return runs + [(i, -1, False) for i in range(stop, n)]

    @property
    def has_state(self) -> bool:
        """True when some layer keeps a recurrent state per sequence (state slots; such a
        model's prefix cannot be taken from cached KV blocks alone)."""
        return bool(self.bigram) or any(s.has_state for s in self.layer_specs)

    @property
    def is_moe(self) -> bool:
        return self.num_experts > 0

    @property
    def q_size(self) -> int:
        return self.num_heads * self.head_dim

    @property
    def kv_size(self) -> int:
        return self.num_kv_heads * self.head_dim

    @property
    def qkv_size(self) -> int:
        return self.q_size + 2 * self.kv_size

    def layer_param_count(self) -> int:
        d, f = self.hidden_size, self.intermediate_size
        if self.is_hybrid:
            from .weights import hybrid_layer_shapes
            import math
            tot = sum(math.prod(s) for i in range(len(self.layer_specs))
                      for s in hybrid_layer_shapes(self, i).values())
            return tot // max(1, len(self.layer_specs))
        if self.arch == "gpt2":
            # c_attn (d x 3d + 3d), c_proj (d x d + d), c_fc (d x f + f), mlp c_proj (f x d + d), 2 LN
            return d * 3 * d + 3 * d + d * d + d + d * f + f + f * d + d + 4 * d
        attn = d * self.qkv_size + self.q_size * d
        mlp = 3 * d * f
        if self.is_moe:
            mlp = self.num_experts * mlp + d * self.num_experts
        return attn + mlp + 2 * d

    def embed_param_count(self) -> int:
        n = self.vocab_size * self.hidden_size
        if self.arch == "gpt2":
            n += self.max_position * self.hidden_size
        return n

    def head_param_count(self) -> int:
        """final norm + lm_head (0 extra for tied embeddings)."""
        n = 2 * self.hidden_size if self.arch == "gpt2" else self.hidden_size
        if not self.tie_embeddings:
            n += self.vocab_size * self.hidden_size
        return n

    def param_count(self) -> int:
        return (self.embed_param_count() + self.num_layers * self.layer_param_count()
                + self.head_param_count())

    def kv_bytes_per_token(self, dtype_bytes: int = 2) -> int:
        if self.is_hybrid:
            return sum(self.cache_row_width(i) for i, _, _ in self.layer_runs()) * dtype_bytes
        return 2 * self.num_layers * self.kv_size * dtype_bytes

    def cache_row_width(self, layer: int) -> int:
        """Cached elements per token of one run of hybrid layer ``layer``."""
        s = self.layer_specs[layer]
        if s.kind == "attention":
            return 2 * s.kv_heads * s.dim           # normed keys + raw keys (the values)
        if s.kind == "latent_attention":
            return 0 if s.kv_from >= 0 else s.kv_rank + s.rot_dim
        if s.kind == "talk_attention":
            return 0 if s.kv_from >= 0 else s.kv_heads * (s.dim + s.vdim)
        if s.kind == "parallel":
            return s.left.kv_heads * (s.left.dim + s.left.vdim)
        return 0

    def to_dict(self) -> dict:
        return asdict(self)

    @classmethod
    def from_dict(cls, d: dict) -> "ModelConfig":
        fields = cls.__dataclass_fields__.keys()
        kw = {k: v for k, v in d.items() if k in fields}
        if kw.get("layer_specs"):
            kw["layer_specs"] = tuple(s if isinstance(s, LayerSpec) else LayerSpec.from_dict(s)
                                      for s in kw["layer_specs"])
        if "loop" in kw:
            kw["loop"] = tuple(kw["loop"] or ())
        if "bigram" in kw:
            kw["bigram"] = tuple(kw["bigram"] or ())
        if "rope_scaling" in kw:         # JSON turned the pairs into lists
            kw["rope_scaling"] = tuple(tuple(p) for p in (kw["rope_scaling"] or ()))
        return cls(**kw)


GPT2 = ModelConfig(
    name="gpt2", arch="gpt2", hidden_size=768, num_layers=12, num_heads=12, num_kv_heads=12,
    head_dim=64, intermediate_size=3072, vocab_size=50257, max_position=1024, norm_eps=1e-5,
    tie_embeddings=True, bos_token_id=50256, eos_token_id=50256, rope_theta=0.0)

LLAMA3_8B = ModelConfig(
    name="llama3-8b", arch="llama", hidden_size=4096, num_layers=32, num_heads=32, num_kv_heads=8,
    head_dim=128, intermediate_size=14336, vocab_size=128256, max_position=8192,
    rope_theta=500000.0, norm_eps=1e-5, bos_token_id=128000, eos_token_id=128001)

LLAMA3_70B = replace(LLAMA3_8B, name="llama3-70b", hidden_size=8192, num_layers=80,
                     num_heads=64, num_kv_heads=8, intermediate_size=28672)

MIXTRAL_8X7B = ModelConfig(
    name="mixtral-8x7b", arch="llama", hidden_size=4096, num_layers=32, num_heads=32,
    num_kv_heads=8, head_dim=128, intermediate_size=14336, vocab_size=32000,
    max_position=32768, rope_theta=1e6, norm_eps=1e-5, num_experts=8, top_k_experts=2,
    bos_token_id=1, eos_token_id=2)

# Tiny variants: same code paths, test-sized. Shapes keep the hardware-friendly
# multiples (head_dim 64/128, hidden multiple of 256) so HIP kernels see real layouts.
LLAMA_TINY = ModelConfig(
    name="llama-tiny", arch="llama", hidden_size=256, num_layers=4, num_heads=4, num_kv_heads=2,
    head_dim=64, intermediate_size=512, vocab_size=1024, max_position=2048,
    rope_theta=10000.0, bos_token_id=1, eos_token_id=2)

LLAMA_TINY128 = replace(LLAMA_TINY, name="llama-tiny128", hidden_size=512, num_heads=4,
                        num_kv_heads=2, head_dim=128, intermediate_size=1024)

# 8 layers: one per stage of an 8-rank pipeline test
LLAMA_TINY8 = replace(LLAMA_TINY, name="llama-tiny8", num_layers=8)

MIXTRAL_TINY = replace(LLAMA_TINY, name="mixtral-tiny", num_experts=4, top_k_experts=2,
                       intermediate_size=256)

# 8 experts: one per rank of an 8-rank expert-parallel test
MIXTRAL_TINY8E = replace(MIXTRAL_TINY, name="mixtral-tiny8e", num_experts=8)

GPT2_TINY = replace(GPT2, name="gpt2-tiny", hidden_size=256, num_layers=2, num_heads=4,
                    num_kv_heads=4, head_dim=64, intermediate_size=1024, vocab_size=1024,
                    max_position=256, bos_token_id=1023, eos_token_id=1023)

def hybrid_config(name: str, width: int, vocab: int, layer_specs, loop=(), norm_groups: int = 1,
                  norm_eps: float = 1e-6, residual_mult: float = 1.0, arch: str = "buborax",
                  max_position: int = 1 << 20, **extra) -> ModelConfig:
    """A hybrid (layer-list) ModelConfig; the llama-shaped fields hold the widest layer's sizes
    (they only feed capacity estimates)."""
    specs = tuple(layer_specs)
    heads = max(s.heads for s in specs)
    return ModelConfig(
        name=name, arch=arch, hidden_size=width, num_layers=len(specs), num_heads=heads,
        num_kv_heads=max(max(s.kv_heads, 1) for s in specs), head_dim=max(s.dim for s in specs),
        intermediate_size=max(s.ff for s in specs), vocab_size=vocab, max_position=max_position,
        rope_theta=0.0, norm_eps=norm_eps, bos_token_id=0, eos_token_id=-1,
        layer_specs=specs, loop=tuple(loop), norm_groups=norm_groups,
        residual_mult=residual_mult, **extra)


# Buborax at test size: every mixer kind, a loop over two layers, grouped norm, GQA in the
# attention layer, a layer without feed-forward
BUBORAX_TINY = hybrid_config(
    "buborax-tiny", width=128, vocab=384,
    layer_specs=(
        LayerSpec("attention", heads=4, kv_heads=2, dim=32, vdim=32, window=24, scale=0.2, ff=192),
        LayerSpec("hgrn2", heads=2, dim=32, vdim=48, ff=192),
        LayerSpec("latent_attention", heads=4, dim=32, vdim=24, window=40, scale=0.15,
                  rot_dim=16, kv_rank=48, rot_dims=8, rot_base=5000.0, ff=0),
        LayerSpec("hgrn2", heads=4, dim=16, vdim=32, ff=160)),
    loop=(1, 3, 2), norm_groups=2, norm_eps=1e-6, residual_mult=0.8)


def _pulunex_layer(ff_kind: str, kv_from: int = -1) -> LayerSpec:
    moe = dict(ff=64, experts=6, identity=2, top=2, shared_ff=96) if ff_kind == "moe" else dict(ff=256)
    return LayerSpec("talk_attention", heads=4, kv_heads=2, dim=32, vdim=48, scale=0.125,
                     chunk=40, kv_from=kv_from, shift=True, ff_kind=ff_kind, **moe)


# Pulunex at test size: a dense layer, routed layers with identity experts and a shared
# expert, and a layer that attends another layer's keys and values
PULUNEX_TINY = hybrid_config(
    "pulunex-tiny", width=128, vocab=384, arch="pulunex", max_position=1024,
    layer_specs=(_pulunex_layer("gelu"), _pulunex_layer("moe"), _pulunex_layer("moe", kv_from=1)),
    norm_eps=1e-6, embed_scale=8.0, logit_scale=0.5, learned_pos=True, scalar_norm=True)

def _risutar_moe(**kw) -> dict:
    return dict(ff_kind="moe", router="logit_topk", expert_act="gelu_erf", **kw)


_RISUTAR_LATENT = dict(heads=3, kv_heads=1, dim=32, vdim=40, scale=0.14, rot_dim=16, kv_rank=48,
                       rot_dims=16, rot_base=5000.0, q_rank=40, head_gate=True, rot_half=True,
                       window=1 << 30)

# Risutar at test size: post-norm layers with bias, hashed bigram embedding, per-layer token
# input, gated linear attention, latent attention with a query latent (one layer on another's
# cache), dense and routed feed-forwards, a layer without feed-forward
RISUTAR_TINY = hybrid_config(
    "risutar-tiny", width=128, vocab=384, arch="risutar",
    layer_specs=(
        LayerSpec("latent_attention", **_RISUTAR_LATENT, ff=192, ff_kind="gated_silu"),
        LayerSpec("gla", heads=2, dim=24, vdim=32, tau=8.0, decay_rank=8,
                  **_risutar_moe(ff=48, experts=5, top=2, shared_ff=64)),
        LayerSpec("latent_attention", **_RISUTAR_LATENT, kv_from=0,
                  **_risutar_moe(ff=64, experts=4, top=1)),
        LayerSpec("gla", heads=4, dim=16, vdim=16, tau=4.0, decay_rank=4, ff=0)),
    norm_eps=1e-6, post_norm=True, postln_alpha=2.0, bigram=(251, 31, 5), side_dim=8)

def _lapunex_moe(**kw) -> dict:
    return dict(ff_kind="moe", router="group_score", expert_act="clamp_swish", **kw)


# Lapunex at test size: hyper-connected streams, lightning layers, a parallel attention +
# matrix-memory layer, dense and routed feed-forwards, a loop without an entry projection
LAPUNEX_TINY = hybrid_config(
    "lapunex-tiny", width=128, vocab=384, arch="lapunex",
    layer_specs=(
        LayerSpec("lightning", heads=2, dim=32, vdim=16, decays=(0.7, 0.97), ff=192,
                  ff_kind="gated_silu"),
        LayerSpec("parallel", heads=4, dim=32, vdim=32,
                  left=LayerSpec("sink_attention", heads=4, kv_heads=2, dim=32, vdim=16,
                                 scale=0.2, rot_dims=8, rot_base=1000.0,
                                 rot_scaling=(4.0, 64.0, 16.0, 1.0)),
                  right=LayerSpec("mlstm", heads=2, dim=16, vdim=32, gate_cap=10.0),
                  left_scale=0.7, right_scale=0.6,
                  **_lapunex_moe(ff=48, experts=6, top=2, router_groups=3, router_keep=2,
                                 router_scale=1.2, act_limit=2.0)),
        LayerSpec("lightning", heads=4, dim=16, vdim=32, decays=(0.5, 0.8, 0.9, 0.99), ff=0)),
    loop=(0, 2, 2), norm_eps=1e-5, embed_scale=6.0, streams=2, norm_offset=1.0,
    loop_entry=False)

_REGISTRY = {c.name: c for c in
             (GPT2, LLAMA3_8B, LLAMA3_70B, MIXTRAL_8X7B, LLAMA_TINY, LLAMA_TINY128,
              LLAMA_TINY8, MIXTRAL_TINY, MIXTRAL_TINY8E, GPT2_TINY, BUBORAX_TINY, PULUNEX_TINY,
              RISUTAR_TINY, LAPUNEX_TINY)}

_ALIASES = {
    "openai-community/gpt2": "gpt2",
    "meta-llama/meta-llama-3-8b": "llama3-8b",
    "meta-llama/llama-3.1-8b": "llama3-8b",
    "meta-llama/meta-llama-3-8b-instruct": "llama3-8b",
    "llama-3-8b": "llama3-8b",
    "llama3_8b": "llama3-8b",
    "meta-llama/meta-llama-3-70b": "llama3-70b",
    "llama-3-70b": "llama3-70b",
    "llama3_70b": "llama3-70b",
    "mistralai/mixtral-8x7b-v0.1": "mixtral-8x7b",
    "mixtral": "mixtral-8x7b",
    "mixtral_8x7b": "mixtral-8x7b",
}


def list_models() -> list[str]:
    return sorted(_REGISTRY)


def get_config(name: str, num_layers: Optional[int] = None) -> ModelConfig:
    key = name.strip().lower()
    key = _ALIASES.get(key, key)
    if key not in _REGISTRY:
        raise KeyError(f"unknown model '{name}'; known: {', '.join(list_models())}")
    cfg = _REGISTRY[key]
    if num_layers is not None:
        cfg = replace(cfg, num_layers=num_layers)
    return cfg


def register(cfg: ModelConfig) -> None:
    _REGISTRY[cfg.name] = cfg
