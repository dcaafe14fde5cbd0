"""Model hyper-parameters for the MI355X decode path.

Mirrors the public surface of the reference ``Config`` dataclass
(/root/reference/lit_gpt/config.py:16-144): the same field names and defaults, the same derived
fields computed in ``__post_init__`` (``head_size``, ``padded_vocab_size``, ``n_query_groups``,
``intermediate_size``, ``rope_n_elem``; reference :63-89), ``from_name`` / ``from_json`` /
``from_checkpoint`` (:91-130) and the ``mlp_class`` / ``norm_class`` indirection (:132-144).

Only the model families this build targets are registered ("fields + the 4 target
configs"): GPT-NeoX/pythia (CPU plumbing config), Llama-2 7B/13B/70B (+chat), Mixtral-8x7B, plus
the tiny configs the test-suite uses.
"""

from __future__ import annotations

import json
import math
from dataclasses import dataclass, field
from pathlib import Path
from typing import Any, Dict, List, Literal, Optional, Type, Union

from lit_gpt.utils import find_multiple


@dataclass
class Config:
    name: str = ""
    hf_config: dict = field(default_factory=dict)
    block_size: int = 4096
    vocab_size: int = 50254
    padding_multiple: int = 512
    padded_vocab_size: Optional[int] = None
    n_layer: int = 16
    n_head: int = 32
    n_embd: int = 4096
    rotary_percentage: float = 0.25
    parallel_residual: bool = True
    bias: bool = True
    lm_head_bias: bool = False
    # MHA: n_query_groups == n_head; MQA: 1; GQA: in between (reference :31-50)
    n_query_groups: Optional[int] = None
    shared_attention_norm: bool = False
    _norm_class: Literal["LayerNorm", "RMSNorm"] = "LayerNorm"
    norm_eps: float = 1e-5
    _mlp_class: Literal["GptNeoxMLP", "LLaMAMLP", "LLaMAMoE"] = "GptNeoxMLP"
    gelu_approximate: str = "none"
    intermediate_size: Optional[int] = None
    rope_condense_ratio: int = 1
    rope_base: int = 10000
    n_expert: int = 0
    n_expert_per_token: int = 0

    def __post_init__(self) -> None:
        if not self.name:
            self.name = self.hf_config.get("name", self.name)
        assert self.n_embd % self.n_head == 0
        self.head_size = self.n_embd // self.n_head
        if self.padded_vocab_size is None:
            self.padded_vocab_size = find_multiple(self.vocab_size, self.padding_multiple)
        else:
            self.vocab_size = min(self.vocab_size, self.padded_vocab_size)
        if self.n_query_groups is None:
            self.n_query_groups = self.n_head
        else:
            assert self.n_head % self.n_query_groups == 0
        if self.intermediate_size is None:
            if self._mlp_class == "LLaMAMLP":
                raise ValueError("The config needs to set the `intermediate_size`")
            self.intermediate_size = 4 * self.n_embd
        self.rope_n_elem = int(self.rotary_percentage * self.head_size)

    @classmethod
    def from_name(cls, name: str, **kwargs: Any) -> "Config":
        conf = name_to_config.get(name)
        if conf is None:
            conf = next((c for c in configs if c["hf_config"].get("name") == name), None)
            if conf is None:
                raise ValueError(f"{name!r} is not a supported config name")
        conf = dict(conf)
        if "condense_ratio" in kwargs:  # legacy spelling
            kwargs["rope_condense_ratio"] = kwargs.pop("condense_ratio")
        conf.update(kwargs)
        return cls(**conf)

    @classmethod
    def from_json(cls, path: Union[str, Path], **kwargs: Any) -> "Config":
        with open(path, encoding="utf-8") as fp:
            loaded = json.load(fp)
        for d in (loaded, kwargs):
            if "condense_ratio" in d:
                d["rope_condense_ratio"] = d.pop("condense_ratio")
        if "org" in loaded:
            loaded["hf_config"] = {"name": loaded["name"], "org": loaded.pop("org")}
        if "org" in kwargs:
            kwargs["hf_config"] = {"name": kwargs.get("name", loaded["name"]), "org": kwargs.pop("org")}
        loaded.update(kwargs)
        return cls(**loaded)

    @classmethod
    def from_checkpoint(cls, path: Path, **kwargs: Any) -> "Config":
        path = Path(path)
        if (path / "lit_config.json").is_file():
            return cls.from_json(path / "lit_config.json", **kwargs)
        if path.name in name_to_config:
            return cls.from_name(path.name, **kwargs)
        raise FileNotFoundError(f"For {str(path)!r} neither 'lit_config.json' nor matching config exists.")

    @property
    def mlp_class(self) -> Type:
        import lit_gpt.model

        return getattr(lit_gpt.model, self._mlp_class)

    @property
    def norm_class(self) -> Type:
        if self._norm_class == "RMSNorm":
            from lit_gpt.rmsnorm import RMSNorm

            return RMSNorm
        import lit_gpt.model

        return getattr(lit_gpt.model, self._norm_class)


# --------------------------------------------------------------------------------------------
# Registry. Values follow the HF configs the reference cites (pythia: config.py:200-260,
# Llama-2: :726-776, Mixtral: :1290-1307).
# --------------------------------------------------------------------------------------------
configs: List[Dict[str, Any]] = []


def _register(name: str, org: str, **kw: Any) -> None:
    configs.append(dict(name=name, hf_config=dict(org=org, name=name), **kw))


for _name, _block, _layers, _embd, _heads in (
    ("pythia-14m", 512, 6, 128, 4),
    ("pythia-31m", 1024, 6, 256, 8),
    ("pythia-70m", 2048, 6, 512, 8),
    ("pythia-160m", 2048, 12, 768, 12),
    ("pythia-410m", 2048, 24, 1024, 16),
    ("pythia-1b", 2048, 16, 2048, 8),
):
    _register(_name, "EleutherAI", block_size=_block, n_layer=_layers, n_embd=_embd, n_head=_heads,
              padding_multiple=128)

_LLAMA2 = dict(vocab_size=32000, padding_multiple=64, rotary_percentage=1.0, parallel_residual=False,
               bias=False, _norm_class="RMSNorm", _mlp_class="LLaMAMLP")
for _kind in ("", "-chat"):
    _register(f"Llama-2-7b{_kind}-hf", "meta-llama", n_layer=32, intermediate_size=11008, **_LLAMA2)
    _register(f"Llama-2-13b{_kind}-hf", "meta-llama", n_layer=40, n_head=40, n_embd=5120,
              intermediate_size=13824, **_LLAMA2)
    _register(f"Llama-2-70b{_kind}-hf", "meta-llama", n_layer=80, n_head=64, n_embd=8192, n_query_groups=8,
              intermediate_size=28672, **_LLAMA2)

for _kind in ("", "Instruct-"):
    _register(f"Mixtral-8x7B-{_kind}v0.1", "mistralai", padded_vocab_size=32000, block_size=32768, n_layer=32,
              n_query_groups=8, rotary_percentage=1.0, parallel_residual=False, bias=False,
              _norm_class="RMSNorm", norm_eps=1e-05, _mlp_class="LLaMAMoE", intermediate_size=14336,
              rope_base=1000000, n_expert=8, n_expert_per_token=2)

name_to_config: Dict[str, Dict[str, Any]] = {c["name"]: c for c in configs}


# --------------------------------------------------------------------------------------------
# Layered models: a ``config.json`` that lists its layers one by one (each with its own sequence mixer and
# feed-forward) instead of repeating one block. ``architecture`` names the design; the registry below maps it to
# the model class, and ``load_config`` picks the configuration class for a checkpoint folder.
# --------------------------------------------------------------------------------------------
@dataclass
class RotarySpec:
    dims: int = 0
    base: float = 10000.0
    # band-wise rescaling of the frequencies for contexts longer than the ``original`` one: wavelengths above
    # original / low are slowed down by ``factor``, those below original / high are kept, the band between blends
    # the two linearly in original / wavelength. Keys: factor, low, high, original.
    scaling: Optional[Dict[str, float]] = None

    def inv_freq(self) -> List[float]:
        """f_i = base^(-2i / dims), i < dims / 2, rescaled band by band when ``scaling`` is set; in double precision
        (rounded once to fp32 by the caller)."""
        out = [float(self.base) ** (-2.0 * i / self.dims) for i in range(self.dims // 2)]
        if self.scaling:
            factor, low, high, orig = (float(self.scaling[k]) for k in ("factor", "low", "high", "original"))
            for i, f in enumerate(out):
                wavelength = 2.0 * math.pi / f
                if wavelength > orig / low:
                    out[i] = f / factor
                elif wavelength >= orig / high:
                    mix = (orig / wavelength - low) / (high - low)
                    out[i] = (1.0 - mix) * f / factor + mix * f
        return out


@dataclass
class MixerSpec:
    kind: str  # one of MIXER_KINDS
    heads: int
    dim: int  # per-head query / key size (latent attention: the unrotated part; attention: of one map)
    vdim: int
    rot: RotarySpec
    decay: Optional[List[float]] = None  # retention: one fixed decay per head
    kv_rank: int = 0  # latent attention: size of the cached latent
    rot_dim: int = 0  # latent attention: rotated query / key part (one key part shared by the heads)
    scale: float = 1.0  # attention score scale
    kv_heads: int = 0  # attention: key / value heads (query head h reads head h // (heads // kv_heads))
    diff: float = 0.0  # differential attention: the constant of lambda; the output is scaled by 1 - diff
    softcap: float = 0.0  # attention: scores pass cap * tanh(s / cap) (0: not)
    mask_size: int = 0  # attention: a query sees keys of its own aligned chunk of this many positions (0: all before it)
    kv_from: Optional[int] = None  # attention: the layer whose cached keys and values this layer reads
    conv: int = 0  # mamba2: taps of the short convolution
    groups: int = 0  # mamba2: groups of heads that share B and C
    norm_groups: int = 1  # mamba2: equal parts of the gated output, each divided by its own root mean square
    state: int = 0  # mamba2: state size N
    q_temp_coef: float = 0.0  # sink attention: the query is multiplied by 1 + coef * ln(floor((p + 1) / every) + 1)
    q_temp_every: int = 0  # (0: no query temperature)
    decay_rank: int = 0  # channel_delta: inner sizes of the low-rank decay and gate maps (a checkpoint's tensors give
    gate_rank: int = 0  # them; these only size random weights, 0: 16)
    left: Optional["MixerSpec"] = None  # parallel: two mixers that read the same input ...
    right: Optional["MixerSpec"] = None
    left_scale: float = 1.0  # ... and are summed with these factors
    right_scale: float = 1.0
    branch_norm: bool = False  # parallel: each branch's output is RMS-normed over the width (weights "left.out" /
    # "right.out") before the weighted sum
    # one-map softmax attention ("sink_attention" and its relatives):
    qk_norm: str = "unit"  # "none" | "unit" (divided by the root mean square) | "weight" (and times "q.norm" / "k.norm")
    sink_kind: str = "learned"  # "none" | "learned" (a scalar per head, "sink") | "one" (a sink of score 0: 1 + sum exp)
    values: str = "own"  # "own" (a value projection) | "keys" (the keys as projected, before their norm)
    head_gate: bool = False  # every head's output times sigmoid(W_g h)_h, one number per head ("g")
    tau: float = 0.0  # gated_linear: the decay is sigmoid(z)^(1 / tau)


@dataclass
class FeedForwardSpec:
    kind: str  # "dense" | "moe"
    ff: int
    experts: int = 0
    top: int = 0
    limit: float = 0.0  # clamped gated unit: bound of the gate (from above) and of the up branch (both sides)
    identity: int = 0  # moe: router outputs beyond ``experts`` that stand for identity experts (output = input)
    shared_ff: int = 0  # moe: size of a shared expert that runs for every token behind a sigmoid gate (0: none)


@dataclass
class LayerSpec:
    mixer: MixerSpec
    mlp: Optional[FeedForwardSpec]


# "channel_delta" / "gated_delta": the gated delta rule with a decay per head and key channel / per head;
# "sink_attention": softmax attention with unit-RMS queries and keys, a query temperature and a sink;
# "rotary_attention": grouped softmax attention with rotary positions (half layout) and a sink of score 0;
# "key_value_attention": softmax attention whose values are the keys as projected, weighted q / k norms, a query
# temperature and a gate per head; "gated_linear": the gated rule without the correction and a decay per key channel,
# S <- diag(alpha) S + k v^T; "lightning": the constant-decay rule on silu(q), silu(k), silu(v);
# "parallel": two of these side by side (which two, the design says)
MIXER_KINDS = ("retention", "latent_attention", "attention", "mamba2", "channel_delta", "gated_delta",
               "sink_attention", "parallel", "rotary_attention", "key_value_attention", "gated_linear", "lightning")
SOFTMAX_KINDS = ("sink_attention", "rotary_attention", "key_value_attention")


@dataclass(frozen=True)
class LayeredDesign:
    """What a design fixes for all its models (everything else is in ``config.json``)."""

    # "parallel": x += mixer(h) + ff(h), one norm; "sequential": x += mixer(norm1 x), then x += ff(norm2 x);
    # "post": the sublayers read x itself and their OUTPUT is normed: x += m norm1(mixer(x)), then x += m norm2(ff(x))
    # "sandwich": normed on the way in and out, with a per-channel scale: x += ls1 * norm1b(mixer(norm1 x)), then
    # x += ls2 * norm2b(ff(norm2 x))
    block: str
    norm_offset: float  # the norm multiplies by offset + stored weight
    tied_head: bool  # logits from the embedding table itself, or from a matrix of their own ("head")
    # "gelu_tanh": W_down(gelu_tanh(gate) * up); "clamped_swish": g sigmoid(1.702 g) (u + 1), clamped;
    # "relu2": W_down relu(W_up h)^2 (no gate)
    dense_ff: str
    norm: str = "rms"  # "rms": x / rms(x) * w; "layer": (x - mean) / sqrt(var + eps) * w + b (tensor "<norm>.b")
    positions: str = "none"  # "learned": a table "pos" whose row p joins the embedding at position p
    # "top_logits": the largest router logits, softmax over the chosen, experts W_down relu(W_up h)^2;
    # "scores": softmax over all router outputs (+ a stored correction for the choice only), weights = the chosen
    # scores as they are, gated experts W_down(silu(W_gate h) * W_up h), optional identity experts
    # "sigmoid": scores = sigmoid of every router output, the largest chosen, the score scales the expert's INPUT,
    # experts W_down relu(W_up h)^2, optional shared expert behind a sigmoid gate per token
    moe: str = "top_logits"
    # layer type (config.json) -> (left kind, right kind, branch_norm) of the designs' two-branch mixers
    pairs: Dict[str, tuple] = field(default_factory=lambda: {"parallel": ("sink_attention", "gated_delta", False)})


DESIGNS: Dict[str, LayeredDesign] = {
    "Bavesun": LayeredDesign("parallel", 1.0, True, "gelu_tanh"),
    "Rigulorn": LayeredDesign("sequential", 0.0, False, "clamped_swish"),
    "Ravelorn": LayeredDesign("post", 0.0, False, "gelu_tanh", norm="layer", positions="learned", moe="scores"),
    "Gatutar": LayeredDesign("sandwich", 0.0, False, "relu2", moe="sigmoid",
                             pairs={"parallel": ("rotary_attention", "gated_linear", True),
                                    "parallel_2": ("key_value_attention", "lightning", True)}),
}


@dataclass
class LayeredConfig:
    architecture: str
    vocab: int
    width: int
    norm_eps: float
    embedding_scale: float
    layers: List[LayerSpec]
    loop_start: int = 0
    loop_stop: int = 0
    loop_times: int = 1
    side_dim: int = 0  # per-layer token input: width of each layer's slice of the second embedding table (0: none)
    name: str = ""
    streams: int = 1  # parallel residual streams (hyper-connections); 1 with no stream weights: the plain residual sum
    stream_weights: bool = False  # the checkpoint holds read / write / mix weights per sublayer
    residual_mult: float = 1.0  # post-norm layers: factor of every normed sublayer output in the residual sum
    logit_softcap: float = 0.0  # logits pass cap * tanh(z / cap) (0: not)
    max_positions: int = 0  # rows of the learned position table (0: the design has none)

    @property
    def design(self) -> LayeredDesign:
        return DESIGNS[self.architecture]

    def __post_init__(self) -> None:
        self.name = self.name or self.architecture
        if self.architecture not in DESIGNS:
            raise ValueError(f"architecture {self.architecture!r} is not registered (known: {sorted(DESIGNS)})")
        if not 1 <= self.streams <= 8:
            raise ValueError(f"{self.streams} residual streams: 1 to 8 are served")
        n = len(self.layers)
        if not (0 <= self.loop_start <= self.loop_stop <= n) or self.loop_times < 1:
            raise ValueError(f"loop [{self.loop_start}, {self.loop_stop}) x {self.loop_times} does not fit {n} layers")
        if self.design.positions == "learned" and self.max_positions < 1:
            raise ValueError("max_positions: the design adds a learned position vector")
        for i, spec in enumerate(self.layers):
            m = spec.mixer
            if m.kind not in MIXER_KINDS:
                raise ValueError(f"layer {i}: unknown mixer {m.kind!r}")
            if spec.mlp is not None and spec.mlp.kind == "moe":
                f = spec.mlp
                if not 0 < f.top <= f.experts + f.identity or f.identity < 0 or f.experts + f.identity > 256:
                    raise ValueError(f"layer {i}: top {f.top} of {f.experts} + {f.identity} experts (at most 256)")
            parts = [m.left, m.right] if m.kind == "parallel" else [m]
            if m.kind == "parallel":
                allowed = {(a, b) for a, b, _ in self.design.pairs.values()}
                if m.left is None or m.right is None or (m.left.kind, m.right.kind) not in allowed:
                    raise ValueError(f"layer {i}: a parallel mixer of this design holds one of {sorted(allowed)}")
            for q in parts:
                if q.kind in ("gated_linear", "lightning"):
                    if q.heads < 1 or not 1 <= q.dim <= 512 or q.vdim < 1:
                        raise ValueError(f"layer {i}: heads {q.heads} / key dim {q.dim} (<= 512) / value dim {q.vdim}")
                    if q.kind == "gated_linear" and not q.tau > 0.0:
                        raise ValueError(f"layer {i}: tau must be positive")
                    if q.kind == "lightning" and (q.decay is None or len(q.decay) != q.heads):
                        raise ValueError(f"layer {i}: one decay per head")
                if q.kind in ("rotary_attention", "key_value_attention"):
                    if q.kv_heads < 1 or q.heads % q.kv_heads or not 1 <= q.dim <= 512 or not 1 <= q.vdim <= 256:
                        raise ValueError(f"layer {i}: heads {q.heads} / key heads {q.kv_heads} / dims {q.dim}, {q.vdim}")
                    if q.rot.dims % 2 or q.rot.dims > q.dim or q.q_temp_every < 0:
                        raise ValueError(f"layer {i}: rotary dims {q.rot.dims} / q_temp.every {q.q_temp_every}")
                    if q.values == "keys" and q.vdim != q.dim:
                        raise ValueError(f"layer {i}: values that are the keys have the keys' size")
                if q.kind in ("channel_delta", "gated_delta"):
                    if q.kv_heads < 1 or q.heads % q.kv_heads or not 1 <= q.dim <= 512 or q.vdim < 1:
                        raise ValueError(f"layer {i}: heads {q.heads} / key heads {q.kv_heads} / key dim {q.dim} (<= 512)")
                    if not 1 <= q.conv <= 16:
                        raise ValueError(f"layer {i}: convolution taps 1..16 are served")
                if q.kind == "sink_attention":
                    if q.kv_heads < 1 or q.heads % q.kv_heads or not 1 <= q.dim <= 512 or not 1 <= q.vdim <= 256:
                        raise ValueError(f"layer {i}: heads {q.heads} / key heads {q.kv_heads} / dims {q.dim}, {q.vdim}")
                    if q.q_temp_every < 0:
                        raise ValueError(f"layer {i}: q_temp.every must be positive")
            if m.kind in ("channel_delta", "gated_delta", "sink_attention", "parallel", "rotary_attention",
                          "key_value_attention", "gated_linear", "lightning"):
                continue
            if m.kind == "retention" and (m.decay is None or len(m.decay) != m.heads):
                raise ValueError(f"layer {i}: retention needs one decay per head")
            if m.kind == "mamba2":
                if m.groups < 1 or m.heads % m.groups or m.norm_groups < 1 or (m.heads * m.vdim) % m.norm_groups:
                    raise ValueError(f"layer {i}: heads {m.heads} / groups {m.groups} / norm groups {m.norm_groups}")
                if not (1 <= m.conv <= 16 and 1 <= m.state <= 256):
                    raise ValueError(f"layer {i}: convolution taps 1..16 and state size 1..256 are served")
                continue
            if m.rot.dims % 2 or m.rot.dims > (m.rot_dim if m.kind == "latent_attention" else m.dim):
                raise ValueError(f"layer {i}: rotary dims {m.rot.dims} do not fit the head")
            if m.kind == "attention":
                if m.kv_heads < 1 or m.heads % m.kv_heads or m.mask_size < 0 or m.vdim > 256:
                    raise ValueError(f"layer {i}: heads {m.heads} / key heads {m.kv_heads} / value dim {m.vdim}")
                if m.kv_from is not None:
                    j = m.kv_from
                    src = self.layers[j].mixer if 0 <= j < i else None
                    if src is None or src.kind != "attention" or src.kv_from is not None:
                        raise ValueError(f"layer {i}: kv_from {j} must name an earlier attention layer with keys of its own")
                    if (src.kv_heads, src.dim, src.vdim) != (m.kv_heads, m.dim, m.vdim):
                        raise ValueError(f"layer {i}: its key heads and sizes differ from layer {j}'s")

    @property
    def layer_runs(self) -> List[int]:
        """Layer index of every layer run in order: layers [loop_start, loop_stop) run loop_times times in a row
        with the same weights (each run with a cache or state of its own), the others once."""
        a, b = self.loop_start, self.loop_stop
        return list(range(a)) + list(range(a, b)) * self.loop_times + list(range(b, len(self.layers)))

    @staticmethod
    def _mixer_spec(kind: str, m: Dict[str, Any], design: Optional[LayeredDesign] = None) -> MixerSpec:
        pairs = (design or DESIGNS["Ravelorn"]).pairs
        if kind in pairs:
            left, right, normed = pairs[kind]
            half = 0.5 if normed else 1.0  # normed branches are averaged
            return MixerSpec(kind="parallel", heads=0, dim=0, vdim=0, rot=RotarySpec(),
                             left=LayeredConfig._mixer_spec(left, m["left"]),
                             right=LayeredConfig._mixer_spec(right, m["right"]),
                             left_scale=float(m.get("left_scale", half)), right_scale=float(m.get("right_scale", half)),
                             branch_norm=normed)
        rot = m.get("rot") or {}
        mask = m.get("mask") or {}
        temp = m.get("q_temp") or {}
        extra = {}
        if kind == "rotary_attention":
            extra = dict(qk_norm="none", sink_kind="one")
        elif kind == "key_value_attention":
            extra = dict(qk_norm="weight", sink_kind="none", values="keys", head_gate=True)
        scaling = rot.get("scaling")
        return MixerSpec(kind=kind, heads=int(m["heads"]), dim=int(m.get("dim", 0)), vdim=int(m["vdim"]),
                         rot=RotarySpec(int(rot.get("dims", 0)), float(rot.get("base", 10000.0)),
                                        {k: float(v) for k, v in scaling.items()} if scaling else None),
                         tau=float(m.get("tau", 0.0)), **extra,
                         decay=[float(x) for x in m["decay"]] if "decay" in m else None,
                         kv_rank=int(m.get("kv_rank", 0)), rot_dim=int(m.get("rot_dim", 0)),
                         scale=float(m.get("scale", 1.0)), kv_heads=int(m.get("kv_heads", m["heads"])),
                         diff=float(m.get("diff", 0.0)), softcap=float(m.get("softcap") or 0.0),
                         mask_size=int(mask.get("size") or 0),
                         kv_from=int(m["kv_from"]) if m.get("kv_from") is not None else None,
                         conv=int(m.get("conv", 0)), groups=int(m.get("groups", 1)),
                         norm_groups=int(m.get("norm_groups", 1)), state=int(m.get("state", 0)),
                         q_temp_coef=float(temp.get("coef", 0.0)), q_temp_every=int(temp.get("every", 0)),
                         decay_rank=int(m.get("decay_rank", 0)), gate_rank=int(m.get("gate_rank", 0)))

    @classmethod
    def from_dict(cls, d: Dict[str, Any]) -> "LayeredConfig":
        layers = []
        design = DESIGNS.get(d["architecture"])
        for entry in d["layers"]:
            m = entry["mixer"]
            mixer = cls._mixer_spec(entry["type"], m, design)
            f = entry.get("mlp")
            if f is None:
                mlp = None
            elif f["kind"] == "dense":
                mlp = FeedForwardSpec("dense", int(f["ff"]), limit=float(f.get("limit") or 0.0))
            elif f["kind"] == "moe":
                mlp = FeedForwardSpec("moe", int(f["expert"]["ff"]), int(f["router"]["experts"]), int(f["router"]["top"]),
                                      identity=int(f["router"].get("identity") or 0),
                                      shared_ff=int((f.get("shared") or {}).get("ff") or 0))
            else:
                raise ValueError(f"unknown feed-forward kind {f['kind']!r}")
            layers.append(LayerSpec(mixer, mlp))
        loop = d.get("loop") or {}
        side = d.get("token_side") or {}
        return cls(architecture=d["architecture"], vocab=int(d["vocab"]), width=int(d["width"]),
                   norm_eps=float(d["norm"]["eps"]), embedding_scale=float((d.get("embedding") or {}).get("scale", 1.0)),
                   layers=layers, loop_start=int(loop.get("start", 0)), loop_stop=int(loop.get("stop", 0)),
                   loop_times=int(loop.get("times", 1)), side_dim=int(side.get("dim", 0)),
                   streams=int(d.get("streams", 1)), stream_weights="streams" in d,
                   residual_mult=float(d.get("residual_mult", 1.0)), logit_softcap=float(d.get("logit_softcap") or 0.0),
                   max_positions=int(d.get("max_positions") or 0))

    @classmethod
    def from_json(cls, path: Union[str, Path]) -> "LayeredConfig":
        with open(path, encoding="utf-8") as fp:
            return cls.from_dict(json.load(fp))


# architecture name (config.json) -> "module:class" of the model that serves it
ARCHITECTURES: Dict[str, str] = {name: "lit_gpt.layered:LayeredGPT"
                                 for name in ("Bavesun", "Rigulorn", "Ravelorn", "Gatutar")}


def load_config(checkpoint_dir: Union[str, Path]) -> Union[Config, LayeredConfig]:
    """The configuration of a checkpoint folder: ``config.json`` with a registered ``architecture`` gives a
    LayeredConfig, anything else goes through ``Config.from_checkpoint`` (lit_config.json or a registered name)."""
    path = Path(checkpoint_dir)
    cj = path / "config.json"
    if cj.is_file():
        with open(cj, encoding="utf-8") as fp:
            d = json.load(fp)
        if d.get("architecture") in ARCHITECTURES:
            return LayeredConfig.from_dict(d)
        if "architecture" in d and not (path / "lit_config.json").is_file():
            raise ValueError(f"architecture {d['architecture']!r} is not registered (known: {sorted(ARCHITECTURES)})")
    return Config.from_checkpoint(path)


def model_class(config: Union[Config, LayeredConfig]) -> Type:
    if isinstance(config, LayeredConfig):
        import importlib

        mod, _, cls = ARCHITECTURES[config.architecture].partition(":")
        return getattr(importlib.import_module(mod), cls)
    import lit_gpt.model

    return lit_gpt.model.GPT
