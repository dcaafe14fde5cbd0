"""LayeredGPT: a decoder whose ``config.json`` lists its layers one by one, each with its own sequence mixer
(``lit_gpt.mixers``) and feed-forward, optionally looping a range of layers with shared weights.

It keeps the serving surface of ``lit_gpt.GPT`` — ``forward(idx, input_pos)``, ``max_seq_length``,
``set_kv_cache`` / ``clear_kv_cache`` — so ``generate.base.generate`` drives it unchanged, and adds the packed-batch
step (``forward_step`` / ``logits``) that ``generate.batch.BatchEngine`` schedules. The residual stream, norms,
attention scores, recurrent states and routers are fp32 in both precisions; ``dtype`` (bf16 or fp32) is the dtype
of the weight matrices and of the cached latent, and picks bf16-operand / fp32-sum products or plain fp32 ones.

The design named by ``config.architecture`` fixes the layer's shape (``config.design``):

* parallel — h = norm(x); x <- x + mixer(h) + ff(h); then the optional per-layer token input. The norm's weight is
  stored around zero (offset 1); every matrix that reads h is one row block of a single fused input projection;
  logits come from the embedding table itself (tied, unscaled) after the final norm.
* post — the sublayers read the residual x itself and their OUTPUT is normed before it joins the residual with a
  constant factor m: x <- x + m norm1(mixer(x)), then x <- x + m norm2(ff(x)) (layer norms with weight and bias).
  A learned position vector joins the embedding; logits pass a tanh soft cap. The norm + residual add of a
  sublayer is one launch that also leaves the bf16 copy of x the next input projection reads.
* sequential — pre-norm sublayers, x <- x + mixer(norm1 x), then x <- x + ff(norm2 x) (a layer may have no
  feed-forward), over ``config.streams`` parallel residual streams: a sublayer reads a weighted sum of the streams
  and its output is written into all of them while a small matrix mixes them (``lit_gpt.mixers.StreamLinks``; one
  stream with unit weights is the plain residual sum). The write-back of a sublayer and the read + norm of the next
  run as one launch. Logits from a matrix of their own (``head``) after the final norm of the streams' sum.
* sandwich — every sublayer is normed on the way in AND on the way out, and its normed output is scaled channel by
  channel before it joins the residual: x <- x + ls1 * norm1b(mixer(norm1 x)), then x <- x + ls2 * norm2b(ff(norm2 x))
  (RMS norms with plain weights). A two-branch mixer whose branches are each normed over the width hands both
  outputs to the boundary launch, which norms and averages them, applies the output norm and the scale, adds the
  residual and leaves the next sublayer's normed input (fp32 or its bf16 copy): one launch per sublayer boundary.
"""

from __future__ import annotations

from pathlib import Path
from typing import Dict, List, Optional, Sequence, Tuple

import torch
import torch.nn as nn

from lit_gpt import seq_ops
from lit_gpt.config import LayeredConfig, LayerSpec
from lit_gpt.mixers import (MIXERS, DenseFeedForward, GatedFeedForward, SparseFeedForward, StepBatch, StreamLinks,
                            TokenSide)
from lit_gpt.rmsnorm import StreamRMSNorm


def _sub(w: Dict[str, torch.Tensor], prefix: str) -> Dict[str, torch.Tensor]:
    return {k[len(prefix):]: v for k, v in w.items() if k.startswith(prefix)}


class LayeredBlock(nn.Module):
    def __init__(self, index: int, spec: LayerSpec, config: LayeredConfig, w: Dict[str, torch.Tensor],
                 side_table: Optional[torch.Tensor], device, dtype) -> None:
        super().__init__()
        W, eps = config.width, config.norm_eps
        self.norm1 = StreamRMSNorm(W, eps=eps, offset=1.0)
        self.norm1.weight = w["norm1"].to(device=device, dtype=torch.float32).contiguous()
        self.mixer = MIXERS[spec.mixer.kind](spec.mixer, W, eps, _sub(w, "mix."), device, dtype)
        self.mlp = None
        if spec.mlp is not None:
            cls = GatedFeedForward if spec.mlp.kind == "dense" else SparseFeedForward
            self.mlp = cls(spec.mlp, W, _sub(w, "mlp."), device, dtype)
        self.side = None
        if side_table is not None and "side.gate" in w:
            self.side = TokenSide(index, config.side_dim, side_table, _sub(w, "side."), eps, device, dtype)
        # one input projection for everything that reads the norm's output
        parts, offsets, at = [], [{}, {}], 0
        for k, mod in enumerate((self.mixer, self.mlp)):
            if mod is None:
                continue
            for name, t in mod.in_parts():
                offsets[k][name] = at
                parts.append(t)
                at += t.shape[0]
                pad = -at % 8  # every part starts on a 32-byte boundary of the fp32 row
                if pad:
                    parts.append(torch.zeros(pad, W, dtype=t.dtype))
                    at += pad
        self.mixer.bind(offsets[0])
        if self.mlp is not None:
            self.mlp.bind(offsets[1])
        self.register_buffer("w_in", torch.cat(parts).to(device=device, dtype=dtype).contiguous())

    def forward(self, x: torch.Tensor, step: StepBatch, cache: nn.Module) -> None:
        """x (T, width) fp32, updated in place."""
        # more than 8 rows run MFMA tiles: with bf16 weights the norm also leaves its output rounded to bf16, which
        # the tiles read at half the traffic (the values they would round the fp32 stream to)
        tiles16 = step.T > 8 and self.w_in.dtype == torch.bfloat16
        h, h16 = self.norm1(x, bf16_copy=True) if tiles16 else (self.norm1(x), None)
        n_in, W = self.w_in.shape
        proj = torch.empty(step.T, n_in, dtype=torch.float32, device=x.device)
        seq_ops.linear(h16 if tiles16 else h, self.w_in, M=step.T, N=n_in, K=W, y=proj, lda=W, ldy=n_in)
        self.mixer(proj, step, cache, x)
        if self.mlp is not None:
            self.mlp(proj, h, x, h16=h16)
        if self.side is not None:
            self.side(x, step.tokens)


def _fuse_rows(parts, width: int, device, dtype) -> Tuple[torch.Tensor, Dict[str, int]]:
    """Row-wise concatenation of the matrices that read one norm output, every part on a 32-byte boundary of the
    fp32 result row; returns the matrix and each part's first row."""
    rows, offsets, at = [], {}, 0
    for name, t in parts:
        offsets[name] = at
        rows.append(t)
        at += t.shape[0]
        pad = -at % 8
        if pad:
            rows.append(torch.zeros(pad, width, dtype=t.dtype))
            at += pad
    return torch.cat(rows).to(device=device, dtype=dtype).contiguous(), offsets


class Sublayer(nn.Module):
    """One pre-norm sublayer of a sequential layer: its norm weight, its links to the residual streams, its fused
    input projection and the module (a mixer or a feed-forward) that turns the projection into the output."""

    def __init__(self, module: nn.Module, norm_w: torch.Tensor, links: StreamLinks, width: int, device, dtype) -> None:
        super().__init__()
        self.module, self.links = module, links
        self.register_buffer("norm_w", norm_w.to(device=device, dtype=torch.float32).contiguous())
        w_in, offsets = _fuse_rows(module.in_parts(), width, device, dtype)
        module.bind(offsets)
        self.register_buffer("w_in", w_in)

    def wants_bf16(self, rows: int) -> bool:
        """Whether the norm that feeds this sublayer should also leave a bf16 copy (bf16 MFMA tiles read it)."""
        return rows > 8 and self.w_in.dtype == torch.bfloat16

    def forward(self, h: torch.Tensor, h16: Optional[torch.Tensor], step: StepBatch, cache) -> torch.Tensor:
        """h (T, width): the normed read of the streams. Returns the sublayer's output (T, width) fp32."""
        n_in, W = self.w_in.shape
        proj = torch.empty(step.T, n_in, dtype=torch.float32, device=h.device)
        seq_ops.linear(h if h16 is None else h16, self.w_in, M=step.T, N=n_in, K=W, y=proj, lda=W, ldy=n_in)
        y = torch.empty(step.T, W, dtype=torch.float32, device=h.device)
        if cache is None:
            self.module(proj, h, y, h16=h16, accumulate=False)
        else:
            self.module(proj, step, cache, y, accumulate=False)
        return y


class SequentialBlock(nn.Module):
    """A pre-norm layer: the mixer sublayer, then the feed-forward sublayer if the layer has one."""

    def __init__(self, index: int, spec: LayerSpec, config: LayeredConfig, w: Dict[str, torch.Tensor], device,
                 dtype) -> None:
        super().__init__()
        W, eps, design = config.width, config.norm_eps, config.design
        if design.norm_offset != 0.0:
            raise NotImplementedError("sequential layers take the norm weight as stored")

        def links(q: int) -> StreamLinks:
            return StreamLinks(config.streams, _sub(w, f"hc{q}.") if config.stream_weights else None, device)

        self.mixer = MIXERS[spec.mixer.kind](spec.mixer, W, eps, _sub(w, "mix."), device, dtype)
        self.sub1 = Sublayer(self.mixer, w["norm1"], links(1), W, device, dtype)
        self.sub2 = None
        if spec.mlp is not None:
            if spec.mlp.kind != "dense":
                raise NotImplementedError("sequential layers serve dense feed-forwards")
            clamp = (1.702, spec.mlp.limit, 1.0) if design.dense_ff == "clamped_swish" else None
            mlp = GatedFeedForward(spec.mlp, W, _sub(w, "mlp."), device, dtype, clamp=clamp)
            self.sub2 = Sublayer(mlp, w["norm2"], links(2), W, device, dtype)

    def sublayers(self) -> List[Sublayer]:
        return [self.sub1] if self.sub2 is None else [self.sub1, self.sub2]


class PostSublayer(nn.Module):
    """One sublayer of a post-norm layer: the fused input projection of everything that reads the residual, the
    module (a mixer or a feed-forward), and the layer norm (weight, bias) its output passes."""

    def __init__(self, module: nn.Module, norm_w: torch.Tensor, norm_b: Optional[torch.Tensor], width: int, device,
                 dtype) -> None:
        super().__init__()
        self.module = module
        if norm_w.numel() != width or (norm_b is not None and norm_b.numel() != width):
            raise ValueError("norm: weight and bias must have the model's width")
        self.register_buffer("norm_w", norm_w.to(device=device, dtype=torch.float32).contiguous())
        self.register_buffer("norm_b", None if norm_b is None else norm_b.to(device=device, dtype=torch.float32).contiguous())
        w_in, offsets = _fuse_rows(module.in_parts(), width, device, dtype)
        module.bind(offsets)
        self.register_buffer("w_in", w_in)

    def forward(self, x: torch.Tensor, x16: Optional[torch.Tensor], step: StepBatch, cache) -> torch.Tensor:
        """x (T, width): the residual (x16: its bf16 copy for the MFMA tiles). Returns the sublayer's output, unnormed."""
        n_in, W = self.w_in.shape
        proj = None
        if self.module.wants_proj(step.T):
            proj = torch.empty(step.T, n_in, dtype=torch.float32, device=x.device)
            seq_ops.linear(x if x16 is None else x16, self.w_in, M=step.T, N=n_in, K=W, y=proj, lda=W, ldy=n_in)
        y = torch.empty(step.T, W, dtype=torch.float32, device=x.device)
        if cache is None:
            self.module(proj, x, y, h16=x16, accumulate=False)
        else:
            self.module(proj, step, cache, y, accumulate=False)
        return y


class PostNormBlock(nn.Module):
    """x <- x + m norm1(mixer(x)), then x <- x + m norm2(ff(x)) when the layer has a feed-forward."""

    def __init__(self, index: int, spec: LayerSpec, config: LayeredConfig, w: Dict[str, torch.Tensor], device,
                 dtype) -> None:
        super().__init__()
        W, eps, design = config.width, config.norm_eps, config.design
        if design.norm != "layer":
            raise NotImplementedError("post-norm layers use layer norms")
        self.mixer = MIXERS[spec.mixer.kind](spec.mixer, W, eps, _sub(w, "mix."), device, dtype)
        self.sub1 = PostSublayer(self.mixer, w["norm1"], w.get("norm1.b"), W, device, dtype)
        self.sub2 = None
        if spec.mlp is not None:
            if spec.mlp.kind != "moe" or design.moe != "scores":
                raise NotImplementedError("post-norm layers serve the score-routed mixture of experts")
            mlp = SparseFeedForward(spec.mlp, W, _sub(w, "mlp."), device, dtype, route="scores")
            self.sub2 = PostSublayer(mlp, w["norm2"], w.get("norm2.b"), W, device, dtype)

    def sublayers(self) -> List[PostSublayer]:
        return [self.sub1] if self.sub2 is None else [self.sub1, self.sub2]


class SandwichSublayer(nn.Module):
    """One sublayer of a sandwich layer: the input norm's weight, the fused input projection of everything that reads
    the normed input (none when the module makes its own product), the module, and the output norm's weight times the
    layer's per-channel scale (folded once, in fp32)."""

    def __init__(self, module: nn.Module, norm_w: torch.Tensor, post_w: torch.Tensor, scale: Optional[torch.Tensor],
                 width: int, device, dtype) -> None:
        super().__init__()
        self.module = module
        for t in (norm_w, post_w) + ((scale,) if scale is not None else ()):
            if t.numel() != width:
                raise ValueError("norm / layer scale: one value per channel of the model's width")
        self.register_buffer("norm_w", norm_w.to(device=device, dtype=torch.float32).contiguous())
        post = post_w.to(device=device, dtype=torch.float32)
        if scale is not None:
            post = post * scale.to(device=device, dtype=torch.float32)
        self.register_buffer("post_w", post.contiguous())
        self.register_buffer("w_in", None)
        parts = module.in_parts()
        if parts:
            self.w_in, offsets = _fuse_rows(parts, width, device, dtype)
            module.bind(offsets)

    def wants_bf16(self, rows: int) -> bool:
        """Whether the norm that feeds this sublayer should leave a bf16 copy (bf16 MFMA tiles read it)."""
        return rows > 8 and self._dtype() == torch.bfloat16

    def _dtype(self):
        return self.w_in.dtype if self.w_in is not None else self.module.w_up.dtype

    def forward(self, h: Optional[torch.Tensor], h16: Optional[torch.Tensor], step: StepBatch, cache):
        """h / h16 (T, width): the normed input (fp32 and / or its bf16 copy). Returns (branches, factor): the
        sublayer's output as one (y, None) pair, or a two-branch mixer's (y, weight) pairs, for the boundary launch."""
        src = h16 if h16 is not None else h
        T, W = src.shape
        proj = None
        if self.w_in is not None and self.module.wants_proj(T):
            n_in = self.w_in.shape[0]
            proj = torch.empty(T, n_in, dtype=torch.float32, device=src.device)
            seq_ops.linear(src, self.w_in, M=T, N=n_in, K=W, y=proj, lda=W, ldy=n_in)
        y = torch.empty(T, W, dtype=torch.float32, device=src.device)
        if cache is None:
            self.module(proj, h, y, h16=h16, accumulate=False)
        elif getattr(self.module, "branch_norm", False):
            return self.module.branches(proj, step, cache, y)
        else:
            self.module(proj, step, cache, y, accumulate=False)
        return [(y, None)], 1.0


class SandwichBlock(nn.Module):
    """x <- x + ls1 * norm1b(mixer(norm1 x)), then x <- x + ls2 * norm2b(ff(norm2 x)) when the layer has a feed-forward."""

    def __init__(self, index: int, spec: LayerSpec, config: LayeredConfig, w: Dict[str, torch.Tensor], device,
                 dtype) -> None:
        super().__init__()
        W, eps, design = config.width, config.norm_eps, config.design
        if design.norm != "rms" or design.norm_offset != 0.0:
            raise NotImplementedError("sandwich layers use RMS norms with plain weights")
        self.mixer = MIXERS[spec.mixer.kind](spec.mixer, W, eps, _sub(w, "mix."), device, dtype)
        self.sub1 = SandwichSublayer(self.mixer, w["norm1"], w["norm1b"], w.get("ls1"), W, device, dtype)
        self.sub2 = None
        if spec.mlp is not None:
            if spec.mlp.kind == "dense":
                if design.dense_ff != "relu2":
                    raise NotImplementedError("sandwich layers serve the ungated relu^2 feed-forward")
                mlp = DenseFeedForward(spec.mlp, W, _sub(w, "mlp."), device, dtype)
            else:
                mlp = SparseFeedForward(spec.mlp, W, _sub(w, "mlp."), device, dtype, route=design.moe)
            self.sub2 = SandwichSublayer(mlp, w["norm2"], w["norm2b"], w.get("ls2"), W, device, dtype)

    def sublayers(self) -> List[SandwichSublayer]:
        return [self.sub1] if self.sub2 is None else [self.sub1, self.sub2]


def _mixer_shapes(p: str, m, W: int) -> Dict[str, Tuple[int, ...]]:
    """Name -> shape of the tensors of a gated delta rule, a sink attention or a pair of them under prefix p."""
    if m.kind == "parallel":
        out = {**_mixer_shapes(p + "left.", m.left, W), **_mixer_shapes(p + "right.", m.right, W)}
        if m.branch_norm:
            out.update({p + "left.out": (W,), p + "right.out": (W,)})
        return out
    if m.kind in ("sink_attention", "rotary_attention", "key_value_attention"):
        out = {p + "q": (m.heads * m.dim, W), p + "k": (m.kv_heads * m.dim, W)}
        if m.values == "own":
            out[p + "v"] = (m.kv_heads * m.vdim, W)
        if m.sink_kind == "learned":
            out[p + "sink"] = (m.heads,)
        out[p + "o"] = (W, m.heads * m.vdim)
        if m.qk_norm == "weight":
            out.update({p + "q.norm": (m.dim,), p + "k.norm": (m.dim,)})
        if m.head_gate:
            out[p + "g"] = (m.heads, W)
        return out
    if m.kind in ("gated_linear", "lightning"):
        qk, v = m.heads * m.dim, m.heads * m.vdim
        out = {p + "q": (qk, W), p + "k": (qk, W), p + "v": (v, W), p + "g": (v, W), p + "o": (W, v)}
        if m.kind == "gated_linear":
            rank = m.decay_rank or 16
            out.update({p + "norm": (m.vdim,), p + "a1": (rank, W), p + "a2": (qk, rank), p + "a2.b": (qk,)})
        else:
            out[p + "norm"] = (v,)
        return out
    qk, v = m.kv_heads * m.dim, m.heads * m.vdim
    out = {p + "q": (qk, W), p + "q.conv": (qk, m.conv), p + "k": (qk, W), p + "k.conv": (qk, m.conv), p + "v": (v, W),
           p + "v.conv": (v, m.conv), p + "b": (m.heads, W), p + "A_log": (m.heads,), p + "norm": (m.vdim,),
           p + "o": (W, v)}
    if m.kind == "channel_delta":
        ra, rg = m.decay_rank or 16, m.gate_rank or 16
        out.update({p + "a1": (ra, W), p + "a2": (m.heads * m.dim, ra), p + "dt_bias": (m.heads * m.dim,),
                    p + "g1": (rg, W), p + "g2": (v, rg)})
    else:
        out.update({p + "a": (m.heads, W), p + "dt_bias": (m.heads,), p + "g": (v, W)})
    return out


class LayeredGPT(nn.Module):
    decode_graph = False  # generate.base.generate steps this model eagerly (its graph executor is GPT's)

    def __init__(self, config: LayeredConfig, weights: Dict[str, torch.Tensor], *, device: torch.device,
                 dtype: torch.dtype = torch.bfloat16) -> None:
        super().__init__()
        if dtype not in (torch.bfloat16, torch.float32):
            raise NotImplementedError(f"dtype {dtype}: the MI355X path computes with bf16 or fp32 weights")
        if torch.device(device).type != "cuda":
            raise RuntimeError("LayeredGPT: this build computes on the MI355X only (no CPU path)")
        self.config, self.dtype, self.device = config, dtype, torch.device(device)
        V, W = config.vocab, config.width
        if tuple(weights["embed"].shape) != (V, W):
            raise ValueError(f"embed: shape {tuple(weights['embed'].shape)}, expected {(V, W)}")
        self.register_buffer("embed", weights["embed"].to(device=device, dtype=dtype).contiguous())
        self.register_buffer("side_embed", None)
        if config.side_dim:
            t = weights["side.embed"]
            if t.shape[0] != V or t.shape[1] < config.side_dim * len(config.layers):
                raise ValueError(f"side.embed: shape {tuple(t.shape)} does not hold {len(config.layers)} slices")
            self.side_embed = t.to(device=device, dtype=dtype).contiguous()
        design = config.design
        self.sequential = design.block == "sequential"
        self.post = design.block == "post"
        self.sandwich = design.block == "sandwich"
        self.register_buffer("pos_table", None)
        if design.positions == "learned":
            t = weights["pos"]
            if tuple(t.shape) != (config.max_positions, W):
                raise ValueError(f"pos: shape {tuple(t.shape)}, expected {(config.max_positions, W)}")
            self.pos_table = t.to(device=device, dtype=dtype).contiguous()
        if self.post:
            if config.side_dim or config.streams != 1:
                raise NotImplementedError("post-norm layers have one residual stream and no per-layer token input")
            self.blocks = nn.ModuleList(PostNormBlock(i, spec, config, _sub(weights, f"l{i}."), device, dtype)
                                        for i, spec in enumerate(config.layers))
        elif self.sandwich:
            if config.side_dim or config.streams != 1:
                raise NotImplementedError("sandwich layers have one residual stream and no per-layer token input")
            self.blocks = nn.ModuleList(SandwichBlock(i, spec, config, _sub(weights, f"l{i}."), device, dtype)
                                        for i, spec in enumerate(config.layers))
        elif self.sequential:
            if config.side_dim:
                raise NotImplementedError("per-layer token inputs belong to the parallel layers")
            self.blocks = nn.ModuleList(SequentialBlock(i, spec, config, _sub(weights, f"l{i}."), device, dtype)
                                        for i, spec in enumerate(config.layers))
            self.register_buffer("stream_ones", torch.ones(config.streams, dtype=torch.float32, device=device))
        else:
            if config.streams != 1:
                raise NotImplementedError("several residual streams belong to the sequential layers")
            self.blocks = nn.ModuleList(
                LayeredBlock(i, spec, config, _sub(weights, f"l{i}."), self.side_embed, device, dtype)
                for i, spec in enumerate(config.layers))
        self.register_buffer("head", None)
        if not design.tied_head:
            if tuple(weights["head"].shape) != (V, W):
                raise ValueError(f"head: shape {tuple(weights['head'].shape)}, expected {(V, W)}")
            self.head = weights["head"].to(device=device, dtype=dtype).contiguous()
        self.register_buffer("final_bias", None)
        if design.norm == "layer":
            self.final_norm = None
            self.register_buffer("final_weight", weights["final.norm"].to(device=device, dtype=torch.float32).contiguous())
            if "final.norm.b" in weights:
                self.final_bias = weights["final.norm.b"].to(device=device, dtype=torch.float32).contiguous()
        else:
            self.final_norm = StreamRMSNorm(W, eps=config.norm_eps, offset=design.norm_offset)
            self.final_norm.weight = weights["final.norm"].to(device=device, dtype=torch.float32).contiguous()
        self.runs: List[int] = config.layer_runs
        self.caches: Optional[nn.ModuleList] = None  # one cache / state per layer run
        self._max_seq_length = 0
        self.eval()

    # ------------------------------------------------------------------------------------------ construction
    @classmethod
    def from_checkpoint(cls, checkpoint_dir, *, device, dtype=torch.bfloat16) -> "LayeredGPT":
        """``config.json`` + ``model.safetensors`` (bf16 matrices [out, in], names l<i>.mix.* / .mlp.* / .side.*)."""
        from lit_gpt.utils import read_safetensors

        path = Path(checkpoint_dir)
        config = LayeredConfig.from_json(path / "config.json")
        return cls(config, read_safetensors(path / "model.safetensors"), device=device, dtype=dtype)

    @staticmethod
    def tensor_shapes(config: LayeredConfig) -> Dict[str, Tuple[int, ...]]:
        """Name -> shape of every checkpoint tensor of a configuration."""
        W, out = config.width, {"embed": (config.vocab, config.width), "final.norm": (config.width,)}
        if not config.design.tied_head:
            out["head"] = (config.vocab, config.width)
        if config.side_dim:
            out["side.embed"] = (config.vocab, config.side_dim * len(config.layers))
        biased = config.design.norm == "layer"
        if biased:
            out["final.norm.b"] = (W,)
        if config.design.positions == "learned":
            out["pos"] = (config.max_positions, W)
        for i, spec in enumerate(config.layers):
            m, p = spec.mixer, f"l{i}."
            out[p + "norm1"] = (W,)
            if spec.mlp is not None and config.design.block != "parallel":
                out[p + "norm2"] = (W,)
            if config.design.block == "sandwich":
                out.update({p + "norm1b": (W,), p + "ls1": (W,)})
                if spec.mlp is not None:
                    out.update({p + "norm2b": (W,), p + "ls2": (W,)})
            if biased:
                out.update({name + ".b": (W,) for name in (p + "norm1", p + "norm2") if name in out})
            if config.stream_weights:
                for q in (1, 2) if spec.mlp is not None else (1,):
                    s = config.streams
                    out.update({p + f"hc{q}.in": (s,), p + f"hc{q}.out": (s,), p + f"hc{q}.mix": (s, s)})
            if m.kind == "retention":
                out.update({p + "mix.q": (m.heads * m.dim, W), p + "mix.k": (m.heads * m.dim, W),
                            p + "mix.v": (m.heads * m.vdim, W), p + "mix.g": (m.heads * m.vdim, W),
                            p + "mix.o": (W, m.heads * m.vdim)})
            elif m.kind == "attention":
                out.update({p + "mix.q": (2 * m.heads * m.dim, W), p + "mix.o": (W, m.heads * m.vdim)})
                if m.kv_from is None:
                    out.update({p + "mix.k": (2 * m.kv_heads * m.dim, W), p + "mix.v": (m.kv_heads * m.vdim, W)})
                out.update({p + f"mix.{n}": (m.dim,) for n in ("lq1", "lk1", "lq2", "lk2")})
            elif m.kind in ("channel_delta", "gated_delta", "sink_attention", "parallel", "rotary_attention",
                            "key_value_attention", "gated_linear", "lightning"):
                out.update(_mixer_shapes(p + "mix.", m, W))
            elif m.kind == "mamba2":
                inner, bc = m.heads * m.vdim, 2 * m.groups * m.state
                out.update({p + "mix.in": (2 * inner + bc + m.heads, W), p + "mix.conv": (inner + bc, m.conv),
                            p + "mix.conv.b": (inner + bc,), p + "mix.dt_bias": (m.heads,), p + "mix.A_log": (m.heads,),
                            p + "mix.D": (m.heads,), p + "mix.norm": (inner,), p + "mix.o": (W, inner)})
            else:
                out.update({p + "mix.q": (m.heads * (m.dim + m.rot_dim), W), p + "mix.dkv": (m.kv_rank + m.rot_dim, W),
                            p + "mix.dkv.norm": (m.kv_rank,), p + "mix.uk": (m.heads * m.dim, m.kv_rank),
                            p + "mix.uv": (m.heads * m.vdim, m.kv_rank), p + "mix.sink": (m.heads,),
                            p + "mix.g": (m.heads * m.vdim, W), p + "mix.o": (W, m.heads * m.vdim)})
            f = spec.mlp
            if f is not None and f.kind == "dense" and config.design.dense_ff == "relu2":
                out.update({p + "mlp.up": (f.ff, W), p + "mlp.down": (W, f.ff)})
            elif f is not None and f.kind == "dense":
                out.update({p + "mlp.gate": (f.ff, W), p + "mlp.up": (f.ff, W), p + "mlp.down": (W, f.ff)})
            elif f is not None:
                gated = config.design.moe == "scores"
                out[p + "mlp.router"] = (f.experts + (f.identity if gated else 0), W)
                if gated:
                    out[p + "mlp.correction"] = (f.experts + f.identity,)
                for e in range(f.experts):
                    if gated:
                        out[p + f"mlp.e{e}.gate"] = (f.ff, W)
                    out.update({p + f"mlp.e{e}.up": (f.ff, W), p + f"mlp.e{e}.down": (W, f.ff)})
                if f.shared_ff:
                    out.update({p + "mlp.shared.up": (f.shared_ff, W), p + "mlp.shared.down": (W, f.shared_ff),
                                p + "mlp.shared.sg": (1, W)})
            if config.side_dim:
                out.update({p + "side.gate": (config.side_dim, W), p + "side.proj": (W, config.side_dim),
                            p + "side.norm": (W,)})
        return out

    @classmethod
    def random_weights(cls, config: LayeredConfig, seed: int = 0) -> Dict[str, torch.Tensor]:
        """Random bf16 checkpoint tensors (matrices ~ N(0, 1/fan_in), norm weights around the design's neutral value,
        sinks ~ N(0, 1), stream weights around the plain residual sum, step sizes and decays in a usable range)."""
        g = torch.Generator().manual_seed(seed)
        out = {}
        neutral = 1.0 - config.design.norm_offset
        for name, shape in cls.tensor_shapes(config).items():
            leaf = name.rsplit(".", 1)[-1]
            if leaf in ("norm1", "norm2", "norm1b", "norm2b") or name == "final.norm":
                t = neutral + 0.1 * torch.randn(shape, generator=g)
            elif leaf in ("ls1", "ls2"):
                t = 0.5 + 0.2 * torch.randn(shape, generator=g)
            elif name.endswith((".left.out", ".right.out", "q.norm", "k.norm")):
                t = 1.0 + 0.2 * torch.randn(shape, generator=g)
            elif name.endswith("a2.b"):
                t = 2.0 + torch.randn(shape, generator=g)
            elif name.endswith(("norm1.b", "norm2.b", "final.norm.b", "correction")):
                t = 0.1 * torch.randn(shape, generator=g)
            elif name == "pos":
                t = 0.5 * shape[1] ** -0.5 * torch.randn(shape, generator=g)
            elif name.endswith(".conv") and len(shape) == 2 and ".mix." in name and "mamba" not in name and \
                    name.rsplit(".", 2)[-2] in ("q", "k", "v"):
                t = torch.randn(shape, generator=g) * 0.7
            elif ".hc" in name:
                s = config.streams
                t = {"in": torch.full(shape, 1.0 / s), "out": torch.ones(shape), "mix": torch.eye(s)}[leaf] + \
                    0.2 * torch.randn(shape, generator=g)
            elif leaf in ("lq1", "lk1", "lq2", "lk2"):
                t = 0.3 * torch.randn(shape, generator=g)
            elif leaf == "A_log":
                t = torch.log(1.0 + 3.0 * torch.rand(shape, generator=g))
            elif leaf == "dt_bias":
                t = -2.0 + torch.randn(shape, generator=g)
            elif leaf == "D":
                t = 1.0 + 0.2 * torch.randn(shape, generator=g)
            elif name.endswith("conv.b"):
                t = 0.2 * torch.randn(shape, generator=g)
            elif name.endswith(".norm"):
                t = 1.0 + 0.1 * torch.randn(shape, generator=g)
            elif name.endswith("sink"):
                t = torch.randn(shape, generator=g)
            elif name.endswith("embed"):
                t = torch.randn(shape, generator=g) * (1.0 if name == "side.embed" else shape[1] ** -0.5)
            else:
                t = torch.randn(shape, generator=g) * shape[1] ** -0.5
            out[name] = t.to(torch.bfloat16)
        return out

    # ------------------------------------------------------------------------------------------ cache
    @property
    def max_seq_length(self) -> int:
        return self._max_seq_length

    @max_seq_length.setter
    def max_seq_length(self, value: int) -> None:
        if self.config.max_positions > 0:  # a learned position table bounds every sequence
            value = min(int(value), self.config.max_positions)
        if self.caches is not None and value != self._max_seq_length:
            self.caches = None  # rebuilt by the next set_kv_cache
        self._max_seq_length = int(value)

    def set_kv_cache(self, batch_size: int, max_seq_length: Optional[int] = None,
                     device: Optional[torch.device] = None, dtype: Optional[torch.dtype] = None) -> None:
        """Caches and states for ``batch_size`` slots of ``max_seq_length`` positions, one per layer run."""
        if max_seq_length is not None:
            self.max_seq_length = max_seq_length
        if self._max_seq_length <= 0:
            raise ValueError("set max_seq_length (or pass it) before set_kv_cache")
        caches, of_layer = [], {}
        for i in self.runs:
            mixer = self.blocks[i].mixer
            src = getattr(mixer, "kv_from", None)
            if src is not None:  # the layer reads the keys and values the named layer has cached (its latest run)
                cache = of_layer[src]
            else:
                cache = mixer.build_cache(batch_size, self._max_seq_length, device or self.device, dtype or self.dtype)
            of_layer[i] = cache
            caches.append(cache)
        self.caches = nn.ModuleList(caches)

    def clear_kv_cache(self) -> None:
        self.caches = None

    @property
    def slots(self) -> int:
        return 0 if self.caches is None else self.caches[0].slots

    def grow_slots(self, slots: int) -> None:
        for c in self.caches:
            c.grow(slots)

    # ------------------------------------------------------------------------------------------ forward
    @torch.inference_mode()
    def forward_step(self, step: StepBatch) -> torch.Tensor:
        """Run the step's tokens through every layer run from the caches and states earlier steps left; returns the
        final residual stream (T, width) fp32 (before the final norm)."""
        if self.caches is None:
            raise TypeError("You need to call `set_kv_cache()`")
        if self.sequential:
            return self._forward_streams(step)
        if self.post:
            return self._forward_post(step)
        if self.sandwich:
            return self._forward_sandwich(step)
        x = seq_ops.embed(step.tokens, self.embed, self.config.embedding_scale)
        for run, layer in enumerate(self.runs):
            self.blocks[layer](x, step, self.caches[run])
        return x

    def _forward_post(self, step: StepBatch, after_layer=None) -> torch.Tensor:
        """The post-norm layers: every sublayer reads the residual itself (for more than 8 rows with bf16 weights its
        bf16 copy, which the embedding and every norm + residual launch leave behind); its output passes the layer
        norm and joins the residual times ``residual_mult`` in one launch. ``after_layer(run, x)``: a hook that sees
        the residual (T, width) after each layer run (for tests)."""
        cfg = self.config
        want16 = step.T > 8 and self.dtype == torch.bfloat16
        got = seq_ops.embed_pos(step.tokens, step.pos, self.embed, self.pos_table, cfg.embedding_scale, bf16_copy=want16)
        x, x16 = got if want16 else (got, None)
        for run, layer in enumerate(self.runs):
            for k, sub in enumerate(self.blocks[layer].sublayers()):
                y = sub(x, x16, step, self.caches[run] if k == 0 else None)
                got = seq_ops.layernorm(y, sub.norm_w, sub.norm_b, eps=cfg.norm_eps, x=x, mult=cfg.residual_mult,
                                        bf16_copy=want16)
                x16 = got[1] if want16 else None
            if after_layer is not None:
                after_layer(run, x)
        return x

    def _forward_sandwich(self, step: StepBatch, after_layer=None) -> torch.Tensor:
        """The sandwich layers. Every boundary between two sublayers is one launch: the branch norms and the average of
        a two-branch mixer, the output norm times the layer scale, the residual add, and the next sublayer's normed
        input (for more than 8 rows with bf16 weights only its bf16 copy, unless the next module also reads it in
        fp32). ``after_layer(run, x)``: a hook that sees the residual (T, width) after each layer run (for tests)."""
        eps = self.config.norm_eps
        x = seq_ops.embed(step.tokens, self.embed, self.config.embedding_scale)
        chain = [(run, sub, self.caches[run] if k == 0 else None)
                 for run, layer in enumerate(self.runs) for k, sub in enumerate(self.blocks[layer].sublayers())]

        def reads(sub):  # (fp32 input wanted, bf16 copy wanted)
            b16 = sub.wants_bf16(step.T)
            return (not b16) or getattr(sub.module, "reads_f32", False), b16

        f32, b16 = reads(chain[0][1])
        h, h16 = seq_ops.sandwich_step(x, next_w=chain[0][1].norm_w, eps=eps, want_f32=f32, bf16_copy=b16)
        for n, (run, sub, cache) in enumerate(chain):
            branches, coef = sub(h, h16, step, cache)
            nxt = chain[n + 1][1] if n + 1 < len(chain) else None
            f32, b16 = reads(nxt) if nxt is not None else (False, False)
            h, h16 = seq_ops.sandwich_step(x, branches=branches, coef=coef, post_w=sub.post_w,
                                           next_w=nxt.norm_w if nxt is not None else None, eps=eps, want_f32=f32,
                                           bf16_copy=b16)
            if after_layer is not None and (nxt is None or chain[n + 1][0] != run):
                after_layer(run, x)
        return x

    def _forward_streams(self, step: StepBatch, after_layer=None) -> torch.Tensor:
        """The sequential layers over the residual streams. Every boundary between two sublayers is one launch: the
        write-back of the one that ran (streams mixed, output added) and the weighted read + norm of the next. The
        last boundary reads the plain sum of the streams, which is returned. ``after_layer(run, x)``: a hook that
        sees the streams (T, s, width) after each layer run (for tests; it costs one extra launch per layer)."""
        eps = self.config.norm_eps
        x = seq_ops.embed_streams(step.tokens, self.embed, self.config.embedding_scale, self.config.streams)
        chain = [(run, sub, self.caches[run] if k == 0 else None)
                 for run, layer in enumerate(self.runs) for k, sub in enumerate(self.blocks[layer].sublayers())]
        first = chain[0][1]
        got = seq_ops.streams_step(x, read=first.links.read, norm_w=first.norm_w, eps=eps,
                                   bf16_copy=first.wants_bf16(step.T))
        for n, (run, sub, cache) in enumerate(chain):
            h, h16 = got if isinstance(got, tuple) else (got, None)
            y = sub(h, h16, step, cache)
            nxt = chain[n + 1] if n + 1 < len(chain) else None
            if after_layer is not None and (nxt is None or nxt[0] != run):
                seq_ops.streams_step(x, y=y, mix=sub.links.mix, out=sub.links.write)
                after_layer(run, x)
                y = None
            kw = dict(y=y, mix=sub.links.mix, out=sub.links.write) if y is not None else {}
            if nxt is None:
                return seq_ops.streams_step(x, read=self.stream_ones, **kw)
            got = seq_ops.streams_step(x, read=nxt[1].links.read, norm_w=nxt[1].norm_w, eps=eps,
                                       bf16_copy=nxt[1].wants_bf16(step.T), **kw)
        raise AssertionError("unreachable")

    @torch.inference_mode()
    def logits(self, x: torch.Tensor, rows: Optional[torch.Tensor] = None) -> torch.Tensor:
        """Final norm and the output product (the embedding table itself, or the design's own matrix) for the given
        rows of the stream (int32 indices; all if None)."""
        if rows is not None:
            x = seq_ops.gather_rows(x, rows)
        if self.final_norm is None:
            h = seq_ops.layernorm(x, self.final_weight, self.final_bias, eps=self.config.norm_eps)
        else:
            h = self.final_norm(x)
        table = self.embed if self.head is None else self.head
        V, W = table.shape
        out = torch.empty(h.shape[0], V, dtype=torch.float32, device=h.device)
        seq_ops.linear(h, table, M=h.shape[0], N=V, K=W, y=out, lda=W, ldy=V)
        if self.config.logit_softcap > 0.0:
            seq_ops.softcap(out, self.config.logit_softcap)
        return out

    def forward(self, idx: torch.Tensor, input_pos: Optional[torch.Tensor] = None, *,
                last_token_only: bool = False) -> torch.Tensor:
        """``GPT.forward``'s calling convention for one sequence in slot 0: (1, T) ids at positions ``input_pos`` (consecutive;
        default 0..T-1, which starts the sequence anew) -> (1, T, vocab) fp32 logits, or (1, 1, vocab)."""
        B, T = idx.shape
        if B != 1:
            raise NotImplementedError("forward() serves one sequence; batches go through generate.batch.BatchEngine")
        dev = idx.device
        if self.caches is None:
            if input_pos is not None:
                raise TypeError("You need to call `set_kv_cache()`")
            self.set_kv_cache(1, max(T, self._max_seq_length))
        if T > self._max_seq_length:
            raise ValueError(f"Cannot forward sequence of length {T}, max seq length is only {self._max_seq_length}.")
        pos = (torch.arange(T, device=dev) if input_pos is None else input_pos.to(dev)).to(torch.int32).contiguous()
        zero = torch.zeros(1, dtype=torch.int32, device=dev)
        step = StepBatch(idx.reshape(-1).to(torch.int32).contiguous(), zero.expand(T).contiguous(), pos,
                         torch.tensor([0, T], dtype=torch.int32, device=dev), zero, pos[:1], T=T, B=1)
        x = self.forward_step(step)
        if last_token_only:
            x = x[-1:].contiguous()
        return self.logits(x).unsqueeze(0)
