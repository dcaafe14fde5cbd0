"""Sequence mixers, feed-forwards and the per-layer token input of the layered models, on ``liblitgpt_seq.so``.

Every module here reads one shared input projection: a layer's norm output ``h`` goes through ONE product with the
row-wise concatenation of all the matrices that read it (the mixer's q / k / v / gate or q / latent / gate, the dense
gate and up matrices, the router), and each module finds its columns in the result by offset. ``in_parts`` lists a
module's rows of that matrix, ``bind`` tells it where they landed. Outputs are accumulated into the fp32 residual
stream ``x`` by the epilogue of the out-projection (or the expert combine), so a layer needs no add kernel.

Mixers here: ``Retention`` (and its preset ``Lightning``: the constant-decay rule on activated projections),
``LatentAttention``, ``DiffAttention``, ``SelectiveScan``, ``GatedDelta`` (the gated delta rule with a decay per head or
per head and key channel), ``GatedLinearAttention`` (the gated rule without the correction), ``SinkAttention`` (one-map
softmax attention: optional q / k norms, rotary positions, a query temperature, a learned or constant sink, values that
are the keys, a gate per head) and ``ParallelMixer`` (two of them side by side on one input projection).

A step is a packed batch (``StepBatch``): the tokens of all sequences row after row, with per-token cache slot and
position and per-sequence row range, slot and first position, all int32 on the device. Sizes, decays, scales, rotary
dims / bases and layouts are constructor parameters; nothing is fixed to one model.
"""

from __future__ import annotations

import math
from dataclasses import dataclass
from typing import Dict, List, Optional, Sequence, Tuple

import torch
import torch.nn as nn

from lit_gpt import seq_ops
from lit_gpt.config import FeedForwardSpec, MixerSpec
from lit_gpt.model import CachePair, HeadKVCache, LatentKVCache, RetentionState, ScanState


@dataclass
class StepBatch:
    tokens: torch.Tensor  # (T,) int32
    slot: torch.Tensor  # (T,) cache slot of each token's sequence
    pos: torch.Tensor  # (T,) position of each token in its sequence
    seq_start: torch.Tensor  # (B + 1,) first row of each sequence, then T
    seq_slot: torch.Tensor  # (B,)
    seq_pos0: torch.Tensor  # (B,) position of each sequence's first row
    T: int
    B: int
    max_len: int = 0  # the most tokens any sequence brings to this step (host side; 0: unknown, taken as T)

    @classmethod
    def build(cls, entries: Sequence[Tuple[int, int, Sequence[int]]], device: torch.device) -> "StepBatch":
        """entries: (slot, first position, token ids) per sequence; one host -> device copy for the whole table."""
        tokens, slot, pos, start, sslot, spos = [], [], [], [0], [], []
        for s, p0, toks in entries:
            n = len(toks)
            if n == 0:
                raise ValueError("a sequence brings no tokens to this step")
            tokens += list(toks)
            slot += [s] * n
            pos += range(p0, p0 + n)
            start.append(start[-1] + n)
            sslot.append(s)
            spos.append(p0)
        T, B = len(tokens), len(entries)
        flat = torch.tensor(tokens + slot + pos + start + sslot + spos, dtype=torch.int32).to(device)
        cut = [T, T, T, B + 1, B, B]
        parts = torch.split(flat, cut)
        return cls(*parts, T=T, B=B, max_len=max(len(e[2]) for e in entries))


def _f32(t: torch.Tensor, device) -> torch.Tensor:
    return t.to(device=device, dtype=torch.float32).contiguous()


def _tiles16(rows: int, weight: torch.Tensor) -> bool:
    """Whether a product of ``rows`` rows with ``weight`` runs bf16 MFMA tiles (more than 8 rows, bf16 weights): its
    producer then hands over the operand already rounded to bf16, at half the traffic."""
    return rows > 8 and weight.dtype == torch.bfloat16


class InputReader(nn.Module):
    """A module that reads columns of the layer's shared input projection."""

    def in_parts(self) -> List[Tuple[str, torch.Tensor]]:
        raise NotImplementedError

    def bind(self, offsets: Dict[str, int]) -> None:
        self.off = dict(offsets)

    def wants_proj(self, rows: int) -> bool:
        """Whether a step of ``rows`` tokens needs the shared input projection made for this module."""
        return True


class Retention(InputReader):
    """A per-head outer-product memory with a constant decay, read by the query (linear attention, scores neither
    normalised nor soft-maxed): per head S_t = decay S_{t-1} + k_t v_t^T,
    o_t = S_t^T q_t, rotary positions (pairs i, i + dims/2) on q and k, k scaled by ``k_scale``; each head's output is
    divided by its root mean square, gated with silu(W_g h) and projected.

    Options (the "lightning" kind sets them): ``act`` an activation on q, k and v as projected; ``k_scale`` (default
    dim^-1/2); ``joint_norm`` the concatenated heads are RMS-normed together with the weight ``norm`` (H dv values)
    instead of head by head without one; ``gate_act`` the gate's activation."""

    def __init__(self, spec: MixerSpec, width: int, eps: float, w: Dict[str, torch.Tensor], device, dtype, *,
                 act: int = seq_ops.ACT_NONE, k_scale: Optional[float] = None, joint_norm: bool = False,
                 gate_act: int = seq_ops.ACT_SILU) -> None:
        super().__init__()
        self.H, self.d, self.dv, self.eps = spec.heads, spec.dim, spec.vdim, eps
        self.rot_dims = spec.rot.dims
        self.k_scale = float(spec.dim) ** -0.5 if k_scale is None else float(k_scale)
        self.act, self.joint_norm, self.gate_act = act, joint_norm, gate_act
        H, d, dv = self.H, self.d, self.dv
        self.register_buffer("norm_w", None)
        if joint_norm:
            if w["norm"].numel() != H * dv:
                raise ValueError(f"{spec.kind}.norm: {w['norm'].numel()} values, expected {H * dv}")
            self.norm_w = _f32(w["norm"], device)
        for name, rows in (("q", H * d), ("k", H * d), ("v", H * dv), ("g", H * dv)):
            if tuple(w[name].shape) != (rows, width):
                raise ValueError(f"retention.{name}: shape {tuple(w[name].shape)}, expected {(rows, width)}")
        self._in = [(n, w[n]) for n in ("q", "k", "v", "g")]
        self.register_buffer("w_o", w["o"].to(device=device, dtype=dtype).contiguous())
        self.register_buffer("decay", torch.tensor(spec.decay, dtype=torch.float64).to(device=device, dtype=torch.float32))
        self.register_buffer("inv_freq", torch.tensor(spec.rot.inv_freq() or [1.0], dtype=torch.float64)
                             .to(device=device, dtype=torch.float32))

    def in_parts(self):
        return self._in

    def build_cache(self, slots: int, max_seq_length: int, device, dtype) -> RetentionState:
        return RetentionState(slots, self.H, self.d, self.dv, device=device)

    def forward(self, proj: torch.Tensor, step: StepBatch, cache: RetentionState, x: torch.Tensor,
                accumulate: bool = True, post: float = 1.0) -> None:
        H, dv = self.H, self.dv
        o = seq_ops.retention(proj, self.off["q"], self.off["k"], self.off["v"], cache.s, self.decay, self.inv_freq,
                              step.seq_start, step.seq_slot, step.seq_pos0, H=H, d=self.d, dv=dv,
                              rot_dims=self.rot_dims, k_scale=self.k_scale, max_len=step.max_len, pos=step.pos,
                              act=self.act)
        if self.joint_norm:  # one "head" of H dv values with a weight
            o = seq_ops.head_gate(o, proj, self.off["g"], H=1, dv=H * dv, unit_norm=True, eps=self.eps,
                                  act=self.gate_act, weight=self.norm_w, post=post,
                                  bf16_copy=_tiles16(step.T, self.w_o))
        else:
            o = seq_ops.head_gate(o, proj, self.off["g"], H=H, dv=dv, unit_norm=True, eps=self.eps, act=self.gate_act,
                                  post=post, bf16_copy=_tiles16(step.T, self.w_o))
        W = x.shape[1]
        seq_ops.linear(o, self.w_o, M=step.T, N=W, K=H * dv, y=x, lda=H * dv, ldy=W, accumulate=accumulate)


class LatentAttention(InputReader):
    """Causal softmax attention whose keys and values are expanded from a cached low-rank latent c (RMS-normed) and
    one rotated key part shared by all heads (interleaved rotary pairs 2i, 2i + 1). The score of head h is
    (q_h . W_uk,h c + q_rot,h . k_rot) * scale; a learned per-head sink scalar adds its exponential to the softmax normaliser. The kernels never expand
    keys or values: the query is mapped through W_uk,h first (one product per head), attention runs over the cached
    rows [c | k_rot] for all heads alike, and W_uv,h maps the weighted latent back. Output gate sigmoid(W_g h)."""

    def __init__(self, spec: MixerSpec, width: int, eps: float, w: Dict[str, torch.Tensor], device, dtype) -> None:
        super().__init__()
        self.H, self.d, self.dr, self.dv, self.r = spec.heads, spec.dim, spec.rot_dim, spec.vdim, spec.kv_rank
        self.eps, self.scale, self.rot_dims, self.dtype = eps, spec.scale, spec.rot.dims, dtype
        H, d, dr, dv, r = self.H, self.d, self.dr, self.dv, self.r
        for name, shape in (("q", (H * (d + dr), width)), ("dkv", (r + dr, width)), ("g", (H * dv, width)),
                            ("uk", (H * d, r)), ("uv", (H * dv, r)), ("o", (width, H * dv))):
            if tuple(w[name].shape) != shape:
                raise ValueError(f"latent_attention.{name}: shape {tuple(w[name].shape)}, expected {shape}")
        self._in = [(n, w[n]) for n in ("q", "dkv", "g")]
        # per head (r, d): the key up-projection transposed, so that q_h (d values) maps to r latent coordinates
        self.register_buffer("w_ukT", w["uk"].to(device=device, dtype=dtype).view(H, d, r).transpose(1, 2).contiguous())
        self.register_buffer("w_uv", w["uv"].to(device=device, dtype=dtype).contiguous())
        self.register_buffer("w_o", w["o"].to(device=device, dtype=dtype).contiguous())
        self.register_buffer("norm_w", _f32(w["dkv.norm"], device))
        self.register_buffer("sink", _f32(w["sink"], device) if "sink" in w else None)
        self.register_buffer("inv_freq", torch.tensor(spec.rot.inv_freq() or [1.0], dtype=torch.float64)
                             .to(device=device, dtype=torch.float32))

    def in_parts(self):
        return self._in

    def build_cache(self, slots: int, max_seq_length: int, device, dtype) -> LatentKVCache:
        return LatentKVCache(slots, max_seq_length, self.r, self.dr, device=device, dtype=dtype)

    def forward(self, proj: torch.Tensor, step: StepBatch, cache: LatentKVCache, x: torch.Tensor,
                accumulate: bool = True) -> None:
        H, d, dr, dv, r = self.H, self.d, self.dr, self.dv, self.r
        T, ld = proj.shape
        q_off = self.off["q"]
        seq_ops.latent_prepare(proj, q_off, self.off["dkv"], cache.c, cache.kr, self.norm_w, self.inv_freq, step.slot,
                               step.pos, H=H, d=d, dr=dr, r=r, rot_dims=self.rot_dims, eps=self.eps)
        qc = torch.empty(T, H * r, dtype=torch.float32, device=proj.device)
        seq_ops.linear(proj, self.w_ukT, M=T, N=r, K=d, y=qc, a_off=q_off, lda=ld, ldy=H * r, batch=H,
                       stride_a=d + dr, stride_w=r * d, stride_y=r)
        if r % 64 == 0 and r <= 512 and T >= 8 * step.B:  # a prompt: 16-token tiles on the matrix cores
            lat = seq_ops.latent_attention_tiles(qc, proj, q_off, cache.c, cache.kr, self.sink, step.seq_start,
                                                 step.seq_slot, step.seq_pos0, step.max_len or T, H=H, d=d, dr=dr,
                                                 r=r, scale=self.scale)
        else:
            lat = seq_ops.latent_attention(qc, proj, q_off, cache.c, cache.kr, self.sink, step.slot, step.pos, H=H,
                                           d=d, dr=dr, r=r, scale=self.scale)
        att = torch.empty(T, H * dv, dtype=torch.float32, device=proj.device)
        seq_ops.linear(lat, self.w_uv, M=T, N=dv, K=r, y=att, lda=H * r, ldy=H * dv, batch=H, stride_a=r,
                       stride_w=dv * r, stride_y=dv)
        att = seq_ops.head_gate(att, proj, self.off["g"], H=H, dv=dv, unit_norm=False, eps=self.eps,
                                act=seq_ops.ACT_SIGMOID, bf16_copy=_tiles16(T, self.w_o))
        W = x.shape[1]
        seq_ops.linear(att, self.w_o, M=T, N=W, K=H * dv, y=x, lda=H * dv, ldy=W, accumulate=accumulate)


class DiffAttention(InputReader):
    """Differential softmax attention with grouped key / value heads. Every query head carries two maps (the q and k
    rows of a head hold map 1 then map 2, ``dim`` rows each); both attend over the same values and are combined as
    o = a1 - lambda a2 with lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + diff (one number per layer), after which the
    head's output is divided by its root mean square and scaled by 1 - diff. Scores (q . k) * scale pass an optional
    tanh soft cap; rotary positions on interleaved pairs (2i, 2i + 1) of the first rot.dims dims of every map; a
    query sees the keys before it in its own chunk of ``mask_size`` positions, chunks aligned to position 0 (0: all
    keys before it). With ``kv_from`` the layer has no key / value projections and attends over the named layer's
    cache (rotated keys, values) with its own queries, mask and constants."""

    def __init__(self, spec: MixerSpec, width: int, eps: float, w: Dict[str, torch.Tensor], device, dtype) -> None:
        super().__init__()
        self.H, self.G, self.d, self.dv, self.eps = spec.heads, spec.kv_heads, spec.dim, spec.vdim, eps
        self.scale, self.cap, self.diff, self.chunk = spec.scale, spec.softcap, spec.diff, spec.mask_size
        self.rot_dims, self.kv_from = spec.rot.dims, spec.kv_from
        H, G, d, dv = self.H, self.G, self.d, self.dv
        shapes = [("q", (2 * H * d, width)), ("o", (width, H * dv))]
        if self.kv_from is None:
            shapes += [("k", (2 * G * d, width)), ("v", (G * dv, width))]
        for name, shape in shapes:
            if tuple(w[name].shape) != shape:
                raise ValueError(f"attention.{name}: shape {tuple(w[name].shape)}, expected {shape}")
        for name in ("lq1", "lk1", "lq2", "lk2"):
            if w[name].numel() != d:
                raise ValueError(f"attention.{name}: {w[name].numel()} values, expected {d}")
        self._in = [(n, w[n]) for n in (("q", "k", "v") if self.kv_from is None else ("q",))]
        dot = lambda a, b: float((w[a].double() * w[b].double()).sum())  # noqa: E731
        self.lam = math.exp(dot("lq1", "lk1")) - math.exp(dot("lq2", "lk2")) + self.diff
        self.register_buffer("w_o", w["o"].to(device=device, dtype=dtype).contiguous())
        self.register_buffer("inv_freq", torch.tensor(spec.rot.inv_freq() or [1.0], dtype=torch.float64)
                             .to(device=device, dtype=torch.float32))

    def in_parts(self):
        return self._in

    def build_cache(self, slots: int, max_seq_length: int, device, dtype) -> HeadKVCache:
        return HeadKVCache(slots, max_seq_length, self.G, 2 * self.d, self.dv, device=device, dtype=dtype)

    def forward(self, proj: torch.Tensor, step: StepBatch, cache: HeadKVCache, x: torch.Tensor,
                accumulate: bool = True) -> None:
        H, G, d, dv = self.H, self.G, self.d, self.dv
        own = self.kv_from is None
        seq_ops.diffattn_prepare(proj, self.off["q"], self.off["k"] if own else -1, self.off["v"] if own else -1,
                                 cache.k, cache.v, self.inv_freq, step.slot, step.pos, H=H, G=G, d=d, dv=dv,
                                 rot_dims=self.rot_dims)
        att = seq_ops.diffattn(proj, self.off["q"], cache.k, cache.v, step.seq_start, step.seq_slot, step.seq_pos0,
                               step.max_len or step.T, H=H, G=G, d=d, dv=dv, chunk=self.chunk, scale=self.scale,
                               cap=self.cap, lam=self.lam, eps=self.eps, post=1.0 - self.diff,
                               bf16_copy=_tiles16(step.T, self.w_o))
        W = x.shape[1]
        seq_ops.linear(att, self.w_o, M=step.T, N=W, K=H * dv, y=x, lda=H * dv, ldy=W, accumulate=accumulate)


class SelectiveScan(InputReader):
    """Selective state-space mixer in the Mamba-2 form. One input projection whose rows are ordered
    [z | x | B | C | dt] (inner = heads * vdim gate and value columns, groups * state columns each for B and C, one step size per head); x, B and C
    pass a short causal per-channel convolution and silu; dt = softplus(dt + bias); per head (heads share B and C in
    groups) S_t = exp(-exp(A_log) dt_t) S_{t-1} + dt_t B_t x_t^T, y_t = S_t^T C_t + D x_t; y is gated with silu(z),
    divided by its root mean square in ``norm_groups`` equal parts, weighted and projected. The state (S and the
    convolution's last taps - 1 inputs) is fp32 and lives in a cache slot."""

    def __init__(self, spec: MixerSpec, width: int, eps: float, w: Dict[str, torch.Tensor], device, dtype) -> None:
        super().__init__()
        self.H, self.dv, self.N, self.G, self.taps = spec.heads, spec.vdim, spec.state, spec.groups, spec.conv
        self.norm_groups, self.eps = spec.norm_groups, eps
        inner, bc = self.H * self.dv, 2 * self.G * self.N
        self.inner, self.channels = inner, inner + bc
        for name, shape in (("in", (2 * inner + bc + self.H, width)), ("conv", (inner + bc, self.taps)),
                            ("conv.b", (inner + bc,)), ("dt_bias", (self.H,)), ("A_log", (self.H,)), ("D", (self.H,)),
                            ("norm", (inner,)), ("o", (width, inner))):
            if tuple(w[name].shape) != shape:
                raise ValueError(f"mamba2.{name}: shape {tuple(w[name].shape)}, expected {shape}")
        self._in = [("in", w["in"])]
        self.register_buffer("conv_w", w["conv"].to(device=device, dtype=dtype).contiguous())
        self.register_buffer("conv_b", w["conv.b"].to(device=device, dtype=dtype).contiguous())
        for name, key in (("dt_bias", "dt_bias"), ("A_log", "A_log"), ("D", "D"), ("norm_w", "norm")):
            self.register_buffer(name, _f32(w[key], device))
        self.register_buffer("w_o", w["o"].to(device=device, dtype=dtype).contiguous())

    def in_parts(self):
        return self._in

    def build_cache(self, slots: int, max_seq_length: int, device, dtype) -> ScanState:
        return ScanState(slots, self.H, self.N, self.dv, self.taps, self.channels, device=device)

    def forward(self, proj: torch.Tensor, step: StepBatch, cache: ScanState, x: torch.Tensor,
                accumulate: bool = True) -> None:
        base, inner = self.off["in"], self.inner
        tables = (step.seq_start, step.seq_slot, step.seq_pos0)
        xbc = seq_ops.conv_silu(proj, base + inner, self.conv_w, self.conv_b, cache.conv, *tables,
                                step.max_len or step.T)
        y = seq_ops.ssm_scan(xbc, proj, base + inner + self.channels, self.dt_bias, self.A_log, self.D, cache.s,
                             *tables, heads=self.H, groups=self.G, N=self.N, dv=self.dv,
                             max_len=step.max_len or step.T)
        g = seq_ops.gated_group_norm(y, proj, base, self.norm_w, groups=self.norm_groups, eps=self.eps,
                                     bf16_copy=_tiles16(step.T, self.w_o))
        W = x.shape[1]
        seq_ops.linear(g, self.w_o, M=step.T, N=W, K=inner, y=x, lda=inner, ldy=W, accumulate=accumulate)


class GatedDelta(InputReader):
    """The gated delta rule: per head an outer-product memory S (dim x vdim, fp32) that is decayed, corrected towards
    the current key's value and read by the query: S <- diag(g) S; u = beta (v - S^T k); S <- S + k u^T; o = S^T q.
    q and k (``kv_heads`` heads shared by groups of value heads) and v pass a short causal per-channel convolution
    (tap ``taps - 1`` weights the token itself, no bias) and silu; q and k become unit vectors per head
    (x / sqrt(sum x^2 + 1e-6)), q also times dim^-1/2; beta = sigmoid(W_b h); g = exp(-exp(A_log) softplus(a + dt_bias)).
    ``per_channel``: a = W_a2 (W_a1 h) with one decay per head and key channel and the output gate is
    sigmoid(W_g2 (W_g1 h)); otherwise a = W_a h with one decay per head and the gate is silu(W_g h). Each head's output
    is divided by its root mean square, times a weight shared by the heads, times the gate, then projected. The state
    (S and the convolution's last taps - 1 inputs) lives in a cache slot."""

    FUSED_ROWS = 8  # one-token steps of up to this many sequences take the fused convolution + preparation launch

    def __init__(self, spec: MixerSpec, width: int, eps: float, w: Dict[str, torch.Tensor], device, dtype,
                 per_channel: Optional[bool] = None) -> None:
        super().__init__()
        self.H, self.G, self.d, self.dv, self.taps, self.eps = spec.heads, spec.kv_heads, spec.dim, spec.vdim, spec.conv, eps
        self.per_channel = spec.kind == "channel_delta" if per_channel is None else per_channel
        H, G, d, dv = self.H, self.G, self.d, self.dv
        self.channels = 2 * G * d + H * dv
        shapes = [("q", (G * d, width)), ("k", (G * d, width)), ("v", (H * dv, width)), ("q.conv", (G * d, self.taps)),
                  ("k.conv", (G * d, self.taps)), ("v.conv", (H * dv, self.taps)), ("b", (H, width)), ("A_log", (H,)),
                  ("norm", (dv,)), ("o", (width, H * dv))]
        if self.per_channel:
            ra, rg = w["a1"].shape[0], w["g1"].shape[0]
            shapes += [("a1", (ra, width)), ("a2", (H * d, ra)), ("g1", (rg, width)), ("g2", (H * dv, rg)),
                       ("dt_bias", (H * d,))]
        else:
            shapes += [("a", (H, width)), ("g", (H * dv, width)), ("dt_bias", (H,))]
        for name, shape in shapes:
            if tuple(w[name].shape) != shape:
                raise ValueError(f"{spec.kind}.{name}: shape {tuple(w[name].shape)}, expected {shape}")
        self._in = [("qkv", torch.cat([w["q"], w["k"], w["v"]])), ("b", w["b"])]
        self._in += [("a1", w["a1"]), ("g1", w["g1"])] if self.per_channel else [("a", w["a"]), ("g", w["g"])]
        if self.per_channel:
            self.register_buffer("w_a2", w["a2"].to(device=device, dtype=dtype).contiguous())
            self.register_buffer("w_g2", w["g2"].to(device=device, dtype=dtype).contiguous())
        self.register_buffer("conv_w", torch.cat([w["q.conv"], w["k.conv"], w["v.conv"]]).to(device=device, dtype=dtype)
                             .contiguous())
        self.register_buffer("conv_b", torch.zeros(self.channels, device=device, dtype=dtype))
        for name, key in (("A_log", "A_log"), ("dt_bias", "dt_bias"), ("norm_w", "norm")):
            self.register_buffer(name, _f32(w[key], device))
        self.register_buffer("w_o", w["o"].to(device=device, dtype=dtype).contiguous())

    def in_parts(self):
        return self._in

    def build_cache(self, slots: int, max_seq_length: int, device, dtype) -> ScanState:
        return ScanState(slots, self.H, self.d, self.dv, self.taps, self.channels, device=device)

    def forward(self, proj: torch.Tensor, step: StepBatch, cache: ScanState, x: torch.Tensor, accumulate: bool = True,
                post: float = 1.0) -> None:
        self.project(self.mix(proj, step, cache, post), x, accumulate)

    def project(self, o: torch.Tensor, x: torch.Tensor, accumulate: bool) -> None:
        """The out-projection of the gated head outputs ``o`` (T, H dv) into x (written or accumulated)."""
        T, W = x.shape
        seq_ops.linear(o, self.w_o, M=T, N=W, K=self.H * self.dv, y=x, lda=self.H * self.dv, ldy=W, accumulate=accumulate)

    def mix(self, proj: torch.Tensor, step: StepBatch, cache: ScanState, post: float = 1.0) -> torch.Tensor:
        """Everything before the out-projection: the gated, normed head outputs times ``post`` (T, H dv), fp32 or the
        bf16 copy the out-projection's MFMA tiles read."""
        H, G, d, dv = self.H, self.G, self.d, self.dv
        T, ld = proj.shape
        tables = (step.seq_start, step.seq_slot, step.seq_pos0)
        kw = dict(H=H, G=G, d=d, per_channel=self.per_channel, q_scale=float(d) ** -0.5)
        if step.max_len == 1 and T <= self.FUSED_ROWS and (not self.per_channel or
                                                           max(self.w_a2.shape[1], self.w_g2.shape[1]) <= 512):
            # one token per sequence (decode): convolution + preparation in one launch, and the second maps of the
            # low-rank decay and gate inside the kernels that consume them
            a_off = self.off["a1"] if self.per_channel else self.off["a"]
            w2 = (self.w_a2, self.w_g2) if self.per_channel else (None, None)
            qkv, dec, beta, kq = seq_ops.delta_step_prepare(proj, self.off["qkv"], self.conv_w, cache.conv, step.seq_slot,
                                                            step.seq_pos0, a_off, self.off["b"], self.A_log,
                                                            self.dt_bias, dv=dv, w_a2=w2[0], **kw)
            gate, g_off, g2 = proj, (self.off["g1"] if self.per_channel else self.off["g"]), w2[1]
        else:
            qkv = seq_ops.conv_silu(proj, self.off["qkv"], self.conv_w, self.conv_b, cache.conv, *tables,
                                    step.max_len or T)
            if self.per_channel:
                ra, rg = self.w_a2.shape[1], self.w_g2.shape[1]
                a = torch.empty(T, H * d, dtype=torch.float32, device=proj.device)
                seq_ops.linear(proj, self.w_a2, M=T, N=H * d, K=ra, y=a, a_off=self.off["a1"], lda=ld, ldy=H * d)
                gate = torch.empty(T, H * dv, dtype=torch.float32, device=proj.device)
                seq_ops.linear(proj, self.w_g2, M=T, N=H * dv, K=rg, y=gate, a_off=self.off["g1"], lda=ld, ldy=H * dv)
                a_off, g_off = 0, 0
            else:
                a, a_off, gate, g_off = proj, self.off["a"], proj, self.off["g"]
            g2 = None
            dec, beta, kq = seq_ops.delta_prepare(qkv, a, a_off, proj, self.off["b"], self.A_log, self.dt_bias, **kw)
        o = seq_ops.gated_delta(qkv, dec, beta, kq, cache.s, *tables, H=H, G=G, d=d, dv=dv,
                                per_channel=self.per_channel)
        act = seq_ops.ACT_SIGMOID if self.per_channel else seq_ops.ACT_SILU
        return seq_ops.head_gate(o, gate, g_off, H=H, dv=dv, unit_norm=True, eps=self.eps, act=act, weight=self.norm_w,
                                 post=post, bf16_copy=_tiles16(T, self.w_o), w_g2=g2)


class SinkAttention(InputReader):
    """Causal softmax attention with grouped key / value heads and no rotation: q and k are divided by their root
    mean square per head (no weight), the query is multiplied by a temperature that grows with its position,
    1 + coef * ln(floor((p + 1) / every) + 1); score = (q . k) * scale; a learned per-head sink scalar adds its
    exponential to the softmax normaliser without contributing a value. The cache holds the normed keys and the
    values.

    The spec's options make its relatives: ``qk_norm`` "none" / "unit" / "weight" (times ``q.norm`` / ``k.norm``, d
    values shared by the heads); rotary positions on the pairs (i, i + rot.dims / 2) of the first ``rot.dims`` dims
    after the norm (frequencies optionally rescaled band by band); ``sink_kind`` "none" / "learned" / "one" (a sink of
    score 0: the denominator is 1 + sum exp); ``values`` "keys": no value projection, the values are the keys as
    projected, before their norm; ``head_gate``: head h's output times sigmoid(W_g h)_h, one number per head."""

    def __init__(self, spec: MixerSpec, width: int, eps: float, w: Dict[str, torch.Tensor], device, dtype) -> None:
        super().__init__()
        self.H, self.G, self.d, self.dv, self.eps = spec.heads, spec.kv_heads, spec.dim, spec.vdim, eps
        self.scale, self.cap, self.chunk = spec.scale, spec.softcap, spec.mask_size
        self.temp_coef, self.temp_every = spec.q_temp_coef, spec.q_temp_every
        self.qk_norm, self.own_values, self.head_gate = spec.qk_norm, spec.values == "own", spec.head_gate
        self.rot_dims = spec.rot.dims
        H, G, d, dv = self.H, self.G, self.d, self.dv
        shapes = [("q", (H * d, width)), ("k", (G * d, width)), ("o", (width, H * dv))]
        shapes += [("v", (G * dv, width))] if self.own_values else []
        shapes += [("g", (H, width))] if self.head_gate else []
        for name, shape in shapes:
            if tuple(w[name].shape) != shape:
                raise ValueError(f"{spec.kind}.{name}: shape {tuple(w[name].shape)}, expected {shape}")
        if not self.own_values and dv != d:
            raise ValueError(f"{spec.kind}: values that are the keys have the keys' size")
        self._in = [(n, w[n]) for n in (("q", "k", "v") if self.own_values else ("q", "k"))]
        self._in += [("g", w["g"])] if self.head_gate else []
        self.register_buffer("sink", None)
        if spec.sink_kind == "one":
            self.sink = torch.zeros(H, dtype=torch.float32, device=device)
        elif spec.sink_kind == "learned" and "sink" in w:
            if w["sink"].numel() != H:
                raise ValueError(f"{spec.kind}.sink: {w['sink'].numel()} values, expected {H}")
            self.sink = _f32(w["sink"], device)
        self.register_buffer("q_norm", None)
        self.register_buffer("k_norm", None)
        if self.qk_norm == "weight":
            if w["q.norm"].numel() != d or w["k.norm"].numel() != d:
                raise ValueError(f"{spec.kind}: q.norm / k.norm hold {d} values")
            self.q_norm, self.k_norm = _f32(w["q.norm"], device), _f32(w["k.norm"], device)
        self.register_buffer("inv_freq", None)
        if self.rot_dims > 0:
            self.inv_freq = torch.tensor(spec.rot.inv_freq(), dtype=torch.float64).to(device=device, dtype=torch.float32)
        self.register_buffer("w_o", w["o"].to(device=device, dtype=dtype).contiguous())

    def in_parts(self):
        return self._in

    def build_cache(self, slots: int, max_seq_length: int, device, dtype) -> HeadKVCache:
        return HeadKVCache(slots, max_seq_length, self.G, self.d, self.dv, device=device, dtype=dtype)

    def forward(self, proj: torch.Tensor, step: StepBatch, cache: HeadKVCache, x: torch.Tensor, accumulate: bool = True,
                post: float = 1.0) -> None:
        H, G, d, dv = self.H, self.G, self.d, self.dv
        seq_ops.normattn_prepare(proj, self.off["q"], self.off["k"], self.off["v" if self.own_values else "k"], cache.k,
                                 cache.v, step.slot, step.pos, H=H, G=G, d=d, dv=dv, eps=self.eps,
                                 temp_coef=self.temp_coef, temp_every=self.temp_every, norm=self.qk_norm != "none",
                                 q_weight=self.q_norm, k_weight=self.k_norm, inv_freq=self.inv_freq,
                                 rot_dims=self.rot_dims)
        att = seq_ops.sinkattn(proj, self.off["q"], cache.k, cache.v, self.sink, step.seq_start, step.seq_slot,
                               step.seq_pos0, step.max_len or step.T, H=H, G=G, d=d, dv=dv, scale=self.scale,
                               chunk=self.chunk, cap=self.cap, post=post, bf16_copy=_tiles16(step.T, self.w_o),
                               gate_off=self.off["g"] if self.head_gate else -1)
        W = x.shape[1]
        seq_ops.linear(att, self.w_o, M=step.T, N=W, K=H * dv, y=x, lda=H * dv, ldy=W, accumulate=accumulate)


class GatedLinearAttention(InputReader):
    """Linear attention with a decay per head and key channel and no correction towards the key's value: per head
    S <- diag(alpha) S + k v^T, o = S^T q (the state S is dim x vdim, fp32, in a cache slot), q = W_q h * dim^-1/2,
    alpha = sigmoid(W_a2 (W_a1 h) + b)^(1 / tau) (a low-rank pair of maps with a bias). Each head's output is RMS-normed
    over vdim with one weight vector for all heads, multiplied by silu(W_g h) and projected. The recurrence is the gated
    delta rule's kernel without its correction, token by token in every step kind."""

    def __init__(self, spec: MixerSpec, width: int, eps: float, w: Dict[str, torch.Tensor], device, dtype) -> None:
        super().__init__()
        self.H, self.d, self.dv, self.eps, self.tau = spec.heads, spec.dim, spec.vdim, eps, float(spec.tau)
        H, d, dv = self.H, self.d, self.dv
        rank = w["a1"].shape[0]
        for name, shape in (("q", (H * d, width)), ("k", (H * d, width)), ("v", (H * dv, width)), ("g", (H * dv, width)),
                            ("a1", (rank, width)), ("a2", (H * d, rank)), ("a2.b", (H * d,)), ("norm", (dv,)),
                            ("o", (width, H * dv))):
            if tuple(w[name].shape) != shape:
                raise ValueError(f"{spec.kind}.{name}: shape {tuple(w[name].shape)}, expected {shape}")
        self._in = [("qkv", torch.cat([w["q"], w["k"], w["v"]])), ("g", w["g"]), ("a1", w["a1"])]
        self.register_buffer("w_a2", w["a2"].to(device=device, dtype=dtype).contiguous())
        self.register_buffer("a_bias", _f32(w["a2.b"], device))
        self.register_buffer("norm_w", _f32(w["norm"], device))
        self.register_buffer("w_o", w["o"].to(device=device, dtype=dtype).contiguous())

    def in_parts(self):
        return self._in

    def build_cache(self, slots: int, max_seq_length: int, device, dtype) -> RetentionState:
        return RetentionState(slots, self.H, self.d, self.dv, device=device)

    def forward(self, proj: torch.Tensor, step: StepBatch, cache: RetentionState, x: torch.Tensor,
                accumulate: bool = True, post: float = 1.0) -> None:
        H, d, dv = self.H, self.d, self.dv
        T, ld = proj.shape
        rank = self.w_a2.shape[1]
        kw = dict(H=H, G=H, d=d, per_channel=True, q_scale=float(d) ** -0.5, unit=False, decay_form=1, tau=self.tau,
                  qkv_off=self.off["qkv"])
        if T <= 8 and rank <= 512:  # few tokens: the second map of the decay inside the preparation launch
            dec, _, kq = seq_ops.delta_prepare(proj, proj, self.off["a1"], None, 0, None, self.a_bias, w_a2=self.w_a2, **kw)
        else:
            a = torch.empty(T, H * d, dtype=torch.float32, device=proj.device)
            seq_ops.linear(proj, self.w_a2, M=T, N=H * d, K=rank, y=a, a_off=self.off["a1"], lda=ld, ldy=H * d)
            dec, _, kq = seq_ops.delta_prepare(proj, a, 0, None, 0, None, self.a_bias, **kw)
        o = seq_ops.gated_delta(proj, dec, None, kq, cache.s, step.seq_start, step.seq_slot, step.seq_pos0, H=H, G=H,
                                d=d, dv=dv, per_channel=True, plain=True, qkv_off=self.off["qkv"])
        o = seq_ops.head_gate(o, proj, self.off["g"], H=H, dv=dv, unit_norm=True, eps=self.eps, act=seq_ops.ACT_SILU,
                              weight=self.norm_w, post=post, bf16_copy=_tiles16(T, self.w_o))
        W = x.shape[1]
        seq_ops.linear(o, self.w_o, M=T, N=W, K=H * dv, y=x, lda=H * dv, ldy=W, accumulate=accumulate)


class Lightning(Retention):
    """The constant-decay rule on activated projections: q = silu(W_q h), k = silu(W_k h), v = silu(W_v h), per head
    S <- decay_h S + k v^T, o = S^T q (no rotation, no key scale); the concatenated heads are RMS-normed together with
    the weight ``norm``, multiplied by sigmoid(W_g h) and projected."""

    def __init__(self, spec: MixerSpec, width: int, eps: float, w: Dict[str, torch.Tensor], device, dtype) -> None:
        super().__init__(spec, width, eps, w, device, dtype, act=seq_ops.ACT_SILU, k_scale=1.0, joint_norm=True,
                         gate_act=seq_ops.ACT_SIGMOID)


class ParallelMixer(InputReader):
    """Two mixers side by side on the same input (tensors under ``left.`` and ``right.``; which kinds, the spec says:
    a sink attention beside a gated delta rule, a rotary attention beside a gated linear attention, ...). Both read
    the layer's one input projection. Plain form: ``left_scale`` * left + ``right_scale`` * right, each factor applied
    where its mixer's last elementwise kernel runs, the second out-projection accumulating onto the first. With
    ``branch_norm`` each branch's output is first RMS-normed over the width with its own weight (``left.out`` /
    ``right.out``): the branches then go to buffers of their own and ``branches()`` hands them, with the weights, to the
    layer's norm + residual launch, which also forms the weighted sum. With ``overlap`` the right mixer's kernels of a
    prompt step run on a second HIP stream (default priority) beside the left's: they touch disjoint columns of the
    projection and different caches; the second stream starts after the projection and is joined before the two
    outputs meet."""

    overlap = True
    OVERLAP_ROWS = 8  # steps of up to this many rows stay on one stream (a captured one-token step gains nothing)
    _side: Dict[int, "torch.cuda.Stream"] = {}

    def __init__(self, spec: MixerSpec, width: int, eps: float, w: Dict[str, torch.Tensor], device, dtype) -> None:
        super().__init__()
        sub = lambda prefix: {k[len(prefix):]: v for k, v in w.items() if k.startswith(prefix)}  # noqa: E731
        self.left = MIXERS[spec.left.kind](spec.left, width, eps, sub("left."), device, dtype)
        self.right = MIXERS[spec.right.kind](spec.right, width, eps, sub("right."), device, dtype)
        self.left_scale, self.right_scale = spec.left_scale, spec.right_scale
        self.branch_norm = spec.branch_norm
        self.register_buffer("left_out", None)
        self.register_buffer("right_out", None)
        if self.branch_norm:
            if spec.left_scale != spec.right_scale:
                raise NotImplementedError("normed branches are summed with one common factor")
            if w["left.out"].numel() != width or w["right.out"].numel() != width:
                raise ValueError("parallel.left.out / right.out: one weight per channel of the model's width")
            self.left_out, self.right_out = _f32(w["left.out"], device), _f32(w["right.out"], device)

    def in_parts(self):
        return [("left." + n, t) for n, t in self.left.in_parts()] + [("right." + n, t) for n, t in self.right.in_parts()]

    def bind(self, offsets: Dict[str, int]) -> None:
        self.left.bind({k[5:]: v for k, v in offsets.items() if k.startswith("left.")})
        self.right.bind({k[6:]: v for k, v in offsets.items() if k.startswith("right.")})

    def build_cache(self, slots: int, max_seq_length: int, device, dtype) -> CachePair:
        return CachePair(self.left.build_cache(slots, max_seq_length, device, dtype),
                         self.right.build_cache(slots, max_seq_length, device, dtype))

    def _side_stream(self, device) -> "torch.cuda.Stream":
        index = device.index or 0
        side = self._side.get(index)
        if side is None:
            side = self._side[index] = torch.cuda.Stream(device=device)
        return side

    def branches(self, proj: torch.Tensor, step: StepBatch, cache: CachePair, y: torch.Tensor):
        """The normed form: the left mixer's output goes to ``y``, the right's to a buffer of its own; returns
        ([(y_left, w_left), (y_right, w_right)], common factor) for the layer's norm + residual launch."""
        yr = torch.empty_like(y)
        if not self.overlap or step.T <= self.OVERLAP_ROWS:
            self.left(proj, step, cache.left, y, accumulate=False)
            self.right(proj, step, cache.right, yr, accumulate=False)
        else:
            main = torch.cuda.current_stream(proj.device)
            side = self._side_stream(proj.device)
            side.wait_stream(main)  # the projection is made
            with torch.cuda.stream(side):
                self.right(proj, step, cache.right, yr, accumulate=False)
            self.left(proj, step, cache.left, y, accumulate=False)
            main.wait_stream(side)
        return [(y, self.left_out), (yr, self.right_out)], self.left_scale

    def forward(self, proj: torch.Tensor, step: StepBatch, cache: CachePair, x: torch.Tensor,
                accumulate: bool = True) -> None:
        if self.branch_norm:
            raise RuntimeError("normed branches meet in the layer's norm launch: call branches()")
        if not self.overlap or step.T <= self.OVERLAP_ROWS or not hasattr(self.right, "mix"):
            self.left(proj, step, cache.left, x, accumulate=accumulate, post=self.left_scale)
            self.right(proj, step, cache.right, x, accumulate=True, post=self.right_scale)
            return
        main = torch.cuda.current_stream(proj.device)
        side = self._side_stream(proj.device)
        side.wait_stream(main)  # the projection is made
        with torch.cuda.stream(side):
            o = self.right.mix(proj, step, cache.right, post=self.right_scale)
        self.left(proj, step, cache.left, x, accumulate=accumulate, post=self.left_scale)
        main.wait_stream(side)
        self.right.project(o, x, accumulate=True)


class StreamLinks(nn.Module):
    """The weights that tie one sublayer to a multi-stream residual: ``read`` (s,) weights of the sum the sublayer
    reads, ``write`` (s,) weights of its output in every stream, ``mix`` (s, s) [from, to] applied to the streams
    at the write-back. Without stored weights: all ones (one stream: the plain residual sum). fp32."""

    def __init__(self, streams: int, w: Optional[Dict[str, torch.Tensor]], device) -> None:
        super().__init__()
        if w:
            if w["in"].numel() != streams or w["out"].numel() != streams or tuple(w["mix"].shape) != (streams, streams):
                raise ValueError(f"stream weights do not fit {streams} streams")
            read, write, mix = w["in"], w["out"], w["mix"]
        else:
            read, write, mix = torch.ones(streams), torch.ones(streams), torch.eye(streams)
        self.register_buffer("read", _f32(read, device))
        self.register_buffer("write", _f32(write, device))
        self.register_buffer("mix", _f32(mix, device))


class GatedFeedForward(InputReader):
    """W_down (act(W_gate h) * (W_up h)); ``act`` one of seq_ops.ACT_*. With ``clamp`` = (alpha, limit, shift) the
    unit is g sigmoid(alpha g) (u + shift) on g = min(W_gate h, limit), u = clamp(W_up h, -limit, limit) instead."""

    def __init__(self, spec: FeedForwardSpec, width: int, w: Dict[str, torch.Tensor], device, dtype,
                 act: int = seq_ops.ACT_GELU_TANH, clamp: Optional[Tuple[float, float, float]] = None) -> None:
        super().__init__()
        self.ff, self.act, self.clamp = spec.ff, act, clamp
        for name, shape in (("gate", (spec.ff, width)), ("up", (spec.ff, width)), ("down", (width, spec.ff))):
            if tuple(w[name].shape) != shape:
                raise ValueError(f"mlp.{name}: shape {tuple(w[name].shape)}, expected {shape}")
        self._in = [("gate", w["gate"]), ("up", w["up"])]
        self.register_buffer("w_down", w["down"].to(device=device, dtype=dtype).contiguous())

    def in_parts(self):
        return self._in

    def forward(self, proj: torch.Tensor, h: torch.Tensor, x: torch.Tensor, h16=None, accumulate: bool = True) -> None:
        # (h: the norm output, fp32 or its bf16 copy; for MFMA tiles with bf16 weights the gated product is rounded
        # where it is made)
        bf16 = _tiles16(proj.shape[0], self.w_down)
        if self.clamp is not None:
            alpha, limit, shift = self.clamp
            a = seq_ops.glu_clamped(proj, self.off["gate"], self.off["up"], self.ff, alpha=alpha, limit=limit,
                                    shift=shift, bf16=bf16)
        else:
            a = seq_ops.glu(proj, self.off["gate"], self.off["up"], self.ff, self.act, bf16=bf16)
        W = x.shape[1]
        seq_ops.linear(a, self.w_down, M=a.shape[0], N=W, K=self.ff, y=x, lda=self.ff, ldy=W, accumulate=accumulate)


class DenseFeedForward(InputReader):
    """W_down act(W_up h) without a gate (``act`` defaults to the square of relu). The unit is the only reader of its
    input, so it makes the up product itself, with the activation in the product's epilogue (for MFMA tiles the
    result is left in bf16, the down product's operand)."""

    def __init__(self, spec: FeedForwardSpec, width: int, w: Dict[str, torch.Tensor], device, dtype,
                 act: int = seq_ops.ACT_RELU2) -> None:
        super().__init__()
        self.ff, self.act = spec.ff, act
        for name, shape in (("up", (spec.ff, width)), ("down", (width, spec.ff))):
            if tuple(w[name].shape) != shape:
                raise ValueError(f"mlp.{name}: shape {tuple(w[name].shape)}, expected {shape}")
        self.register_buffer("w_up", w["up"].to(device=device, dtype=dtype).contiguous())
        self.register_buffer("w_down", w["down"].to(device=device, dtype=dtype).contiguous())

    def in_parts(self):
        return []

    def wants_proj(self, rows: int) -> bool:
        return False

    def forward(self, proj, h: Optional[torch.Tensor], x: torch.Tensor, h16: Optional[torch.Tensor] = None,
                accumulate: bool = True) -> None:
        """h: the normed input in fp32, or None when only its bf16 copy ``h16`` was made (MFMA tiles)."""
        T, W = x.shape
        F = self.ff
        bf16 = _tiles16(T, self.w_down)
        src = h16 if (bf16 and h16 is not None) else h
        a = torch.empty(T, F, dtype=torch.bfloat16 if bf16 else torch.float32, device=x.device)
        seq_ops.linear(src, self.w_up, M=T, N=F, K=W, y=a, lda=W, ldy=F, act=self.act)
        seq_ops.linear(a, self.w_down, M=T, N=W, K=F, y=x, lda=F, ldy=W, accumulate=accumulate)


class SparseFeedForward(InputReader):
    """Mixture of experts with an fp32 router, in one of two forms.

    ``route = "top_logits"``: the ``top`` largest logits are chosen, weights = softmax restricted to the chosen
    logits, expert = W_down act(W_up h) (``act`` defaults to the square of relu).
    ``route = "scores"``: scores = softmax over ALL router outputs; the ``top`` largest of score + ``correction``
    (a stored vector that shifts the choice only) are chosen; the weights are the chosen scores as they are;
    expert = W_down (act(W_gate h) * W_up h) (``act`` defaults to silu); the last ``identity`` router outputs are
    identity experts without matrices, whose output is the input itself.
    ``route = "sigmoid"``: scores = sigmoid of every router output on its own; the ``top`` largest are chosen; the
    chosen score multiplies the expert's INPUT, expert = W_down relu(W_up (s h))^2. Since s > 0 that equals
    s^2 W_down relu(W_up h)^2, which is what runs: the routing launch hands out s^2 as the weight of the expert's
    output (another activation than the square of relu is refused). With ``shared_ff`` a shared expert of the same
    form (``shared.up`` / ``shared.down``) runs for every token and is added times sigmoid(W_sg h), one number per
    token (``shared.sg``); its up matrix, its gate row and the router are one fused input projection.

    Few (token, choice) pairs (decode) stream only the chosen experts' rows through two GEMV launches. A prompt
    sorts its pairs by expert on the device and runs two grouped products over the expert ranges, then sums each
    token's choices in routing order."""

    STREAM_PAIRS = 48  # up to this many (token, choice) pairs the streaming form runs
    reads_f32 = True  # the streaming experts and the in-launch router read the fp32 input itself

    def __init__(self, spec: FeedForwardSpec, width: int, w: Dict[str, torch.Tensor], device, dtype,
                 act: Optional[int] = None, route: str = "top_logits") -> None:
        super().__init__()
        if route not in ("top_logits", "scores", "sigmoid"):
            raise ValueError(f"unknown routing {route!r}")
        self.E, self.top, self.ff, self.route = spec.experts, spec.top, spec.ff, route
        self.gated = route == "scores"
        self.n_router = spec.experts + (spec.identity if self.gated else 0)
        self.act = act if act is not None else (seq_ops.ACT_SILU if self.gated else seq_ops.ACT_RELU2)
        if route == "sigmoid" and self.act != seq_ops.ACT_RELU2:
            raise NotImplementedError("a score on the expert's input is served for the square of relu")
        self.shared_ff = spec.shared_ff if route == "sigmoid" else 0
        if tuple(w["router"].shape) != (self.n_router, width):
            raise ValueError(f"mlp.router: shape {tuple(w['router'].shape)}, expected {(self.n_router, width)}")
        self._in = [("router", w["router"])]
        self.register_buffer("w_shared_down", None)
        if self.shared_ff:
            Fs = self.shared_ff
            for name, shape in (("shared.up", (Fs, width)), ("shared.down", (width, Fs)), ("shared.sg", (1, width))):
                if tuple(w[name].shape) != shape:
                    raise ValueError(f"mlp.{name}: shape {tuple(w[name].shape)}, expected {shape}")
            self._in += [("shared.up", w["shared.up"]), ("shared.sg", w["shared.sg"])]
            self.w_shared_down = w["shared.down"].to(device=device, dtype=dtype).contiguous()
        up = torch.stack([torch.cat([w[f"e{e}.gate"], w[f"e{e}.up"]]) if self.gated else w[f"e{e}.up"]
                          for e in range(self.E)])
        down = torch.stack([w[f"e{e}.down"] for e in range(self.E)])
        rows = 2 * spec.ff if self.gated else spec.ff
        if tuple(up.shape) != (self.E, rows, width) or tuple(down.shape) != (self.E, width, spec.ff):
            raise ValueError("mlp experts: unexpected shapes")
        self.register_buffer("w_up", up.to(device=device, dtype=dtype).contiguous())  # gated: gate rows, then up rows
        self.register_buffer("w_down", down.to(device=device, dtype=dtype).contiguous())
        # (steps with few tokens compute the router's logits inside the routing launch, from this copy)
        fused_router = self.gated or (route == "sigmoid" and not self.shared_ff)
        self.register_buffer("w_router", w["router"].to(device=device, dtype=dtype).contiguous() if fused_router else None)
        self.register_buffer("correction", None)
        if self.gated and "correction" in w:
            if w["correction"].numel() != self.n_router:
                raise ValueError(f"mlp.correction: {w['correction'].numel()} values, expected {self.n_router}")
            self.correction = _f32(w["correction"], device)

    def in_parts(self):
        return self._in

    def wants_proj(self, rows: int) -> bool:
        """Whether a step of ``rows`` tokens needs the layer's input projection (the router logits) made for it."""
        return not (self.w_router is not None and rows * self.top <= self.STREAM_PAIRS)

    def forward(self, proj: Optional[torch.Tensor], h: torch.Tensor, x: torch.Tensor,
                h16: Optional[torch.Tensor] = None, accumulate: bool = True) -> None:
        """h: the sublayer's input (fp32); h16: its bf16 copy when the layer made one (the grouped products read it).
        ``proj`` None (score routing, few tokens): the router's logits are made inside the routing launch."""
        T, W = h.shape
        E, top, F = self.E, self.top, self.ff
        sig = self.route == "sigmoid"
        if proj is None:
            ids, wts = seq_ops.moe_router(h, self.w_router, top, self.correction, sigmoid=sig, square=sig)
        elif sig:
            ids, wts = seq_ops.moe_route_scores(proj, self.off["router"], self.n_router, top, sigmoid=True, square=True)
        elif self.gated:
            ids, wts = seq_ops.moe_route_scores(proj, self.off["router"], self.n_router, top, self.correction)
        else:
            ids, wts = seq_ops.moe_route(proj, self.off["router"], E, top)
        if T * top <= self.STREAM_PAIRS:
            a = seq_ops.moe_up(h, self.w_up, ids, self.act, gated=self.gated)
            seq_ops.moe_down(a, self.w_down, ids, wts, x, h, accumulate=accumulate)
            self._shared(proj, x)
            return
        pairs = T * top
        z_start, tok_of, where = seq_ops.moe_sort(ids, self.n_router)
        a_dtype = torch.bfloat16 if self.w_down.dtype == torch.bfloat16 else torch.float32
        if self.gated:
            gu = torch.empty(pairs, 2 * F, dtype=torch.float32, device=h.device)
            seq_ops.linear(h if h16 is None else h16, self.w_up, M=pairs, N=2 * F, K=W, y=gu, lda=W, ldy=2 * F, batch=E,
                           stride_w=2 * F * W, a_rows=tok_of, z_start=z_start)
            a = seq_ops.glu(gu, 0, F, F, self.act, bf16=a_dtype == torch.bfloat16)
        else:
            a = torch.empty(pairs, F, dtype=a_dtype, device=h.device)
            seq_ops.linear(h if h16 is None else h16, self.w_up, M=pairs, N=F, K=W, y=a, lda=W, ldy=F, batch=E,
                           stride_w=F * W, act=self.act, a_rows=tok_of, z_start=z_start)
        y = torch.empty(pairs, W, dtype=torch.float32, device=h.device)
        seq_ops.linear(a, self.w_down, M=pairs, N=W, K=F, y=y, lda=F, ldy=W, batch=E, stride_w=W * F, z_start=z_start)
        identity = self.n_router > E
        seq_ops.moe_combine(y, where, wts, x, ids=ids if identity else None, n_real=E, h=h if identity else None,
                            accumulate=accumulate)
        self._shared(proj, x)

    def _shared(self, proj: Optional[torch.Tensor], x: torch.Tensor) -> None:
        """x += sigmoid(W_sg h) * W_down act(W_up h) of the shared expert: the gate scales the activated rows (one
        number per row), then the down product accumulates."""
        if not self.shared_ff:
            return
        T, W = x.shape
        Fs = self.shared_ff
        a = seq_ops.act_rows(proj, self.off["shared.up"], Fs, self.act, gate_off=self.off["shared.sg"],
                             bf16=_tiles16(T, self.w_shared_down))
        seq_ops.linear(a, self.w_shared_down, M=T, N=W, K=Fs, y=x, lda=Fs, ldy=W, accumulate=True)


class TokenSide(nn.Module):
    """Per-layer token input: e = this layer's slice of a second embedding table at the token,
    y = W_proj (gelu_tanh(W_gate x) * e), x <- x + y / rms(y) * w (plain weight). Reads the stream after the
    layer's feed-forward; a looped layer uses the same slice in every pass."""

    def __init__(self, layer: int, dim: int, table: torch.Tensor, w: Dict[str, torch.Tensor], eps: float, device,
                 dtype) -> None:
        super().__init__()
        self.col0, self.dim, self.eps = layer * dim, dim, eps
        self.table = table  # shared by all layers (owned by the model)
        self.register_buffer("w_gate", w["gate"].to(device=device, dtype=dtype).contiguous())
        self.register_buffer("w_proj", w["proj"].to(device=device, dtype=dtype).contiguous())
        self.register_buffer("norm_w", _f32(w["norm"], device))

    def forward(self, x: torch.Tensor, tokens: torch.Tensor) -> None:
        seq_ops.token_side(x, tokens, self.table, self.col0, self.w_gate, self.w_proj, self.norm_w, self.eps)


MIXERS = {"retention": Retention, "latent_attention": LatentAttention, "attention": DiffAttention,
          "mamba2": SelectiveScan, "channel_delta": GatedDelta, "gated_delta": GatedDelta,
          "sink_attention": SinkAttention, "parallel": ParallelMixer, "rotary_attention": SinkAttention,
          "key_value_attention": SinkAttention, "gated_linear": GatedLinearAttention, "lightning": Lightning}
