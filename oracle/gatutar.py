"""Plain, slow CPU implementation of the Gatutar design: one function per mechanism, float64 by default.

It is the oracle the GPU kernels are tested against and shares no code with ``lit_gpt``. It takes the raw
``config.json`` dictionary and a ``{name: tensor}`` dictionary of weights and walks a sequence token by token
wherever the design is recurrent or causal, so that nothing here depends on a chunking, a cache layout or a batch.

The design in short. ``x = embed[token]``. Every layer is a *sandwich*: each sublayer is normed on the way in and on
the way out and its normed output is scaled channel by channel before it joins the residual,
``x += ls1 * N1b(mixer(N1 x))``, then ``x += ls2 * N2b(ff(N2 x))`` (RMS norms with a plain weight). A mixer is a pair
of branches on the same input whose outputs are each RMS-normed over the width and averaged:

* ``parallel`` - *left*: causal softmax attention, grouped key/value heads, rotary positions in the half layout on the
  first ``rot.dims`` dims with band-wise rescaled frequencies, and a softmax whose denominator holds an extra 1 (a
  sink of score 0 without a value). *right*: gated linear attention, ``S <- diag(alpha) S + k v^T``, ``o = S^T q`` with a
  decay per key channel ``alpha = sigmoid(low-rank(h) + b)^(1/tau)``; per-head RMS norm, ``silu`` gate.
* ``parallel_2`` - *left*: causal softmax attention whose values are the keys as projected, weighted RMS norm on q and
  k per head, no rotation, a query temperature that grows with the position, a sigmoid gate per head. *right*:
  linear attention with one constant decay per head on ``silu`` q / k / v; RMS norm over all heads at once, sigmoid gate.

Feed-forward: ``W_down relu(W_up h)^2``, dense or as a mixture of such experts chosen by the largest sigmoid router
scores; the score scales the expert's INPUT; a shared expert with a sigmoid gate per token is added.

Notation: ``W`` width, ``H`` heads, ``G`` key heads, ``d`` key dim, ``dv`` value dim.
"""

from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

DT = torch.float64


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def relu2(z: torch.Tensor) -> torch.Tensor:
    return torch.relu(z) ** 2


def rms_norm(x: torch.Tensor, w: Optional[torch.Tensor], eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last axis, times w."""
    y = x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)
    return y if w is None else y * w


def scaled_frequencies(rot: dict) -> List[float]:
    """f_i = base^(-2i/dims); with ``scaling`` long wavelengths are slowed down by ``factor``, short ones kept, and
    the band between blends the two linearly in original / wavelength."""
    dims = int(rot["dims"])
    out = []
    sc = rot.get("scaling")
    for i in range(dims // 2):
        f = float(rot["base"]) ** (-2.0 * i / dims)
        if sc:
            factor, low, high, orig = float(sc["factor"]), float(sc["low"]), float(sc["high"]), float(sc["original"])
            wl = 2.0 * math.pi / f
            if wl < orig / high:
                pass
            elif wl > orig / low:
                f = f / factor
            else:
                s = (orig / wl - low) / (high - low)
                f = (1.0 - s) * f / factor + s * f
        out.append(f)
    return out


def rotate_half(x: torch.Tensor, pos: int, freqs: List[float]) -> torch.Tensor:
    """x (..., dim): dim i is paired with i + n for i < n = len(freqs); the rest passes."""
    n = len(freqs)
    out = x.clone()
    for i, f in enumerate(freqs):
        a = pos * f
        c, s = math.cos(a), math.sin(a)
        u, v = x[..., i], x[..., i + n]
        out[..., i] = u * c - v * s
        out[..., i + n] = v * c + u * s
    return out


def softmax_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, scale: float, extra_one: bool) -> torch.Tensor:
    """q (T, H, d), k (T, G, d), v (T, G, dv), causal. ``extra_one``: 1 is added to the softmax denominator."""
    T, H, d = q.shape
    G = k.shape[1]
    out = torch.zeros(T, H, v.shape[2], dtype=q.dtype)
    for t in range(T):
        for h in range(H):
            g = h // (H // G)
            s = (k[: t + 1, g] @ q[t, h]) * scale
            e = torch.exp(s)
            den = e.sum() + (1.0 if extra_one else 0.0)
            out[t, h] = (e / den) @ v[: t + 1, g]
    return out


def rope_attention(h: torch.Tensor, m: dict, w: Dict[str, torch.Tensor], pos0: int = 0) -> torch.Tensor:
    """The left branch of ``parallel``. h (T, W) -> (T, W)."""
    T = h.shape[0]
    H, G, d, dv = int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"])
    q = (h @ w["q"].T).view(T, H, d)
    k = (h @ w["k"].T).view(T, G, d)
    v = (h @ w["v"].T).view(T, G, dv)
    rot = m.get("rot")
    if rot and int(rot["dims"]) > 0:
        freqs = scaled_frequencies(rot)
        q = torch.stack([rotate_half(q[t], pos0 + t, freqs) for t in range(T)])
        k = torch.stack([rotate_half(k[t], pos0 + t, freqs) for t in range(T)])
    o = softmax_attention(q, k, v, float(m["scale"]), extra_one=True)
    return o.reshape(T, H * dv) @ w["o"].T


def normed_key_attention(h: torch.Tensor, m: dict, w: Dict[str, torch.Tensor], eps: float, pos0: int = 0) -> torch.Tensor:
    """The left branch of ``parallel_2``: values are the keys as projected."""
    T = h.shape[0]
    H, G, d = int(m["heads"]), int(m["kv_heads"]), int(m["dim"])
    q = (h @ w["q"].T).view(T, H, d)
    k = (h @ w["k"].T).view(T, G, d)
    v = k.clone()
    q = rms_norm(q, w["q.norm"], eps)
    k = rms_norm(k, w["k.norm"], eps)
    temp = m.get("q_temp")
    if temp:
        for t in range(T):
            p = pos0 + t
            q[t] = q[t] * (1.0 + float(temp["coef"]) * math.log((p + 1) // int(temp["every"]) + 1))
    o = softmax_attention(q, k, v, float(m["scale"]), extra_one=False)
    gate = torch.sigmoid(h @ w["g"].T)  # (T, H)
    o = o * gate.unsqueeze(-1)
    return o.reshape(T, H * d) @ w["o"].T


def linear_recurrence(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, alpha: torch.Tensor,
                      state: Optional[torch.Tensor] = None) -> torch.Tensor:
    """S_t = diag(alpha_t) S_(t-1) + k_t v_t^T, o_t = S_t^T q_t per head. q, k, alpha (T, H, d), v (T, H, dv)."""
    T, H, d = q.shape
    dv = v.shape[2]
    S = torch.zeros(H, d, dv, dtype=q.dtype) if state is None else state
    out = torch.zeros(T, H, dv, dtype=q.dtype)
    for t in range(T):
        S = alpha[t].unsqueeze(-1) * S + k[t].unsqueeze(-1) * v[t].unsqueeze(-2)
        out[t] = torch.einsum("hdv,hd->hv", S, q[t])
    return out


def gated_linear_attention(h: torch.Tensor, m: dict, w: Dict[str, torch.Tensor], eps: float) -> torch.Tensor:
    """The right branch of ``parallel``."""
    T = h.shape[0]
    H, d, dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    q = (h @ w["q"].T).view(T, H, d) * d ** -0.5
    k = (h @ w["k"].T).view(T, H, d)
    v = (h @ w["v"].T).view(T, H, dv)
    z = (h @ w["a1"].T) @ w["a2"].T + w["a2.b"]
    alpha = torch.sigmoid(z).view(T, H, d) ** (1.0 / float(m["tau"]))
    o = linear_recurrence(q, k, v, alpha)
    o = rms_norm(o, w["norm"], eps).reshape(T, H * dv)
    o = o * silu(h @ w["g"].T)
    return o @ w["o"].T


def lightning_attention(h: torch.Tensor, m: dict, w: Dict[str, torch.Tensor], eps: float) -> torch.Tensor:
    """The right branch of ``parallel_2``."""
    T = h.shape[0]
    H, d, dv = int(m["heads"]), int(m["dim"]), int(m["vdim"])
    q = silu(h @ w["q"].T).view(T, H, d)
    k = silu(h @ w["k"].T).view(T, H, d)
    v = silu(h @ w["v"].T).view(T, H, dv)
    decay = torch.tensor([float(x) for x in m["decay"]], dtype=h.dtype)
    alpha = decay.view(1, H, 1).expand(T, H, d)
    o = linear_recurrence(q, k, v, alpha).reshape(T, H * dv)
    o = rms_norm(o, w["norm"], eps)
    o = o * torch.sigmoid(h @ w["g"].T)
    return o @ w["o"].T


def _sub(w: Dict[str, torch.Tensor], prefix: str) -> Dict[str, torch.Tensor]:
    return {k[len(prefix):]: v for k, v in w.items() if k.startswith(prefix)}


def mixer(kind: str, h: torch.Tensor, m: dict, w: Dict[str, torch.Tensor], eps: float) -> torch.Tensor:
    """Both branches, each RMS-normed over the width with its own weight, averaged."""
    wl, wr = _sub(w, "left."), _sub(w, "right.")
    if kind == "parallel":
        left = rope_attention(h, m["left"], wl)
        right = gated_linear_attention(h, m["right"], wr, eps)
    elif kind == "parallel_2":
        left = normed_key_attention(h, m["left"], wl, eps)
        right = lightning_attention(h, m["right"], wr, eps)
    else:
        raise ValueError(kind)
    return 0.5 * (rms_norm(left, w["left.out"], eps) + rms_norm(right, w["right.out"], eps))


def expert(h: torch.Tensor, w: Dict[str, torch.Tensor]) -> torch.Tensor:
    return relu2(h @ w["up"].T) @ w["down"].T


def feed_forward(h: torch.Tensor, f: dict, w: Dict[str, torch.Tensor]) -> torch.Tensor:
    if f["kind"] == "dense":
        return expert(h, w)
    E, top = int(f["router"]["experts"]), int(f["router"]["top"])
    scores = torch.sigmoid(h @ w["router"].T)  # (T, E)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        order = sorted(range(E), key=lambda e: (-float(scores[t, e]), e))[:top]
        for e in order:
            out[t] += expert((scores[t, e] * h[t]).unsqueeze(0), _sub(w, f"e{e}."))[0]
    if f.get("shared"):
        gate = torch.sigmoid(h @ w["shared.sg"].T)  # (T, 1)
        out = out + gate * expert(h, _sub(w, "shared."))
    return out


def forward(config: dict, weights: Dict[str, torch.Tensor], tokens: List[int], dtype=DT, layers_out: Optional[list] = None
            ) -> torch.Tensor:
    """Logits (T, vocab) of one sequence from position 0. ``layers_out``: receives the residual after every layer."""
    w = {k: v.to(dtype) for k, v in weights.items()}
    eps = float(config["norm"]["eps"])
    x = w["embed"][torch.tensor(tokens)]
    for i, layer in enumerate(config["layers"]):
        lw = _sub(w, f"l{i}.")
        y = mixer(layer["type"], rms_norm(x, lw["norm1"], eps), layer["mixer"], _sub(lw, "mix."), eps)
        x = x + rms_norm(y, lw["norm1b"], eps) * lw["ls1"]
        if layer.get("mlp"):
            y = feed_forward(rms_norm(x, lw["norm2"], eps), layer["mlp"], _sub(lw, "mlp."))
            x = x + rms_norm(y, lw["norm2b"], eps) * lw["ls2"]
        if layers_out is not None:
            layers_out.append(x.clone())
    return rms_norm(x, w["final.norm"], eps) @ w["head"].T
