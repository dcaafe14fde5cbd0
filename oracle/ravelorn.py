"""Plain, slow CPU implementation of the Ravelorn design: one function per mechanism, float64 by default.

It is the oracle the GPU kernels are tested against and shares no code with ``lit_gpt``. It takes the raw
``config.json`` dictionary and a ``{name: tensor}`` dictionary of weights and walks a sequence token by token
wherever the design is recurrent or causal, so that nothing here depends on a chunking, a cache layout or a batch.

The design in short. Token embedding plus a learned position vector. Every sublayer reads the residual ``x`` itself
and its OUTPUT is normed (layer norm with weight and bias) before it joins the residual with a constant factor:
``x += m LN1(mixer(x))``, ``x += m LN2(ff(x))``. Mixers:

* ``channel_delta`` - a gated delta rule whose decay is per head AND key channel. Per head the memory S (d x dv)
  goes ``S <- diag(g) S``, ``u = beta (v - S^T k)``, ``S <- S + k u^T``, ``o = S^T q``. q / k / v pass a short causal
  per-channel convolution and silu, q and k become unit vectors per head (q also times d^-1/2), the decay is
  ``exp(-exp(A_log) softplus(low-rank(h) + bias))``, the output is divided by its root mean square per head, weighted
  and gated by ``sigmoid(low-rank(h))``.
* ``parallel`` - two mixers on the same input, summed with fixed scales: *left* a causal softmax attention with
  grouped key/value heads, q and k divided by their root mean square, a position-dependent query temperature and a
  per-head sink in the softmax normaliser; *right* a gated delta rule with one decay per head and a ``silu`` gate.

Feed-forward: a mixture of gated (silu) experts; the router's softmax runs over all outputs, a stored correction
shifts the scores for the choice only, the weights are the chosen scores as they are, and the last few router
outputs are identity experts (their output is the input). Logits: final layer norm, head matrix, tanh soft cap.

Notation: ``W`` width, ``H`` heads, ``G`` key heads, ``d`` key dim, ``dv`` value dim.
"""

from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch

DT = torch.float64


def silu(z: torch.Tensor) -> torch.Tensor:
    return z * torch.sigmoid(z)


def softplus(z: torch.Tensor) -> torch.Tensor:
    return torch.where(z > 30.0, z, torch.log1p(torch.exp(torch.clamp(z, max=30.0))))


def rms_unit(x: torch.Tensor, eps: float) -> torch.Tensor:
    """x / sqrt(mean(x^2) + eps) over the last axis."""
    return x / torch.sqrt((x * x).mean(-1, keepdim=True) + eps)


def layer_norm(x: torch.Tensor, w: torch.Tensor, b: torch.Tensor, eps: float) -> torch.Tensor:
    mu = x.mean(-1, keepdim=True)
    var = ((x - mu) ** 2).mean(-1, keepdim=True)
    return (x - mu) / torch.sqrt(var + eps) * w + b


def causal_conv_silu(u: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """u (T, C), weight (C, taps): out[t] = silu(sum_j weight[:, j] u[t - (taps - 1 - j)]), zeros before the start."""
    T, C = u.shape
    taps = weight.shape[1]
    out = torch.zeros_like(u)
    for t in range(T):
        acc = torch.zeros(C, dtype=u.dtype)
        for j in range(taps):
            src = t - (taps - 1 - j)
            if src >= 0:
                acc = acc + weight[:, j] * u[src]
        out[t] = silu(acc)
    return out


def delta_rule(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, beta: torch.Tensor, g: torch.Tensor) -> torch.Tensor:
    """One head, token by token. q, k (T, d); v (T, dv); beta (T,); g (T, d) decay of each key channel's row of S
    (a per-head decay is the same number in every column). Returns o (T, dv)."""
    T, d = q.shape
    S = torch.zeros(d, v.shape[1], dtype=q.dtype)
    out = []
    for t in range(T):
        S = g[t][:, None] * S
        u = beta[t] * (v[t] - S.T @ k[t])
        S = S + torch.outer(k[t], u)
        out.append(S.T @ q[t])
    return torch.stack(out)


def gated_delta(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, eps: float, per_channel: bool) -> torch.Tensor:
    """The gated delta rule mixer on h (T, W). ``per_channel``: the decay comes from the low-rank pair a1 / a2 with
    one value per head and key channel and the gate is sigmoid(g2 g1 h); otherwise one decay per head from ``a`` and
    the gate is silu(g h)."""
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = causal_conv_silu(h @ w["q"].T, w["q.conv"]).view(T, G, d)
    k = causal_conv_silu(h @ w["k"].T, w["k.conv"]).view(T, G, d)
    v = causal_conv_silu(h @ w["v"].T, w["v.conv"]).view(T, H, dv)
    q = q / torch.sqrt((q * q).sum(-1, keepdim=True) + 1e-6) * d ** -0.5
    k = k / torch.sqrt((k * k).sum(-1, keepdim=True) + 1e-6)
    beta = torch.sigmoid(h @ w["b"].T)  # (T, H)
    rate = torch.exp(w["A_log"])  # (H,)
    if per_channel:
        a = ((h @ w["a1"].T) @ w["a2"].T + w["dt_bias"]).view(T, H, d)
        g = torch.exp(-rate[None, :, None] * softplus(a))
        gate = torch.sigmoid((h @ w["g1"].T) @ w["g2"].T).view(T, H, dv)
    else:
        a = h @ w["a"].T + w["dt_bias"]  # (T, H)
        g = torch.exp(-rate[None, :] * softplus(a))[:, :, None].expand(T, H, d)
        gate = silu(h @ w["g"].T).view(T, H, dv)
    outs = []
    for hd in range(H):
        kv = hd // (H // G)
        o = delta_rule(q[:, kv], k[:, kv], v[:, hd], beta[:, hd], g[:, hd])
        outs.append(rms_unit(o, eps) * w["norm"] * gate[:, hd])
    return torch.cat(outs, dim=-1) @ w["o"].T


def sink_attention(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, eps: float) -> torch.Tensor:
    """Causal softmax attention with grouped key / value heads, unit-RMS q and k, a query temperature that grows
    with the position, and exp(sink) of the head joining the normaliser."""
    H, G, d, dv = m["heads"], m["kv_heads"], m["dim"], m["vdim"]
    T = h.shape[0]
    q = rms_unit((h @ w["q"].T).view(T, H, d), eps)
    k = rms_unit((h @ w["k"].T).view(T, G, d), eps)
    v = (h @ w["v"].T).view(T, G, dv)
    qt = m.get("q_temp")
    out = torch.zeros(T, H, dv, dtype=h.dtype)
    for t in range(T):
        temp = 1.0 + qt["coef"] * math.log((t + 1) // qt["every"] + 1) if qt else 1.0
        for hd in range(H):
            kv = hd // (H // G)
            s = (k[: t + 1, kv] @ (q[t, hd] * temp)) * m["scale"]
            sink = w["sink"][hd] if "sink" in w else None
            mx = s.max() if sink is None else torch.maximum(s.max(), sink)
            e = torch.exp(s - mx)
            den = e.sum() + (torch.exp(sink - mx) if sink is not None else 0.0)
            out[t, hd] = (e / den) @ v[: t + 1, kv]
    return out.reshape(T, H * dv) @ w["o"].T


def parallel_mixer(h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, eps: float) -> torch.Tensor:
    left = sink_attention(h, _sub(w, "left."), m["left"], eps)
    right = gated_delta(h, _sub(w, "right."), m["right"], eps, per_channel=False)
    return m["left_scale"] * left + m["right_scale"] * right


def route(h: torch.Tensor, w: Dict[str, torch.Tensor], top: int):
    """Scores over all router outputs, the ``top`` largest of score + correction, weights = the scores themselves."""
    s = torch.softmax(h @ w["router"].T, dim=-1)
    choice = s + w["correction"] if "correction" in w else s
    idx = torch.topk(choice, top, dim=-1).indices
    return idx, torch.gather(s, -1, idx)


def moe_ff(h: torch.Tensor, w: Dict[str, torch.Tensor], f: dict) -> torch.Tensor:
    E, top = f["router"]["experts"], f["router"]["top"]
    idx, wt = route(h, w, top)
    out = torch.zeros_like(h)
    for t in range(h.shape[0]):
        for e, p in zip(idx[t].tolist(), wt[t]):
            if e >= E:  # an identity expert
                out[t] += p * h[t]
            else:
                a = silu(w[f"e{e}.gate"] @ h[t]) * (w[f"e{e}.up"] @ h[t])
                out[t] += p * (w[f"e{e}.down"] @ a)
    return out


def _sub(w: Dict[str, torch.Tensor], prefix: str) -> Dict[str, torch.Tensor]:
    return {k[len(prefix):]: v for k, v in w.items() if k.startswith(prefix)}


def mixer(kind: str, h: torch.Tensor, w: Dict[str, torch.Tensor], m: dict, eps: float) -> torch.Tensor:
    if kind == "channel_delta":
        return gated_delta(h, w, m, eps, per_channel=True)
    if kind == "parallel":
        return parallel_mixer(h, w, m, eps)
    raise ValueError(f"unknown mixer {kind!r}")


def forward(config: dict, weights: Dict[str, torch.Tensor], tokens: List[int], dtype=DT,
            layers_out: Optional[list] = None) -> torch.Tensor:
    """Logits (T, vocab) of one sequence from position 0. ``layers_out``: a list that receives the residual after
    every layer."""
    w = {k: (v.to(dtype) if v.is_floating_point() else v) for k, v in weights.items()}
    eps, mult = config["norm"]["eps"], config["residual_mult"]
    T = len(tokens)
    x = w["embed"][torch.tensor(tokens)] + w["pos"][:T]
    for i, layer in enumerate(config["layers"]):
        lw = _sub(w, f"l{i}.")
        y = mixer(layer["type"], x, _sub(lw, "mix."), layer["mixer"], eps)
        x = x + mult * layer_norm(y, lw["norm1"], lw["norm1.b"], eps)
        if layer.get("mlp") is not None:
            y = moe_ff(x, _sub(lw, "mlp."), layer["mlp"])
            x = x + mult * layer_norm(y, lw["norm2"], lw["norm2.b"], eps)
        if layers_out is not None:
            layers_out.append(x.clone())
    z = layer_norm(x, w["final.norm"], w["final.norm.b"], eps) @ w["head"].T
    cap = config.get("logit_softcap")
    return cap * torch.tanh(z / cap) if cap else z
