"""Python view of ``liblitgpt_seq.so`` (declared in ``include/litgpt_seq.h``): the kernels of the layered models.

Same conventions as ``lit_gpt.ops``: thin wrappers that check device / dtype / contiguity, pass raw device pointers,
launch on torch's current HIP stream (capturable into a HIP graph) and raise on a non-zero return code. There is
no CPU path. Activations are fp32; a weight is a bf16 or an fp32 tensor and its dtype picks the kernel: bf16 weights
take the activation rounded to bf16 with fp32 sums (MFMA tiles, streaming GEMVs), fp32 weights run plain fp32 FMA.

The library is separate from ``liblitgpt_amd.so`` so that serving a layered model compiles a few small sources only;
``build_library`` runs that ``make`` target when the library is missing.
"""

from __future__ import annotations

import ctypes
import os
import subprocess
from pathlib import Path
from typing import Optional

import torch

from lit_gpt.ops import NativeLibraryError, _dev, _opt, _stream

LIB_PATH = Path(os.environ.get("LGS_LIB", Path(__file__).resolve().parent / "_lib" / "liblitgpt_seq.so"))
CSRC = Path(__file__).resolve().parent.parent / "csrc"

ACT_NONE, ACT_RELU2, ACT_GELU_TANH, ACT_SILU, ACT_SIGMOID = 0, 1, 2, 3, 4

_P, _I, _L, _F = ctypes.c_void_p, ctypes.c_int, ctypes.c_long, ctypes.c_float

SIGNATURES = {
    "lgs_version": [],
    "lgs_last_error_string": [],
    "lgs_linear": [_P, _L, _L, _P, _I, _L, _P, _L, _L, _I, _I, _I, _I, _I, _I, _P, _P, _I, _I, _P],
    "lgs_embed": [_P, _P, _I, _F, _P, _I, _I, _I, _P],
    "lgs_rmsnorm": [_P, _L, _P, _F, _F, _P, _L, _I, _I, _I, _P, _P],
    "lgs_gather_rows": [_P, _P, _P, _I, _I, _P],
    "lgs_retention": [_P, _P, _P, _L, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _F, _I, _P, _I, _I, _P, _I, _P],
    "lgs_head_gate": [_P, _P, _L, _I, _I, _I, _I, _F, _I, _P, _F, _P, _P, _I, _I, _P],
    "lgs_latent_prepare": [_P, _L, _I, _I, _P, _I, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _F, _P],
    "lgs_latent_attention": [_P, _P, _L, _I, _P, _I, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _F, _I, _P, _P],
    "lgs_latent_attention_tiles": [_P, _P, _L, _I, _P, _I, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _F, _P],
    "lgs_glu": [_P, _P, _L, _P, _I, _I, _I, _I, _P],
    "lgs_moe_route": [_P, _L, _I, _I, _I, _P, _P, _P],
    "lgs_moe_route_scores": [_P, _L, _I, _I, _I, _P, _P, _P, _I, _I, _P],
    "lgs_moe_router": [_P, _L, _P, _I, _I, _I, _I, _I, _P, _P, _P, _I, _I, _P],
    "lgs_act_rows": [_P, _L, _P, _L, _P, _I, _I, _I, _I, _P],
    "lgs_sandwich_step": [_P, _P, _P, _P, _P, _F, _P, _P, _P, _P, _F, _I, _I, _P],
    "lgs_moe_up": [_P, _L, _P, _I, _P, _P, _I, _I, _I, _I, _I, _I, _I, _P],
    "lgs_moe_down": [_P, _P, _I, _P, _P, _P, _L, _I, _I, _I, _I, _I, _P, _L, _I, _P],
    "lgs_moe_sort": [_P, _I, _I, _I, _P, _P, _P, _P, _P],
    "lgs_moe_combine": [_P, _P, _P, _P, _L, _I, _I, _I, _P, _I, _P, _L, _I, _P],
    "lgs_token_side": [_P, _P, _P, _I, _L, _I, _P, _P, _P, _I, _I, _I, _I, _F, _P],
    "lgs_embed_streams": [_P, _P, _I, _F, _P, _I, _I, _I, _I, _P],
    "lgs_streams_step": [_P, _P, _P, _P, _P, _P, _P, _P, _F, _I, _I, _I, _P],
    "lgs_diffattn_prepare": [_P, _L, _I, _I, _I, _P, _P, _I, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _P],
    "lgs_diffattn": [_P, _L, _P, _P, _I, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _I, _F, _F, _F, _F,
                     _F, _P],
    "lgs_conv_silu": [_P, _L, _P, _P, _I, _P, _P, _P, _P, _P, _I, _I, _I, _I, _P],
    "lgs_ssm_scan": [_P, _L, _P, _L, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _P, _P, _I, _P],
    "lgs_gated_group_norm": [_P, _P, _L, _P, _F, _P, _P, _I, _I, _I, _P],
    "lgs_glu_clamped": [_P, _P, _L, _P, _I, _I, _I, _F, _F, _F, _P],
    "lgs_embed_pos": [_P, _P, _P, _P, _I, _F, _P, _P, _I, _I, _I, _I, _P],
    "lgs_layernorm": [_P, _P, _P, _F, _F, _I, _P, _P, _I, _I, _P],
    "lgs_softcap": [_P, _L, _F, _P],
    "lgs_normattn_prepare": [_P, _L, _I, _I, _I, _P, _P, _I, _P, _P, _I, _I, _I, _I, _I, _I, _F, _F, _I, _I, _P, _P, _P,
                             _I, _P],
    "lgs_sinkattn": [_P, _L, _P, _P, _I, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _I, _F, _F, _F, _P,
                     _L, _P],
    "lgs_delta_prepare": [_P, _L, _P, _L, _P, _L, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _F, _F, _P, _I, _I, _I, _I, _F,
                          _P],
    "lgs_delta_step_prepare": [_P, _L, _P, _I, _I, _P, _P, _P, _P, _P, _L, _P, _L, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I,
                               _I, _F, _F, _P, _I, _I, _P],
    "lgs_gated_delta": [_P, _L, _P, _P, _P, _P, _P, _P, _P, _P, _I, _I, _I, _I, _I, _I, _I, _I, _P],
}
_RESTYPES = {"lgs_last_error_string": ctypes.c_char_p}

_lib: Optional[ctypes.CDLL] = None


def _user_lib_path() -> Path:
    """Where the library goes when the checkout's own folders cannot be written to."""
    home = Path(os.environ.get("XDG_CACHE_HOME") or Path(os.environ.get("HOME") or "/tmp") / ".cache")
    return home / "litgpt_amd" / "liblitgpt_seq.so"


def build_library() -> Path:
    """Compile the library (``make seq``: hipcc --offload-arch=gfx950) unless it is there already: in-tree, or, when
    the tree's folders are not writable for this user, under the user's cache folder."""
    global LIB_PATH
    if LIB_PATH.is_file():
        return LIB_PATH
    jobs = str(min(16, os.cpu_count() or 8))
    try:
        subprocess.run(["make", "-C", str(CSRC), f"-j{jobs}", "seq"], check=True, stdout=subprocess.DEVNULL,
                       stderr=subprocess.PIPE)
    except (subprocess.CalledProcessError, OSError) as first:
        alt = _user_lib_path()
        if not alt.is_file():
            try:
                alt.parent.mkdir(parents=True, exist_ok=True)
                subprocess.run(["make", "-C", str(CSRC), f"-j{jobs}", "seq", f"SEQ_BUILD={alt.parent / 'build'}",
                                f"SEQ_OUT={alt}"], check=True, stdout=subprocess.DEVNULL, stderr=subprocess.PIPE)
            except (subprocess.CalledProcessError, OSError) as second:
                err = getattr(second, "stderr", b"") or getattr(first, "stderr", b"") or b""
                raise NativeLibraryError("building liblitgpt_seq.so failed:\n" + err.decode(errors="replace")[-2000:])
        LIB_PATH = alt
    return LIB_PATH


def load_library() -> ctypes.CDLL:
    global _lib, LIB_PATH
    if _lib is not None:
        return _lib
    if not LIB_PATH.is_file() and _user_lib_path().is_file():
        LIB_PATH = _user_lib_path()
    if not LIB_PATH.is_file():
        raise NativeLibraryError(f"HIP library not found at {LIB_PATH}. Build it with `make -C lit-gpt_amd/csrc seq` "
                                 "(hipcc --offload-arch=gfx950). There is no CPU fallback.")
    lib = ctypes.CDLL(str(LIB_PATH))
    for name, argtypes in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.argtypes = argtypes
        fn.restype = _RESTYPES.get(name, ctypes.c_int)
    _lib = lib
    return lib


def _check(rc: int) -> None:
    if rc != 0:
        msg = load_library().lgs_last_error_string()
        raise RuntimeError(f"liblitgpt_seq error {rc}: {msg.decode() if msg else ''}")


def _wf32(w: torch.Tensor, name: str) -> int:
    if w.dtype not in (torch.bfloat16, torch.float32):
        raise TypeError(f"{name}: weights are bf16 or fp32, got {w.dtype}")
    return int(w.dtype == torch.float32)


F32, I32 = torch.float32, torch.int32


def linear(a: torch.Tensor, w: torch.Tensor, *, M: int, N: int, K: int, y: torch.Tensor, a_off: int = 0, lda: int,
           y_off: int = 0, ldy: int, batch: int = 1, stride_a: int = 0, stride_w: int = 0, stride_y: int = 0,
           accumulate: bool = False, act: int = ACT_NONE, a_rows: Optional[torch.Tensor] = None,
           z_start: Optional[torch.Tensor] = None) -> torch.Tensor:
    """y[z] (+)= act(a[z] w[z]^T) over ``batch`` strided operands; offsets and strides count elements. With
    ``z_start`` (batch + 1 int32 row bounds) batch z owns that range of a row list of at most M rows, whose A rows
    are ``a_rows`` (or the list places themselves) and whose Y rows are the list places. ``a`` may be a producer's
    bf16 copy (``rmsnorm(bf16_copy=True)``, ``glu(bf16=True)``) for the MFMA tiles with bf16 weights."""
    a16 = a.dtype == torch.bfloat16
    ap = _dev(a, "a", torch.bfloat16 if a16 else F32) + (2 if a16 else 4) * a_off
    y16 = y.dtype == torch.bfloat16  # the result feeds another bf16 product
    yp = _dev(y, "y", torch.bfloat16 if y16 else F32) + (2 if y16 else 4) * y_off
    need_a = a_off + (batch - 1) * stride_a + (0 if a_rows is not None else (M - 1) * lda) + K
    need_y = y_off + (batch - 1) * stride_y * (0 if z_start is not None else 1) + (M - 1) * ldy + N
    if a.numel() < need_a or y.numel() < need_y or w.numel() < (batch - 1) * stride_w + N * K:
        raise ValueError("linear: an operand is smaller than the sizes and strides say")
    _check(load_library().lgs_linear(ap, lda, stride_a, _dev(w, "w"), _wf32(w, "w"), stride_w, yp, ldy, stride_y,
                                     M, N, K, batch, int(accumulate), act, _opt(a_rows, "a_rows", I32),
                                     _opt(z_start, "z_start", I32), int(a16), int(y16), _stream()))
    return y


def embed(tokens: torch.Tensor, table: torch.Tensor, scale: float) -> torch.Tensor:
    T, (V, W) = tokens.numel(), table.shape
    x = torch.empty(T, W, dtype=F32, device=tokens.device)
    _check(load_library().lgs_embed(_dev(tokens, "tokens", I32), _dev(table, "table"), _wf32(table, "table"),
                                    float(scale), x.data_ptr(), T, W, V, _stream()))
    return x


def rmsnorm(x: torch.Tensor, weight: Optional[torch.Tensor], *, offset: float, eps: float,
            out: Optional[torch.Tensor] = None, bf16_copy: bool = False):
    """Rows of a contiguous (rows, n) tensor: x / sqrt(mean(x^2) + eps) * (offset + weight) (no weight: unit RMS).
    ``bf16_copy``: also returns the result rounded to bf16 (the operand of the bf16 MFMA products): (y, y_bf16)."""
    rows, n = x.shape
    y = out if out is not None else torch.empty_like(x)
    yb = torch.empty(rows, n, dtype=torch.bfloat16, device=x.device) if bf16_copy else None
    if weight is not None and weight.numel() != n:
        raise ValueError("rmsnorm: weight size")
    _check(load_library().lgs_rmsnorm(_dev(x, "x", F32), n, _opt(weight, "weight", F32), float(offset), float(eps),
                                      _dev(y, "y", F32), n, rows, 1, n, _opt(yb, "y_bf16", torch.bfloat16),
                                      _stream()))
    return (y, yb) if bf16_copy else y


def gather_rows(x: torch.Tensor, rows: torch.Tensor) -> torch.Tensor:
    y = torch.empty(rows.numel(), x.shape[1], dtype=F32, device=x.device)
    _check(load_library().lgs_gather_rows(_dev(x, "x", F32), _dev(rows, "rows", I32), y.data_ptr(), rows.numel(),
                                          x.shape[1], _stream()))
    return y


def retention(proj: torch.Tensor, q_off: int, k_off: int, v_off: int, state: torch.Tensor, decay: torch.Tensor,
              inv_freq: Optional[torch.Tensor], seq_start: torch.Tensor, seq_slot: torch.Tensor,
              seq_pos0: torch.Tensor, *, H: int, d: int, dv: int, rot_dims: int, k_scale: float,
              chunked: Optional[bool] = None, max_len: int = 0, pos: Optional[torch.Tensor] = None,
              act: int = ACT_NONE) -> torch.Tensor:
    """proj (T, ld) holds q, k (H * d each) and v (H * dv) at the given column offsets; state (slots, H, d, dv) fp32
    is read (unless a sequence starts at position 0) and left at the step's last token. Returns o (T, H * dv).
    ``chunked`` picks the prompt form (64-token chunks as matrix products) over the token-by-token scan; by default
    steps that bring 8 or more tokens per sequence on average take it. ``max_len`` (the most tokens any sequence
    brings; 0: unknown) lets the prompt form run its chunks side by side when a sequence has more than one. The
    prompt form needs ``pos`` (T,) and rotates / scales the q and k columns of ``proj`` in place. ``act``: an activation
    on q, k and v as projected, ahead of the rotation and the scale (the prompt form applies it in place)."""
    T, ld = proj.shape
    B = seq_slot.numel()
    if tuple(state.shape[1:]) != (H, d, dv) or seq_start.numel() != B + 1 or decay.numel() != H:
        raise ValueError("retention: state / sequence table shapes")
    if max(q_off, k_off) + H * d > ld or v_off + H * dv > ld:
        raise ValueError("retention: projections outside the row")
    out = torch.empty(T, H * dv, dtype=F32, device=proj.device)
    base = _dev(proj, "proj", F32)
    if chunked is None:
        chunked = T >= 8 * B and pos is not None
    if chunked and (pos is None or pos.numel() != T):
        raise ValueError("retention: the prompt form needs the rows' positions")
    ws, max_chunks = None, 0
    if chunked and d <= 128 and max_len > 64:
        max_chunks = (max_len + 63) // 64
        ws = torch.empty(B * max_chunks * H * d * dv, dtype=F32, device=proj.device)
    _check(load_library().lgs_retention(base + 4 * q_off, base + 4 * k_off, base + 4 * v_off, ld,
                                        _dev(state, "state", F32), _dev(decay, "decay", F32),
                                        _opt(inv_freq, "inv_freq", F32), _dev(seq_start, "seq_start", I32),
                                        _dev(seq_slot, "seq_slot", I32), _dev(seq_pos0, "seq_pos0", I32),
                                        out.data_ptr(), B, H, d, dv, rot_dims, float(k_scale), int(bool(chunked)),
                                        _opt(ws, "ws", F32), max_chunks, T, _opt(pos, "pos", I32), int(act),
                                        _stream()))
    return out


def head_gate(o: torch.Tensor, proj: torch.Tensor, g_off: int, *, H: int, dv: int, unit_norm: bool, eps: float,
              act: int, bf16_copy: bool = False, weight: Optional[torch.Tensor] = None,
              post: float = 1.0, w_g2: Optional[torch.Tensor] = None) -> torch.Tensor:
    """In place on o (T, H * dv): per head optional unit RMS, times ``weight`` (dv values shared by the heads), times
    act(gate), the gate at proj[:, g_off:], times ``post``. With ``w_g2`` (H dv, rank) the columns of ``proj`` at
    ``g_off`` are the rank inner values of a low-rank gate and the gate's input is w_g2 times them (the form of steps
    with few tokens). Returns o, or with ``bf16_copy`` its rounding to bf16 (the operand of a bf16 MFMA product)."""
    T, ld = proj.shape
    cols = H * dv if w_g2 is None else w_g2.shape[1]
    if o.shape != (T, H * dv) or g_off + cols > ld or (weight is not None and weight.numel() != dv) or \
            (w_g2 is not None and w_g2.shape[0] != H * dv):
        raise ValueError("head_gate: shapes")
    o16 = torch.empty(T, H * dv, dtype=torch.bfloat16, device=o.device) if bf16_copy else None
    _check(load_library().lgs_head_gate(_dev(o, "o", F32), _dev(proj, "proj", F32) + 4 * g_off, ld, T, H, dv,
                                        int(unit_norm), float(eps), act, _opt(weight, "weight", F32), float(post),
                                        _opt(o16, "o_bf16", torch.bfloat16), _opt(w_g2, "w_g2"),
                                        0 if w_g2 is None else w_g2.shape[1], 0 if w_g2 is None else _wf32(w_g2, "w_g2"),
                                        _stream()))
    return o16 if bf16_copy else o


def latent_prepare(proj: torch.Tensor, q_off: int, kv_off: int, cache_c: torch.Tensor, cache_kr: torch.Tensor,
                   norm_w: torch.Tensor, inv_freq: Optional[torch.Tensor], slot: torch.Tensor, pos: torch.Tensor, *,
                   H: int, d: int, dr: int, r: int, rot_dims: int, eps: float) -> None:
    T, ld = proj.shape
    slots, S = cache_c.shape[:2]
    if tuple(cache_c.shape) != (slots, S, r) or tuple(cache_kr.shape) != (slots, S, dr) or norm_w.numel() != r:
        raise ValueError("latent_prepare: cache shapes")
    if q_off + H * (d + dr) > ld or kv_off + r + dr > ld or slot.numel() != T or pos.numel() != T:
        raise ValueError("latent_prepare: projections outside the row")
    _check(load_library().lgs_latent_prepare(_dev(proj, "proj", F32), ld, q_off, kv_off, _dev(cache_c, "cache_c"),
                                             _wf32(cache_c, "cache_c"), _dev(cache_kr, "cache_kr", F32),
                                             _dev(norm_w, "norm_w", F32), _opt(inv_freq, "inv_freq", F32),
                                             _dev(slot, "slot", I32), _dev(pos, "pos", I32), T, H, d, dr, r, rot_dims,
                                             S, float(eps), _stream()))


def latent_attention(qc: torch.Tensor, proj: torch.Tensor, q_off: int, cache_c: torch.Tensor, cache_kr: torch.Tensor,
                     sink: Optional[torch.Tensor], slot: torch.Tensor, pos: torch.Tensor, *, H: int, d: int, dr: int,
                     r: int, scale: float, splits: Optional[int] = None) -> torch.Tensor:
    """Softmax attention of every (token, head) over its sequence's cached rows up to the token's position, in the
    latent space. ``splits``: workgroups per (token, head); by default enough of them to fill the chip when the
    step has few rows (decode), one when it has many (a prompt)."""
    T, ld = proj.shape
    S = cache_c.shape[1]
    if qc.shape != (T, H * r) or (sink is not None and sink.numel() != H):
        raise ValueError("latent_attention: shapes")
    out = torch.empty(T, H * r, dtype=F32, device=proj.device)
    if splits is None:
        splits = max(1, min(32, 1024 // (T * H)))
    part = torch.empty(T * H * splits * (r + 2), dtype=F32, device=proj.device) if splits > 1 else None
    _check(load_library().lgs_latent_attention(_dev(qc, "qc", F32), _dev(proj, "proj", F32), ld, q_off,
                                               _dev(cache_c, "cache_c"), _wf32(cache_c, "cache_c"),
                                               _dev(cache_kr, "cache_kr", F32), _opt(sink, "sink", F32),
                                               _dev(slot, "slot", I32), _dev(pos, "pos", I32), out.data_ptr(), T, H,
                                               d, dr, r, S, float(scale), splits, _opt(part, "part", F32), _stream()))
    return out


def latent_attention_tiles(qc: torch.Tensor, proj: torch.Tensor, q_off: int, cache_c: torch.Tensor,
                           cache_kr: torch.Tensor, sink: Optional[torch.Tensor], seq_start: torch.Tensor,
                           seq_slot: torch.Tensor, seq_pos0: torch.Tensor, max_len: int, *, H: int, d: int, dr: int,
                           r: int, scale: float) -> torch.Tensor:
    """The prompt form of ``latent_attention``: tiles of 16 consecutive tokens of a sequence against key tiles of 16
    cached rows on fp32 MFMA. ``max_len``: the most tokens any sequence brings to this step. r % 64 == 0."""
    T, ld = proj.shape
    B = seq_slot.numel()
    S = cache_c.shape[1]
    if qc.shape != (T, H * r) or (sink is not None and sink.numel() != H) or seq_start.numel() != B + 1:
        raise ValueError("latent_attention_tiles: shapes")
    out = torch.empty(T, H * r, dtype=F32, device=proj.device)
    _check(load_library().lgs_latent_attention_tiles(
        _dev(qc, "qc", F32), _dev(proj, "proj", F32), ld, q_off, _dev(cache_c, "cache_c"), _wf32(cache_c, "cache_c"),
        _dev(cache_kr, "cache_kr", F32), _opt(sink, "sink", F32), _dev(seq_start, "seq_start", I32),
        _dev(seq_slot, "seq_slot", I32), _dev(seq_pos0, "seq_pos0", I32), out.data_ptr(), B, int(max_len), H, d, dr, r,
        S, float(scale), _stream()))
    return out


def glu(proj: torch.Tensor, a_off: int, b_off: int, n: int, act: int, bf16: bool = False) -> torch.Tensor:
    """act(proj[:, a_off:a_off + n]) * proj[:, b_off:b_off + n]; ``bf16``: rounded to bf16 (a bf16 product's operand)."""
    T, ld = proj.shape
    if max(a_off, b_off) + n > ld:
        raise ValueError("glu: columns outside the row")
    out = torch.empty(T, n, dtype=torch.bfloat16 if bf16 else F32, device=proj.device)
    base = _dev(proj, "proj", F32)
    _check(load_library().lgs_glu(base + 4 * a_off, base + 4 * b_off, ld, out.data_ptr(), int(bf16), T, n, act,
                                  _stream()))
    return out


def moe_route(proj: torch.Tensor, z_off: int, E: int, top: int):
    T, ld = proj.shape
    if z_off + E > ld:
        raise ValueError("moe_route: router logits outside the row")
    ids = torch.empty(T, top, dtype=I32, device=proj.device)
    wts = torch.empty(T, top, dtype=F32, device=proj.device)
    _check(load_library().lgs_moe_route(_dev(proj, "proj", F32) + 4 * z_off, ld, T, E, top, ids.data_ptr(),
                                        wts.data_ptr(), _stream()))
    return ids, wts


def moe_route_scores(proj: torch.Tensor, z_off: int, E: int, top: int, bias: Optional[torch.Tensor] = None,
                     sigmoid: bool = False, square: bool = False):
    """Softmax over all E router outputs at proj[:, z_off:] (``sigmoid``: the sigmoid of every output on its own); the
    ``top`` largest of score + ``bias`` are chosen (lowest index first among equals); the weights are the chosen scores
    themselves, not renormalised (``square``: their squares)."""
    T, ld = proj.shape
    if z_off + E > ld or (bias is not None and bias.numel() != E):
        raise ValueError("moe_route_scores: router logits outside the row, or the correction's size")
    ids = torch.empty(T, top, dtype=I32, device=proj.device)
    wts = torch.empty(T, top, dtype=F32, device=proj.device)
    _check(load_library().lgs_moe_route_scores(_dev(proj, "proj", F32) + 4 * z_off, ld, T, E, top,
                                               _opt(bias, "bias", F32), ids.data_ptr(), wts.data_ptr(), int(sigmoid),
                                               int(square), _stream()))
    return ids, wts


def act_rows(proj: torch.Tensor, off: int, n: int, act: int, gate_off: int = -1, bf16: bool = False) -> torch.Tensor:
    """act(proj[:, off:off + n]), times sigmoid(proj[:, gate_off]) row by row when ``gate_off`` >= 0; ``bf16``: rounded
    to bf16 (a bf16 product's operand)."""
    T, ld = proj.shape
    if off + n > ld or gate_off >= ld:
        raise ValueError("act_rows: columns outside the row")
    out = torch.empty(T, n, dtype=torch.bfloat16 if bf16 else F32, device=proj.device)
    base = _dev(proj, "proj", F32)
    _check(load_library().lgs_act_rows(base + 4 * off, ld, base + 4 * gate_off if gate_off >= 0 else None, ld,
                                       out.data_ptr(), int(bf16), T, n, act, _stream()))
    return out


def sandwich_step(x: torch.Tensor, *, branches=(), coef: float = 1.0, post_w: Optional[torch.Tensor] = None,
                  next_w: Optional[torch.Tensor] = None, eps: float, want_f32: bool = True, bf16_copy: bool = False):
    """One boundary between sublayers that are normed on the way in and out, in place on the residual x (T, W).
    ``branches``: up to two (y, w) pairs of the sublayer that ran, each y (T, W) RMS-normed with weight w (w None: taken
    as it is); their sum times ``coef`` is RMS-normed with ``post_w`` (the output norm's weight times the layer's
    per-channel scale) and added to x. With ``next_w`` the next sublayer's input rmsnorm(x) * next_w is returned as
    (h fp32 or None, h bf16 or None)."""
    T, W = x.shape
    ys = [(None, None), (None, None)]
    for i, (y, w) in enumerate(branches):
        if i > 1 or y.shape != (T, W) or (w is not None and w.numel() != W):
            raise ValueError("sandwich_step: at most two branches of the residual's shape")
        ys[i] = (y, w)
    if (ys[0][0] is not None and (post_w is None or post_w.numel() != W)) or (next_w is not None and next_w.numel() != W):
        raise ValueError("sandwich_step: norm weights")
    h = torch.empty(T, W, dtype=F32, device=x.device) if next_w is not None and (want_f32 or not bf16_copy) else None
    h16 = torch.empty(T, W, dtype=torch.bfloat16, device=x.device) if next_w is not None and bf16_copy else None
    _check(load_library().lgs_sandwich_step(_dev(x, "x", F32), _opt(ys[0][0], "y0", F32), _opt(ys[0][1], "w0", F32),
                                            _opt(ys[1][0], "y1", F32), _opt(ys[1][1], "w1", F32), float(coef),
                                            _opt(post_w, "post_w", F32), _opt(next_w, "next_w", F32),
                                            _opt(h, "h", F32), _opt(h16, "h_bf16", torch.bfloat16), float(eps), T, W,
                                            _stream()))
    return h, h16


def moe_router(h: torch.Tensor, w: torch.Tensor, top: int, bias: Optional[torch.Tensor] = None, sigmoid: bool = False,
               square: bool = False):
    """``moe_route_scores`` of the router logits w h, both in one launch (steps with few tokens). w (E, K)."""
    T, K = h.shape
    E = w.shape[0]
    if w.shape[1] != K or (bias is not None and bias.numel() != E):
        raise ValueError("moe_router: shapes")
    ids = torch.empty(T, top, dtype=I32, device=h.device)
    wts = torch.empty(T, top, dtype=F32, device=h.device)
    _check(load_library().lgs_moe_router(_dev(h, "h", F32), K, _dev(w, "w"), _wf32(w, "w"), T, K, E, top,
                                         _opt(bias, "bias", F32), ids.data_ptr(), wts.data_ptr(), int(sigmoid),
                                         int(square), _stream()))
    return ids, wts


def moe_up(h: torch.Tensor, up: torch.Tensor, ids: torch.Tensor, act: int, gated: bool = False) -> torch.Tensor:
    """up (E, F, K), or with ``gated`` (E, 2 F, K): F gate rows, then F up rows -> act(gate h) * (up h). Pairs whose
    expert id is >= E (experts without matrices) are left untouched."""
    T, K = h.shape
    E, F, K2 = up.shape
    if gated:
        F //= 2
    top = ids.shape[1]
    if K2 != K or ids.shape[0] != T:
        raise ValueError("moe_up: shapes")
    buf = torch.empty(T * top, F, dtype=F32, device=h.device)
    _check(load_library().lgs_moe_up(_dev(h, "h", F32), K, _dev(up, "up"), _wf32(up, "up"), _dev(ids, "ids", I32),
                                     buf.data_ptr(), T, top, F, K, act, int(gated), E, _stream()))
    return buf


def moe_down(actbuf: torch.Tensor, down: torch.Tensor, ids: torch.Tensor, wts: torch.Tensor, x: torch.Tensor,
             h: torch.Tensor, accumulate: bool = True) -> None:
    """x (+)= sum over a token's choices of weight * down[expert] act; a choice whose id is >= the number of stored
    experts is an identity expert and contributes weight * h."""
    T, top = ids.shape
    E, N, F = down.shape
    if actbuf.shape != (T * top, F) or x.shape != (T, N) or h.shape != (T, N):
        raise ValueError("moe_down: shapes")
    _check(load_library().lgs_moe_down(_dev(actbuf, "actbuf", F32), _dev(down, "down"), _wf32(down, "down"),
                                       _dev(ids, "ids", I32), _dev(wts, "wts", F32), _dev(x, "x", F32), N, T, top, N,
                                       F, E, _dev(h, "h", F32), N, int(accumulate), _stream()))


def moe_sort(ids: torch.Tensor, E: int):
    T, top = ids.shape
    dev = ids.device
    z_start = torch.empty(E + 1, dtype=I32, device=dev)
    tok_of = torch.empty(T * top, dtype=I32, device=dev)
    where = torch.empty(T * top, dtype=I32, device=dev)
    ws = torch.zeros(2 * E, dtype=I32, device=dev)
    _check(load_library().lgs_moe_sort(_dev(ids, "ids", I32), T * top, top, E, z_start.data_ptr(), tok_of.data_ptr(),
                                       where.data_ptr(), ws.data_ptr(), _stream()))
    return z_start, tok_of, where


def moe_combine(y: torch.Tensor, where: torch.Tensor, wts: torch.Tensor, x: torch.Tensor, *,
                ids: Optional[torch.Tensor] = None, n_real: int = 0, h: Optional[torch.Tensor] = None,
                accumulate: bool = True) -> None:
    """x (+)= sum_k wts[:, k] * y[where[:, k]]; with ``ids`` a choice whose id is >= ``n_real`` (an identity expert)
    contributes the token's input ``h`` instead."""
    T, top = wts.shape
    N = x.shape[1]
    if y.shape != (T * top, N) or where.numel() != T * top or (ids is not None and (h is None or h.shape != (T, N))):
        raise ValueError("moe_combine: shapes")
    _check(load_library().lgs_moe_combine(_dev(y, "y", F32), _dev(where, "where", I32), _dev(wts, "wts", F32),
                                          _dev(x, "x", F32), N, T, top, N, _opt(ids, "ids", I32), int(n_real),
                                          _opt(h, "h", F32), N, int(accumulate), _stream()))


def token_side(x: torch.Tensor, tokens: torch.Tensor, table: torch.Tensor, col0: int, gate_w: torch.Tensor,
               proj_w: torch.Tensor, norm_w: torch.Tensor, eps: float) -> None:
    T, W = x.shape
    dim = gate_w.shape[0]
    V, ld = table.shape
    if gate_w.shape != (dim, W) or proj_w.shape != (W, dim) or norm_w.numel() != W or col0 + dim > ld:
        raise ValueError("token_side: shapes")
    if len({table.dtype, gate_w.dtype, proj_w.dtype}) != 1:
        raise TypeError("token_side: weights of one dtype expected")
    _check(load_library().lgs_token_side(_dev(x, "x", F32), _dev(tokens, "tokens", I32), _dev(table, "table"),
                                         _wf32(table, "table"), ld, col0, _dev(gate_w, "gate_w"),
                                         _dev(proj_w, "proj_w"), _dev(norm_w, "norm_w", F32), T, W, dim, V,
                                         float(eps), _stream()))


def embed_streams(tokens: torch.Tensor, table: torch.Tensor, scale: float, streams: int) -> torch.Tensor:
    """(T, streams, W) fp32: every stream starts as the scaled embedding row."""
    T, (V, W) = tokens.numel(), table.shape
    x = torch.empty(T, streams, W, dtype=F32, device=tokens.device)
    _check(load_library().lgs_embed_streams(_dev(tokens, "tokens", I32), _dev(table, "table"), _wf32(table, "table"),
                                            float(scale), x.data_ptr(), T, W, V, streams, _stream()))
    return x


def streams_step(x: torch.Tensor, *, y: Optional[torch.Tensor] = None, mix: Optional[torch.Tensor] = None,
                 out: Optional[torch.Tensor] = None, read: Optional[torch.Tensor] = None,
                 norm_w: Optional[torch.Tensor] = None, eps: float = 0.0, bf16_copy: bool = False):
    """One sublayer boundary of a multi-stream residual x (T, s, W), in place: with ``y`` (T, W) the write-back
    x_j <- sum_i mix[i, j] x_i + out[j] y; then with ``read`` (s,) the next sublayer's input
    h = rmsnorm(sum_j read[j] x_j) * norm_w (no ``norm_w``: the weighted sum itself). Returns None without a read,
    else h, or (h, h_bf16) with ``bf16_copy``."""
    T, s, W = x.shape
    if y is not None and (y.shape != (T, W) or mix is None or out is None or mix.numel() != s * s or out.numel() != s):
        raise ValueError("streams_step: write-back shapes")
    if read is not None and (read.numel() != s or (norm_w is not None and norm_w.numel() != W)):
        raise ValueError("streams_step: read shapes")
    h = torch.empty(T, W, dtype=F32, device=x.device) if read is not None else None
    h16 = torch.empty(T, W, dtype=torch.bfloat16, device=x.device) if read is not None and bf16_copy else None
    _check(load_library().lgs_streams_step(_dev(x, "x", F32), _opt(y, "y", F32), _opt(mix, "mix", F32),
                                           _opt(out, "out", F32), _opt(read, "read", F32), _opt(norm_w, "norm_w", F32),
                                           _opt(h, "h", F32), _opt(h16, "h_bf16", torch.bfloat16), float(eps), T, W, s,
                                           _stream()))
    if read is None:
        return None
    return (h, h16) if bf16_copy else h


def diffattn_prepare(proj: torch.Tensor, q_off: int, k_off: int, v_off: int, cache_k: Optional[torch.Tensor],
                     cache_v: Optional[torch.Tensor], inv_freq: Optional[torch.Tensor], slot: torch.Tensor,
                     pos: torch.Tensor, *, H: int, G: int, d: int, dv: int, rot_dims: int) -> None:
    """Rotates the query maps of ``proj`` in place; with key / value columns (``k_off`` >= 0) the rotated keys and
    the values go to the cache rows (slot, position). cache_k (slots, S, G, 2 d), cache_v (slots, S, G, dv)."""
    T, ld = proj.shape
    S = 1
    if k_off >= 0:
        slots, S = cache_k.shape[:2]
        if tuple(cache_k.shape) != (slots, S, G, 2 * d) or tuple(cache_v.shape) != (slots, S, G, dv) or \
                cache_k.dtype != cache_v.dtype:
            raise ValueError("diffattn_prepare: cache shapes")
    if slot.numel() != T or pos.numel() != T:
        raise ValueError("diffattn_prepare: one slot and position per row")
    f32 = _wf32(cache_k, "cache_k") if k_off >= 0 else 1
    _check(load_library().lgs_diffattn_prepare(_dev(proj, "proj", F32), ld, q_off, k_off, v_off,
                                               _dev(cache_k, "cache_k") if k_off >= 0 else None,
                                               _dev(cache_v, "cache_v") if k_off >= 0 else None, f32,
                                               _opt(inv_freq, "inv_freq", F32), _dev(slot, "slot", I32),
                                               _dev(pos, "pos", I32), T, H, G, d, dv, rot_dims, S, _stream()))


def diffattn(proj: torch.Tensor, q_off: int, cache_k: torch.Tensor, cache_v: torch.Tensor, seq_start: torch.Tensor,
             seq_slot: torch.Tensor, seq_pos0: torch.Tensor, max_len: int, *, H: int, G: int, d: int, dv: int,
             chunk: int, scale: float, cap: float, lam: float, eps: float, post: float, bf16_copy: bool = False,
             splits: Optional[int] = None) -> torch.Tensor:
    """Differential attention of every row of a packed batch over its sequence's cached keys and values; the
    rotated queries are the 2 H d columns of ``proj`` at ``q_off``. Returns (T, H dv) fp32, or with ``bf16_copy``
    its rounding to bf16 (the out-projection's MFMA operand). ``splits``: workgroups per (token, head) when every
    sequence brings one token (default: enough to fill the chip, at least 128 keys each)."""
    T, ld = proj.shape
    B = seq_slot.numel()
    slots, S = cache_k.shape[:2]
    if tuple(cache_k.shape) != (slots, S, G, 2 * d) or tuple(cache_v.shape) != (slots, S, G, dv):
        raise ValueError("diffattn: cache shapes")
    if seq_start.numel() != B + 1 or q_off + 2 * H * d > ld or not 1 <= max_len <= T:
        raise ValueError("diffattn: step table / query columns")
    out = torch.empty(T, H * dv, dtype=F32, device=proj.device)
    out16 = torch.empty(T, H * dv, dtype=torch.bfloat16, device=proj.device) if bf16_copy else None
    if max_len > 1:
        splits = 1
    elif splits is None:
        span = min(S, chunk) if chunk > 0 else S
        splits = max(1, min(64, 512 // max(1, B * H), (span + 127) // 128))
    part = torch.empty(T * H * splits * (4 + 2 * dv), dtype=F32, device=proj.device) if splits > 1 else None
    _check(load_library().lgs_diffattn(_dev(proj, "proj", F32) + 4 * q_off, ld, _dev(cache_k, "cache_k"),
                                       _dev(cache_v, "cache_v"), _wf32(cache_k, "cache_k"),
                                       _dev(seq_start, "seq_start", I32), _dev(seq_slot, "seq_slot", I32),
                                       _dev(seq_pos0, "seq_pos0", I32), out.data_ptr(),
                                       _opt(out16, "out_bf16", torch.bfloat16), _opt(part, "part", F32), splits, B,
                                       int(max_len), H, G, d, dv, S, int(chunk), float(scale), float(cap), float(lam),
                                       float(eps), float(post), _stream()))
    return out16 if bf16_copy else out


def conv_silu(proj: torch.Tensor, off: int, weight: torch.Tensor, bias: torch.Tensor, state: torch.Tensor,
              seq_start: torch.Tensor, seq_slot: torch.Tensor, seq_pos0: torch.Tensor, max_len: int) -> torch.Tensor:
    """silu(causal per-channel convolution + bias) of the C columns of ``proj`` at ``off`` over a packed batch;
    weight (C, taps): column taps - 1 weights the token itself, column 0 the oldest input. state (slots, taps - 1, C)
    fp32 carries every sequence's last inputs from step to step. Returns (T, C) fp32."""
    T, ld = proj.shape
    C, taps = weight.shape
    B = seq_slot.numel()
    if off + C > ld or bias.numel() != C or tuple(state.shape[1:]) != (max(1, taps - 1), C) or weight.dtype != bias.dtype:
        raise ValueError("conv_silu: shapes")
    out = torch.empty(T, C, dtype=F32, device=proj.device)
    _check(load_library().lgs_conv_silu(_dev(proj, "proj", F32) + 4 * off, ld, _dev(weight, "weight"),
                                        _dev(bias, "bias"), _wf32(weight, "weight"), _dev(state, "state", F32),
                                        _dev(seq_start, "seq_start", I32), _dev(seq_slot, "seq_slot", I32),
                                        _dev(seq_pos0, "seq_pos0", I32), out.data_ptr(), B, int(max_len), C, taps,
                                        _stream()))
    return out


def ssm_scan(xbc: torch.Tensor, proj: torch.Tensor, dt_off: int, dt_bias: torch.Tensor, A_log: torch.Tensor,
             D: torch.Tensor, state: torch.Tensor, seq_start: torch.Tensor, seq_slot: torch.Tensor,
             seq_pos0: torch.Tensor, *, heads: int, groups: int, N: int, dv: int, max_len: int = 0,
             chunked: Optional[bool] = None) -> torch.Tensor:
    """The selective scan over a packed batch: xbc (T, heads dv + 2 groups N) after the convolution, raw step sizes
    in the ``heads`` columns of ``proj`` at ``dt_off``; state (slots, heads, N, dv) fp32. Returns y (T, heads dv).
    ``chunked`` picks the prompt form (64-token chunks as matrix products, all chunks side by side; N <= 128) over
    the token-by-token walk; by default steps in which a sequence brings more than 16 tokens (``max_len``) take it."""
    T, ldx = xbc.shape
    B = seq_slot.numel()
    if ldx != heads * dv + 2 * groups * N or tuple(state.shape[1:]) != (heads, N, dv) or proj.shape[0] != T:
        raise ValueError("ssm_scan: shapes")
    if dt_off + heads > proj.shape[1] or min(dt_bias.numel(), A_log.numel(), D.numel()) != heads:
        raise ValueError("ssm_scan: per-head parameters")
    y = torch.empty(T, heads * dv, dtype=F32, device=xbc.device)
    if chunked is None:
        chunked = max_len > 16 and N <= 128
    ws, wdec, max_chunks = None, None, 0
    if chunked:
        if not 0 < max_len <= T or N > 128:
            raise ValueError("ssm_scan: the prompt form needs the longest sequence's token count and N <= 128")
        max_chunks = (max_len + 63) // 64
        ws = torch.empty(B * max_chunks * heads * N * dv, dtype=F32, device=xbc.device)
        wdec = torch.empty(B * max_chunks * heads, dtype=F32, device=xbc.device)
    _check(load_library().lgs_ssm_scan(_dev(xbc, "xbc", F32), ldx, _dev(proj, "proj", F32) + 4 * dt_off,
                                       proj.shape[1], _dev(dt_bias, "dt_bias", F32), _dev(A_log, "A_log", F32),
                                       _dev(D, "D", F32), _dev(state, "state", F32), _dev(seq_start, "seq_start", I32),
                                       _dev(seq_slot, "seq_slot", I32), _dev(seq_pos0, "seq_pos0", I32), y.data_ptr(),
                                       B, heads, groups, N, dv, _opt(ws, "ws", F32), _opt(wdec, "wdec", F32),
                                       max_chunks, _stream()))
    return y


def gated_group_norm(y: torch.Tensor, proj: torch.Tensor, z_off: int, weight: torch.Tensor, *, groups: int,
                     eps: float, bf16_copy: bool = False) -> torch.Tensor:
    """unit_rms_per_group(y * silu(z)) * weight with z the columns of ``proj`` at ``z_off``; (T, inner) fp32 or, with
    ``bf16_copy``, its rounding to bf16."""
    T, inner = y.shape
    if z_off + inner > proj.shape[1] or weight.numel() != inner or inner % groups:
        raise ValueError("gated_group_norm: shapes")
    out = torch.empty(T, inner, dtype=F32, device=y.device)
    out16 = torch.empty(T, inner, dtype=torch.bfloat16, device=y.device) if bf16_copy else None
    _check(load_library().lgs_gated_group_norm(_dev(y, "y", F32), _dev(proj, "proj", F32) + 4 * z_off, proj.shape[1],
                                               _dev(weight, "weight", F32), float(eps), out.data_ptr(),
                                               _opt(out16, "out_bf16", torch.bfloat16), T, inner, groups, _stream()))
    return out16 if bf16_copy else out


def glu_clamped(proj: torch.Tensor, a_off: int, b_off: int, n: int, *, alpha: float, limit: float, shift: float,
                bf16: bool = False) -> torch.Tensor:
    """g sigmoid(alpha g) (u + shift) with g = min(proj[:, a_off:], limit), u = clamp(proj[:, b_off:], +-limit)."""
    T, ld = proj.shape
    if max(a_off, b_off) + n > ld:
        raise ValueError("glu_clamped: columns outside the row")
    out = torch.empty(T, n, dtype=torch.bfloat16 if bf16 else F32, device=proj.device)
    base = _dev(proj, "proj", F32)
    _check(load_library().lgs_glu_clamped(base + 4 * a_off, base + 4 * b_off, ld, out.data_ptr(), int(bf16), T, n,
                                          float(alpha), float(limit), float(shift), _stream()))
    return out


def embed_pos(tokens: torch.Tensor, pos: torch.Tensor, table: torch.Tensor, pos_table: torch.Tensor, scale: float,
              bf16_copy: bool = False):
    """x[t] = table[tokens[t]] * scale + pos_table[pos[t]] (T, W) fp32; with ``bf16_copy`` also its rounding."""
    T, (V, W) = tokens.numel(), table.shape
    if pos.numel() != T or pos_table.shape[1] != W or pos_table.dtype != table.dtype:
        raise ValueError("embed_pos: shapes")
    x = torch.empty(T, W, dtype=F32, device=tokens.device)
    x16 = torch.empty(T, W, dtype=torch.bfloat16, device=tokens.device) if bf16_copy else None
    _check(load_library().lgs_embed_pos(_dev(tokens, "tokens", I32), _dev(pos, "pos", I32), _dev(table, "table"),
                                        _dev(pos_table, "pos_table"), _wf32(table, "table"), float(scale),
                                        x.data_ptr(), _opt(x16, "x_bf16", torch.bfloat16), T, W, V,
                                        pos_table.shape[0], _stream()))
    return (x, x16) if bf16_copy else x


def layernorm(y: torch.Tensor, weight: torch.Tensor, bias: Optional[torch.Tensor], *, eps: float,
              x: Optional[torch.Tensor] = None, mult: float = 1.0, bf16_copy: bool = False):
    """Layer norm of the rows of y (rows, n): (y - mean) / sqrt(var + eps) * weight + bias, var the mean of the squared
    deviations. With ``x`` the result joins a residual in place, x += mult * norm (a sublayer's normed output);
    without, it is returned times ``mult``. ``bf16_copy``: also the rounding of the result (of the new x) to bf16."""
    rows, n = y.shape
    if weight.numel() != n or (bias is not None and bias.numel() != n) or (x is not None and x.shape != y.shape):
        raise ValueError("layernorm: shapes")
    out = x if x is not None else torch.empty_like(y)
    o16 = torch.empty(rows, n, dtype=torch.bfloat16, device=y.device) if bf16_copy else None
    _check(load_library().lgs_layernorm(_dev(y, "y", F32), _dev(weight, "weight", F32), _opt(bias, "bias", F32),
                                        float(eps), float(mult), int(x is not None), _dev(out, "x", F32),
                                        _opt(o16, "x_bf16", torch.bfloat16), rows, n, _stream()))
    return (out, o16) if bf16_copy else out


def softcap(z: torch.Tensor, cap: float) -> torch.Tensor:
    """In place: cap * tanh(z / cap)."""
    _check(load_library().lgs_softcap(_dev(z, "z", F32), z.numel(), float(cap), _stream()))
    return z


def normattn_prepare(proj: torch.Tensor, q_off: int, k_off: int, v_off: int, cache_k: torch.Tensor,
                     cache_v: torch.Tensor, slot: torch.Tensor, pos: torch.Tensor, *, H: int, G: int, d: int, dv: int,
                     eps: float, temp_coef: float = 0.0, temp_every: int = 0, norm: bool = True,
                     q_weight: Optional[torch.Tensor] = None, k_weight: Optional[torch.Tensor] = None,
                     inv_freq: Optional[torch.Tensor] = None, rot_dims: int = 0) -> None:
    """Queries normed (``norm``: divided by their root mean square, times ``q_weight`` (d,) if given), rotated on the
    pairs (i, i + rot_dims / 2) and multiplied by the position's query temperature, in place in ``proj``; keys normed
    (``k_weight``) and rotated alike, and the values, into the cache rows (slot, position). cache_k (slots, S, G, d),
    cache_v (slots, S, G, dv). ``v_off == k_off`` (with dv == d): the values are the keys as projected."""
    T, ld = proj.shape
    slots, S = cache_k.shape[:2]
    if tuple(cache_k.shape) != (slots, S, G, d) or tuple(cache_v.shape) != (slots, S, G, dv) or \
            cache_k.dtype != cache_v.dtype:
        raise ValueError("normattn_prepare: cache shapes")
    if slot.numel() != T or pos.numel() != T:
        raise ValueError("normattn_prepare: one slot and position per row")
    if any(w is not None and w.numel() != d for w in (q_weight, k_weight)) or rot_dims % 2 or rot_dims > d or \
            (rot_dims > 0 and (inv_freq is None or inv_freq.numel() < rot_dims // 2)):
        raise ValueError("normattn_prepare: norm weights of d values, rotary frequencies for rot_dims / 2 pairs")
    _check(load_library().lgs_normattn_prepare(_dev(proj, "proj", F32), ld, q_off, k_off, v_off,
                                               _dev(cache_k, "cache_k"), _dev(cache_v, "cache_v"),
                                               _wf32(cache_k, "cache_k"), _dev(slot, "slot", I32),
                                               _dev(pos, "pos", I32), T, H, G, d, dv, S, float(eps), float(temp_coef),
                                               int(temp_every), int(norm), _opt(q_weight, "q_weight", F32),
                                               _opt(k_weight, "k_weight", F32), _opt(inv_freq, "inv_freq", F32),
                                               int(rot_dims), _stream()))


def sinkattn(proj: torch.Tensor, q_off: int, cache_k: torch.Tensor, cache_v: torch.Tensor,
             sink: Optional[torch.Tensor], seq_start: torch.Tensor, seq_slot: torch.Tensor, seq_pos0: torch.Tensor,
             max_len: int, *, H: int, G: int, d: int, dv: int, scale: float, chunk: int = 0, cap: float = 0.0,
             post: float = 1.0, bf16_copy: bool = False, splits: Optional[int] = None,
             gate_off: int = -1) -> torch.Tensor:
    """Causal softmax attention of every row of a packed batch over its sequence's cached keys and values, grouped
    key / value heads, with exp(sink[h]) in the normaliser; the prepared queries are the H d columns of ``proj`` at
    ``q_off``. ``gate_off`` >= 0: head h's output is multiplied by sigmoid(proj[:, gate_off + h]). Returns (T, H dv)
    fp32 times ``post``, or with ``bf16_copy`` its rounding to bf16."""
    T, ld = proj.shape
    B = seq_slot.numel()
    slots, S = cache_k.shape[:2]
    if tuple(cache_k.shape) != (slots, S, G, d) or tuple(cache_v.shape) != (slots, S, G, dv):
        raise ValueError("sinkattn: cache shapes")
    if seq_start.numel() != B + 1 or q_off + H * d > ld or not 1 <= max_len <= T or \
            (sink is not None and sink.numel() != H) or gate_off + H > ld:
        raise ValueError("sinkattn: step table / query columns / sink / head gates")
    out = torch.empty(T, H * dv, dtype=F32, device=proj.device)
    out16 = torch.empty(T, H * dv, dtype=torch.bfloat16, device=proj.device) if bf16_copy else None
    if max_len > 1:
        splits = 1
    elif splits is None:
        span = min(S, chunk) if chunk > 0 else S
        splits = max(1, min(64, 512 // max(1, B * H), (span + 127) // 128))
    part = torch.empty(T * H * splits * (2 + dv), dtype=F32, device=proj.device) if splits > 1 else None
    _check(load_library().lgs_sinkattn(_dev(proj, "proj", F32) + 4 * q_off, ld, _dev(cache_k, "cache_k"),
                                       _dev(cache_v, "cache_v"), _wf32(cache_k, "cache_k"), _opt(sink, "sink", F32),
                                       _dev(seq_start, "seq_start", I32), _dev(seq_slot, "seq_slot", I32),
                                       _dev(seq_pos0, "seq_pos0", I32), out.data_ptr(),
                                       _opt(out16, "out_bf16", torch.bfloat16), _opt(part, "part", F32), splits, B,
                                       int(max_len), H, G, d, dv, S, int(chunk), float(scale), float(cap), float(post),
                                       _dev(proj, "proj", F32) + 4 * gate_off if gate_off >= 0 else None, ld,
                                       _stream()))
    return out16 if bf16_copy else out


def delta_prepare(qkv: torch.Tensor, a: torch.Tensor, a_off: int, b: torch.Tensor, b_off: int, A_log: torch.Tensor,
                  dt_bias: torch.Tensor, *, H: int, G: int, d: int, per_channel: bool, q_scale: float,
                  norm_eps: float = 1e-6, w_a2: Optional[torch.Tensor] = None, unit: bool = True,
                  decay_form: int = 0, tau: float = 1.0, qkv_off: int = 0):
    """qkv (T, ld) holds q | k (G d each) from column ``qkv_off``. ``unit``: q and k become unit vectors per head in
    place (q also times ``q_scale``); otherwise q is only scaled. ``decay_form`` 1: the decays are
    sigmoid(a + dt_bias)^(1 / tau) (``A_log`` None). ``b`` None: no betas. The raw decay
    inputs are the H d (``per_channel``) or H columns of ``a`` at ``a_off`` - or, with ``w_a2`` (H d or H, rank), w_a2
    times the rank columns there; the raw betas are the H columns of ``b`` at ``b_off``. Returns (dec, beta, kq):
    exp(-exp(A_log) softplus(a + dt_bias)) (T, H d) or (T, H), sigmoid(b) (T, H), and k . q of the prepared vectors
    per key head (T, G)."""
    T, ld = qkv.shape
    n = H * d if per_channel else H
    cols = n if w_a2 is None else w_a2.shape[1]
    if a.shape[0] != T or a_off + cols > a.shape[1] or (b is not None and (b.shape[0] != T or b_off + H > b.shape[1])) or \
            (decay_form == 0 and (A_log is None or A_log.numel() != H)) or dt_bias.numel() != n or \
            ld < qkv_off + 2 * G * d or (w_a2 is not None and w_a2.shape[0] != n) or decay_form not in (0, 1):
        raise ValueError("delta_prepare: shapes")
    dec = torch.empty(T, n, dtype=F32, device=qkv.device)
    beta = torch.empty(T, H, dtype=F32, device=qkv.device) if b is not None else None
    kq = torch.empty(T, G, dtype=F32, device=qkv.device)
    _check(load_library().lgs_delta_prepare(_dev(qkv, "qkv", F32) + 4 * qkv_off, ld, _dev(a, "a", F32) + 4 * a_off,
                                            a.shape[1], _dev(b, "b", F32) + 4 * b_off if b is not None else None,
                                            b.shape[1] if b is not None else 0, _opt(A_log, "A_log", F32),
                                            _dev(dt_bias, "dt_bias", F32), dec.data_ptr(), _opt(beta, "beta", F32),
                                            kq.data_ptr(), T, H, G, d, int(per_channel), float(q_scale),
                                            float(norm_eps), _opt(w_a2, "w_a2"), 0 if w_a2 is None else w_a2.shape[1],
                                            0 if w_a2 is None else _wf32(w_a2, "w_a2"), int(unit), int(decay_form),
                                            float(tau), _stream()))
    return dec, beta, kq


def delta_step_prepare(proj: torch.Tensor, off: int, conv_w: torch.Tensor, conv_state: torch.Tensor,
                       seq_slot: torch.Tensor, seq_pos0: torch.Tensor, a_off: int, b_off: int, A_log: torch.Tensor,
                       dt_bias: torch.Tensor, *, H: int, G: int, d: int, dv: int, per_channel: bool, q_scale: float,
                       norm_eps: float = 1e-6, w_a2: Optional[torch.Tensor] = None):
    """``conv_silu`` (without a bias) and ``delta_prepare`` in one launch for a step in which every sequence brings
    one token: row b of ``proj`` belongs to sequence b; its q | k | v channels start at ``off``, the raw decay inputs
    (or their rank inner values, with ``w_a2``) at ``a_off`` and the raw betas at ``b_off`` of the same row.
    Returns (qkv (B, C), dec, beta, kq)."""
    B, ld = proj.shape
    C, taps = conv_w.shape
    n = H * d if per_channel else H
    cols = n if w_a2 is None else w_a2.shape[1]
    if C != 2 * G * d + H * dv or off + C > ld or seq_slot.numel() != B or seq_pos0.numel() != B or \
            tuple(conv_state.shape[1:]) != (max(1, taps - 1), C) or a_off + cols > ld or b_off + H > ld or \
            A_log.numel() != H or dt_bias.numel() != n or (w_a2 is not None and w_a2.shape[0] != n):
        raise ValueError("delta_step_prepare: shapes")
    dev = proj.device
    qkv = torch.empty(B, C, dtype=F32, device=dev)
    dec = torch.empty(B, n, dtype=F32, device=dev)
    beta = torch.empty(B, H, dtype=F32, device=dev)
    kq = torch.empty(B, G, dtype=F32, device=dev)
    base = _dev(proj, "proj", F32)
    _check(load_library().lgs_delta_step_prepare(
        base + 4 * off, ld, _dev(conv_w, "conv_w"), _wf32(conv_w, "conv_w"), taps, _dev(conv_state, "conv_state", F32),
        _dev(seq_slot, "seq_slot", I32), _dev(seq_pos0, "seq_pos0", I32), qkv.data_ptr(), base + 4 * a_off, ld,
        base + 4 * b_off, ld, _dev(A_log, "A_log", F32), _dev(dt_bias, "dt_bias", F32), dec.data_ptr(), beta.data_ptr(),
        kq.data_ptr(), B, H, G, d, dv, int(per_channel), float(q_scale), float(norm_eps), _opt(w_a2, "w_a2"),
        0 if w_a2 is None else w_a2.shape[1], 0 if w_a2 is None else _wf32(w_a2, "w_a2"), _stream()))
    return qkv, dec, beta, kq


def gated_delta(qkv: torch.Tensor, dec: torch.Tensor, beta: Optional[torch.Tensor], kq: torch.Tensor,
                state: torch.Tensor, seq_start: torch.Tensor, seq_slot: torch.Tensor, seq_pos0: torch.Tensor, *, H: int,
                G: int, d: int, dv: int, per_channel: bool, lanes: int = 0, plain: bool = False,
                qkv_off: int = 0) -> torch.Tensor:
    """The gated delta rule over a packed batch, token by token: S <- diag(dec) S; u = beta (v - S^T k);
    S <- S + k u^T; o = S^T q. qkv (T, 2 G d + H dv) prepared rows, kq (T, G) their k . q (``delta_prepare``); state
    (slots, H, d, dv) fp32 is read unless a sequence starts at position 0 and left at the step's last token. Returns
    o (T, H dv). ``lanes``: lanes that share one state column (4, 8, 16; 0: chosen from the sizes). ``plain``: the
    rule without the correction, S <- diag(dec) S + k v^T, o = S^T q (``beta`` None). ``qkv_off``: the first column of
    q | k | v in wider rows."""
    T, ld = qkv.shape
    B = seq_slot.numel()
    if ld < qkv_off + 2 * G * d + H * dv or tuple(state.shape[1:]) != (H, d, dv) or seq_start.numel() != B + 1 or \
            dec.shape != (T, H * d if per_channel else H) or (not plain and (beta is None or beta.shape != (T, H))) or \
            kq.shape != (T, G):
        raise ValueError("gated_delta: shapes")
    out = torch.empty(T, H * dv, dtype=F32, device=qkv.device)
    _check(load_library().lgs_gated_delta(_dev(qkv, "qkv", F32) + 4 * qkv_off, ld, _dev(dec, "dec", F32),
                                          _opt(beta, "beta", F32) if plain else _dev(beta, "beta", F32),
                                          _dev(kq, "kq", F32), _dev(state, "state", F32), _dev(seq_start, "seq_start", I32),
                                          _dev(seq_slot, "seq_slot", I32), _dev(seq_pos0, "seq_pos0", I32),
                                          out.data_ptr(), B, H, G, d, dv, int(per_channel), int(lanes), int(plain),
                                          _stream()))
    return out
