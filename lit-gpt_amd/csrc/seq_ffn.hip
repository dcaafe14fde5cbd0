// Feed-forward parts of the layered models.
//
//   lgs_glu              out = act(a) * b over two column ranges of one projection (the dense gated feed-forward)
//   lgs_glu_clamped      out = g sigmoid(alpha g) (u + shift) with g = min(a, limit), u = clamp(b, -limit, limit)
//   lgs_moe_route        per token: the `top` largest router logits (fp32, lowest index first among equals) and the
//                        softmax over just those
//   lgs_moe_route_scores per token: softmax over all router outputs (or the sigmoid of each on its own); the choice
//                        adds a stored correction to the scores, the weights are the chosen scores themselves (or
//                        their squares: a score on the input of an expert with a relu^2 activation)
//   lgs_act_rows         out = act(a) times an optional sigmoid gate of one number per row (an ungated unit whose
//                        up-projection is part of a fused product: the shared expert)
//   lgs_moe_up / _down   the routed experts as streaming GEMVs over (token, choice) pairs: only the chosen experts'
//                        rows are read; the down kernel sums a token's choices in their routing order and adds the
//                        result to the residual stream (the decode form; a prompt runs grouped products instead)
//   lgs_moe_sort / lgs_moe_combine   the prompt form: a counting sort of the (token, choice) pairs by
//                        expert, whose ranges drive lgs_linear's grouped products, and the weighted sum back
//   lgs_token_side       per-layer token input: x += unit_rms(proj(gelu_tanh(gate x) * e[token])) * w
#include "seq_common.h"

namespace lgs {

// the dot products of one activation row (fp32, rounded as the weights' precision asks) with two weight rows of n
// elements; `vec` (n % 8 == 0 and 16-byte aligned rows) takes 16-byte loads
template <bool WF32>
__device__ __forceinline__ void dot2(const float* __restrict__ x, const void* __restrict__ w, size_t r0, size_t r1, int n,
                                     bool vec, int lane, float& a0, float& a1) {
  a0 = a1 = 0.0f;
  if (vec) {
#pragma unroll 2
    for (int k = lane * 8; k < n; k += 512) {
      float u[8], v[8];
      wload8<WF32>(w, r0 + k, u);
      wload8<WF32>(w, r1 + k, v);
      const float4 xa = *(const float4*)(x + k), xb = *(const float4*)(x + k + 4);
      const float xs[8] = {xa.x, xa.y, xa.z, xa.w, xb.x, xb.y, xb.z, xb.w};
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const float xe = aop<WF32>(xs[e]);
        a0 = fmaf(xe, u[e], a0);
        a1 = fmaf(xe, v[e], a1);
      }
    }
  } else {
    for (int k = lane; k < n; k += 64) {
      const float xe = aop<WF32>(x[k]);
      a0 = fmaf(xe, wload<WF32>(w, r0 + k), a0);
      a1 = fmaf(xe, wload<WF32>(w, r1 + k), a1);
    }
  }
  a0 = wave_sum(a0);
  a1 = wave_sum(a1);
}

__global__ void __launch_bounds__(256) glu_kernel(const float* __restrict__ a, const float* __restrict__ b, long ld,
                                                  float* __restrict__ out, uint16_t* __restrict__ out16, int n, int act) {
  const size_t t = blockIdx.x;
  const int i = blockIdx.y * 256 + threadIdx.x;
  if (i >= n) return;
  const float v = act_f(act, a[t * ld + i]) * b[t * ld + i];
  if (out16) out16[t * n + i] = f2bf(v);  // the operand of a bf16 product: rounded here instead of at its load
  else out[t * n + i] = v;
}

// grid (T, ceil(n / 256)): g = min(a, limit), u = clamp(b, -limit, limit); out = g sigmoid(alpha g) (u + shift)
// (limit <= 0: no clamps)
__global__ void __launch_bounds__(256) glu_clamped_kernel(const float* __restrict__ a, const float* __restrict__ b,
                                                          long ld, float* __restrict__ out, uint16_t* __restrict__ out16,
                                                          int n, float alpha, float limit, float shift) {
  const size_t t = blockIdx.x;
  const int i = blockIdx.y * 256 + threadIdx.x;
  if (i >= n) return;
  float g = a[t * ld + i], u = b[t * ld + i];
  if (limit > 0.0f) {
    g = fminf(g, limit);
    u = fminf(fmaxf(u, -limit), limit);
  }
  const float v = g * sigmoid_f(alpha * g) * (u + shift);
  if (out16) out16[t * n + i] = f2bf(v);
  else out[t * n + i] = v;
}

// one wave per token; lane holds logits lane + 64 e (E <= 256)
__global__ void __launch_bounds__(64) moe_route_kernel(const float* __restrict__ z, long ld, int E, int top,
                                                       int* __restrict__ ids, float* __restrict__ wts) {
  const int t = blockIdx.x, lane = threadIdx.x;
  float v[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) v[e] = lane + 64 * e < E ? z[(size_t)t * ld + lane + 64 * e] : -INFINITY;
  float first = 0.0f, den = 0.0f;
  for (int k = 0; k < top; ++k) {
    float best = -INFINITY;
    int bi = 0x7fffffff;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int i = lane + 64 * e;
      if (i < E && (v[e] > best || (v[e] == best && i < bi))) {
        best = v[e];
        bi = i;
      }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ob = __shfl_xor(best, o);
      const int oi = __shfl_xor(bi, o);
      if (ob > best || (ob == best && oi < bi)) {
        best = ob;
        bi = oi;
      }
    }
    if (k == 0) first = best;
    const float w = expf(best - first);  // the first pick is the maximum
    den += w;
    if (lane == 0) {
      ids[(size_t)t * top + k] = bi;
      wts[(size_t)t * top + k] = w;
    }
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (lane + 64 * e == bi) v[e] = -INFINITY;
  }
  __syncthreads();
  if (lane == 0)
    for (int k = 0; k < top; ++k) wts[(size_t)t * top + k] /= den;
}

// one wave: s = softmax(z) over all E outputs (z: the token's router logits, global or LDS), or with `sigmoid`
// s = sigmoid(z) of every output on its own; the `top` largest of s + bias (lowest index first among equals) are
// chosen, and their weights are s itself: not renormalised, without the bias; `square`: s^2 (the weight of an expert
// whose INPUT is scaled by s when its activation is the square of relu: relu(s a)^2 = s^2 relu(a)^2 for s > 0)
__device__ __forceinline__ void route_scores_wave(const float* z, int E, int top, const float* __restrict__ bias,
                                                  int* __restrict__ ids, float* __restrict__ wts, int lane,
                                                  bool sigmoid = false, bool square = false) {
  float s[4], c[4], mx = -INFINITY;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    s[e] = lane + 64 * e < E ? z[lane + 64 * e] : -INFINITY;
    mx = fmaxf(mx, s[e]);
  }
  mx = wave_max(mx);
  float den = 0.0f;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    if (sigmoid) s[e] = lane + 64 * e < E ? sigmoid_f(s[e]) : 0.0f;
    else s[e] = lane + 64 * e < E ? expf(s[e] - mx) : 0.0f;
    den += s[e];
  }
  den = sigmoid ? 1.0f : wave_sum(den);
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int i = lane + 64 * e;
    s[e] /= den;
    c[e] = i < E ? s[e] + (bias ? bias[i] : 0.0f) : -INFINITY;
  }
  for (int k = 0; k < top; ++k) {
    float best = -INFINITY, bs = 0.0f;
    int bi = 0x7fffffff;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int i = lane + 64 * e;
      if (i < E && (c[e] > best || (c[e] == best && i < bi))) {
        best = c[e];
        bs = s[e];
        bi = i;
      }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ob = __shfl_xor(best, o), os = __shfl_xor(bs, o);
      const int oi = __shfl_xor(bi, o);
      if (ob > best || (ob == best && oi < bi)) {
        best = ob;
        bs = os;
        bi = oi;
      }
    }
    if (lane == 0) {
      ids[k] = bi;
      wts[k] = square ? bs * bs : bs;
    }
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if (lane + 64 * e == bi) c[e] = -INFINITY;
  }
}

__global__ void __launch_bounds__(64) moe_route_scores_kernel(const float* __restrict__ z, long ld, int E, int top,
                                                              const float* __restrict__ bias, int* __restrict__ ids,
                                                              float* __restrict__ wts, int sigmoid, int square) {
  const size_t t = blockIdx.x;
  route_scores_wave(z + t * ld, E, top, bias, ids + t * top, wts + t * top, threadIdx.x, sigmoid != 0, square != 0);
}

// grid (T, ceil(n / 256)): out[t][i] = act(a[t * ld + i]) * (gate ? sigmoid(gate[t * ldg]) : 1): the activation of an
// ungated unit whose up-projection is part of a fused product, with an optional gate of one number per row
__global__ void __launch_bounds__(256) act_rows_kernel(const float* __restrict__ a, long ld,
                                                       const float* __restrict__ gate, long ldg,
                                                       float* __restrict__ out, uint16_t* __restrict__ out16, int n,
                                                       int act) {
  const size_t t = blockIdx.x;
  const int i = blockIdx.y * 256 + threadIdx.x;
  if (i >= n) return;
  float v = act_f(act, a[t * ld + i]);
  if (gate) v *= sigmoid_f(gate[t * ldg]);
  if (out16) out16[t * n + i] = f2bf(v);
  else out[t * n + i] = v;
}

// grid (T), 1024 threads: the router's logits of one token (wave w takes outputs w, w + 16, ...; fp32 sums, the
// operand rounded as the weights' precision asks, 16-byte weight loads where the rows allow) and the routing above,
// in one launch: the form of steps with few tokens
template <bool WF32>
__global__ void __launch_bounds__(1024) moe_router_kernel(const float* __restrict__ h, long ldh, const void* __restrict__ w,
                                                          int K, int E, int top, const float* __restrict__ bias,
                                                          int* __restrict__ ids, float* __restrict__ wts, int sigmoid,
                                                          int square) {
  __shared__ float z[256];
  const size_t t = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const float* x = h + t * ldh;
  const bool vec = (K & 7) == 0 && (ldh & 3) == 0 && ((uintptr_t)h & 15) == 0;
  for (int e = wave; e < E; e += 16) {
    float a0, a1;
    dot2<WF32>(x, w, (size_t)e * K, (size_t)e * K, K, vec, lane, a0, a1);
    if (lane == 0) z[e] = a0;
  }
  __syncthreads();
  if (wave == 0) route_scores_wave(z, E, top, bias, ids + t * top, wts + t * top, lane, sigmoid != 0, square != 0);
}

// grid (ceil(F / 8), pairs): pair = token * top + choice; act[pair][f] = act(up_e[f] . h_token); GATED: an expert's
// matrix holds F gate rows, then F up rows, and act[pair][f] = act(gate_e[f] . h) * (up_e[f] . h), 4 per workgroup.
// Pairs whose expert id is >= n_real (experts without matrices) are skipped.
template <bool WF32, bool GATED>
__global__ void __launch_bounds__(256) moe_up_kernel(const float* __restrict__ h, long ldh, const void* __restrict__ up,
                                                     const int* __restrict__ ids, float* __restrict__ actbuf, int top,
                                                     int F, int K, int act, int n_real) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int pair = blockIdx.y, f0 = (blockIdx.x * 4 + wave) * (GATED ? 1 : 2);
  if (f0 >= F) return;
  const int e = ids[pair];
  if (e >= n_real) return;
  const float* hr = h + (size_t)(pair / top) * ldh;
  const size_t rows = GATED ? 2 * (size_t)F : (size_t)F;
  const size_t w0 = ((size_t)e * rows + f0) * K, w1 = ((size_t)e * rows + (GATED ? F + f0 : min(f0 + 1, F - 1))) * K;
  float a0, a1;
  dot2<WF32>(hr, up, w0, w1, K, (K & 7) == 0 && (ldh & 3) == 0 && ((uintptr_t)h & 15) == 0, lane, a0, a1);
  if (lane == 0) {
    if (GATED) {
      actbuf[(size_t)pair * F + f0] = act_f(act, a0) * a1;
    } else {
      actbuf[(size_t)pair * F + f0] = act_f(act, a0);
      if (f0 + 1 < F) actbuf[(size_t)pair * F + f0 + 1] = act_f(act, a1);
    }
  }
}

// grid (ceil(N / 8), T): x[t][n] (+)= sum_k wts[t][k] * (down_e(t,k)[n] . act[t * top + k]), k ascending; an expert
// id >= n_real is an identity expert: its output is the token's input hin[t][n] itself
template <bool WF32>
__global__ void __launch_bounds__(256) moe_down_kernel(const float* __restrict__ actbuf, const void* __restrict__ down,
                                                       const int* __restrict__ ids, const float* __restrict__ wts,
                                                       float* __restrict__ x, long ldx, int top, int N, int F,
                                                       int n_real, const float* __restrict__ hin, long ldh,
                                                       int accumulate) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int t = blockIdx.y, n0 = (blockIdx.x * 4 + wave) * 2;
  if (n0 >= N) return;
  float y0 = 0.0f, y1 = 0.0f;
  for (int k = 0; k < top; ++k) {
    const int e = ids[(size_t)t * top + k];
    if (e >= n_real) {  // (the whole wave takes this branch)
      const float w = wts[(size_t)t * top + k];
      y0 = fmaf(w, hin[(size_t)t * ldh + n0], y0);
      y1 = fmaf(w, hin[(size_t)t * ldh + min(n0 + 1, N - 1)], y1);
      continue;
    }
    const float* ar = actbuf + ((size_t)t * top + k) * F;
    const size_t w0 = ((size_t)e * N + n0) * F, w1 = ((size_t)e * N + min(n0 + 1, N - 1)) * F;
    float a0, a1;
    dot2<WF32>(ar, down, w0, w1, F, (F & 7) == 0, lane, a0, a1);
    const float w = wts[(size_t)t * top + k];
    y0 = fmaf(w, a0, y0);
    y1 = fmaf(w, a1, y1);
  }
  if (lane == 0) {
    x[(size_t)t * ldx + n0] = accumulate ? x[(size_t)t * ldx + n0] + y0 : y0;
    if (n0 + 1 < N) x[(size_t)t * ldx + n0 + 1] = accumulate ? x[(size_t)t * ldx + n0 + 1] + y1 : y1;
  }
}

// Counting sort of the pairs by expert in three launches. ws: 2 E ints (counts, cursors), zero on entry.
// z_start[E + 1] expert ranges in the sorted list, tok_of[i] the token (row of h) of sorted entry i, where[pair] the
// sorted place of a pair. The order inside an expert's range is whatever the atomics give: every row of the grouped
// products is computed on its own, so the sums do not depend on it.
__global__ void __launch_bounds__(256) moe_count_kernel(const int* __restrict__ ids, int pairs, int E, int* __restrict__ ws) {
  __shared__ int lh[256];
  lh[threadIdx.x] = 0;
  __syncthreads();
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < pairs) atomicAdd(&lh[ids[i]], 1);
  __syncthreads();
  if (threadIdx.x < E && lh[threadIdx.x]) atomicAdd(&ws[threadIdx.x], lh[threadIdx.x]);
}

__global__ void __launch_bounds__(256) moe_scan_kernel(int E, int* __restrict__ ws, int* __restrict__ z_start) {
  __shared__ int cnt[256];
  const int tid = threadIdx.x;
  cnt[tid] = tid < E ? ws[tid] : 0;
  __syncthreads();
  if (tid == 0) {
    int at = 0;
    for (int e = 0; e < E; ++e) {
      z_start[e] = at;
      at += cnt[e];
    }
    z_start[E] = at;
  }
  if (tid < E) {
    ws[tid] = 0;      // counts: zero again for the next call
    ws[E + tid] = 0;  // cursors
  }
}

__global__ void __launch_bounds__(256) moe_place_kernel(const int* __restrict__ ids, int pairs, int top, int E,
                                                        const int* __restrict__ z_start, int* __restrict__ ws,
                                                        int* __restrict__ tok_of, int* __restrict__ where) {
  __shared__ int lh[256], base[256];
  lh[threadIdx.x] = 0;
  __syncthreads();
  const int i = blockIdx.x * 256 + threadIdx.x;
  int e = 0, rank = 0;
  if (i < pairs) {
    e = ids[i];
    rank = atomicAdd(&lh[e], 1);
  }
  __syncthreads();
  if (threadIdx.x < E && lh[threadIdx.x]) base[threadIdx.x] = atomicAdd(&ws[E + threadIdx.x], lh[threadIdx.x]);
  __syncthreads();
  if (i < pairs) {
    const int at = z_start[e] + base[e] + rank;
    tok_of[at] = i / top;
    where[i] = at;
  }
}

// grid (ceil(N / 256), T): x[t] (+)= sum_k wts[t][k] * y[where[t * top + k]], k ascending; with ids, a choice whose
// expert id is >= n_real (an identity expert) contributes the token's input hin[t] instead of a row of y
__global__ void __launch_bounds__(256) moe_combine_kernel(const float* __restrict__ y, const int* __restrict__ where,
                                                          const float* __restrict__ wts, float* __restrict__ x, long ldx,
                                                          int top, int N, const int* __restrict__ ids, int n_real,
                                                          const float* __restrict__ hin, long ldh, int accumulate) {
  const int t = blockIdx.y, n = blockIdx.x * 256 + threadIdx.x;
  if (n >= N) return;
  float s = 0.0f;
  for (int k = 0; k < top; ++k) {
    const size_t pair = (size_t)t * top + k;
    const float v = ids && ids[pair] >= n_real ? hin[(size_t)t * ldh + n] : y[(size_t)where[pair] * N + n];
    s = fmaf(wts[pair], v, s);
  }
  x[(size_t)t * ldx + n] = accumulate ? x[(size_t)t * ldx + n] + s : s;
}

// grid (T): LDS holds the row x (W floats), the gated slice (dim floats) and the projection y (W floats)
template <bool WF32>
__global__ void __launch_bounds__(256) token_side_kernel(float* __restrict__ x, const int* __restrict__ tok,
                                                         const void* __restrict__ table, long ld_table, int col0,
                                                         const void* __restrict__ gate_w, const void* __restrict__ proj_w,
                                                         const float* __restrict__ norm_w, int W, int dim, int vocab,
                                                         float eps) {
  extern __shared__ float sh[];
  __shared__ float red[4];
  float* xs = sh;
  float* ys = sh + W;
  float* gs = sh + 2 * W;
  const int t = blockIdx.x, tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  float* xr = x + (size_t)t * W;
  int id = tok[t];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
  for (int i = tid; i < W; i += 256) xs[i] = aop<WF32>(xr[i]);
  __syncthreads();
  for (int j = wave; j < dim; j += 4) {
    float a = 0.0f;
    for (int k = lane; k < W; k += 64) a = fmaf(xs[k], wload<WF32>(gate_w, (size_t)j * W + k), a);
    a = wave_sum(a);
    if (lane == 0) gs[j] = aop<WF32>(gelu_tanh_f(a) * wload<WF32>(table, (size_t)id * ld_table + col0 + j));
  }
  __syncthreads();
  float ss = 0.0f;
  for (int n = tid; n < W; n += 256) {
    float a = 0.0f;
    for (int j = 0; j < dim; ++j) a = fmaf(gs[j], wload<WF32>(proj_w, (size_t)n * dim + j), a);
    ys[n] = a;
    ss = fmaf(a, a, ss);
  }
  ss = block_sum_256(ss, red);
  const float rstd = 1.0f / sqrtf(ss / (float)W + eps);
  for (int n = tid; n < W; n += 256) xr[n] += ys[n] * rstd * norm_w[n];
}

}  // namespace lgs

extern "C" int lgs_glu(const float* a, const float* b, long ld, void* out, int out_bf16, int T, int n, int act,
                       hipStream_t stream) {
  LGA_CHECK_ARG(a && b && out && T > 0 && n > 0 && (n + 255) / 256 <= 65535, "lgs_glu: bad arguments");
  lgs::glu_kernel<<<dim3(T, (n + 255) / 256), 256, 0, stream>>>(a, b, ld, out_bf16 ? nullptr : (float*)out,
                                                                 out_bf16 ? (uint16_t*)out : nullptr, n, act);
  LGA_LAUNCH_RETURN();
}

extern "C" int lgs_glu_clamped(const float* a, const float* b, long ld, void* out, int out_bf16, int T, int n,
                               float alpha, float limit, float shift, hipStream_t stream) {
  LGA_CHECK_ARG(a && b && out && T > 0 && n > 0 && (n + 255) / 256 <= 65535, "lgs_glu_clamped: bad arguments");
  lgs::glu_clamped_kernel<<<dim3(T, (n + 255) / 256), 256, 0, stream>>>(
      a, b, ld, out_bf16 ? nullptr : (float*)out, out_bf16 ? (uint16_t*)out : nullptr, n, alpha, limit, shift);
  LGA_LAUNCH_RETURN();
}

extern "C" int lgs_moe_route(const float* z, long ld, int T, int E, int top, int* ids, float* wts,
                             hipStream_t stream) {
  LGA_CHECK_ARG(z && ids && wts && T > 0, "lgs_moe_route: bad arguments");
  LGA_CHECK_ARG(E > 0 && E <= 256 && top > 0 && top <= E, "lgs_moe_route: experts must be <= 256 and top <= experts");
  lgs::moe_route_kernel<<<T, 64, 0, stream>>>(z, ld, E, top, ids, wts);
  LGA_LAUNCH_RETURN();
}

extern "C" int lgs_moe_route_scores(const float* z, long ld, int T, int E, int top, const float* bias, int* ids,
                                    float* wts, int sigmoid, int square, hipStream_t stream) {
  LGA_CHECK_ARG(z && ids && wts && T > 0, "lgs_moe_route_scores: bad arguments");
  LGA_CHECK_ARG(E > 0 && E <= 256 && top > 0 && top <= E,
                "lgs_moe_route_scores: experts must be <= 256 and top <= experts");
  lgs::moe_route_scores_kernel<<<T, 64, 0, stream>>>(z, ld, E, top, bias, ids, wts, sigmoid, square);
  LGA_LAUNCH_RETURN();
}

extern "C" int lgs_act_rows(const float* a, long ld, const float* gate, long ldg, void* out, int out_bf16, int T, int n,
                            int act, hipStream_t stream) {
  LGA_CHECK_ARG(a && out && T > 0 && n > 0 && ld >= n && act >= 0 && act <= lgs::kActSigmoid, "lgs_act_rows: bad arguments");
  const dim3 grid(T, (n + 255) / 256);
  lgs::act_rows_kernel<<<grid, 256, 0, stream>>>(a, ld, gate, ldg, out_bf16 ? nullptr : (float*)out,
                                                 out_bf16 ? (uint16_t*)out : nullptr, n, act);
  LGA_LAUNCH_RETURN();
}

extern "C" int lgs_moe_router(const float* h, long ldh, const void* w, int w_f32, int T, int K, int E, int top,
                              const float* bias, int* ids, float* wts, int sigmoid, int square, hipStream_t stream) {
  LGA_CHECK_ARG(h && w && ids && wts && T > 0 && K > 0 && ldh >= K, "lgs_moe_router: bad arguments");
  LGA_CHECK_ARG(E > 0 && E <= 256 && top > 0 && top <= E, "lgs_moe_router: experts must be <= 256 and top <= experts");
  if (w_f32) lgs::moe_router_kernel<true><<<T, 1024, 0, stream>>>(h, ldh, w, K, E, top, bias, ids, wts, sigmoid, square);
  else lgs::moe_router_kernel<false><<<T, 1024, 0, stream>>>(h, ldh, w, K, E, top, bias, ids, wts, sigmoid, square);
  LGA_LAUNCH_RETURN();
}

extern "C" int lgs_moe_up(const float* h, long ldh, const void* up, int w_f32, const int* ids, float* actbuf, int T,
                          int top, int F, int K, int act, int gated, int n_real, hipStream_t stream) {
  LGA_CHECK_ARG(h && up && ids && actbuf && T > 0 && top > 0 && F > 0 && K > 0 && (long)T * top <= 65535 && n_real > 0,
                "lgs_moe_up: bad arguments");
  if (gated) {
    const dim3 grid((F + 3) / 4, T * top);
    if (w_f32) lgs::moe_up_kernel<true, true><<<grid, 256, 0, stream>>>(h, ldh, up, ids, actbuf, top, F, K, act, n_real);
    else lgs::moe_up_kernel<false, true><<<grid, 256, 0, stream>>>(h, ldh, up, ids, actbuf, top, F, K, act, n_real);
  } else {
    const dim3 grid((F + 7) / 8, T * top);
    if (w_f32) lgs::moe_up_kernel<true, false><<<grid, 256, 0, stream>>>(h, ldh, up, ids, actbuf, top, F, K, act, n_real);
    else lgs::moe_up_kernel<false, false><<<grid, 256, 0, stream>>>(h, ldh, up, ids, actbuf, top, F, K, act, n_real);
  }
  LGA_LAUNCH_RETURN();
}

extern "C" int lgs_moe_down(const float* actbuf, const void* down, int w_f32, const int* ids, const float* wts,
                            float* x, long ldx, int T, int top, int N, int F, int n_real, const float* hin, long ldh,
                            int accumulate, hipStream_t stream) {
  LGA_CHECK_ARG(actbuf && down && ids && wts && x && T > 0 && T <= 65535 && top > 0 && N > 0 && F > 0 && n_real > 0 && hin,
                "lgs_moe_down: bad arguments");
  const dim3 grid((N + 7) / 8, T);
  if (w_f32)
    lgs::moe_down_kernel<true><<<grid, 256, 0, stream>>>(actbuf, down, ids, wts, x, ldx, top, N, F, n_real, hin, ldh,
                                                         accumulate);
  else
    lgs::moe_down_kernel<false><<<grid, 256, 0, stream>>>(actbuf, down, ids, wts, x, ldx, top, N, F, n_real, hin, ldh,
                                                          accumulate);
  LGA_LAUNCH_RETURN();
}

extern "C" int lgs_moe_sort(const int* ids, int pairs, int top, int E, int* z_start, int* tok_of, int* where, int* ws,
                            hipStream_t stream) {
  LGA_CHECK_ARG(ids && z_start && tok_of && where && ws && pairs > 0 && top > 0 && E > 0 && E <= 256,
                "lgs_moe_sort: experts must be <= 256");
  const int blocks = (pairs + 255) / 256;
  lgs::moe_count_kernel<<<blocks, 256, 0, stream>>>(ids, pairs, E, ws);
  lgs::moe_scan_kernel<<<1, 256, 0, stream>>>(E, ws, z_start);
  lgs::moe_place_kernel<<<blocks, 256, 0, stream>>>(ids, pairs, top, E, z_start, ws, tok_of, where);
  LGA_LAUNCH_RETURN();
}

extern "C" int lgs_moe_combine(const float* y, const int* where, const float* wts, float* x, long ldx, int T, int top,
                               int N, const int* ids, int n_real, const float* hin, long ldh, int accumulate,
                               hipStream_t stream) {
  LGA_CHECK_ARG(y && where && wts && x && T > 0 && T <= 65535 && top > 0 && N > 0, "lgs_moe_combine: bad arguments");
  LGA_CHECK_ARG(!ids || hin, "lgs_moe_combine: identity experts need the tokens' inputs");
  lgs::moe_combine_kernel<<<dim3((N + 255) / 256, T), 256, 0, stream>>>(y, where, wts, x, ldx, top, N, ids, n_real, hin,
                                                                          ldh, accumulate);
  LGA_LAUNCH_RETURN();
}

extern "C" int lgs_token_side(float* x, const int* tokens, const void* table, int w_f32, long ld_table, int col0,
                              const void* gate_w, const void* proj_w, const float* norm_w, int T, int W, int dim,
                              int vocab, float eps, hipStream_t stream) {
  LGA_CHECK_ARG(x && tokens && table && gate_w && proj_w && norm_w && T > 0 && W > 0 && dim > 0 && vocab > 0,
                "lgs_token_side: bad arguments");
  const size_t lds = (size_t)(2 * W + dim) * sizeof(float);
  LGA_CHECK_ARG(lds <= 64 * 1024, "lgs_token_side: width too large for one workgroup's LDS");
  if (w_f32)
    lgs::token_side_kernel<true><<<T, 256, lds, stream>>>(x, tokens, table, ld_table, col0, gate_w, proj_w, norm_w, W,
                                                          dim, vocab, eps);
  else
    lgs::token_side_kernel<false><<<T, 256, lds, stream>>>(x, tokens, table, ld_table, col0, gate_w, proj_w, norm_w, W,
                                                           dim, vocab, eps);
  LGA_LAUNCH_RETURN();
}
