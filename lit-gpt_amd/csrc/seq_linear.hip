// Linear layers, embedding and RMS norms of the layered models: fp32 activations, bf16 or fp32 weights.
//
//   lgs_linear     Y[z] (+)= act(A[z] W[z]^T): one entry point for every projection. Up to 8 rows run a streaming
//                  GEMV (a wave per pair of output columns, 16-B weight loads, fp32 sums); more rows run 128x128
//                  tiles of v_mfma_f32_16x16x32_bf16 (bf16 weights; A is rounded to bf16 while it is staged into
//                  LDS) or 64x64 fp32 FMA tiles (fp32 weights). `batch` with strides runs per-head products (the
//                  latent attention's absorbed key and value maps); `z_start` / `a_rows` make it a grouped product
//                  over row ranges of a sorted list (sparse experts during a prompt).
//   lgs_embed      x[t] = table[token[t]] * scale
//   lgs_rmsnorm    y = x / sqrt(mean(x^2) + eps) * (offset + w), rows with strides (whole rows, or heads)
#include "seq_common.h"

namespace lgs {

typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef float f32x4_t __attribute__((ext_vector_type(4)));

struct LinArgs {
  const float* a;
  long lda, sa;
  const void* w;
  long sw;
  float* y;
  long ldy, sy;
  int M, N, K;
  int accumulate, act;
  const int* a_rows;   // row r of the list reads A row a_rows[r] (null: r)
  const int* z_start;  // batch z owns list rows [z_start[z], z_start[z + 1]) (null: rows [0, M) in every batch)
  const uint16_t* a16;  // MFMA tiles only: A as bf16 (a producer's rounded copy) instead of fp32 `a`
  uint16_t* y16;        // MFMA tiles only: Y written as bf16 (the operand of a following bf16 product), no accumulate
};

// ------------------------------------------------------------------------------------------------ GEMV, M <= 8
// R output columns per wave: 4 for tall matrices (more loads in flight per lane), fewer for short ones (more waves)
template <bool WF32, int MT, int R>
__global__ void __launch_bounds__(256) lin_gemv_kernel(LinArgs p) {
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int z = blockIdx.y;
  const int n0 = (blockIdx.x * 4 + wave) * R;
  if (n0 >= p.N) return;
  const float* a = p.a + (size_t)z * p.sa;
  const size_t wbase = (size_t)z * p.sw;
  float acc[MT][R];
#pragma unroll
  for (int m = 0; m < MT; ++m)
#pragma unroll
    for (int r = 0; r < R; ++r) acc[m][r] = 0.0f;
  const int K = p.K;
  const bool vec = (K % 8 == 0) && (p.lda % 4 == 0) && (((uintptr_t)a) % 16 == 0) && (p.sw % 8 == 0) &&
                   (((uintptr_t)p.w) % 16 == 0);
  int rows[R];
#pragma unroll
  for (int r = 0; r < R; ++r) rows[r] = min(n0 + r, p.N - 1);
  if (vec) {
#pragma unroll 2
    for (int k = lane * 8; k < K; k += 512) {
      float wv[R][8];
#pragma unroll
      for (int r = 0; r < R; ++r) {
        const size_t off = wbase + (size_t)rows[r] * K + k;
        if (WF32) {
          const float4 lo = *(const float4*)((const float*)p.w + off), hi = *(const float4*)((const float*)p.w + off + 4);
          wv[r][0] = lo.x; wv[r][1] = lo.y; wv[r][2] = lo.z; wv[r][3] = lo.w;
          wv[r][4] = hi.x; wv[r][5] = hi.y; wv[r][6] = hi.z; wv[r][7] = hi.w;
        } else {
          const uint4 q = *(const uint4*)((const uint16_t*)p.w + off);
          wv[r][0] = bflo(q.x); wv[r][1] = bfhi(q.x); wv[r][2] = bflo(q.y); wv[r][3] = bfhi(q.y);
          wv[r][4] = bflo(q.z); wv[r][5] = bfhi(q.z); wv[r][6] = bflo(q.w); wv[r][7] = bfhi(q.w);
        }
      }
#pragma unroll
      for (int m = 0; m < MT; ++m) {
        if (m < p.M) {
          const float* ar = a + (size_t)m * p.lda + k;
          const float4 lo = *(const float4*)ar, hi = *(const float4*)(ar + 4);
          const float av[8] = {lo.x, lo.y, lo.z, lo.w, hi.x, hi.y, hi.z, hi.w};
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const float x = aop<WF32>(av[e]);
#pragma unroll
            for (int r = 0; r < R; ++r) acc[m][r] = fmaf(x, wv[r][e], acc[m][r]);
          }
        }
      }
    }
  } else {
    for (int k = lane; k < K; k += 64) {
      float wv[R];
#pragma unroll
      for (int r = 0; r < R; ++r) wv[r] = wload<WF32>(p.w, wbase + (size_t)rows[r] * K + k);
#pragma unroll
      for (int m = 0; m < MT; ++m)
        if (m < p.M) {
          const float x = aop<WF32>(a[(size_t)m * p.lda + k]);
#pragma unroll
          for (int r = 0; r < R; ++r) acc[m][r] = fmaf(x, wv[r], acc[m][r]);
        }
    }
  }
#pragma unroll
  for (int m = 0; m < MT; ++m)
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const float s = wave_sum(acc[m][r]);
      if (lane == 0 && m < p.M && n0 + r < p.N) {
        float* yp = p.y + (size_t)z * p.sy + (size_t)m * p.ldy + n0 + r;
        const float v = act_f(p.act, s);
        *yp = p.accumulate ? *yp + v : v;
      }
    }
}

// ------------------------------------------------------------------------------------------------ MFMA tiles
constexpr int BM = 128, BN = 128, BK = 64;
constexpr int TILE_BYTES = BM * BK * 2;
__device__ __forceinline__ int swz(int row, int chunk) { return row * 128 + 16 * (chunk ^ (row & 7)); }

// VEC: K % 8 == 0 and 16-B aligned rows of A and W (vector loads); otherwise element loads with k guards.
// A16: A arrives as bf16 (half the operand traffic of the fp32 stream; the same values the fp32 path would round to)
template <bool VEC, bool A16>
__global__ void __launch_bounds__(256) lin_mfma_kernel(LinArgs p) {
  __shared__ __attribute__((aligned(16))) unsigned char lds[2 * 2 * TILE_BYTES];  // [buf][A|W]
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int wm = wave >> 1, wn = wave & 1;
  const int z = blockIdx.z;
  const int r_lo = p.z_start ? p.z_start[z] : 0;
  const int Mz = p.z_start ? p.z_start[z + 1] - r_lo : p.M;
  const int m0 = blockIdx.y * BM, n0 = blockIdx.x * BN;
  if (m0 >= Mz) return;
  const float* abase = A16 ? nullptr : p.a + (size_t)z * p.sa;
  const uint16_t* abase16 = A16 ? p.a16 + (size_t)z * p.sa : nullptr;
  const uint16_t* wbase = (const uint16_t*)p.w + (size_t)z * p.sw;
  const int K = p.K, nk = (K + BK - 1) / BK;
  const int t_row = tid >> 1, t_half = tid & 1;
  const int lr = r_lo + min(m0 + t_row, Mz - 1);  // rows past the end repeat the last one (never stored)
  const size_t arow_off = (size_t)(p.a_rows ? p.a_rows[lr] : lr) * p.lda;
  const float* arow = abase + arow_off;
  const uint16_t* arow16 = abase16 + arow_off;
  const uint16_t* wrow = wbase + (size_t)min(n0 + t_row, p.N - 1) * K;

  uint4 areg[4], wreg[4];
  auto gload = [&](int kt) {
    const int k0 = kt * BK + t_half * 32;
    if (VEC) {
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        const int k = k0 + c * 8;
        if (k < K) {
          if (A16) {
            areg[c] = *(const uint4*)(arow16 + k);
          } else {
            const float4 lo = *(const float4*)(arow + k), hi = *(const float4*)(arow + k + 4);
            areg[c] = make_uint4(pack2(lo.x, lo.y), pack2(lo.z, lo.w), pack2(hi.x, hi.y), pack2(hi.z, hi.w));
          }
          wreg[c] = *(const uint4*)(wrow + k);
        } else {
          areg[c] = make_uint4(0, 0, 0, 0);
          wreg[c] = make_uint4(0, 0, 0, 0);
        }
      }
    } else {
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        uint32_t av[4], wv[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int k = k0 + c * 8 + 2 * e;
          const uint32_t w0 = k < K ? wrow[k] : 0, w1 = k + 1 < K ? wrow[k + 1] : 0;
          if (A16) {
            const uint32_t b0 = k < K ? arow16[k] : 0, b1 = k + 1 < K ? arow16[k + 1] : 0;
            av[e] = b0 | (b1 << 16);
          } else {
            const float a0 = k < K ? arow[k] : 0.0f, a1 = k + 1 < K ? arow[k + 1] : 0.0f;
            av[e] = pack2(a0, a1);
          }
          wv[e] = w0 | (w1 << 16);
        }
        areg[c] = make_uint4(av[0], av[1], av[2], av[3]);
        wreg[c] = make_uint4(wv[0], wv[1], wv[2], wv[3]);
      }
    }
  };
  auto lstore = [&](int buf) {
    unsigned char* A = lds + buf * (2 * TILE_BYTES);
    unsigned char* B = A + TILE_BYTES;
#pragma unroll
    for (int c = 0; c < 4; ++c) {
      *(uint4*)(A + swz(t_row, t_half * 4 + c)) = areg[c];
      *(uint4*)(B + swz(t_row, t_half * 4 + c)) = wreg[c];
    }
  };

  f32x4_t acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  gload(0);
  lstore(0);
  __syncthreads();
  const int fr = lane & 15, fk = lane >> 4;
  for (int kt = 0; kt < nk; ++kt) {
    const int cur = kt & 1;
    if (kt + 1 < nk) gload(kt + 1);
    const unsigned char* A = lds + cur * (2 * TILE_BYTES);
    const unsigned char* B = A + TILE_BYTES;
#pragma unroll
    for (int sub = 0; sub < 2; ++sub) {
      bf16x8_t af[4], bfr[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        af[i] = *(const bf16x8_t*)(A + swz(wm * 64 + i * 16 + fr, sub * 4 + fk));
        bfr[i] = *(const bf16x8_t*)(B + swz(wn * 64 + i * 16 + fr, sub * 4 + fk));
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(af[i], bfr[j], acc[i][j], 0, 0, 0);
    }
    if (kt + 1 < nk) lstore(cur ^ 1);
    __syncthreads();
  }

#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int n = n0 + wn * 64 + j * 16 + fr;
    if (n >= p.N) continue;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int m = m0 + wm * 64 + i * 16 + fk * 4 + r;
        if (m >= Mz) continue;
        const size_t at = (size_t)z * p.sy + (size_t)(r_lo + m) * p.ldy + n;
        const float v = act_f(p.act, acc[i][j][r]);
        if (p.y16) p.y16[at] = f2bf(v);
        else p.y[at] = p.accumulate ? p.y[at] + v : v;
      }
  }
}

// ------------------------------------------------------------------------------------------------ fp32 tiles
// 64x64 outputs per workgroup, 16 deep; thread (ty, tx) owns rows ty + 16 i and columns tx + 16 j; k ascending
template <bool WF32>
__global__ void __launch_bounds__(256) lin_fma_kernel(LinArgs p) {
  __shared__ float As[16][65];
  __shared__ float Ws[16][65];
  const int tid = threadIdx.x, tx = tid & 15, ty = tid >> 4;
  const int z = blockIdx.z;
  const int r_lo = p.z_start ? p.z_start[z] : 0;
  const int Mz = p.z_start ? p.z_start[z + 1] - r_lo : p.M;
  const int m0 = blockIdx.y * 64, n0 = blockIdx.x * 64;
  if (m0 >= Mz) return;
  const float* abase = p.a + (size_t)z * p.sa;
  const size_t wz = (size_t)z * p.sw;
  const int K = p.K;
  // staging: thread loads column k = tid & 15 of rows (tid >> 4) + 16 i
  const int sk = tid & 15, sr = tid >> 4;
  const float* arows[4];
  size_t wrows[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int lr = r_lo + min(m0 + sr + 16 * i, Mz - 1);
    arows[i] = abase + (size_t)(p.a_rows ? p.a_rows[lr] : lr) * p.lda;
    wrows[i] = wz + (size_t)min(n0 + sr + 16 * i, p.N - 1) * K;
  }
  float acc[4][4];
#pragma unroll
  for (int i = 0; i < 4; ++i)
#pragma unroll
    for (int j = 0; j < 4; ++j) acc[i][j] = 0.0f;
  for (int k0 = 0; k0 < K; k0 += 16) {
    const int k = k0 + sk;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      As[sk][sr + 16 * i] = k < K ? aop<WF32>(arows[i][k]) : 0.0f;
      Ws[sk][sr + 16 * i] = k < K ? wload<WF32>(p.w, wrows[i] + k) : 0.0f;
    }
    __syncthreads();
#pragma unroll
    for (int kk = 0; kk < 16; ++kk) {
      float av[4], wv[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        av[i] = As[kk][ty + 16 * i];
        wv[i] = Ws[kk][tx + 16 * i];
      }
#pragma unroll
      for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = fmaf(av[i], wv[j], acc[i][j]);
    }
    __syncthreads();
  }
  float* ybase = p.y + (size_t)z * p.sy;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int m = m0 + ty + 16 * i;
    if (m >= Mz) continue;
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int n = n0 + tx + 16 * j;
      if (n >= p.N) continue;
      float* yp = ybase + (size_t)(r_lo + m) * p.ldy + n;
      const float v = act_f(p.act, acc[i][j]);
      *yp = p.accumulate ? *yp + v : v;
    }
  }
}

// ------------------------------------------------------------------------------------------------ row kernels
template <bool WF32>
__global__ void __launch_bounds__(256) embed_kernel(const int* __restrict__ tok, const void* __restrict__ table,
                                                    float* __restrict__ x, int W, int vocab, float scale) {
  const int t = blockIdx.x;
  int id = tok[t];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);  // the host validates ids; never read out of bounds
  for (int i = threadIdx.x; i < W; i += 256) x[(size_t)t * W + i] = wload<WF32>(table, (size_t)id * W + i) * scale;
}

// x[t] = table[tok[t]] * scale + ptable[pos[t]] (a learned position vector, not scaled); x16: optional rounded copy
template <bool WF32>
__global__ void __launch_bounds__(256) embed_pos_kernel(const int* __restrict__ tok, const int* __restrict__ pos,
                                                        const void* __restrict__ table, const void* __restrict__ ptable,
                                                        float* __restrict__ x, uint16_t* __restrict__ x16, int W, int vocab,
                                                        int positions, float scale) {
  const int t = blockIdx.x;
  int id = tok[t], ps = pos[t];
  id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);  // the host validates ids and positions
  ps = ps < 0 ? 0 : (ps >= positions ? positions - 1 : ps);
  for (int i = threadIdx.x; i < W; i += 256) {
    const float v = fmaf(wload<WF32>(table, (size_t)id * W + i), scale, wload<WF32>(ptable, (size_t)ps * W + i));
    x[(size_t)t * W + i] = v;
    if (x16) x16[(size_t)t * W + i] = f2bf(v);
  }
}

// Layer norm of a sublayer's output joining the residual: x[r] (+)= mult * ((y - mean) / sqrt(var + eps) * w + b),
// var = mean of the squared deviations (two passes over the row, which stays in registers up to 256 * CPT columns).
// x16: optional copy of the new x rounded to bf16 (the next product's operand). grid (rows).
template <int CPT>
__global__ void __launch_bounds__(256) layernorm_kernel(const float* __restrict__ y, const float* __restrict__ w,
                                                        const float* __restrict__ b, float eps, float mult, int accumulate,
                                                        float* __restrict__ x, uint16_t* __restrict__ x16, int n) {
  __shared__ float red[4];
  const size_t r = blockIdx.x;
  const float* yr = y + r * n;
  float v[CPT];
  float s = 0.0f;
#pragma unroll
  for (int e = 0; e < CPT; ++e) {
    const int i = threadIdx.x + 256 * e;
    v[e] = i < n ? yr[i] : 0.0f;
    s += v[e];
  }
  for (int i = threadIdx.x + 256 * CPT; i < n; i += 256) s += yr[i];
  const float mean = block_sum_256(s, red) / (float)n;
  float q = 0.0f;
#pragma unroll
  for (int e = 0; e < CPT; ++e) {
    const float dlt = threadIdx.x + 256 * e < n ? v[e] - mean : 0.0f;
    q = fmaf(dlt, dlt, q);
  }
  for (int i = threadIdx.x + 256 * CPT; i < n; i += 256) {
    const float dlt = yr[i] - mean;
    q = fmaf(dlt, dlt, q);
  }
  const float rstd = 1.0f / sqrtf(block_sum_256(q, red) / (float)n + eps);
  auto put = [&](int i, float val) {
    float o = mult * fmaf((val - mean) * rstd, w[i], b ? b[i] : 0.0f);
    if (accumulate) o += x[r * n + i];
    x[r * n + i] = o;
    if (x16) x16[r * n + i] = f2bf(o);
  };
#pragma unroll
  for (int e = 0; e < CPT; ++e)
    if (threadIdx.x + 256 * e < n) put(threadIdx.x + 256 * e, v[e]);
  for (int i = threadIdx.x + 256 * CPT; i < n; i += 256) put(i, yr[i]);
}

// z <- cap * tanh(z / cap)
__global__ void __launch_bounds__(256) softcap_kernel(float* __restrict__ z, size_t n, float cap) {
  const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
  if (i < n) z[i] = cap * tanhf(z[i] / cap);
}

// grid (rows, groups): group g of row r is x[r * ldx + g * n .. + n); weight (may be null) is indexed within a group
__global__ void __launch_bounds__(256) rmsnorm_kernel(const float* __restrict__ x, long ldx, const float* __restrict__ w,
                                                      float offset, float eps, float* __restrict__ y, long ldy, int n,
                                                      uint16_t* __restrict__ y16) {
  __shared__ float red[4];
  const float* xr = x + (size_t)blockIdx.x * ldx + (size_t)blockIdx.y * n;
  float* yr = y + (size_t)blockIdx.x * ldy + (size_t)blockIdx.y * n;
  float ss = 0.0f;
  for (int i = threadIdx.x; i < n; i += 256) ss = fmaf(xr[i], xr[i], ss);
  ss = block_sum_256(ss, red);
  const float rstd = 1.0f / sqrtf(ss / (float)n + eps);
  uint16_t* yb = y16 ? y16 + (size_t)blockIdx.x * ldy + (size_t)blockIdx.y * n : nullptr;
  for (int i = threadIdx.x; i < n; i += 256) {
    const float v = xr[i] * rstd * (w ? offset + w[i] : 1.0f);
    yr[i] = v;
    if (yb) yb[i] = f2bf(v);  // the rounded copy the matrix cores read
  }
}

// y[i] = x[rows[i]] (row gather of the positions whose logits are asked for)
__global__ void __launch_bounds__(256) gather_rows_kernel(const float* __restrict__ x, const int* __restrict__ rows,
                                                          float* __restrict__ y, int W) {
  const size_t src = (size_t)rows[blockIdx.x] * W, dst = (size_t)blockIdx.x * W;
  for (int i = threadIdx.x; i < W; i += 256) y[dst + i] = x[src + i];
}

}  // namespace lgs

extern "C" int lgs_linear(const void* a_any, long lda, long stride_a, const void* w, int w_f32, long stride_w, void* y_any,
                          long ldy, long stride_y, int M, int N, int K, int batch, int accumulate, int act,
                          const int* a_rows, const int* z_start, int a_bf16, int y_bf16, hipStream_t stream) {
  const float* a = (const float*)a_any;  // (bf16 when a_bf16)
  float* y = (float*)y_any;              // (bf16 when y_bf16)
  LGA_CHECK_ARG(a && w && y, "lgs_linear: null pointer");
  LGA_CHECK_ARG(!a_bf16 || (!w_f32 && (M > 8 || z_start || a_rows)),
                "lgs_linear: a bf16 A operand goes with bf16 weights on the MFMA tiles (more than 8 rows)");
  LGA_CHECK_ARG(M > 0 && N > 0 && K > 0 && batch > 0 && batch <= 65535, "lgs_linear: bad sizes");
  LGA_CHECK_ARG(lda >= K && ldy >= N, "lgs_linear: row strides shorter than the rows");
  LGA_CHECK_ARG(act >= 0 && act <= lgs::kActSigmoid, "lgs_linear: unknown activation");
  LGA_CHECK_ARG(!y_bf16 || (!w_f32 && !accumulate && (M > 8 || z_start || a_rows)),
                "lgs_linear: a bf16 result comes from the MFMA tiles (bf16 weights, more than 8 rows, no accumulate)");
  lgs::LinArgs p{a, lda, stride_a, w, stride_w, y, ldy, stride_y, M, N, K, accumulate, act, a_rows, z_start,
                 a_bf16 ? (const uint16_t*)a : nullptr, y_bf16 ? (uint16_t*)y : nullptr};
  if (M <= 8 && !z_start && !a_rows) {
    const int R = N >= 16384 ? 4 : (N >= 4096 ? 2 : 1);
    const dim3 grid((N + 4 * R - 1) / (4 * R), batch);
#define LGS_GEMV_R(MT, RR)                                                              \
  do {                                                                                  \
    if (w_f32) lgs::lin_gemv_kernel<true, MT, RR><<<grid, 256, 0, stream>>>(p);         \
    else lgs::lin_gemv_kernel<false, MT, RR><<<grid, 256, 0, stream>>>(p);              \
  } while (0)
#define LGS_GEMV(MT)                 \
  do {                               \
    if (R == 4) LGS_GEMV_R(MT, 4);   \
    else if (R == 2) LGS_GEMV_R(MT, 2); \
    else LGS_GEMV_R(MT, 1);          \
  } while (0)
    if (M == 1) LGS_GEMV(1);
    else if (M == 2) LGS_GEMV(2);
    else if (M <= 4) LGS_GEMV(4);
    else LGS_GEMV(8);
#undef LGS_GEMV
#undef LGS_GEMV_R
    LGA_LAUNCH_RETURN();
  }
  if (w_f32) {
    const dim3 grid((N + 63) / 64, (M + 63) / 64, batch);
    LGA_CHECK_ARG(grid.y <= 65535, "lgs_linear: too many rows");
    lgs::lin_fma_kernel<true><<<grid, 256, 0, stream>>>(p);
    LGA_LAUNCH_RETURN();
  }
  const dim3 grid((N + lgs::BN - 1) / lgs::BN, (M + lgs::BM - 1) / lgs::BM, batch);
  LGA_CHECK_ARG(grid.y <= 65535, "lgs_linear: too many rows");
  const int am = a_bf16 ? 8 : 4;  // elements per 16 bytes of A
  const bool vec = K % 8 == 0 && lda % am == 0 && stride_a % am == 0 && stride_w % 8 == 0 && (uintptr_t)a % 16 == 0 &&
                   (uintptr_t)w % 16 == 0;
  if (a_bf16) {
    if (vec) lgs::lin_mfma_kernel<true, true><<<grid, 256, 0, stream>>>(p);
    else lgs::lin_mfma_kernel<false, true><<<grid, 256, 0, stream>>>(p);
  } else {
    if (vec) lgs::lin_mfma_kernel<true, false><<<grid, 256, 0, stream>>>(p);
    else lgs::lin_mfma_kernel<false, false><<<grid, 256, 0, stream>>>(p);
  }
  LGA_LAUNCH_RETURN();
}

extern "C" int lgs_embed(const int* tokens, const void* table, int w_f32, float scale, float* x, int T, int W,
                         int vocab, hipStream_t stream) {
  LGA_CHECK_ARG(tokens && table && x && T > 0 && W > 0 && vocab > 0, "lgs_embed: bad arguments");
  if (w_f32) lgs::embed_kernel<true><<<T, 256, 0, stream>>>(tokens, table, x, W, vocab, scale);
  else lgs::embed_kernel<false><<<T, 256, 0, stream>>>(tokens, table, x, W, vocab, scale);
  LGA_LAUNCH_RETURN();
}

extern "C" int lgs_embed_pos(const int* tokens, const int* pos, const void* table, const void* pos_table, int w_f32,
                             float scale, float* x, void* x_bf16, int T, int W, int vocab, int positions,
                             hipStream_t stream) {
  LGA_CHECK_ARG(tokens && pos && table && pos_table && x && T > 0 && W > 0 && vocab > 0 && positions > 0,
                "lgs_embed_pos: bad arguments");
  if (w_f32)
    lgs::embed_pos_kernel<true><<<T, 256, 0, stream>>>(tokens, pos, table, pos_table, x, (uint16_t*)x_bf16, W, vocab,
                                                       positions, scale);
  else
    lgs::embed_pos_kernel<false><<<T, 256, 0, stream>>>(tokens, pos, table, pos_table, x, (uint16_t*)x_bf16, W, vocab,
                                                        positions, scale);
  LGA_LAUNCH_RETURN();
}

extern "C" int lgs_layernorm(const float* y, const float* weight, const float* bias, float eps, float mult,
                             int accumulate, float* x, void* x_bf16, int rows, int n, hipStream_t stream) {
  LGA_CHECK_ARG(y && weight && x && rows > 0 && n > 0, "lgs_layernorm: bad arguments");
  if (n <= 1024)
    lgs::layernorm_kernel<4><<<rows, 256, 0, stream>>>(y, weight, bias, eps, mult, accumulate, x, (uint16_t*)x_bf16, n);
  else
    lgs::layernorm_kernel<16><<<rows, 256, 0, stream>>>(y, weight, bias, eps, mult, accumulate, x, (uint16_t*)x_bf16, n);
  LGA_LAUNCH_RETURN();
}

extern "C" int lgs_softcap(float* z, long n, float cap, hipStream_t stream) {
  LGA_CHECK_ARG(z && n > 0 && cap > 0.0f, "lgs_softcap: bad arguments");
  lgs::softcap_kernel<<<(unsigned)((n + 255) / 256), 256, 0, stream>>>(z, (size_t)n, cap);
  LGA_LAUNCH_RETURN();
}

extern "C" int lgs_rmsnorm(const float* x, long ldx, const float* weight, float offset, float eps, float* y, long ldy,
                           int rows, int groups, int n, void* y_bf16, hipStream_t stream) {
  LGA_CHECK_ARG(x && y && rows > 0 && groups > 0 && groups <= 65535 && n > 0, "lgs_rmsnorm: bad arguments");
  lgs::rmsnorm_kernel<<<dim3(rows, groups), 256, 0, stream>>>(x, ldx, weight, offset, eps, y, ldy, n,
                                                              (uint16_t*)y_bf16);
  LGA_LAUNCH_RETURN();
}

extern "C" int lgs_gather_rows(const float* x, const int* rows, float* y, int n_rows, int W, hipStream_t stream) {
  LGA_CHECK_ARG(x && rows && y && n_rows > 0 && W > 0, "lgs_gather_rows: bad arguments");
  lgs::gather_rows_kernel<<<n_rows, 256, 0, stream>>>(x, rows, y, W);
  LGA_LAUNCH_RETURN();
}
