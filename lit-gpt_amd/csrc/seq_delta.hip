// Gated delta rule of the layered models: a per-head outer-product memory S (d x dv, fp32, one per cache slot) that is
// decayed, corrected towards the value of the current key, and read by the query:
//   S <- diag(g) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q
// g is one number per head, or one per head and key channel (the rows of S). Query / key heads may be shared by
// groups of value heads (head h reads q / k head h / (H / G)). Everything that enters the recurrence is fp32.
// The same kernels serve the plain gated rule without the correction, S <- diag(g) S + k v^T (gated linear attention:
// u = v, no beta), whose decay is sigmoid(raw + bias)^(1 / tau) and whose q is only scaled.
//
//   lgs_delta_prepare   per token: q and k (after their convolution) become unit vectors per head, q times q_scale
//                       (or q is only scaled); beta = sigmoid(raw); g = exp(-exp(A_log) softplus(raw + dt_bias)) or
//                       sigmoid(raw + bias)^(1 / tau); k . q per key head. Steps of few rows spread the decays (each
//                       a low-rank product) over workgroups of their own
//   lgs_delta_step_prepare  the same for a step in which every sequence brings one token, with the short convolution
//                       of q | k | v (and the shift of its stored inputs) in the same launch
//   lgs_gated_delta     the recurrence, token by token for every step kind. The columns of S never mix, so a column
//                       is owned by LPC adjacent lanes that hold d / LPC of its rows in registers; the two dot
//                       products over the rows (both against the decayed state: o = S'^T q + u (k . q)) are summed
//                       inside those lanes with DPP adds (no LDS, no barrier);
//                       q, k, g, v, beta of 16 tokens at a time are staged in LDS, the next 16 prefetched in registers
//                       (8 at a time for key dims above 256)
#include "seq_common.h"

namespace lgs {

__device__ __forceinline__ float softplus_d(float z) { return z > 20.0f ? z : log1pf(expf(z)); }

struct DeltaPrepArgs {
  float* qkv;  // [T][ld]: q [G][d] | k [G][d] | v [H][dv] after the convolution; q and k are normalised in place
  long ld;
  const float* a;  // raw decay inputs, row stride lda: [H][d] (per_channel) or [H]
  long lda;
  const float* b;  // raw beta inputs [H], row stride ldb
  long ldb;
  const float *A_log, *dt_bias;  // [H]; [H][d] or [H]
  float* dec;                    // [T][H][d] or [T][H]
  float* beta;                   // [T][H]
  float* kq;                     // [T][G]: k . q of the prepared vectors
  int H, G, d, per_channel;
  float q_scale, norm_eps;
  // optional second map of a low-rank decay input: a holds `rank` values per row and the raw input of entry i is
  // w_a2[i] . a (w_a2 [H d or H][rank], bf16 or fp32)
  const void* w_a2;
  int rank, a2_f32;
  // unit: q and k become unit vectors (0: q is only scaled, k stays as it is). decay_form 0:
  // exp(-exp(A_log) softplus(raw + dt_bias)); 1: sigmoid(raw + dt_bias)^(1 / tau) (A_log unused). b NULL: no betas.
  int unit, decay_form;
  float tau;
  // the fused one-token form only: the convolution's inputs u [B][ldu] (C = 2 G d + H dv channels), its weights
  // [C][taps] and its slot-indexed history [slots][taps - 1][C]
  const float* u;
  long ldu;
  const void* conv_w;
  int conv_f32, taps, C;
  float* conv_state;
  const int *seq_slot, *seq_pos0;
};

// the decay of one entry from its raw input z (bias added): form 0 exp(-exp(A_log[head]) softplus(z)); form 1
// sigmoid(z)^(1 / tau) = exp(-softplus(-z) / tau)
__device__ __forceinline__ float decay_of(const DeltaPrepArgs& p, float z, int head) {
  if (p.decay_form == 1) return expf(-softplus_d(-z) / p.tau);
  return expf(-expf(p.A_log[head]) * softplus_d(z));
}

// One row's preparation by a whole workgroup: wave w makes the vectors w, w + 4, ... of the 2 G query / key heads
// unit vectors; all threads walk the decays and betas; then k . q per key head.
constexpr int kMaxRank = 512;  // inner size of a low-rank second map that is folded into a consuming kernel

// part 0 of a row's work: the vectors (wave w takes the vectors w, w + 4, ...), the betas and k . q per key head;
// part y >= 1: the decays [256 (y - 1), 256 y) - with `whole` (one workgroup per row) all of them
template <bool A2F32>
__device__ __forceinline__ void delta_prepare_row(const DeltaPrepArgs& p, size_t t, int part, bool whole) {
  __shared__ float a1[kMaxRank];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int d = p.d;
  float* row = p.qkv + t * p.ld;
  if (part > 0 || whole) {
    if (p.w_a2) {
      for (int r = threadIdx.x; r < p.rank; r += 256) a1[r] = aop<A2F32>(p.a[t * p.lda + r]);
      __syncthreads();
    }
    const int dc = p.per_channel ? d : 1, n = p.H * dc;
    const int lo = whole ? 0 : 256 * (part - 1), hi = whole ? n : min(n, lo + 256);
    for (int i = lo + threadIdx.x; i < hi; i += 256) {
      const float raw = p.w_a2 ? lowrank_dot<A2F32>(p.w_a2, i, a1, p.rank) : p.a[t * p.lda + i];
      p.dec[t * n + i] = decay_of(p, raw + p.dt_bias[i], i / dc);
    }
    if (!whole) return;
  }
  for (int vec = wave; vec < 2 * p.G; vec += 4) {
    float* x = row + (size_t)vec * d;
    float s = vec < p.G ? p.q_scale : 1.0f;
    if (p.unit) {
      float ss = 0.0f;
      for (int i = lane; i < d; i += 64) ss = fmaf(x[i], x[i], ss);
      ss = wave_sum(ss);
      s = s / sqrtf(ss + p.norm_eps);
    }
    if (s != 1.0f)
      for (int i = lane; i < d; i += 64) x[i] *= s;
  }
  if (p.b)
    for (int h = threadIdx.x; h < p.H; h += 256) p.beta[t * p.H + h] = sigmoid_f(p.b[t * p.ldb + h]);
  __syncthreads();  // the prepared vectors of all heads are written
  for (int g = wave; g < p.G; g += 4) {
    const float *q = row + (size_t)g * d, *k = row + (size_t)(p.G + g) * d;
    float s = 0.0f;
    for (int i = lane; i < d; i += 64) s = fmaf(q[i], k[i], s);
    s = wave_sum(s);
    if (lane == 0) p.kq[t * p.G + g] = s;
  }
}

// grid (T), or for steps of few rows (T, 1 + ceil(n / 256)): the decays in workgroups of their own
template <bool A2F32>
__global__ void __launch_bounds__(256) delta_prepare_kernel(DeltaPrepArgs p) {
  delta_prepare_row<A2F32>(p, blockIdx.x, blockIdx.y, gridDim.y == 1);
}

// One channel of the short convolution for a one-token step: the weighted sum of the token's input and the slot's
// stored inputs (zeros before the sequence's start), which are shifted by one; returns silu of the sum.
template <bool WF32>
__device__ __forceinline__ float conv_step_channel(const DeltaPrepArgs& p, int b, int c, int pos0, float* st) {
  const int taps = p.taps, hist = taps - 1, C = p.C;
  const float cur = p.u[(size_t)b * p.ldu + c];
  float acc = wload<WF32>(p.conv_w, (size_t)c * taps + hist) * cur;
  float prev = cur;  // walks the history from the newest stored input to the oldest, shifting it on the way
  for (int j = hist - 1; j >= 0; --j) {
    const float x = pos0 - (hist - j) >= 0 ? st[(size_t)j * C + c] : 0.0f;
    acc = fmaf(wload<WF32>(p.conv_w, (size_t)c * taps + j), x, acc);
    st[(size_t)j * C + c] = prev;
    prev = x;
  }
  return acc / (1.0f + expf(-acc));
}

// The one-token step (every sequence brings one token; row b belongs to sequence b): convolution + silu of the
// token's q | k | v channels and the row's preparation in one launch. grid (B, G + ceil(H dv / 256) + ceil(n / 256)):
// workgroup y < G convolves and normalises q and k of key head y and leaves their k . q; the next ones convolve 256
// value channels each; the last ones make 256 decays each (the first of them also the betas).
template <bool WF32, bool A2F32>
__global__ void __launch_bounds__(256) delta_step_prepare_kernel(DeltaPrepArgs p) {
  __shared__ float buf[2 * 512];
  __shared__ float red[4];
  const int b = blockIdx.x, y = blockIdx.y, tid = threadIdx.x;
  const int d = p.d, G = p.G, C = p.C, hist = p.taps - 1;
  const int pos0 = p.seq_pos0[b];
  float* st = p.conv_state + (size_t)p.seq_slot[b] * max(hist, 1) * C;
  float* row = p.qkv + (size_t)b * p.ld;
  const int nv = C - 2 * G * d, parts_v = (nv + 255) / 256;
  if (y < G) {
    for (int i = tid; i < 2 * d; i += 256) {
      const int c = i < d ? y * d + i : (G + y) * d + (i - d);
      buf[i] = conv_step_channel<WF32>(p, b, c, pos0, st);
    }
    __syncthreads();
    float sq = 0.0f, sk = 0.0f;
    for (int i = tid; i < d; i += 256) {
      sq = fmaf(buf[i], buf[i], sq);
      sk = fmaf(buf[d + i], buf[d + i], sk);
    }
    sq = block_sum_256(sq, red);
    sk = block_sum_256(sk, red);
    const float fq = p.q_scale / sqrtf(sq + p.norm_eps), fk = 1.0f / sqrtf(sk + p.norm_eps);
    float kq = 0.0f;
    for (int i = tid; i < d; i += 256) {
      const float qn = buf[i] * fq, kn = buf[d + i] * fk;
      row[(size_t)y * d + i] = qn;
      row[(size_t)(G + y) * d + i] = kn;
      kq = fmaf(qn, kn, kq);
    }
    kq = block_sum_256(kq, red);
    if (tid == 0) p.kq[(size_t)b * G + y] = kq;
  } else if (y < G + parts_v) {
    const int c = 2 * G * d + (y - G) * 256 + tid;
    if (c < C) row[c] = conv_step_channel<WF32>(p, b, c, pos0, st);
  } else {
    const int blk = y - G - parts_v;
    const int dc = p.per_channel ? d : 1, n = p.H * dc;
    if (p.w_a2) {
      for (int r = tid; r < p.rank; r += 256) buf[r] = aop<A2F32>(p.a[(size_t)b * p.lda + r]);
      __syncthreads();
    }
    const int i = blk * 256 + tid;
    if (i < n) {
      const float raw = p.w_a2 ? lowrank_dot<A2F32>(p.w_a2, i, buf, p.rank) : p.a[(size_t)b * p.lda + i];
      p.dec[(size_t)b * n + i] = decay_of(p, raw + p.dt_bias[i], i / dc);
    }
    if (blk == 0)
      for (int h = tid; h < p.H; h += 256) p.beta[(size_t)b * p.H + h] = sigmoid_f(p.b[(size_t)b * p.ldb + h]);
  }
}

struct DeltaArgs {
  const float* qkv;  // [T][ld]: unit q [G][d] | unit k [G][d] | v [H][dv]
  long ld;
  const float* dec;   // [T][H][dc], dc = d or 1
  const float* beta;  // [T][H]
  const float* kq;    // [T][G]
  float* state;       // [slots][H][d][dv]
  const int *seq_start, *seq_slot, *seq_pos0;
  float* out;  // [T][H * dv]
  int H, G, d, dv, per_channel;
  int ncb, items;  // column blocks per head; work items = B * H * ncb
};
// DELTA false: the plain gated rule S <- diag(g) S + k v^T (u = v: no correction towards the key's value, no beta)

template <int CTRL>
__device__ __forceinline__ float dpp_f(float v) {
  return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, 0xf, 0xf, false));
}
// sum over LPC adjacent lanes (aligned, inside a row of 16 lanes); every lane of the group gets the sum. The order
// of the additions is fixed: neighbours, pairs, then the mirrored halves. Two values at once: their steps interleave.
template <int LPC>
__device__ __forceinline__ void lanes_sum2(float& a, float& b) {
  float x = dpp_f<0xB1>(a), y = dpp_f<0xB1>(b);
  a += x, b += y;
  x = dpp_f<0x4E>(a), y = dpp_f<0x4E>(b);
  a += x, b += y;
  if (LPC >= 8) {
    x = dpp_f<0x141>(a), y = dpp_f<0x141>(b);
    a += x, b += y;
  }
  if (LPC >= 16) {
    x = dpp_f<0x140>(a), y = dpp_f<0x140>(b);
    a += x, b += y;
  }
}

// grid (B * H * ceil(dv / CW) rounded up to 8), CW = 256 / LPC columns per workgroup. Lane l of a wave: r = l % LPC, column
// l / LPC of the wave's 64 / LPC; the lane holds the rows 4 (r + LPC j) + e, j < NR4, e < 4, of its column.
template <int NR4, int LPC, bool DELTA>
__global__ void __launch_bounds__(256) gated_delta_kernel(DeltaArgs p) {
  constexpr int DP = 4 * NR4 * LPC;      // rows, padded
  constexpr int CW = 256 / LPC;          // columns per workgroup
  constexpr int ROW = 3 * DP + CW + 4;   // staged floats per token: q | k | g | v | beta (rows stay 16-byte aligned)
  constexpr int kDeltaTB = DP > 256 ? 8 : (DP > 128 ? 16 : 32);  // tokens staged at a time
  constexpr int EPT = (ROW + 255) / 256;       // staged entries per thread and token
  __shared__ __attribute__((aligned(16))) float st[kDeltaTB * ROW];
  __shared__ float os[kDeltaTB][CW];
  const int tid = threadIdx.x;
  const int r = tid % LPC, cw = tid / LPC;  // cw: column inside the workgroup
  // Workgroups are dealt to the 8 XCDs in turn. The column blocks of one (sequence, head) read the same q, k and
  // decays, so consecutive work items go to ONE XCD (and its L2): item = xcd * per_xcd + turn.
  const int per_xcd = (p.items + 7) / 8;
  const int item = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
  if (item >= p.items) return;
  const int cblk = item % p.ncb, hd = (item / p.ncb) % p.H, b = item / (p.ncb * p.H);
  const int col = cblk * CW + cw;
  const int d = p.d, dv = p.dv, H = p.H;
  const bool live = col < dv;
  const int g = hd / (H / p.G);
  const int r0 = p.seq_start[b], n = p.seq_start[b + 1] - r0;
  const int dc = p.per_channel ? d : 1;
  float* sp = p.state + (((size_t)p.seq_slot[b] * H + hd) * d) * dv;
  const bool fresh = p.seq_pos0[b] == 0;
  float S[NR4][4];
#pragma unroll
  for (int j = 0; j < NR4; ++j)
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      const int row = 4 * (r + LPC * j) + e;
      S[j][e] = (!fresh && live && row < d) ? sp[(size_t)row * dv + col] : 0.0f;
    }
  // Entry e = tid + 256 i of a token's staged row comes from one place whatever the token: a pointer to it at the
  // sequence's first row, the distance to the next token's, and the value of an entry that has no source (padding).
  // (an entry without a source loads a valid address all the same, so that the loads carry no branches)
  const float* src[EPT];
  long step[EPT];
  float pad[EPT];
  bool has[EPT];
#pragma unroll
  for (int i = 0; i < EPT; ++i) {
    const int e = tid + 256 * i;
    src[i] = nullptr, step[i] = 0, pad[i] = 0.0f;
    if (e < 2 * DP) {  // q, then k
      const int c = e < DP ? e : e - DP;
      if (c < d) src[i] = p.qkv + (size_t)r0 * p.ld + (size_t)((e < DP ? g : p.G + g)) * d + c, step[i] = p.ld;
    } else if (e < 3 * DP) {
      const int c = e - 2 * DP;
      pad[i] = 1.0f;
      if (c < d) src[i] = p.dec + ((size_t)r0 * H + hd) * dc + (dc == 1 ? 0 : c), step[i] = (long)H * dc;
    } else if (e < 3 * DP + CW) {
      const int c = cblk * CW + (e - 3 * DP);
      if (c < dv) src[i] = p.qkv + (size_t)r0 * p.ld + (size_t)2 * p.G * d + (size_t)hd * dv + c, step[i] = p.ld;
    } else if (e == 3 * DP + CW && DELTA) {
      src[i] = p.beta + (size_t)r0 * H + hd, step[i] = H;
    } else if (e == 3 * DP + CW + 1) {
      src[i] = p.kq + (size_t)r0 * p.G + g, step[i] = p.G;
    }
    has[i] = src[i] != nullptr;
    if (!has[i]) src[i] = p.kq + (size_t)r0 * p.G + g;
  }
  float pre[kDeltaTB][EPT];
  auto prefetch = [&](int t0) {
#pragma unroll
    for (int t = 0; t < kDeltaTB; ++t)
#pragma unroll
      for (int i = 0; i < EPT; ++i) {
        const float v = src[i][(size_t)min(t0 + t, n - 1) * step[i]];
        pre[t][i] = has[i] ? v : pad[i];
      }
  };
  prefetch(0);

  for (int t0 = 0; t0 < n; t0 += kDeltaTB) {
    const int nb = min(kDeltaTB, n - t0);
    __syncthreads();  // the previous batch's reads of st and os are done
#pragma unroll
    for (int t = 0; t < kDeltaTB; ++t)
#pragma unroll
      for (int i = 0; i < EPT; ++i)
        if (tid + 256 * i < ROW) st[t * ROW + tid + 256 * i] = pre[t][i];
    __syncthreads();
    if (t0 + kDeltaTB < n) prefetch(t0 + kDeltaTB);
    // With S' = diag(g) S the output is o = S'^T q + u (k . q): both products with S' run side by side and share one
    // round of lane sums, and the write S' + k u^T leaves the output's dependent chain. Four partial sums per product
    // keep the chains short; two tokens per trip let one token's tail overlap the next one's decay.
#pragma unroll 2
    for (int t = 0; t < nb; ++t) {
      const float* row = st + t * ROW;
      float4 k4[NR4];
      float ka = 0.0f, kb = 0.0f, kc = 0.0f, kd = 0.0f, oa = 0.0f, ob = 0.0f, oc = 0.0f, od = 0.0f;
#pragma unroll
      for (int j = 0; j < NR4; ++j) {
        const int at = 4 * (r + LPC * j);
        k4[j] = *(const float4*)(row + DP + at);
        const float4 g4 = *(const float4*)(row + 2 * DP + at);
        const float4 q4 = *(const float4*)(row + at);
        S[j][0] *= g4.x;
        S[j][1] *= g4.y;
        S[j][2] *= g4.z;
        S[j][3] *= g4.w;
        if (DELTA) {
          ka = fmaf(S[j][0], k4[j].x, ka);
          kb = fmaf(S[j][1], k4[j].y, kb);
          kc = fmaf(S[j][2], k4[j].z, kc);
          kd = fmaf(S[j][3], k4[j].w, kd);
        }
        oa = fmaf(S[j][0], q4.x, oa);
        ob = fmaf(S[j][1], q4.y, ob);
        oc = fmaf(S[j][2], q4.z, oc);
        od = fmaf(S[j][3], q4.w, od);
      }
      float ks = (ka + kb) + (kc + kd), qs = (oa + ob) + (oc + od);
      lanes_sum2<LPC>(ks, qs);
      const float u = DELTA ? row[3 * DP + CW] * (row[3 * DP + cw] - ks) : row[3 * DP + cw];
      if (r == 0) os[t][cw] = fmaf(u, row[3 * DP + CW + 1], qs);
#pragma unroll
      for (int j = 0; j < NR4; ++j) {
        S[j][0] = fmaf(k4[j].x, u, S[j][0]);
        S[j][1] = fmaf(k4[j].y, u, S[j][1]);
        S[j][2] = fmaf(k4[j].z, u, S[j][2]);
        S[j][3] = fmaf(k4[j].w, u, S[j][3]);
      }
    }
    __syncthreads();
    for (int i = tid; i < nb * CW; i += 256) {
      const int t = i / CW, c = i % CW;
      if (cblk * CW + c < dv)
        p.out[(size_t)(r0 + t0 + t) * H * dv + (size_t)hd * dv + cblk * CW + c] = os[t][c];
    }
  }
  if (live) {
#pragma unroll
    for (int j = 0; j < NR4; ++j)
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const int row = 4 * (r + LPC * j) + e;
        if (row < d) sp[(size_t)row * dv + col] = S[j][e];
      }
  }
}

template <int LPC, bool DELTA>
static bool gated_delta_launch(DeltaArgs p, int B, hipStream_t stream) {
  p.ncb = (p.dv + 256 / LPC - 1) / (256 / LPC);
  p.items = B * p.H * p.ncb;
  const dim3 grid((p.items + 7) / 8 * 8);
  const int nr4 = (p.d + 4 * LPC - 1) / (4 * LPC);
  if (nr4 <= 1) gated_delta_kernel<1, LPC, DELTA><<<grid, 256, 0, stream>>>(p);
  else if (nr4 <= 2) gated_delta_kernel<2, LPC, DELTA><<<grid, 256, 0, stream>>>(p);
  else if (nr4 <= 4) gated_delta_kernel<4, LPC, DELTA><<<grid, 256, 0, stream>>>(p);
  else if (nr4 <= 8) gated_delta_kernel<8, LPC, DELTA><<<grid, 256, 0, stream>>>(p);
  else return false;
  return true;
}

}  // namespace lgs

extern "C" int lgs_delta_prepare(float* qkv, long ld, const float* a, long lda, const float* b, long ldb,
                                 const float* A_log, const float* dt_bias, float* dec, float* beta, float* kq, int T,
                                 int H, int G, int d, int per_channel, float q_scale, float norm_eps, const void* w_a2,
                                 int rank, int a2_f32, int unit, int decay_form, float tau, hipStream_t stream) {
  LGA_CHECK_ARG(qkv && a && dt_bias && dec && kq && T > 0 && (!b || beta), "lgs_delta_prepare: bad arguments");
  LGA_CHECK_ARG((decay_form == 0 && A_log) || (decay_form == 1 && tau > 0.0f),
                "lgs_delta_prepare: decay form 0 needs A_log, form 1 a positive tau");
  LGA_CHECK_ARG(H > 0 && G > 0 && H % G == 0 && d > 0 && ld >= 2L * G * d, "lgs_delta_prepare: bad sizes");
  LGA_CHECK_ARG(!w_a2 || (rank > 0 && rank <= lgs::kMaxRank), "lgs_delta_prepare: inner size of the decay map 1..512");
  lgs::DeltaPrepArgs p{qkv, ld, a, lda, b, ldb, A_log, dt_bias, dec, beta, kq, H, G, d, per_channel ? 1 : 0, q_scale,
                       norm_eps, w_a2, rank, a2_f32, unit ? 1 : 0, decay_form, tau, nullptr, 0, nullptr, 0, 0, 0, nullptr,
                       nullptr, nullptr};
  // few rows (decode): the decays - with a low-rank second map a product each - spread over workgroups of their own
  const int n = per_channel ? H * d : H;
  const dim3 grid(T, T <= 64 && n > 256 ? 1 + (n + 255) / 256 : 1);
  if (a2_f32) lgs::delta_prepare_kernel<true><<<grid, 256, 0, stream>>>(p);
  else lgs::delta_prepare_kernel<false><<<grid, 256, 0, stream>>>(p);
  LGA_LAUNCH_RETURN();
}

extern "C" int lgs_delta_step_prepare(const float* u, long ldu, const void* conv_w, int conv_f32, int taps,
                                      float* conv_state, const int* seq_slot, const int* seq_pos0, float* qkv,
                                      const float* a, long lda, const float* b, long ldb, const float* A_log,
                                      const float* dt_bias, float* dec, float* beta, float* kq, int B, int H, int G,
                                      int d, int dv, int per_channel, float q_scale, float norm_eps, const void* w_a2,
                                      int rank, int a2_f32, hipStream_t stream) {
  LGA_CHECK_ARG(u && conv_w && conv_state && seq_slot && seq_pos0 && qkv && a && b && A_log && dt_bias && dec && beta &&
                    kq && B > 0,
                "lgs_delta_step_prepare: bad arguments");
  LGA_CHECK_ARG(H > 0 && G > 0 && H % G == 0 && d > 0 && dv > 0 && taps >= 1 && taps <= 16,
                "lgs_delta_step_prepare: bad sizes (taps 1..16)");
  LGA_CHECK_ARG(!w_a2 || (rank > 0 && rank <= lgs::kMaxRank),
                "lgs_delta_step_prepare: inner size of the decay map 1..512");
  const int C = 2 * G * d + H * dv;
  LGA_CHECK_ARG(ldu >= C, "lgs_delta_step_prepare: channels outside the row");
  lgs::DeltaPrepArgs p{qkv, C, a, lda, b, ldb, A_log, dt_bias, dec, beta, kq, H, G, d, per_channel ? 1 : 0, q_scale,
                       norm_eps, w_a2, rank, a2_f32, 1, 0, 1.0f, u, ldu, conv_w, conv_f32, taps, C, conv_state, seq_slot,
                       seq_pos0};
  const int n = per_channel ? H * d : H;
  const dim3 grid(B, G + (H * dv + 255) / 256 + (n + 255) / 256);
  LGA_CHECK_ARG(d <= 512 && grid.y <= 65535, "lgs_delta_step_prepare: key dim <= 512");
  if (conv_f32) {
    if (a2_f32) lgs::delta_step_prepare_kernel<true, true><<<grid, 256, 0, stream>>>(p);
    else lgs::delta_step_prepare_kernel<true, false><<<grid, 256, 0, stream>>>(p);
  } else {
    if (a2_f32) lgs::delta_step_prepare_kernel<false, true><<<grid, 256, 0, stream>>>(p);
    else lgs::delta_step_prepare_kernel<false, false><<<grid, 256, 0, stream>>>(p);
  }
  LGA_LAUNCH_RETURN();
}

extern "C" int lgs_gated_delta(const float* qkv, long ld, const float* dec, const float* beta, const float* kq,
                               float* state, const int* seq_start, const int* seq_slot, const int* seq_pos0, float* out,
                               int B, int H, int G, int d, int dv, int per_channel, int lanes, int plain,
                               hipStream_t stream) {
  LGA_CHECK_ARG(qkv && dec && (beta || plain) && kq && state && seq_start && seq_slot && seq_pos0 && out,
                "lgs_gated_delta: null pointer");
  LGA_CHECK_ARG(B > 0 && H > 0 && G > 0 && H % G == 0 && d > 0 && d <= 512 && dv > 0,
                "lgs_gated_delta: bad sizes (key dim <= 512)");
  LGA_CHECK_ARG(ld >= 2L * G * d + (long)H * dv, "lgs_gated_delta: q | k | v outside the row");
  LGA_CHECK_ARG((long)B * H * ((dv + 15) / 16) < (1L << 30), "lgs_gated_delta: too many columns");
  lgs::DeltaArgs p{qkv, ld, dec, beta, kq, state, seq_start, seq_slot, seq_pos0, out, H, G, d, dv, per_channel ? 1 : 0,
                   0, 0};
  // lanes per column: more lanes shorten a token's dependent chain and multiply the waves; by default as many as
  // keep the launch within about two waves per SIMD, and at least enough for 32 rows per lane
  int lpc = lanes;
  if (lpc == 0) {
    const long cols = (long)B * H * dv;
    lpc = cols * 16 / 64 <= 2048 ? 16 : cols * 8 / 64 <= 2048 ? 8 : 4;
    while (lpc > 4 && 4 * lpc > d) lpc >>= 1;
  }
  while (lpc < 16 && d > 32 * lpc) lpc <<= 1;
  bool ok;
  if (lpc == 4) ok = plain ? lgs::gated_delta_launch<4, false>(p, B, stream) : lgs::gated_delta_launch<4, true>(p, B, stream);
  else if (lpc == 8) ok = plain ? lgs::gated_delta_launch<8, false>(p, B, stream) : lgs::gated_delta_launch<8, true>(p, B, stream);
  else if (lpc == 16) ok = plain ? lgs::gated_delta_launch<16, false>(p, B, stream) : lgs::gated_delta_launch<16, true>(p, B, stream);
  else ok = false;
  LGA_CHECK_ARG(ok, "lgs_gated_delta: lanes per column must be 4, 8 or 16 and cover the key dim");
  LGA_LAUNCH_RETURN();
}
