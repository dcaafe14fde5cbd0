// Sequence mixers of the layered models, all sums in fp32.
//
//   lgs_retention        decayed linear attention: an optional activation on q, k and v, rotary (half layout) on q
//                        and k, k scaled, then per head S <- decay S + k v^T, o = S^T q, the state S (d x dv fp32)
//                        carried per cache slot
//   lgs_head_gate        per head: optional unit RMS of o, times act(g): the retention's output norm + silu gate and
//                        the latent attention's sigmoid gate
//   lgs_latent_prepare   latent attention, per token: RMS-normed latent c and the rotated shared key part go to the
//                        cache rows (slot, position); the queries' rotated parts are rotated in place (interleaved)
//   lgs_latent_attention softmax attention in the latent space: every head's query has been mapped through its key
//                        up-projection, so all heads read the same cached rows [c | k_rot]; scores, the sink's
//                        share of the denominator and the weighted sum of c are fp32; the value up-projection
//                        follows as a per-head product
#include "seq_common.h"

namespace lgs {

// ------------------------------------------------------------------------------------------------ retention
struct RetArgs {
  const float* q;  // row t, head h at q[t * ld + h * d]
  const float* k;
  const float* v;  // v[t * ld + h * dv]
  long ld;
  float* state;          // [slots][H][d][dv]
  const float* decay;    // [H]
  const float* inv_freq; // [rot_dims / 2]
  const int* seq_start;  // [B + 1] rows
  const int* seq_slot;   // [B]
  const int* seq_pos0;   // [B] position of the sequence's first row in this step
  float* out;            // [T][H * dv]
  int H, d, dv, rot_dims;
  float k_scale;
  float* ws;       // chunk-parallel prompt form: [B * max_chunks][H][d][dv] local sums, then chunk-start states
  int max_chunks;  // chunks of 64 tokens of the longest sequence
  int act;         // activation on q, k and v as projected (ahead of the rotation and the key scale)
};

// grid (B, H, ceil(dv / 64)): a workgroup owns 64 columns of one head's state; wave w owns rows [w NR, (w + 1) NR)
template <int NR>
__global__ void __launch_bounds__(256) retention_scan_kernel(RetArgs p) {
  __shared__ float qs[512], ks[512];
  __shared__ float part[4][64];
  const int b = blockIdx.x, h = blockIdx.y, col = blockIdx.z * 64 + (threadIdx.x & 63);
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int d = p.d, dv = p.dv, half = p.rot_dims / 2;
  const int t0 = p.seq_start[b], t1 = p.seq_start[b + 1];
  const int pos0 = p.seq_pos0[b];
  const float lam = p.decay[h];
  const bool live = col < dv;
  float* sp = p.state + (((size_t)p.seq_slot[b] * p.H + h) * d) * dv + col;
  float S[NR];
#pragma unroll
  for (int i = 0; i < NR; ++i) {
    const int row = wave * NR + i;
    S[i] = (pos0 > 0 && live && row < d) ? sp[(size_t)row * dv] : 0.0f;  // a sequence starts from the zero state
  }
  for (int t = t0; t < t1; ++t) {
    const float pos = (float)(pos0 + (t - t0));
    for (int tid = threadIdx.x; tid < d; tid += 256) {
      const float* qr = p.q + (size_t)t * p.ld + (size_t)h * d;
      const float* kr = p.k + (size_t)t * p.ld + (size_t)h * d;
      float qo = act_f(p.act, qr[tid]), ko = act_f(p.act, kr[tid]);
      if (tid < p.rot_dims) {
        const int j = tid < half ? tid : tid - half;
        float sn, cs;
        sincosf(pos * p.inv_freq[j], &sn, &cs);
        if (tid < half) {
          qo = qo * cs - act_f(p.act, qr[tid + half]) * sn;
          ko = ko * cs - act_f(p.act, kr[tid + half]) * sn;
        } else {
          qo = qo * cs + act_f(p.act, qr[tid - half]) * sn;
          ko = ko * cs + act_f(p.act, kr[tid - half]) * sn;
        }
      }
      qs[tid] = qo;
      ks[tid] = ko * p.k_scale;
    }
    __syncthreads();
    const float vt = live ? act_f(p.act, p.v[(size_t)t * p.ld + (size_t)h * dv + col]) : 0.0f;
    float o = 0.0f;
#pragma unroll
    for (int i = 0; i < NR; ++i) {
      const int row = wave * NR + i;
      if (row < d) {
        S[i] = fmaf(lam, S[i], ks[row] * vt);
        o = fmaf(S[i], qs[row], o);
      }
    }
    part[wave][lane] = o;
    __syncthreads();
    if (wave == 0 && live)
      p.out[(size_t)t * p.H * dv + (size_t)h * dv + col] = (part[0][lane] + part[1][lane]) + (part[2][lane] + part[3][lane]);
  }
  if (live) {
#pragma unroll
    for (int i = 0; i < NR; ++i) {
      const int row = wave * NR + i;
      if (row < d) sp[(size_t)row * dv] = S[i];
    }
  }
}

// The prompt form: the same recurrence over chunks of 64 tokens as fp32 matrix products (v_mfma_f32_16x16x4_f32).
// With S the state at the chunk's start, n its token count and i, j local positions:
//   o_i = decay^(i+1) S^T q_i + sum_{j <= i} decay^(i-j) (q_i . k_j) v_j,   S' = decay^n S + sum_j decay^(n-1-j) k_j v_j^T
// MODE 0, grid (B, H, ceil(dv / 64)): a workgroup keeps 64 columns of the state in LDS and walks its sequence's
// chunks one after the other. With a workspace the chunks run side by side instead, grid (B * max_chunks, H, ..):
// MODE 1 leaves every chunk's local sum (the second term of S') in the workspace, retention_carry_kernel turns these
// into the state at each chunk's start (a short elementwise recurrence over the chunks, which also leaves the final
// state), and MODE 2 computes the outputs of every chunk from its start state.
// LDS (floats): Q, K [64][DP], V [64][80], scores [64][66], S [DPAD][80], powers of the decay [66]; d <= 128.
typedef float f32x4_t __attribute__((ext_vector_type(4)));
constexpr int kRC = 64, kVS = 80, kAS = 66;

// grid (T, H): the activation on q, k and v, rotary on q and k (pairs i, i + rot_dims / 2) and the key scale, all in
// place, ahead of the chunk kernels
__global__ void __launch_bounds__(64) retention_rope_kernel(float* __restrict__ q, float* __restrict__ k,
                                                            float* __restrict__ v, long ld,
                                                            const float* __restrict__ inv_freq,
                                                            const int* __restrict__ pos, int d, int dv, int rot_dims,
                                                            float k_scale, int act) {
  const int t = blockIdx.x, h = blockIdx.y, half = rot_dims / 2;
  float* qr = q + (size_t)t * ld + (size_t)h * d;
  float* kr = k + (size_t)t * ld + (size_t)h * d;
  const float fpos = (float)pos[t];
  for (int i = threadIdx.x; i < d; i += 64) {
    if (i < half) {
      float sn, cs;
      sincosf(fpos * inv_freq[i], &sn, &cs);
      const float qu = act_f(act, qr[i]), qv = act_f(act, qr[i + half]);
      const float ku = act_f(act, kr[i]), kv = act_f(act, kr[i + half]);
      qr[i] = qu * cs - qv * sn;
      qr[i + half] = qv * cs + qu * sn;
      kr[i] = (ku * cs - kv * sn) * k_scale;
      kr[i + half] = (kv * cs + ku * sn) * k_scale;
    } else if (i >= rot_dims) {
      if (act != kActNone) qr[i] = act_f(act, qr[i]);
      kr[i] = act_f(act, kr[i]) * k_scale;
    }
  }
  if (act != kActNone) {
    float* vr = v + (size_t)t * ld + (size_t)h * dv;
    for (int i = threadIdx.x; i < dv; i += 64) vr[i] = act_f(act, vr[i]);
  }
}

// DPC: the key dim padded to 16 when it is 64 or 128 (constant trip counts), 0 for any other
template <int MODE, int DPC>
__global__ void __launch_bounds__(256) retention_chunk_kernel(RetArgs p) {
  extern __shared__ float lds[];
  const int b = MODE == 0 ? blockIdx.x : blockIdx.x / p.max_chunks;
  const int cidx = MODE == 0 ? 0 : blockIdx.x % p.max_chunks;
  const int h = blockIdx.y, col0 = blockIdx.z * 64;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int d = p.d, dv = p.dv;
  const int DPAD = DPC ? DPC : (d + 15) / 16 * 16, DT = DPAD / 16, DP = DPAD + 2;
  int dshift = 4;
  while ((1 << dshift) < DPAD) ++dshift;
  const int DPOW = 1 << dshift;
  float* Qs = lds;
  float* Ks = Qs + kRC * DP;
  float* Vs = Ks + kRC * DP;
  float* As = Vs + kRC * kVS;
  float* Ss = As + kRC * kAS;
  float* pw = Ss + DPAD * kVS;
  const int t0 = p.seq_start[b], t1 = p.seq_start[b + 1];
  if (MODE != 0 && t0 + cidx * kRC >= t1) return;
  const int pos0 = p.seq_pos0[b];
  const float lam = p.decay[h];
  // MODE 0: the slot's state; MODE 1 / 2: this chunk's tile of the workspace
  float* sp = MODE == 0 ? p.state + (((size_t)p.seq_slot[b] * p.H + h) * d) * dv
                        : p.ws + (((size_t)blockIdx.x * p.H + h) * d) * dv;
  if (MODE != 1)
    for (int i = tid; i < DPAD * 64; i += 256) {
      const int row = i >> 6, c = i & 63;
      Ss[row * kVS + c] = ((MODE == 2 || pos0 > 0) && row < d && col0 + c < dv) ? sp[(size_t)row * dv + col0 + c] : 0.0f;
    }
  if (tid <= 64) pw[tid] = powf(lam, (float)tid);
  const int fr = lane & 15, fk = lane >> 4;
  const int t_end = MODE == 0 ? t1 : min(t1, t0 + (cidx + 1) * kRC);
  for (int tc = t0 + cidx * kRC; tc < t_end; tc += kRC) {
    const int n = min(kRC, t1 - tc);
    // ---- load (q and k were rotated and scaled in place beforehand); rows past n and dims past d are zero
    for (int i = tid; i < kRC * DPOW; i += 256) {
      const int row = i >> dshift, dd = i & (DPOW - 1);
      if (dd >= DPAD) continue;
      const bool in = row < n && dd < d;
      const size_t at = (size_t)(tc + row) * p.ld + (size_t)h * d + dd;
      if (MODE != 1) Qs[row * DP + dd] = in ? p.q[at] : 0.0f;
      Ks[row * DP + dd] = in ? p.k[at] : 0.0f;
    }
    for (int i = tid; i < kRC * 64; i += 256) {
      const int row = i >> 6, c = i & 63;
      Vs[row * kVS + c] = (row < n && col0 + c < dv) ? p.v[(size_t)(tc + row) * p.ld + (size_t)h * dv + col0 + c] : 0.0f;
    }
    __syncthreads();
    // ---- wave w owns tokens 16 w .. 16 w + 15: decayed causal scores, and the carried state's share of o
    const int ti = wave;
    if (MODE != 1) {
      // the four key blocks as independent chains (blocks right of the diagonal are skipped and left zero)
      f32x4_t acc[4];
#pragma unroll
      for (int tj = 0; tj < 4; ++tj) acc[tj] = f32x4_t{0.f, 0.f, 0.f, 0.f};
      const float* qa = Qs + (ti * 16 + fr) * DP + fk;
      const float* kb = Ks + fr * DP + fk;
#pragma unroll 2
      for (int k = 0; k < DPAD; k += 4) {
        const float a = qa[k];
#pragma unroll
        for (int tj = 0; tj < 4; ++tj)
          if (tj <= ti) acc[tj] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, kb[tj * 16 * DP + k], acc[tj], 0, 0, 0);
      }
#pragma unroll
      for (int tj = 0; tj < 4; ++tj)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int i = ti * 16 + fk * 4 + r, j = tj * 16 + fr;
          As[i * kAS + j] = j <= i ? acc[tj][r] * pw[i - j] : 0.0f;
        }
    f32x4_t o[4];
#pragma unroll
    for (int c = 0; c < 4; ++c) o[c] = f32x4_t{0.f, 0.f, 0.f, 0.f};
#pragma unroll 4
    for (int k = 0; k < DPAD; k += 4) {
      const float a = Qs[(ti * 16 + fr) * DP + k + fk];
#pragma unroll
      for (int c = 0; c < 4; ++c)
        o[c] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, Ss[(k + fk) * kVS + c * 16 + fr], o[c], 0, 0, 0);
    }
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
      for (int r = 0; r < 4; ++r) o[c][r] *= pw[ti * 16 + fk * 4 + r + 1];
    __syncthreads();
    // ---- o += scores . V (keys up to the wave's last token), then out
#pragma unroll 4
    for (int k = 0; k < (ti + 1) * 16; k += 4) {
      const float a = As[(ti * 16 + fr) * kAS + k + fk];
#pragma unroll
      for (int c = 0; c < 4; ++c)
        o[c] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, Vs[(k + fk) * kVS + c * 16 + fr], o[c], 0, 0, 0);
    }
#pragma unroll
    for (int c = 0; c < 4; ++c)
#pragma unroll
      for (int r = 0; r < 4; ++r) {
        const int i = ti * 16 + fk * 4 + r, col = col0 + c * 16 + fr;
        if (i < n && col < dv) p.out[(size_t)(tc + i) * p.H * dv + (size_t)h * dv + col] = o[c][r];
      }
    }
    // ---- state: S' = decay^n S + sum_j decay^(n-1-j) k_j v_j^T; each element of S belongs to one lane
    const float pn = pw[n];
    for (int td = wave; td < DT && MODE != 2; td += 4) {
      f32x4_t s[4];
#pragma unroll
      for (int c = 0; c < 4; ++c)
#pragma unroll
        for (int r = 0; r < 4; ++r) s[c][r] = MODE == 1 ? 0.0f : pn * Ss[(td * 16 + fk * 4 + r) * kVS + c * 16 + fr];
#pragma unroll 4
      for (int k = 0; k < kRC; k += 4) {
        const int j = k + fk;
        const float a = j < n ? Ks[j * DP + td * 16 + fr] * pw[n - 1 - j] : 0.0f;
#pragma unroll
        for (int c = 0; c < 4; ++c)
          s[c] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, Vs[j * kVS + c * 16 + fr], s[c], 0, 0, 0);
      }
#pragma unroll
      for (int c = 0; c < 4; ++c)
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const int row = td * 16 + fk * 4 + r, col = c * 16 + fr;
          if (MODE == 0) Ss[row * kVS + col] = s[c][r];
          else if (row < d && col0 + col < dv) sp[(size_t)row * dv + col0 + col] = s[c][r];
        }
    }
    __syncthreads();
  }
  if (MODE == 0)
    for (int i = tid; i < DPAD * 64; i += 256) {
      const int row = i >> 6, c = i & 63;
      if (row < d && col0 + c < dv) sp[(size_t)row * dv + col0 + c] = Ss[row * kVS + c];
    }
}

// grid (B, H, ceil(d dv / 256)): one state element per thread walks its sequence's chunks: the workspace's local
// sums become the states at the chunks' starts, and the state after the last chunk goes back to the slot
__global__ void __launch_bounds__(256) retention_carry_kernel(RetArgs p) {
  const int b = blockIdx.x, h = blockIdx.y;
  const int e = blockIdx.z * 256 + threadIdx.x;
  if (e >= p.d * p.dv) return;
  const int len = p.seq_start[b + 1] - p.seq_start[b];
  const float lam = p.decay[h];
  const float p64 = powf(lam, (float)kRC);
  float* sp = p.state + ((size_t)p.seq_slot[b] * p.H + h) * p.d * p.dv + e;
  float S = p.seq_pos0[b] > 0 ? *sp : 0.0f;
  const int chunks = (len + kRC - 1) / kRC;
  for (int c = 0; c < chunks; ++c) {
    float* w = p.ws + (((size_t)b * p.max_chunks + c) * p.H + h) * p.d * p.dv + e;
    const float u = *w;
    *w = S;
    const int n = min(kRC, len - c * kRC);
    S = fmaf(n == kRC ? p64 : powf(lam, (float)n), S, u);
  }
  *sp = S;
}

static size_t retention_chunk_lds(int d) {
  const int DPAD = (d + 15) / 16 * 16, DP = DPAD + 2;
  return (size_t)(2 * kRC * DP + kRC * kVS + kRC * kAS + DPAD * kVS + 66) * sizeof(float);
}

// grid (T, H): o[t][h][:] <- (unit ? o / rms(o) : o) * w[:] * act(g[t * ldg + h * dv + :]) * post
// (w: optional weight shared by the heads; o16: optional rounded copy, the operand of the out-projection's bf16
// MFMA tiles). With w_g2 ([H dv][rank], bf16 or fp32) the gate's input is the second map of a low-rank gate:
// g holds `rank` values per row and entry i's input is w_g2[i] . g.
template <bool G2F32>
__global__ void __launch_bounds__(256) head_gate_kernel(float* __restrict__ o, const float* __restrict__ g, long ldg,
                                                        int H, int dv, int unit, float eps, int act,
                                                        const float* __restrict__ w, float post,
                                                        uint16_t* __restrict__ o16, const void* __restrict__ w_g2,
                                                        int rank) {
  __shared__ float red[4];
  __shared__ float g1[512];
  const int t = blockIdx.x, h = blockIdx.y;
  float* orow = o + ((size_t)t * H + h) * dv;
  const float* grow = g + (size_t)t * ldg + (size_t)h * dv;
  if (w_g2) {
    for (int r = threadIdx.x; r < rank; r += 256) g1[r] = aop<G2F32>(g[(size_t)t * ldg + r]);
    __syncthreads();
  }
  float rstd = 1.0f;
  if (unit) {
    float ss = 0.0f;
    for (int i = threadIdx.x; i < dv; i += 256) ss = fmaf(orow[i], orow[i], ss);
    ss = block_sum_256(ss, red);
    rstd = 1.0f / sqrtf(ss / (float)dv + eps);
  }
  for (int i = threadIdx.x; i < dv; i += 256) {
    float v = orow[i] * rstd;
    if (w) v *= w[i];
    const float gin = w_g2 ? lowrank_dot<G2F32>(w_g2, (size_t)h * dv + i, g1, rank) : grow[i];
    v *= act_f(act, gin);
    if (post != 1.0f) v *= post;
    orow[i] = v;
    if (o16) o16[((size_t)t * H + h) * dv + i] = f2bf(v);
  }
}

// ------------------------------------------------------------------------------------------------ latent attention
struct LatPrepArgs {
  float* proj;  // row t: queries at q_off (head h at h * (d + dr): d unrotated, dr rotated), latent row at kv_off
  long ld;
  int q_off, kv_off;
  void* cache_c;    // [slots][S][r] bf16 or fp32
  float* cache_kr;  // [slots][S][dr]
  const float* norm_w;    // [r]
  const float* inv_freq;  // [rot_dims / 2]
  const int* slot;        // [T]
  const int* pos;         // [T]
  int H, d, dr, r, rot_dims, max_seq;
  float eps;
};

template <bool CF32>
__global__ void __launch_bounds__(256) latent_prepare_kernel(LatPrepArgs p) {
  __shared__ float red[4];
  const int t = blockIdx.x, tid = threadIdx.x;
  const int ps = p.pos[t];
  if (ps < 0 || ps >= p.max_seq) return;  // the host sizes the cache; never write out of bounds
  float* row = p.proj + (size_t)t * p.ld;
  const float* kv = row + p.kv_off;
  const size_t crow = (size_t)p.slot[t] * p.max_seq + ps;
  float ss = 0.0f;
  for (int i = tid; i < p.r; i += 256) ss = fmaf(kv[i], kv[i], ss);
  ss = block_sum_256(ss, red);
  const float rstd = 1.0f / sqrtf(ss / (float)p.r + p.eps);
  for (int i = tid; i < p.r; i += 256) {
    const float c = kv[i] * rstd * p.norm_w[i];
    if (CF32) ((float*)p.cache_c)[crow * p.r + i] = c;
    else ((uint16_t*)p.cache_c)[crow * p.r + i] = f2bf(c);
  }
  const float fpos = (float)ps;
  const int half = p.rot_dims / 2;
  float* kro = p.cache_kr + crow * p.dr;
  for (int i = tid; i < p.dr; i += 256) {
    if (i >= p.rot_dims) kro[i] = kv[p.r + i];
    else if ((i & 1) == 0) {
      float sn, cs;
      sincosf(fpos * p.inv_freq[i >> 1], &sn, &cs);
      const float u = kv[p.r + i], v = kv[p.r + i + 1];
      kro[i] = u * cs - v * sn;
      kro[i + 1] = v * cs + u * sn;
    }
  }
  for (int it = tid; it < p.H * half; it += 256) {
    const int h = it / half, i = it % half;
    float* qr = row + p.q_off + (size_t)h * (p.d + p.dr) + p.d + 2 * i;
    float sn, cs;
    sincosf(fpos * p.inv_freq[i], &sn, &cs);
    const float u = qr[0], v = qr[1];
    qr[0] = u * cs - v * sn;
    qr[1] = v * cs + u * sn;
  }
}

struct LatAttArgs {
  const float* qc;    // [T][H][r] queries mapped into the latent space
  const float* proj;  // rotated query part of head h at proj[t * ld + q_off + h * (d + dr) + d]
  long ld;
  int q_off;
  const void* cache_c;
  const float* cache_kr;
  const float* sink;  // [H] or null
  const int* slot;
  const int* pos;
  float* out;  // [T][H][r]
  int H, d, dr, r, max_seq;
  float scale;
};

// grid (T, H, splits): split z of (token, head) owns an equal share of the keys 0 .. pos; its wave w walks keys
// lo + w, lo + w + 4, ... four at a time (their loads in flight together) with an online softmax; lanes hold dims
// lane + 64 e. One split finishes in place (the sink joins the denominator); several leave (max, sum, weighted sum)
// per split in `part` [T][H][splits][r + 2] for latent_combine_kernel.
template <bool CF32, int NR>
__global__ void __launch_bounds__(256) latent_attention_kernel(LatAttArgs p, float* __restrict__ part) {
  __shared__ float sm[4], sl[4];
  extern __shared__ float sacc[];  // [4][r]
  constexpr int U = 4;
  const int t = blockIdx.x, h = blockIdx.y, z = blockIdx.z, splits = gridDim.z;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int r = p.r, dr = p.dr;
  const int last = min(p.pos[t], p.max_seq - 1);
  const int share = (last + splits) / splits;  // ceil((last + 1) / splits)
  const int lo = z * share, hi = min(last, lo + share - 1);
  const size_t base = (size_t)p.slot[t] * p.max_seq;
  const float* qc = p.qc + ((size_t)t * p.H + h) * r;
  const float* qr = p.proj + (size_t)t * p.ld + p.q_off + (size_t)h * (p.d + dr) + p.d;
  float q[NR], qrot[2], acc[NR];
#pragma unroll
  for (int e = 0; e < NR; ++e) {
    q[e] = lane + 64 * e < r ? qc[lane + 64 * e] : 0.0f;
    acc[e] = 0.0f;
  }
#pragma unroll
  for (int e = 0; e < 2; ++e) qrot[e] = lane + 64 * e < dr ? qr[lane + 64 * e] : 0.0f;
  float m = -INFINITY, l = 0.0f;
  for (int j0 = lo + wave; j0 <= hi; j0 += 4 * U) {
    float c[U][NR], dot[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int j = min(j0 + 4 * u, hi);  // a key past the end repeats the last one and gets no weight
      dot[u] = 0.0f;
#pragma unroll
      for (int e = 0; e < NR; ++e) {
        const int i = lane + 64 * e;
        c[u][e] = i < r ? (CF32 ? ((const float*)p.cache_c)[(base + j) * r + i]
                                : bf2f(((const uint16_t*)p.cache_c)[(base + j) * r + i]))
                        : 0.0f;
      }
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        const int i = lane + 64 * e;
        if (i < dr) dot[u] = fmaf(qrot[e], p.cache_kr[(base + j) * dr + i], dot[u]);
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int e = 0; e < NR; ++e) dot[u] = fmaf(q[e], c[u][e], dot[u]);
      dot[u] = wave_sum(dot[u]) * p.scale;
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (j0 + 4 * u > hi) break;
      const float mn = fmaxf(m, dot[u]);
      const float corr = expf(m - mn), w = expf(dot[u] - mn);
      l = l * corr + w;
#pragma unroll
      for (int e = 0; e < NR; ++e) acc[e] = acc[e] * corr + w * c[u][e];
      m = mn;
    }
  }
  if (lane == 0) {
    sm[wave] = m;
    sl[wave] = l;
  }
#pragma unroll
  for (int e = 0; e < NR; ++e)
    if (lane + 64 * e < r) sacc[wave * r + lane + 64 * e] = acc[e];
  __syncthreads();
  const bool fin = splits == 1;
  const float snk = (fin && p.sink) ? p.sink[h] : -INFINITY;
  const float mx = fmaxf(fmaxf(fmaxf(sm[0], sm[1]), fmaxf(sm[2], sm[3])), snk);
  float f[4], den = (fin && p.sink) ? expf(snk - mx) : 0.0f;
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    f[w] = sl[w] > 0.0f ? expf(sm[w] - mx) : 0.0f;
    den += sl[w] * f[w];
  }
  if (fin) {
    float* o = p.out + ((size_t)t * p.H + h) * r;
    for (int i = threadIdx.x; i < r; i += 256)
      o[i] = ((sacc[i] * f[0] + sacc[r + i] * f[1]) + (sacc[2 * r + i] * f[2] + sacc[3 * r + i] * f[3])) / den;
  } else {
    float* o = part + (((size_t)t * p.H + h) * splits + z) * (r + 2);
    if (threadIdx.x == 0) {
      o[0] = mx;
      o[1] = den;
    }
    for (int i = threadIdx.x; i < r; i += 256)
      o[2 + i] = (sacc[i] * f[0] + sacc[r + i] * f[1]) + (sacc[2 * r + i] * f[2] + sacc[3 * r + i] * f[3]);
  }
}

// The same walk with 16-byte loads: lane holds the 8 consecutive latent dims 8 lane .. 8 lane + 7 (r % 8 == 0,
// r <= 512), so a cached row is one load instruction per wave instead of r / 64.
template <bool CF32>
__global__ void __launch_bounds__(256) latent_attention_vec_kernel(LatAttArgs p, float* __restrict__ part) {
  __shared__ float sm[4], sl[4];
  extern __shared__ float sacc[];  // [4][r]
  constexpr int U = 4;
  const int t = blockIdx.x, h = blockIdx.y, z = blockIdx.z, splits = gridDim.z;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int r = p.r, dr = p.dr;
  const int last = min(p.pos[t], p.max_seq - 1);
  const int share = (last + splits) / splits;
  const int lo = z * share, hi = min(last, lo + share - 1);
  const size_t base = (size_t)p.slot[t] * p.max_seq;
  const bool live = 8 * lane < r;
  const float* qc = p.qc + ((size_t)t * p.H + h) * r + 8 * lane;
  const float* qr = p.proj + (size_t)t * p.ld + p.q_off + (size_t)h * (p.d + dr) + p.d;
  float q[8], qrot[2], acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    q[e] = live ? qc[e] : 0.0f;
    acc[e] = 0.0f;
  }
#pragma unroll
  for (int e = 0; e < 2; ++e) qrot[e] = lane + 64 * e < dr ? qr[lane + 64 * e] : 0.0f;
  float m = -INFINITY, l = 0.0f;
  for (int j0 = lo + wave; j0 <= hi; j0 += 4 * U) {
    float c[U][8], dot[U];
#pragma unroll
    for (int u = 0; u < U; ++u) {
      const int j = min(j0 + 4 * u, hi);
      if (!live) {
#pragma unroll
        for (int e = 0; e < 8; ++e) c[u][e] = 0.0f;
      } else if (CF32) {
        const float4 a = *(const float4*)((const float*)p.cache_c + (base + j) * r + 8 * lane);
        const float4 b = *(const float4*)((const float*)p.cache_c + (base + j) * r + 8 * lane + 4);
        c[u][0] = a.x; c[u][1] = a.y; c[u][2] = a.z; c[u][3] = a.w;
        c[u][4] = b.x; c[u][5] = b.y; c[u][6] = b.z; c[u][7] = b.w;
      } else {
        const uint4 w = *(const uint4*)((const uint16_t*)p.cache_c + (base + j) * r + 8 * lane);
        c[u][0] = bflo(w.x); c[u][1] = bfhi(w.x); c[u][2] = bflo(w.y); c[u][3] = bfhi(w.y);
        c[u][4] = bflo(w.z); c[u][5] = bfhi(w.z); c[u][6] = bflo(w.w); c[u][7] = bfhi(w.w);
      }
      dot[u] = 0.0f;
#pragma unroll
      for (int e = 0; e < 2; ++e) {
        const int i = lane + 64 * e;
        if (i < dr) dot[u] = fmaf(qrot[e], p.cache_kr[(base + j) * dr + i], dot[u]);
      }
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
#pragma unroll
      for (int e = 0; e < 8; ++e) dot[u] = fmaf(q[e], c[u][e], dot[u]);
      dot[u] = wave_sum(dot[u]) * p.scale;
    }
#pragma unroll
    for (int u = 0; u < U; ++u) {
      if (j0 + 4 * u > hi) break;
      const float mn = fmaxf(m, dot[u]);
      const float corr = expf(m - mn), w = expf(dot[u] - mn);
      l = l * corr + w;
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] = acc[e] * corr + w * c[u][e];
      m = mn;
    }
  }
  if (lane == 0) {
    sm[wave] = m;
    sl[wave] = l;
  }
  if (live) {
#pragma unroll
    for (int e = 0; e < 8; ++e) sacc[wave * r + 8 * lane + e] = acc[e];
  }
  __syncthreads();
  const bool fin = splits == 1;
  const float snk = (fin && p.sink) ? p.sink[h] : -INFINITY;
  const float mx = fmaxf(fmaxf(fmaxf(sm[0], sm[1]), fmaxf(sm[2], sm[3])), snk);
  float f[4], den = (fin && p.sink) ? expf(snk - mx) : 0.0f;
#pragma unroll
  for (int w = 0; w < 4; ++w) {
    f[w] = sl[w] > 0.0f ? expf(sm[w] - mx) : 0.0f;
    den += sl[w] * f[w];
  }
  if (fin) {
    float* o = p.out + ((size_t)t * p.H + h) * r;
    for (int i = threadIdx.x; i < r; i += 256)
      o[i] = ((sacc[i] * f[0] + sacc[r + i] * f[1]) + (sacc[2 * r + i] * f[2] + sacc[3 * r + i] * f[3])) / den;
  } else {
    float* o = part + (((size_t)t * p.H + h) * splits + z) * (r + 2);
    if (threadIdx.x == 0) {
      o[0] = mx;
      o[1] = den;
    }
    for (int i = threadIdx.x; i < r; i += 256)
      o[2 + i] = (sacc[i] * f[0] + sacc[r + i] * f[1]) + (sacc[2 * r + i] * f[2] + sacc[3 * r + i] * f[3]);
  }
}

// The prompt form: 16 consecutive tokens of one sequence and one head per workgroup, key tiles of 16 cached rows
// staged in LDS as fp32, both products on v_mfma_f32_16x16x4_f32. The four waves split the score product over the
// latent / rotated dims (partial 16x16 tiles summed through LDS) and the weighted sum over the r output columns
// (NT tiles of 16 per wave); each runs the same online softmax on the summed scores. A wave keeps its share of the
// 16 queries in registers (one value per lane and score instruction), so LDS holds the key tile only and three
// workgroups fit a CU. The next key tile travels in registers while the current one is multiplied; the longest
// tiles (the sequence's last tokens) are launched first. r % 64 == 0.
struct LatTileArgs {
  LatAttArgs a;
  const int* seq_start;
  const int* seq_slot;
  const int* seq_pos0;
};

template <bool CF32, int NT>
__global__ void __launch_bounds__(256) latent_attention_tile_kernel(LatTileArgs tp) {
  extern __shared__ float lds[];
  const LatAttArgs& p = tp.a;
  const int b = blockIdx.z, h = blockIdx.y;
  const int tile = gridDim.x - 1 - blockIdx.x;
  const int t0 = tp.seq_start[b] + tile * 16, t1 = tp.seq_start[b + 1];
  if (t0 >= t1) return;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, fr = lane & 15, fk = lane >> 4;
  const int r = p.r, dr = p.dr, D = r + dr;
  const int DQ = (D + 15) / 16 * 4;             // dims per wave in the score product (multiple of 4)
  const int KP = (4 * DQ + 31) / 32 * 32 + 2;   // row stride of the Q and key tiles (conflict-free 16 x 4 reads)
  float* Kt = lds;                  // [16][KP]
  float* Sp = Kt + 16 * KP;         // [4][16][17] partial scores
  float* Pw = Sp + 4 * 16 * 17;     // [4][16][17] each wave's copy of the weights
  const int rows = min(16, t1 - t0);
  const int pos_first = tp.seq_pos0[b] + tile * 16;
  const int pos_last = min(pos_first + rows - 1, p.max_seq - 1);
  const size_t base = (size_t)tp.seq_slot[b] * p.max_seq;
  // this lane's query operands: row fr, dims wave DQ + fk + 4 i (the latent part, then the rotated part, then zeros)
  constexpr int NQ = 40;  // (512 + 128) / 16
  float qreg[NQ];
#pragma unroll
  for (int i = 0; i < NQ; ++i) {
    const int dd = wave * DQ + fk + 4 * i;
    float v = 0.0f;
    if (4 * i < DQ && fr < rows) {
      if (dd < r) v = p.qc[((size_t)(t0 + fr) * p.H + h) * r + dd];
      else if (dd < D) v = p.proj[(size_t)(t0 + fr) * p.ld + p.q_off + (size_t)h * (p.d + dr) + p.d + (dd - r)];
    }
    qreg[i] = v;
  }
  for (int i = tid; i < 16 * KP; i += 256) Kt[i] = 0.0f;  // the padding columns stay zero
  constexpr int NC = CF32 ? 8 : 4;  // 16-B loads of the latent part per thread (r <= 512)
  uint4 creg[NC];
  float kreg[8];
  const int cvec = CF32 ? r / 4 : r / 8;  // 16-B vectors per cached latent row
  // which key of a tile, and which part of its row, each of this thread's loads covers (fixed for the whole kernel:
  // no integer division inside the tile loop); key -1 marks a load this thread does not have
  int ckey[NC], coff[NC], kkey[8], koff[8];
#pragma unroll
  for (int i = 0; i < NC; ++i) {
    const int idx = tid + 256 * i;
    ckey[i] = idx < 16 * cvec ? idx / cvec : -1;
    coff[i] = (idx % cvec) * (CF32 ? 4 : 8);
  }
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int idx = tid + 256 * i;
    kkey[i] = idx < 16 * dr ? idx / dr : -1;
    koff[i] = dr ? idx % dr : 0;
  }
  auto gload = [&](int kt) {
#pragma unroll
    for (int i = 0; i < NC; ++i)
      if (ckey[i] >= 0) {
        const size_t row = base + min(kt * 16 + ckey[i], p.max_seq - 1);
        creg[i] = CF32 ? *(const uint4*)((const float*)p.cache_c + row * r + coff[i])
                       : *(const uint4*)((const uint16_t*)p.cache_c + row * r + coff[i]);
      }
#pragma unroll
    for (int i = 0; i < 8; ++i)
      if (kkey[i] >= 0) kreg[i] = p.cache_kr[(base + min(kt * 16 + kkey[i], p.max_seq - 1)) * dr + koff[i]];
  };
  auto lstore = [&]() {
#pragma unroll
    for (int i = 0; i < NC; ++i)
      if (ckey[i] >= 0) {
        float* dst = Kt + ckey[i] * KP + coff[i];
        const uint32_t w[4] = {creg[i].x, creg[i].y, creg[i].z, creg[i].w};
        if (CF32) {  // (rows are 8-byte aligned: KP is even)
          ((float2*)dst)[0] = make_float2(__uint_as_float(w[0]), __uint_as_float(w[1]));
          ((float2*)dst)[1] = make_float2(__uint_as_float(w[2]), __uint_as_float(w[3]));
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) ((float2*)dst)[e] = make_float2(bflo(w[e]), bfhi(w[e]));
        }
      }
#pragma unroll
    for (int i = 0; i < 8; ++i)
      if (kkey[i] >= 0) Kt[kkey[i] * KP + r + koff[i]] = kreg[i];
  };
  f32x4_t o[NT];
#pragma unroll
  for (int c = 0; c < NT; ++c) o[c] = f32x4_t{0.f, 0.f, 0.f, 0.f};
  float m[4], l[4];
  int prow[4];
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    m[j] = -INFINITY;
    l[j] = 0.0f;
    prow[j] = min(pos_first + fk * 4 + j, pos_last);  // rows past the sequence's end repeat the last (not stored)
  }
  const int nkt = pos_last / 16 + 1;
  gload(0);
  __syncthreads();  // Kt's zero padding
  for (int kt = 0; kt < nkt; ++kt) {
    lstore();
    __syncthreads();
    if (kt + 1 < nkt) gload(kt + 1);
    // partial scores over this wave's dims
    // (four independent chains, so that LDS reads and matrix instructions overlap)
    f32x4_t sacc = {0.f, 0.f, 0.f, 0.f}, s1 = sacc, s2 = sacc, s3 = sacc;
    const float* kb = Kt + fr * KP + wave * DQ + fk;
#pragma unroll
    for (int i = 0; i < NQ; i += 4) {
      if (4 * i >= DQ) break;
      sacc = __builtin_amdgcn_mfma_f32_16x16x4f32(qreg[i], kb[4 * i], sacc, 0, 0, 0);
      if (4 * (i + 1) < DQ) s1 = __builtin_amdgcn_mfma_f32_16x16x4f32(qreg[i + 1], kb[4 * i + 4], s1, 0, 0, 0);
      if (4 * (i + 2) < DQ) s2 = __builtin_amdgcn_mfma_f32_16x16x4f32(qreg[i + 2], kb[4 * i + 8], s2, 0, 0, 0);
      if (4 * (i + 3) < DQ) s3 = __builtin_amdgcn_mfma_f32_16x16x4f32(qreg[i + 3], kb[4 * i + 12], s3, 0, 0, 0);
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) sacc[j] = (sacc[j] + s1[j]) + (s2[j] + s3[j]);
#pragma unroll
    for (int j = 0; j < 4; ++j) Sp[(wave * 16 + fk * 4 + j) * 17 + fr] = sacc[j];
    __syncthreads();
    float pj[4], corr[4];
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const int row = fk * 4 + j;
      float sc = ((Sp[row * 17 + fr] + Sp[(16 + row) * 17 + fr]) + (Sp[(32 + row) * 17 + fr] + Sp[(48 + row) * 17 + fr])) *
                 p.scale;
      if (kt * 16 + fr > prow[j]) sc = -INFINITY;
      float mx = sc;
#pragma unroll
      for (int x = 8; x > 0; x >>= 1) mx = fmaxf(mx, __shfl_xor(mx, x));
      const float mn = fmaxf(m[j], mx);
      const float w = expf(sc - mn);
      float sum = w;
#pragma unroll
      for (int x = 8; x > 0; x >>= 1) sum += __shfl_xor(sum, x);
      corr[j] = expf(m[j] - mn);
      l[j] = l[j] * corr[j] + sum;
      m[j] = mn;
      pj[j] = w;
      Pw[(wave * 16 + row) * 17 + fr] = w;
    }
#pragma unroll
    for (int c = 0; c < NT; ++c)
#pragma unroll
      for (int j = 0; j < 4; ++j) o[c][j] *= corr[j];
    __syncthreads();
    // weighted sum of the cached latents: this wave's NT column tiles
    const float* pa = Pw + (wave * 16 + fr) * 17 + fk;
#pragma unroll
    for (int k = 0; k < 16; k += 4) {
      const float a = pa[k];
      const float* vb = Kt + (k + fk) * KP + wave * NT * 16 + fr;
#pragma unroll
      for (int c = 0; c < NT; ++c) o[c] = __builtin_amdgcn_mfma_f32_16x16x4f32(a, vb[c * 16], o[c], 0, 0, 0);
    }
    __syncthreads();  // Kt and Sp are free for the next tile
  }
  const float snk = p.sink ? p.sink[h] : -INFINITY;
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    const int row = fk * 4 + j;
    if (row >= rows) continue;
    const float mx = fmaxf(m[j], snk);
    const float f = expf(m[j] - mx);
    const float den = l[j] * f + (p.sink ? expf(snk - mx) : 0.0f);
    float* orow = p.out + ((size_t)(t0 + row) * p.H + h) * r + wave * NT * 16 + fr;
#pragma unroll
    for (int c = 0; c < NT; ++c) orow[c * 16] = o[c][j] * f / den;
  }
}

// grid (T, H): merges the splits' partial softmaxes and the sink
__global__ void __launch_bounds__(256) latent_combine_kernel(const float* __restrict__ part, const float* __restrict__ sink,
                                                             float* __restrict__ out, int H, int r, int splits) {
  const int t = blockIdx.x, h = blockIdx.y;
  const float* pp = part + ((size_t)t * H + h) * splits * (r + 2);
  const float snk = sink ? sink[h] : -INFINITY;
  float mx = snk;
  for (int z = 0; z < splits; ++z)
    if (pp[(size_t)z * (r + 2) + 1] > 0.0f) mx = fmaxf(mx, pp[(size_t)z * (r + 2)]);
  float den = sink ? expf(snk - mx) : 0.0f;
  for (int z = 0; z < splits; ++z) {
    const float lz = pp[(size_t)z * (r + 2) + 1];
    if (lz > 0.0f) den += lz * expf(pp[(size_t)z * (r + 2)] - mx);
  }
  for (int i = threadIdx.x; i < r; i += 256) {
    float a = 0.0f;
    for (int z = 0; z < splits; ++z) {
      const float lz = pp[(size_t)z * (r + 2) + 1];
      if (lz > 0.0f) a += pp[(size_t)z * (r + 2) + 2 + i] * expf(pp[(size_t)z * (r + 2)] - mx);
    }
    out[((size_t)t * H + h) * r + i] = a / den;
  }
}

}  // namespace lgs

extern "C" int lgs_retention(float* q, float* k, float* v, long ld, float* state, const float* decay,
                             const float* inv_freq, const int* seq_start, const int* seq_slot, const int* seq_pos0,
                             float* out, int B, int H, int d, int dv, int rot_dims, float k_scale, int chunked,
                             float* ws, int max_chunks, int T_rows, const int* pos, int act, hipStream_t stream) {
  LGA_CHECK_ARG(act >= 0 && act <= lgs::kActSigmoid, "lgs_retention: unknown activation");
  LGA_CHECK_ARG(q && k && v && state && decay && seq_start && seq_slot && seq_pos0 && out, "lgs_retention: null pointer");
  LGA_CHECK_ARG(B > 0 && H > 0 && H <= 65535 && d > 0 && d <= 512 && dv > 0, "lgs_retention: head dim must be in [1, 512]");
  LGA_CHECK_ARG(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= d && (rot_dims == 0 || inv_freq),
                "lgs_retention: bad rotary dims");
  LGA_CHECK_ARG(!ws || max_chunks > 0, "lgs_retention: a workspace needs the longest sequence's chunk count");
  lgs::RetArgs p{q, k, v, ld, state, decay, inv_freq, seq_start, seq_slot, seq_pos0, out, H, d, dv, rot_dims, k_scale,
                 ws, max_chunks, act};
  const dim3 grid(B, H, (dv + 63) / 64);
  if (chunked && d <= 128) {  // a prompt: chunks of 64 tokens as fp32 matrix products
    LGA_CHECK_ARG(T_rows > 0 && pos, "lgs_retention: the prompt form needs the row count and the rows' positions");
    if (rot_dims > 0 || k_scale != 1.0f || act != lgs::kActNone) {
      lgs::retention_rope_kernel<<<dim3(T_rows, H), 64, 0, stream>>>(q, k, v, ld, inv_freq, pos, d, dv, rot_dims, k_scale,
                                                                     act);
      p.act = lgs::kActNone;  // applied in place: the chunk kernels read the activated values
    }
    const size_t lds = lgs::retention_chunk_lds(d);
    const bool side = ws && (long)B * H * ((dv + 63) / 64) < lga::num_cu() && (long)B * max_chunks <= 1 << 24;
    const dim3 cgrid(side ? B * max_chunks : B, H, (dv + 63) / 64);
#define LGS_RET(MODE, DPC, G)                                                                                          \
  do {                                                                                                                 \
    if (hipFuncSetAttribute((const void*)lgs::retention_chunk_kernel<MODE, DPC>,                                       \
                            hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) {                     \
      lga_set_error("lgs_retention: cannot reserve the chunk kernel's LDS");                                           \
      return (int)hipErrorInvalidValue;                                                                                \
    }                                                                                                                  \
    lgs::retention_chunk_kernel<MODE, DPC><<<G, 256, lds, stream>>>(p);                                                \
  } while (0)
#define LGS_RET_D(MODE, G)              \
  do {                                  \
    if (d == 128) LGS_RET(MODE, 128, G); \
    else if (d == 64) LGS_RET(MODE, 64, G); \
    else LGS_RET(MODE, 0, G);           \
  } while (0)
    if (side) {  // few sequences and heads: the chunks side by side
      LGS_RET_D(1, cgrid);
      lgs::retention_carry_kernel<<<dim3(B, H, (d * dv + 255) / 256), 256, 0, stream>>>(p);
      LGS_RET_D(2, cgrid);
    } else {
      LGS_RET_D(0, cgrid);
    }
#undef LGS_RET_D
#undef LGS_RET
    LGA_LAUNCH_RETURN();
  }
  if (d <= 64) lgs::retention_scan_kernel<16><<<grid, 256, 0, stream>>>(p);
  else if (d <= 128) lgs::retention_scan_kernel<32><<<grid, 256, 0, stream>>>(p);
  else if (d <= 256) lgs::retention_scan_kernel<64><<<grid, 256, 0, stream>>>(p);
  else lgs::retention_scan_kernel<128><<<grid, 256, 0, stream>>>(p);
  LGA_LAUNCH_RETURN();
}

extern "C" int lgs_head_gate(float* o, const float* g, long ldg, int T, int H, int dv, int unit_norm, float eps,
                             int act, const float* weight, float post, void* o_bf16, const void* w_g2, int rank,
                             int g2_f32, hipStream_t stream) {
  LGA_CHECK_ARG(o && g && T > 0 && H > 0 && H <= 65535 && dv > 0 && (!w_g2 || (rank > 0 && rank <= 512)),
                "lgs_head_gate: bad arguments (inner size of a low-rank gate 1..512)");
  if (g2_f32)
    lgs::head_gate_kernel<true><<<dim3(T, H), 256, 0, stream>>>(o, g, ldg, H, dv, unit_norm, eps, act, weight, post,
                                                                (uint16_t*)o_bf16, w_g2, rank);
  else
    lgs::head_gate_kernel<false><<<dim3(T, H), 256, 0, stream>>>(o, g, ldg, H, dv, unit_norm, eps, act, weight, post,
                                                                 (uint16_t*)o_bf16, w_g2, rank);
  LGA_LAUNCH_RETURN();
}

extern "C" int lgs_latent_prepare(float* proj, long ld, int q_off, int kv_off, void* cache_c, int cache_f32,
                                  float* cache_kr, const float* norm_w, const float* inv_freq, const int* slot,
                                  const int* pos, int T, int H, int d, int dr, int r, int rot_dims, int max_seq,
                                  float eps, hipStream_t stream) {
  LGA_CHECK_ARG(proj && cache_c && cache_kr && norm_w && slot && pos, "lgs_latent_prepare: null pointer");
  LGA_CHECK_ARG(T > 0 && H > 0 && d >= 0 && dr >= 0 && r > 0 && max_seq > 0, "lgs_latent_prepare: bad sizes");
  LGA_CHECK_ARG(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= dr && (rot_dims == 0 || inv_freq),
                "lgs_latent_prepare: bad rotary dims");
  lgs::LatPrepArgs p{proj, ld, q_off, kv_off, cache_c, cache_kr, norm_w, inv_freq, slot, pos,
                     H, d, dr, r, rot_dims, max_seq, eps};
  if (cache_f32) lgs::latent_prepare_kernel<true><<<T, 256, 0, stream>>>(p);
  else lgs::latent_prepare_kernel<false><<<T, 256, 0, stream>>>(p);
  LGA_LAUNCH_RETURN();
}

extern "C" int lgs_latent_attention(const float* qc, const float* proj, long ld, int q_off, const void* cache_c,
                                    int cache_f32, const float* cache_kr, const float* sink, const int* slot,
                                    const int* pos, float* out, int T, int H, int d, int dr, int r, int max_seq,
                                    float scale, int splits, float* part, hipStream_t stream) {
  LGA_CHECK_ARG(qc && proj && cache_c && cache_kr && slot && pos && out, "lgs_latent_attention: null pointer");
  LGA_CHECK_ARG(T > 0 && H > 0 && H <= 65535 && r > 0 && r <= 1024 && dr >= 0 && dr <= 128 && max_seq > 0,
                "lgs_latent_attention: latent rank must be <= 1024 and the rotated part <= 128");
  LGA_CHECK_ARG(splits >= 1 && splits <= 256 && (splits == 1 || part),
                "lgs_latent_attention: splits in [1, 256], with a workspace of T * H * splits * (r + 2) floats");
  lgs::LatAttArgs p{qc, proj, ld, q_off, cache_c, cache_kr, sink, slot, pos, out, H, d, dr, r, max_seq, scale};
  const dim3 grid(T, H, splits);
  const size_t lds = (size_t)4 * r * sizeof(float);
#define LGS_LAT(NR)                                                                                    \
  do {                                                                                                 \
    if (cache_f32) lgs::latent_attention_kernel<true, NR><<<grid, 256, lds, stream>>>(p, part);        \
    else lgs::latent_attention_kernel<false, NR><<<grid, 256, lds, stream>>>(p, part);                 \
  } while (0)
  if (r % 8 == 0 && r <= 512 && (uintptr_t)cache_c % 16 == 0 && (uintptr_t)qc % 16 == 0) {  // 16-byte row loads
    if (cache_f32) lgs::latent_attention_vec_kernel<true><<<grid, 256, lds, stream>>>(p, part);
    else lgs::latent_attention_vec_kernel<false><<<grid, 256, lds, stream>>>(p, part);
  } else if (r <= 128) LGS_LAT(2);
  else if (r <= 256) LGS_LAT(4);
  else if (r <= 512) LGS_LAT(8);
  else LGS_LAT(16);
#undef LGS_LAT
  if (splits > 1) lgs::latent_combine_kernel<<<dim3(T, H), 256, 0, stream>>>(part, sink, out, H, r, splits);
  LGA_LAUNCH_RETURN();
}

extern "C" int lgs_latent_attention_tiles(const float* qc, const float* proj, long ld, int q_off, const void* cache_c,
                                          int cache_f32, const float* cache_kr, const float* sink,
                                          const int* seq_start, const int* seq_slot, const int* seq_pos0, float* out,
                                          int B, int max_len, int H, int d, int dr, int r, int max_seq, float scale,
                                          hipStream_t stream) {
  LGA_CHECK_ARG(qc && proj && cache_c && cache_kr && seq_start && seq_slot && seq_pos0 && out,
                "lgs_latent_attention_tiles: null pointer");
  LGA_CHECK_ARG(B > 0 && B <= 65535 && max_len > 0 && H > 0 && H <= 65535 && max_seq > 0,
                "lgs_latent_attention_tiles: bad sizes");
  LGA_CHECK_ARG(r > 0 && r <= 512 && r % 64 == 0 && dr >= 0 && dr <= 128,
                "lgs_latent_attention_tiles: latent rank must be a multiple of 64 up to 512, the rotated part <= 128");
  lgs::LatTileArgs p{{qc, proj, ld, q_off, cache_c, cache_kr, sink, nullptr, nullptr, out, H, d, dr, r, max_seq, scale},
                     seq_start, seq_slot, seq_pos0};
  const int D = r + dr, DQ = (D + 15) / 16 * 4, KP = (4 * DQ + 31) / 32 * 32 + 2;
  const size_t lds = (size_t)(16 * KP + 2 * 4 * 16 * 17) * sizeof(float);
  const dim3 grid((max_len + 15) / 16, H, B);
  const void* fn = nullptr;
#define LGS_TILE(NT)                                                                                   \
  case NT:                                                                                             \
    fn = cache_f32 ? (const void*)lgs::latent_attention_tile_kernel<true, NT>                          \
                   : (const void*)lgs::latent_attention_tile_kernel<false, NT>;                        \
    break;
  switch (r / 64) {
    LGS_TILE(1) LGS_TILE(2) LGS_TILE(3) LGS_TILE(4) LGS_TILE(5) LGS_TILE(6) LGS_TILE(7) LGS_TILE(8)
  }
#undef LGS_TILE
  if (lds > 48 * 1024 &&
      hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds) != hipSuccess) {
    lga_set_error("lgs_latent_attention_tiles: cannot reserve the kernel's LDS");
    return (int)hipErrorInvalidValue;
  }
  void* args[] = {(void*)&p};
  hipError_t e = hipLaunchKernel(fn, grid, dim3(256), args, lds, stream);
  if (e != hipSuccess) {
    lga_set_error(hipGetErrorString(e));
    return (int)e;
  }
  LGA_LAUNCH_RETURN();
}
