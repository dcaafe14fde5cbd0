// Softmax attention of the layered models over cached keys and values: scores, weights and sums in fp32.
//
// Differential attention (two maps per head): a query head carries two maps (q1, q2), a key head two key maps
// (k1, k2); both maps are softmax attentions over the same values, combined as o = a1 - lambda a2, divided by the
// head's root mean square and scaled. Sink attention (one map per head): a plain softmax attention whose normaliser
// also holds exp(sink) of the head. In both, query head h reads key/value head h / (H / G); scores are
// (q . k) * scale, optionally soft-capped (cap * tanh(s / cap)); a query at position i sees keys lo(i) <= j <= i with
// lo(i) = i - i % chunk for a chunked mask (chunks are aligned to the sequence's position 0) and 0 without one.
//
//   lgs_diffattn_prepare  per token: rotary (interleaved pairs 2i, 2i + 1 of the first rot_dims dims of every map)
//                         on the queries in place and on the keys on their way into the cache; values into the cache.
//                         Without key / value columns (a layer that reads another layer's cache) only the queries.
//   lgs_normattn_prepare  per token: queries optionally divided by their root mean square (optionally weighted),
//                         optionally rotated (pairs i, i + rot_dims / 2) and multiplied by a temperature that grows
//                         with the position, in place; keys normed and rotated alike on their way into the cache;
//                         values (own columns, or the keys as projected) into the cache.
//   lgs_diffattn,         QT consecutive queries of one sequence and one head per workgroup (8 with two maps, 16 with
//   lgs_sinkattn          one) against key tiles of 256 cached rows: a thread per key for the scores, an online
//                         softmax per (query, map), a thread per value column for the weighted sums. One query per
//                         workgroup (decode) can spread its keys over several workgroups, merged by a second launch.
#include "seq_common.h"

namespace lgs {

struct AttnPrepArgs {
  float* proj;
  long ld;
  int q_off, k_off, v_off;  // k_off < 0: queries only
  void* cache_k;            // [slots][S][G][2 d]
  void* cache_v;            // [slots][S][G][dv]
  const float* inv_freq;    // [rot_dims / 2]
  const int *slot, *pos;
  int H, G, d, dv, rot_dims, S;
};

template <bool CF32>
__device__ __forceinline__ void cstore(void* c, size_t i, float v) {
  if (CF32) ((float*)c)[i] = v;
  else ((uint16_t*)c)[i] = f2bf(v);
}
template <bool CF32>
__device__ __forceinline__ float cload(const void* c, size_t i) {
  return CF32 ? ((const float*)c)[i] : bf2f(((const uint16_t*)c)[i]);
}

// grid (T): threads walk (vector, pair) items: 2 H query maps, then 2 G key maps, then the value columns
template <bool CF32>
__global__ void __launch_bounds__(256) diffattn_prepare_kernel(AttnPrepArgs p) {
  const size_t t = blockIdx.x;
  const int pos = p.pos[t];
  float* row = p.proj + t * p.ld;
  const int d = p.d, half = d / 2 + (d & 1), rp = p.rot_dims / 2;
  const int nq = 2 * p.H * half, nk = p.k_off >= 0 ? 2 * p.G * half : 0;
  const size_t crow = ((size_t)p.slot[t] * p.S + pos) * p.G;
  for (int it = threadIdx.x; it < nq + nk; it += 256) {
    const bool isk = it >= nq;
    const int e = isk ? it - nq : it;
    const int vec = e / half, i = e % half;
    float* src = row + (isk ? p.k_off : p.q_off) + vec * d + 2 * i;
    const bool pair = 2 * i + 1 < d;
    float u = src[0], v = pair ? src[1] : 0.0f;
    if (i < rp) {
      float sn, cs;
      sincosf((float)pos * p.inv_freq[i], &sn, &cs);
      const float nu = u * cs - v * sn, nv = v * cs + u * sn;
      u = nu;
      v = nv;
    }
    if (isk) {
      const size_t at = crow * 2 * d + (size_t)vec * d + 2 * i;
      cstore<CF32>(p.cache_k, at, u);
      if (pair) cstore<CF32>(p.cache_k, at + 1, v);
    } else {
      src[0] = u;
      if (pair) src[1] = v;
    }
  }
  if (p.k_off >= 0) {
    const int nv = p.G * p.dv;
    for (int i = threadIdx.x; i < nv; i += 256) cstore<CF32>(p.cache_v, crow * p.dv + i, row[p.v_off + i]);
  }
}

struct NormPrepArgs {
  float* proj;
  long ld;
  int q_off, k_off, v_off;
  void* cache_k;  // [slots][S][G][d]
  void* cache_v;  // [slots][S][G][dv]
  const int *slot, *pos;
  int H, G, d, dv, S, temp_every;
  float eps, temp_coef;
  int norm;                // 0: q and k as projected; 1: divided by their root mean square
  const float *q_w, *k_w;  // optional weights [d] of the two norms, shared by the heads
  const float* inv_freq;   // [rot_dims / 2]: rotary positions on pairs (i, i + rot_dims / 2) after the norm
  int rot_dims;
};

// grid (T): wave w takes the vectors w, w + 4, ... of the H query heads (normed, rotated and multiplied by the
// position's query temperature, in place) and of the G key heads (normed and rotated on their way into the cache);
// then all threads copy the values into the cache. The value columns may be the key columns themselves (values = the
// keys as projected): the keys are never changed in place.
template <bool CF32>
__global__ void __launch_bounds__(256) normattn_prepare_kernel(NormPrepArgs p) {
  const size_t t = blockIdx.x;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int pos = p.pos[t], d = p.d, half = p.rot_dims / 2;
  if (pos < 0 || pos >= p.S) return;  // the host sizes the cache; never write out of bounds
  float* row = p.proj + t * p.ld;
  const size_t crow = ((size_t)p.slot[t] * p.S + pos) * p.G;
  const float temp = p.temp_every > 0 ? 1.0f + p.temp_coef * logf((float)((pos + 1) / p.temp_every + 1)) : 1.0f;
  const float fpos = (float)pos;
  for (int vec = wave; vec < p.H + p.G; vec += 4) {
    const bool isk = vec >= p.H;
    float* x = row + (isk ? p.k_off + (size_t)(vec - p.H) * d : p.q_off + (size_t)vec * d);
    const float* w = isk ? p.k_w : p.q_w;
    float s = isk ? 1.0f : temp;  // the norm's factor and the query temperature as one number
    if (p.norm) {
      float ss = 0.0f;
      for (int i = lane; i < d; i += 64) ss = fmaf(x[i], x[i], ss);
      ss = wave_sum(ss);
      s = s / sqrtf(ss / (float)d + p.eps);
    }
    const size_t kat = (crow + (vec - p.H)) * d;
    for (int i = lane; i < half; i += 64) {  // a lane owns both members of a rotated pair
      float u = x[i] * s, v = x[i + half] * s;
      if (w) u *= w[i], v *= w[i + half];
      float sn, cs;
      sincosf(fpos * p.inv_freq[i], &sn, &cs);
      const float a = u * cs - v * sn, b = v * cs + u * sn;
      if (isk) {
        cstore<CF32>(p.cache_k, kat + i, a);
        cstore<CF32>(p.cache_k, kat + i + half, b);
      } else {
        x[i] = a;
        x[i + half] = b;
      }
    }
    for (int i = p.rot_dims + lane; i < d; i += 64) {
      float u = x[i] * s;
      if (w) u *= w[i];
      if (isk) cstore<CF32>(p.cache_k, kat + i, u);
      else x[i] = u;
    }
  }
  __syncthreads();
  const int nv = p.G * p.dv;
  for (int i = threadIdx.x; i < nv; i += 256) cstore<CF32>(p.cache_v, crow * p.dv + i, row[p.v_off + i]);
}

struct AttnArgs {
  const float* q;  // prepared queries at q + row * ld + h * MAPS d
  long ld;
  const void* cache_k;
  const void* cache_v;
  const int *seq_start, *seq_slot, *seq_pos0;
  float* out;       // [T][H * dv]
  uint16_t* out16;  // optional bf16 copy
  float* part;      // splits > 1: [T][H][splits][MAPS (2 + dv)]
  int H, G, d, dv, S, chunk, tiles;
  float scale, cap, lambda, eps, post;
  const float* sink;  // one map: exp(sink[h]) joins the softmax normaliser (NULL: no sink)
  const float* gate;  // one map: the head's output is multiplied by sigmoid(gate[row * ldg + h]) (NULL: not)
  long ldg;
};

constexpr int kKeyTile = 256;
// row stride of the score / weight tile in LDS, [key][(query, map)]: a key's weights for all queries and maps lie
// side by side, so the value phase fetches them with 16-byte reads
template <int NR>
constexpr int score_stride() { return NR <= 2 ? 4 : NR + 4; }

// two maps: o = a1 / l1 - lambda a2 / l2 over the head, unit RMS, times post. Called by all 256 threads; thread
// c < dv owns column c (dv <= 256).
__device__ __forceinline__ void diff_finish(float a1, float a2, float l1, float l2, const AttnArgs& p, size_t row, int h,
                                            float* red) {
  const int c = threadIdx.x;
  const float o = c < p.dv ? a1 / l1 - p.lambda * (a2 / l2) : 0.0f;
  const float ss = block_sum_256(o * o, red);
  const float v = o / sqrtf(ss / (float)p.dv + p.eps) * p.post;
  if (c < p.dv) {
    const size_t at = row * p.H * p.dv + (size_t)h * p.dv + c;
    p.out[at] = v;
    if (p.out16) p.out16[at] = f2bf(v);
  }
}

// one map: o = a / (l + exp(sink - m)) times post, with a and l relative to the running maximum m
__device__ __forceinline__ void sink_finish(float a, float m, float l, const AttnArgs& p, size_t row, int h) {
  const int c = threadIdx.x;
  float den = l, num = a;
  if (p.sink) {
    const float s = p.sink[h], top = fmaxf(m, s);
    const float w = m == -INFINITY ? 0.0f : expf(m - top);
    den = l * w + expf(s - top);
    num = a * w;
  }
  if (c < p.dv) {
    float v = num / den * p.post;
    if (p.gate) v *= sigmoid_f(p.gate[row * p.ldg + h]);
    const size_t at = row * p.H * p.dv + (size_t)h * p.dv + c;
    p.out[at] = v;
    if (p.out16) p.out16[at] = f2bf(v);
  }
}

// grid (B * tiles, H, splits). MAPS maps per head (2: differential attention, 1: plain softmax attention with an
// optional sink). LDS: queries [QT][MAPS d], scores / weights [256][QT MAPS + 4], per (query, map) the running
// maximum, normaliser and the rescale of the current tile, and the cross-subset sums of the value phase.
template <int QT, int MAPS, bool CF32>
__global__ void __launch_bounds__(256) diffattn_kernel(AttnArgs p) {
  extern __shared__ float lds[];
  __shared__ float red[4];
  constexpr int NR = QT * MAPS;  // (query, map) rows
  const int d = p.d, dv = p.dv, d2 = MAPS * d;
  float* qs = lds;                       // [QT][d2]
  constexpr int SCS = score_stride<NR>();
  float* sc = qs + QT * d2;              // [kKeyTile][SCS]: scores, then weights, of key x (query, map)
  float* mrow = sc + kKeyTile * SCS;     // [NR] running maximum
  float* lrow = mrow + NR;               // [NR] running normaliser
  float* arow = lrow + NR;               // [NR] rescale of what was summed before this tile
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int b = blockIdx.x / p.tiles, tile = blockIdx.x % p.tiles;
  const int h = blockIdx.y, g = h / (p.H / p.G);
  const int r0 = p.seq_start[b] + tile * QT;
  const int rend = p.seq_start[b + 1];
  if (r0 >= rend) return;
  const int nq = min(QT, rend - r0);
  const int pos_first = p.seq_pos0[b] + tile * QT, pos_last = pos_first + nq - 1;
  const size_t slot = p.seq_slot[b];
  const int chunk = p.chunk;
  int lo = chunk > 0 ? pos_first - pos_first % chunk : 0, hi = pos_last + 1;
  if (gridDim.z > 1) {  // (QT == 1) an equal share of the keys, in whole numbers
    const int n = hi - lo, per = (n + gridDim.z - 1) / gridDim.z;
    lo += blockIdx.z * per;
    hi = min(hi, lo + per);
  }
  for (int i = tid; i < nq * d2; i += 256) qs[i] = p.q[(size_t)(r0 + i / d2) * p.ld + (size_t)h * d2 + i % d2];
  if (tid < NR) {
    mrow[tid] = -INFINITY;
    lrow[tid] = 0.0f;
  }
  // value phase: thread owns column `col` and every KS-th key of a tile, starting at `ks`
  int ncol = 64;
  while (ncol < dv) ncol <<= 1;  // dv <= 256
  const int KS = 256 / ncol, col = tid % ncol, ks = tid / ncol;
  float acc[QT][MAPS];
#pragma unroll
  for (int i = 0; i < QT; ++i)
#pragma unroll
    for (int m = 0; m < MAPS; ++m) acc[i][m] = 0.0f;
  __syncthreads();

  for (int k0 = lo; k0 < hi; k0 += kKeyTile) {
    const int nk = min(kKeyTile, hi - k0);
    // ---- scores of key k0 + tid against every query and map
    {
      float s[QT][MAPS];
#pragma unroll
      for (int i = 0; i < QT; ++i)
#pragma unroll
        for (int m = 0; m < MAPS; ++m) s[i][m] = 0.0f;
      if (tid < nk) {
        const size_t kr = ((slot * p.S + k0 + tid) * p.G + g) * d2;
        if ((d & 3) == 0) {
#pragma unroll
          for (int m = 0; m < MAPS; ++m)
            for (int e = 0; e < d; e += 4) {
              float kv[4];
              if (CF32) {
                const float4 t4 = *(const float4*)((const float*)p.cache_k + kr + m * d + e);
                kv[0] = t4.x, kv[1] = t4.y, kv[2] = t4.z, kv[3] = t4.w;
              } else {
                const uint2 t2 = *(const uint2*)((const uint16_t*)p.cache_k + kr + m * d + e);
                kv[0] = bflo(t2.x), kv[1] = bfhi(t2.x), kv[2] = bflo(t2.y), kv[3] = bfhi(t2.y);
              }
#pragma unroll
              for (int i = 0; i < QT; ++i) {
                const float4 q4 = *(const float4*)(qs + i * d2 + m * d + e);
                s[i][m] = fmaf(q4.x, kv[0], s[i][m]);
                s[i][m] = fmaf(q4.y, kv[1], s[i][m]);
                s[i][m] = fmaf(q4.z, kv[2], s[i][m]);
                s[i][m] = fmaf(q4.w, kv[3], s[i][m]);
              }
            }
        } else {
#pragma unroll
          for (int m = 0; m < MAPS; ++m)
            for (int e = 0; e < d; ++e) {
              const float kv = cload<CF32>(p.cache_k, kr + m * d + e);
#pragma unroll
              for (int i = 0; i < QT; ++i) s[i][m] = fmaf(qs[i * d2 + m * d + e], kv, s[i][m]);
            }
        }
      }
      const int kpos = k0 + tid;
#pragma unroll
      for (int i = 0; i < QT; ++i) {
        const int qpos = pos_first + i;
        const int qlo = chunk > 0 ? qpos - qpos % chunk : 0;
        const bool see = tid < nk && i < nq && kpos <= qpos && kpos >= qlo;
#pragma unroll
        for (int m = 0; m < MAPS; ++m) {
          float v = s[i][m] * p.scale;
          if (p.cap > 0.0f) v = p.cap * tanhf(v / p.cap);
          sc[tid * SCS + MAPS * i + m] = see ? v : -INFINITY;
        }
      }
    }
    __syncthreads();
    // ---- online softmax: wave w owns rows w, w + 4, ... of the (query, map) rows
    for (int r = wave; r < NR; r += 4) {
      float* srow = sc + r;
      float v[4], mx = -INFINITY;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        v[e] = srow[(lane + 64 * e) * SCS];
        mx = fmaxf(mx, v[e]);
      }
      mx = wave_max(mx);
      const float mo = mrow[r], mn = fmaxf(mo, mx);
      float sum = 0.0f;
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        const float w = mn == -INFINITY ? 0.0f : expf(v[e] - mn);  // (a masked key: exp(-inf) = 0)
        srow[(lane + 64 * e) * SCS] = w;
        sum += w;
      }
      sum = wave_sum(sum);
      if (lane == 0) {
        const float a = mo == -INFINITY ? 0.0f : expf(mo - mn);
        arow[r] = a;
        lrow[r] = lrow[r] * a + sum;
        mrow[r] = mn;
      }
    }
    __syncthreads();
    // ---- weighted sums of the values
    {
#pragma unroll
      for (int i = 0; i < QT; ++i)
#pragma unroll
        for (int m = 0; m < MAPS; ++m) acc[i][m] *= arow[MAPS * i + m];
      if (col < dv) {
#pragma unroll 4
        for (int j = ks; j < nk; j += KS) {
          const float v = cload<CF32>(p.cache_v, ((slot * p.S + k0 + j) * p.G + g) * dv + col);
          float w[NR];
          if (NR == 1) {
            w[0] = sc[j * SCS];
          } else if (NR == 2) {
            const float2 t = *(const float2*)(sc + j * SCS);
            w[0] = t.x, w[NR - 1] = t.y;
          } else {
#pragma unroll
            for (int e = 0; e + 3 < NR; e += 4) {
              const float4 t = *(const float4*)(sc + j * SCS + e);
              w[e] = t.x, w[e + 1] = t.y, w[e + 2] = t.z, w[e + 3] = t.w;
            }
          }
#pragma unroll
          for (int i = 0; i < QT; ++i)
#pragma unroll
            for (int m = 0; m < MAPS; ++m) acc[i][m] = fmaf(w[MAPS * i + m], v, acc[i][m]);
        }
      }
    }
    __syncthreads();
  }
  // ---- sum the key subsets (fixed order), then finish or leave the split's partial result
  float* xs = sc;  // [KS][NR][ncol] = 256 * NR floats <= the score tile
  if (KS > 1) {
#pragma unroll
    for (int i = 0; i < QT; ++i)
#pragma unroll
      for (int m = 0; m < MAPS; ++m) xs[(ks * NR + MAPS * i + m) * ncol + col] = acc[i][m];
    __syncthreads();
  }
  for (int i = 0; i < nq; ++i) {
    float a[MAPS];
#pragma unroll
    for (int m = 0; m < MAPS; ++m) a[m] = 0.0f;
    if (KS > 1) {
      if (tid < ncol)
        for (int z = 0; z < KS; ++z)
#pragma unroll
          for (int m = 0; m < MAPS; ++m) a[m] += xs[(z * NR + MAPS * i + m) * ncol + tid];
    } else {
#pragma unroll
      for (int e = 0; e < QT; ++e)  // (static indexing keeps acc in registers)
        if (e == i)
#pragma unroll
          for (int m = 0; m < MAPS; ++m) a[m] = acc[e][m];
    }
    if (gridDim.z > 1) {
      float* pr = p.part + (((size_t)(r0 + i) * p.H + h) * gridDim.z + blockIdx.z) * (MAPS * (2 + dv));
      if (tid < MAPS) pr[2 * tid] = mrow[tid], pr[2 * tid + 1] = lrow[tid];
      if (tid < dv)
#pragma unroll
        for (int m = 0; m < MAPS; ++m) pr[2 * MAPS + m * dv + tid] = a[m];
    } else if (MAPS == 2) {
      diff_finish(a[0], a[MAPS - 1], lrow[MAPS * i], lrow[MAPS * i + MAPS - 1], p, (size_t)(r0 + i), h, red);
    } else {
      sink_finish(a[0], mrow[i], lrow[i], p, (size_t)(r0 + i), h);
    }
  }
}

// grid (T, H): merges the splits of one (token, head) in split order and finishes
template <int MAPS>
__global__ void __launch_bounds__(256) diffattn_combine_kernel(AttnArgs p, int splits) {
  __shared__ float red[4];
  const size_t t = blockIdx.x;
  const int h = blockIdx.y, dv = p.dv, c = threadIdx.x;
  const int stride = MAPS * (2 + dv);
  const float* pr = p.part + ((t * p.H + h) * splits) * stride;
  float mx[MAPS], l[MAPS], a[MAPS];
#pragma unroll
  for (int m = 0; m < MAPS; ++m) mx[m] = -INFINITY, l[m] = 0.0f, a[m] = 0.0f;
  for (int z = 0; z < splits; ++z)
#pragma unroll
    for (int m = 0; m < MAPS; ++m) mx[m] = fmaxf(mx[m], pr[(size_t)z * stride + 2 * m]);
  for (int z = 0; z < splits; ++z) {
    const float* q = pr + (size_t)z * stride;
#pragma unroll
    for (int m = 0; m < MAPS; ++m) {
      const float w = q[2 * m] == -INFINITY ? 0.0f : expf(q[2 * m] - mx[m]);
      l[m] = fmaf(q[2 * m + 1], w, l[m]);
      if (c < dv) a[m] = fmaf(q[2 * MAPS + m * dv + c], w, a[m]);
    }
  }
  if (MAPS == 2) diff_finish(a[0], a[MAPS - 1], l[0], l[MAPS - 1], p, t, h, red);
  else sink_finish(a[0], mx[0], l[0], p, t, h);
}

template <int QT, int MAPS>
static size_t diffattn_lds(int d) {
  return sizeof(float) * ((size_t)QT * MAPS * d + (size_t)kKeyTile * score_stride<QT * MAPS>() + 3 * QT * MAPS);
}

template <int QT, int MAPS>
static int diffattn_launch(const AttnArgs& p, int cache_f32, dim3 grid, hipStream_t stream) {
  const size_t lds = diffattn_lds<QT, MAPS>(p.d);
  auto* fn = cache_f32 ? diffattn_kernel<QT, MAPS, true> : diffattn_kernel<QT, MAPS, false>;
  if (lds > 48 * 1024) {
    const hipError_t e = hipFuncSetAttribute((const void*)fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
    if (e != hipSuccess) {
      lga_set_error(hipGetErrorString(e));
      return (int)e;
    }
  }
  fn<<<grid, 256, lds, stream>>>(p);
  return 0;
}

}  // namespace lgs

extern "C" int lgs_diffattn_prepare(float* proj, long ld, int q_off, int k_off, int v_off, void* cache_k, void* cache_v,
                                    int cache_f32, const float* inv_freq, const int* slot, const int* pos, int T, int H,
                                    int G, int d, int dv, int rot_dims, int max_seq, hipStream_t stream) {
  LGA_CHECK_ARG(proj && slot && pos && T > 0, "lgs_diffattn_prepare: bad arguments");
  LGA_CHECK_ARG(H > 0 && G > 0 && H % G == 0 && d > 0 && dv > 0,
                "lgs_diffattn_prepare: heads must be a multiple of the key heads");
  LGA_CHECK_ARG(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= d && (rot_dims == 0 || inv_freq),
                "lgs_diffattn_prepare: rotary dims");
  LGA_CHECK_ARG(k_off < 0 || (cache_k && cache_v && v_off >= 0 && max_seq > 0), "lgs_diffattn_prepare: cache");
  LGA_CHECK_ARG(q_off >= 0 && q_off + 2L * H * d <= ld, "lgs_diffattn_prepare: queries outside the row");
  LGA_CHECK_ARG(k_off < 0 || (k_off + 2L * G * d <= ld && v_off + (long)G * dv <= ld),
                "lgs_diffattn_prepare: keys or values outside the row");
  lgs::AttnPrepArgs p{proj, ld, q_off, k_off, v_off, cache_k, cache_v, inv_freq, slot, pos, H, G, d, dv, rot_dims, max_seq};
  if (cache_f32) lgs::diffattn_prepare_kernel<true><<<T, 256, 0, stream>>>(p);
  else lgs::diffattn_prepare_kernel<false><<<T, 256, 0, stream>>>(p);
  LGA_LAUNCH_RETURN();
}

extern "C" int lgs_diffattn(const float* q, long ld, const void* cache_k, const void* cache_v, int cache_f32,
                            const int* seq_start, const int* seq_slot, const int* seq_pos0, float* out, void* out_bf16,
                            float* part, int splits, int B, int max_len, int H, int G, int d, int dv, int max_seq,
                            int chunk, float scale, float cap, float lambda, float eps, float post, hipStream_t stream) {
  LGA_CHECK_ARG(q && cache_k && cache_v && seq_start && seq_slot && seq_pos0 && out, "lgs_diffattn: null pointer");
  LGA_CHECK_ARG(B > 0 && max_len > 0 && H > 0 && H <= 65535 && G > 0 && H % G == 0, "lgs_diffattn: bad sizes");
  LGA_CHECK_ARG(d > 0 && d <= 512 && dv > 0 && dv <= 256, "lgs_diffattn: key dim <= 512, value dim <= 256");
  LGA_CHECK_ARG(ld >= 2L * H * d && chunk >= 0 && max_seq > 0, "lgs_diffattn: bad sizes");
  LGA_CHECK_ARG(splits >= 1 && splits <= 64 && (splits == 1 || (part && max_len == 1)),
                "lgs_diffattn: splits need one token per sequence and a workspace");
  lgs::AttnArgs p{q, ld, cache_k, cache_v, seq_start, seq_slot, seq_pos0, out, (uint16_t*)out_bf16, part,
                  H, G, d, dv, max_seq, chunk, 0, scale, cap, lambda, eps, post, nullptr, nullptr, 0};
  int rc;
  if (max_len == 1) {
    p.tiles = 1;
    rc = lgs::diffattn_launch<1, 2>(p, cache_f32, dim3(B, H, splits), stream);
    if (rc == 0 && splits > 1) lgs::diffattn_combine_kernel<2><<<dim3(B, H), 256, 0, stream>>>(p, splits);
  } else {
    p.tiles = (max_len + 7) / 8;
    LGA_CHECK_ARG((long)B * p.tiles < (1L << 31), "lgs_diffattn: too many tiles");
    rc = lgs::diffattn_launch<8, 2>(p, cache_f32, dim3(B * p.tiles, H, 1), stream);
  }
  if (rc) return rc;
  LGA_LAUNCH_RETURN();
}

extern "C" int lgs_normattn_prepare(float* proj, long ld, int q_off, int k_off, int v_off, void* cache_k, void* cache_v,
                                    int cache_f32, const int* slot, const int* pos, int T, int H, int G, int d, int dv,
                                    int max_seq, float eps, float temp_coef, int temp_every, int norm, const float* q_w,
                                    const float* k_w, const float* inv_freq, int rot_dims, hipStream_t stream) {
  LGA_CHECK_ARG(proj && slot && pos && cache_k && cache_v && T > 0 && max_seq > 0, "lgs_normattn_prepare: bad arguments");
  LGA_CHECK_ARG(H > 0 && G > 0 && H % G == 0 && d > 0 && dv > 0 && temp_every >= 0,
                "lgs_normattn_prepare: heads must be a multiple of the key heads");
  LGA_CHECK_ARG(q_off >= 0 && q_off + (long)H * d <= ld && k_off >= 0 && k_off + (long)G * d <= ld && v_off >= 0 &&
                    v_off + (long)G * dv <= ld,
                "lgs_normattn_prepare: queries, keys or values outside the row");
  LGA_CHECK_ARG(rot_dims >= 0 && rot_dims % 2 == 0 && rot_dims <= d && (rot_dims == 0 || inv_freq),
                "lgs_normattn_prepare: rotary dims");
  lgs::NormPrepArgs p{proj, ld, q_off, k_off, v_off, cache_k, cache_v, slot, pos, H, G, d, dv, max_seq, temp_every, eps,
                      temp_coef, norm ? 1 : 0, q_w, k_w, inv_freq, rot_dims};
  if (cache_f32) lgs::normattn_prepare_kernel<true><<<T, 256, 0, stream>>>(p);
  else lgs::normattn_prepare_kernel<false><<<T, 256, 0, stream>>>(p);
  LGA_LAUNCH_RETURN();
}

extern "C" int lgs_sinkattn(const float* q, long ld, const void* cache_k, const void* cache_v, int cache_f32,
                            const float* sink, const int* seq_start, const int* seq_slot, const int* seq_pos0, float* out,
                            void* out_bf16, float* part, int splits, int B, int max_len, int H, int G, int d, int dv,
                            int max_seq, int chunk, float scale, float cap, float post, const float* gate, long ldg,
                            hipStream_t stream) {
  LGA_CHECK_ARG(q && cache_k && cache_v && seq_start && seq_slot && seq_pos0 && out, "lgs_sinkattn: null pointer");
  LGA_CHECK_ARG(!gate || ldg >= H, "lgs_sinkattn: the head gates' row stride");
  LGA_CHECK_ARG(B > 0 && max_len > 0 && H > 0 && H <= 65535 && G > 0 && H % G == 0, "lgs_sinkattn: bad sizes");
  LGA_CHECK_ARG(d > 0 && d <= 512 && dv > 0 && dv <= 256, "lgs_sinkattn: key dim <= 512, value dim <= 256");
  LGA_CHECK_ARG(ld >= (long)H * d && chunk >= 0 && max_seq > 0, "lgs_sinkattn: bad sizes");
  LGA_CHECK_ARG(splits >= 1 && splits <= 64 && (splits == 1 || (part && max_len == 1)),
                "lgs_sinkattn: splits need one token per sequence and a workspace");
  lgs::AttnArgs p{q, ld, cache_k, cache_v, seq_start, seq_slot, seq_pos0, out, (uint16_t*)out_bf16, part,
                  H, G, d, dv, max_seq, chunk, 0, scale, cap, 0.0f, 0.0f, post, sink, gate, ldg};
  int rc;
  if (max_len == 1) {
    p.tiles = 1;
    rc = lgs::diffattn_launch<1, 1>(p, cache_f32, dim3(B, H, splits), stream);
    if (rc == 0 && splits > 1) lgs::diffattn_combine_kernel<1><<<dim3(B, H), 256, 0, stream>>>(p, splits);
  } else {
    p.tiles = (max_len + 15) / 16;
    LGA_CHECK_ARG((long)B * p.tiles < (1L << 31), "lgs_sinkattn: too many tiles");
    rc = lgs::diffattn_launch<16, 1>(p, cache_f32, dim3(B * p.tiles, H, 1), stream);
  }
  if (rc) return rc;
  LGA_LAUNCH_RETURN();
}
