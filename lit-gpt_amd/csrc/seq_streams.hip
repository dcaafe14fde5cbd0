// Multi-stream residual (hyper-connections) of the layered models, fp32 throughout.
//
// The residual is kept in `s` parallel streams x[t][0 .. s)[W]. A sublayer reads a fixed weighted sum of the
// streams, u = sum_i a[i] x_i, through an RMS norm; its output y goes back into every stream while the streams
// are mixed: x_j <- sum_i m[i][j] x_i + b[j] y. With s = 1, a = b = m = 1 this is the ordinary residual sum.
//
//   lgs_embed_streams   x[t][j] = table[tokens[t]] * scale for every stream j
//   lgs_streams_step    one launch per sublayer boundary: the write-back of the sublayer that just ran (optional)
//                       followed by the read + norm of the next one (optional), so the streams are read once
//   lgs_sandwich_step   the boundary of layers whose sublayers are normed on the way in and out (one stream): the
//                       norms and the average of up to two branch outputs, the output norm times the layer scale,
//                       the residual add and the next sublayer's input norm in one launch
#include "seq_common.h"

namespace lgs {

constexpr int kMaxStreams = 8;

template <bool WF32>
__global__ void __launch_bounds__(256) embed_streams_kernel(const int* __restrict__ tokens, const void* __restrict__ table,
                                                            float scale, float* __restrict__ x, int W, int streams) {
  const size_t t = blockIdx.x;
  const size_t src = (size_t)tokens[t] * W;
  for (int i = threadIdx.x; i < W; i += 256) {
    const float v = wload<WF32>(table, src + i) * scale;
    for (int j = 0; j < streams; ++j) x[(t * streams + j) * W + i] = v;
  }
}

struct StreamArgs {
  float* x;          // [T][s][W]
  const float* y;    // [T][W] sublayer output to write back (null: no write-back)
  const float* mix;  // [s][s] indexed [from][to]
  const float* out;  // [s]
  const float* in;   // [s] read weights of the next sublayer (null: no read)
  const float* w;    // [W] norm weight of the next sublayer (null: the weighted sum itself is the result)
  float* h;          // [T][W] normed read
  uint16_t* h16;     // optional bf16 copy of h
  float eps;
  int W, s;
};

// grid (T): a workgroup owns a token; thread i owns columns i, i + 256, ... in every stream
__global__ void __launch_bounds__(256) streams_step_kernel(StreamArgs p) {
  __shared__ float red[4];
  __shared__ float cm[kMaxStreams * kMaxStreams], cb[kMaxStreams], ca[kMaxStreams];
  const int s = p.s, W = p.W;
  if (threadIdx.x < s * s) cm[threadIdx.x] = p.mix ? p.mix[threadIdx.x] : 0.0f;
  if (threadIdx.x < s) {
    cb[threadIdx.x] = p.out ? p.out[threadIdx.x] : 0.0f;
    ca[threadIdx.x] = p.in ? p.in[threadIdx.x] : 0.0f;
  }
  __syncthreads();
  float* xt = p.x + (size_t)blockIdx.x * s * W;
  const float* yt = p.y ? p.y + (size_t)blockIdx.x * W : nullptr;
  float ss = 0.0f;
  for (int i = threadIdx.x; i < W; i += 256) {
    float v[kMaxStreams];
#pragma unroll
    for (int j = 0; j < kMaxStreams; ++j) v[j] = j < s ? xt[(size_t)j * W + i] : 0.0f;
    if (yt) {
      const float y = yt[i];
      float nv[kMaxStreams];
#pragma unroll
      for (int j = 0; j < kMaxStreams; ++j) {
        float acc = 0.0f;
#pragma unroll
        for (int k = 0; k < kMaxStreams; ++k)
          if (k < s && j < s) acc = fmaf(cm[k * s + j], v[k], acc);
        nv[j] = j < s ? fmaf(cb[j], y, acc) : 0.0f;
      }
#pragma unroll
      for (int j = 0; j < kMaxStreams; ++j) {
        v[j] = nv[j];
        if (j < s) xt[(size_t)j * W + i] = nv[j];
      }
    }
    if (p.in) {
      float u = 0.0f;
#pragma unroll
      for (int j = 0; j < kMaxStreams; ++j)
        if (j < s) u = fmaf(ca[j], v[j], u);
      ss = fmaf(u, u, ss);
      p.h[(size_t)blockIdx.x * W + i] = u;  // normed below
    }
  }
  if (!p.in || !p.w) return;
  ss = block_sum_256(ss, red);
  const float rstd = 1.0f / sqrtf(ss / (float)W + p.eps);
  for (int i = threadIdx.x; i < W; i += 256) {
    const size_t at = (size_t)blockIdx.x * W + i;
    const float v = p.h[at] * rstd * p.w[i];  // (each thread re-reads what it wrote itself)
    p.h[at] = v;
    if (p.h16) p.h16[at] = f2bf(v);
  }
}

// The same step with a token's columns in registers: thread i owns columns i + 256 c, c < CPT (W <= 256 CPT), of
// SMAX >= s streams. All loads are issued before the first use and the normed read is written from registers, so a
// one-token step is one round trip to memory instead of one per column block.
// (NT threads per token: 256 for prompts, 1024 for steps of a few tokens, whose one workgroup per token is then
// four times shorter.)
template <int SMAX, int CPT, int NT>
__global__ void __launch_bounds__(NT) streams_step_reg_kernel(StreamArgs p) {
  __shared__ float red[NT / 64];
  __shared__ float cm[kMaxStreams * kMaxStreams], cb[kMaxStreams], ca[kMaxStreams];
  const int s = p.s, W = p.W;
  if (threadIdx.x < s * s) cm[threadIdx.x] = p.mix ? p.mix[threadIdx.x] : 0.0f;
  if (threadIdx.x < s) {
    cb[threadIdx.x] = p.out ? p.out[threadIdx.x] : 0.0f;
    ca[threadIdx.x] = p.in ? p.in[threadIdx.x] : 0.0f;
  }
  float* xt = p.x + (size_t)blockIdx.x * s * W;
  const float* yt = p.y ? p.y + (size_t)blockIdx.x * W : nullptr;
  float v[SMAX][CPT], y[CPT], nw[CPT];
#pragma unroll
  for (int c = 0; c < CPT; ++c) {
    const int i = threadIdx.x + NT * c;
#pragma unroll
    for (int j = 0; j < SMAX; ++j) v[j][c] = (j < s && i < W) ? xt[(size_t)j * W + i] : 0.0f;
    y[c] = (yt && i < W) ? yt[i] : 0.0f;
    nw[c] = (p.in && p.w && i < W) ? p.w[i] : 1.0f;
  }
  __syncthreads();
  float u[CPT], ss = 0.0f;
#pragma unroll
  for (int c = 0; c < CPT; ++c) {
    const int i = threadIdx.x + NT * c;
    if (yt) {
      float nv[SMAX];
#pragma unroll
      for (int j = 0; j < SMAX; ++j) {
        float acc = 0.0f;
#pragma unroll
        for (int k = 0; k < SMAX; ++k)
          if (k < s && j < s) acc = fmaf(cm[k * s + j], v[k][c], acc);
        nv[j] = j < s ? fmaf(cb[j], y[c], acc) : 0.0f;
      }
#pragma unroll
      for (int j = 0; j < SMAX; ++j) {
        v[j][c] = nv[j];
        if (j < s && i < W) xt[(size_t)j * W + i] = nv[j];
      }
    }
    float a = 0.0f;
#pragma unroll
    for (int j = 0; j < SMAX; ++j)
      if (j < s) a = fmaf(ca[j], v[j][c], a);
    u[c] = a;
    ss = fmaf(a, a, ss);
  }
  if (!p.in) return;
  float rstd = 1.0f;
  if (p.w) {
    ss = wave_sum(ss);
    if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = ss;
    __syncthreads();
    ss = 0.0f;
#pragma unroll
    for (int w = 0; w < NT / 64; ++w) ss += red[w];
    rstd = 1.0f / sqrtf(ss / (float)W + p.eps);
  }
#pragma unroll
  for (int c = 0; c < CPT; ++c) {
    const int i = threadIdx.x + NT * c;
    if (i >= W) continue;
    const size_t at = (size_t)blockIdx.x * W + i;
    const float r = p.w ? u[c] * rstd * nw[c] : u[c];
    p.h[at] = r;
    if (p.h16) p.h16[at] = f2bf(r);
  }
}

template <int SMAX>
static bool streams_step_reg(const StreamArgs& p, int T, hipStream_t stream) {
  if (T <= 32 && p.W > 512) {
    if (p.W <= 2048) streams_step_reg_kernel<SMAX, 2, 1024><<<T, 1024, 0, stream>>>(p);
    else if (p.W <= 4096) streams_step_reg_kernel<SMAX, 4, 1024><<<T, 1024, 0, stream>>>(p);
    else if (p.W <= 8192) streams_step_reg_kernel<SMAX, 8, 1024><<<T, 1024, 0, stream>>>(p);
    else return false;
    return true;
  }
  if (p.W <= 1024) streams_step_reg_kernel<SMAX, 4, 256><<<T, 256, 0, stream>>>(p);
  else if (p.W <= 2048) streams_step_reg_kernel<SMAX, 8, 256><<<T, 256, 0, stream>>>(p);
  else if (p.W <= 4096 && SMAX <= 4) streams_step_reg_kernel<SMAX, 16, 256><<<T, 256, 0, stream>>>(p);
  else return false;
  return true;
}

// ------------------------------------------------------------------------------------------------ sandwich norms
// One boundary between two sublayers of a layer whose sublayers are normed on the way in AND on the way out.
// With y0 (the sublayer that ran; up to two branches): b_i = w_i ? y_i / rms(y_i) * w_i : y_i, s = coef * sum_i b_i,
// x <- x + s / rms(s) * post_w (post_w: the output norm's weight times the layer's per-channel scale). Then with
// next_w: h = x / rms(x) * next_w, the next sublayer's input (fp32 and / or its bf16 rounding). Every root mean
// square has eps inside the root. grid (rows); a row lives in registers up to 256 * CPT columns, else it is re-read.
struct SandwichArgs {
  float* x;
  const float *y0, *w0, *y1, *w1;
  float coef;
  const float* post_w;
  const float* next_w;
  float* h;
  uint16_t* h16;
  float eps;
  int n;
};

// sums of two values over the 256 threads of a workgroup at once (`red` holds 8 floats)
__device__ __forceinline__ void block_sum2_256(float& u, float& v, float* red) {
  u = wave_sum(u);
  v = wave_sum(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) {
    red[threadIdx.x >> 6] = u;
    red[4 + (threadIdx.x >> 6)] = v;
  }
  __syncthreads();
  u = (red[0] + red[1]) + (red[2] + red[3]);
  v = (red[4] + red[5]) + (red[6] + red[7]);
}

template <int CPT>
__global__ void __launch_bounds__(256) sandwich_step_kernel(SandwichArgs p) {
  __shared__ float red[8];
  const size_t r = blockIdx.x;
  const int n = p.n, tid = threadIdx.x;
  float* xr = p.x + r * n;
  const float inv_n = 1.0f / (float)n;
  // every operand of the registers' share of the row is fetched up front, so that the reductions below wait for
  // one batch of loads only
  float xv[CPT], av[CPT], bv[CPT], w0[CPT], w1[CPT], wp[CPT], wn[CPT];
  const float *a = p.y0 ? p.y0 + r * n : nullptr, *b = p.y1 ? p.y1 + r * n : nullptr;
#pragma unroll
  for (int e = 0; e < CPT; ++e) {
    const int i = tid + 256 * e;
    const bool in = i < n;
    xv[e] = in ? xr[i] : 0.0f;
    av[e] = (a && in) ? a[i] : 0.0f;
    bv[e] = (b && in) ? b[i] : 0.0f;
    w0[e] = (a && p.w0 && in) ? p.w0[i] : 1.0f;
    w1[e] = (b && p.w1 && in) ? p.w1[i] : 1.0f;
    wp[e] = (a && in) ? p.post_w[i] : 0.0f;
    wn[e] = (p.next_w && in) ? p.next_w[i] : 0.0f;
  }
  if (a) {
    float sa = 0.0f, sb = 0.0f;
#pragma unroll
    for (int e = 0; e < CPT; ++e) {
      sa = fmaf(av[e], av[e], sa);
      sb = fmaf(bv[e], bv[e], sb);
    }
    for (int i = tid + 256 * CPT; i < n; i += 256) {
      sa = fmaf(a[i], a[i], sa);
      if (b) sb = fmaf(b[i], b[i], sb);
    }
    float ra = 1.0f, rb = 1.0f;
    if (p.w0 || (b && p.w1)) {
      block_sum2_256(sa, sb, red);
      if (p.w0) ra = 1.0f / sqrtf(sa * inv_n + p.eps);
      if (b && p.w1) rb = 1.0f / sqrtf(sb * inv_n + p.eps);
    }
    auto joined = [&](float ya, float yb, float wa, float wb) {
      float s = p.w0 ? ya * ra * wa : ya;
      if (b) s += p.w1 ? yb * rb * wb : yb;
      return s * p.coef;
    };
    auto joined_at = [&](int i) {
      return joined(a[i], b ? b[i] : 0.0f, p.w0 ? p.w0[i] : 1.0f, (b && p.w1) ? p.w1[i] : 1.0f);
    };
    float ss = 0.0f;
#pragma unroll
    for (int e = 0; e < CPT; ++e) {
      av[e] = tid + 256 * e < n ? joined(av[e], bv[e], w0[e], w1[e]) : 0.0f;  // (av now holds the joined value)
      ss = fmaf(av[e], av[e], ss);
    }
    for (int i = tid + 256 * CPT; i < n; i += 256) {
      const float s = joined_at(i);
      ss = fmaf(s, s, ss);
    }
    const float rs = 1.0f / sqrtf(block_sum_256(ss, red) * inv_n + p.eps);
#pragma unroll
    for (int e = 0; e < CPT; ++e) {
      const int i = tid + 256 * e;
      if (i < n) {
        xv[e] = fmaf(av[e] * rs, wp[e], xv[e]);
        xr[i] = xv[e];
      }
    }
    for (int i = tid + 256 * CPT; i < n; i += 256) xr[i] = fmaf(joined_at(i) * rs, p.post_w[i], xr[i]);
  }
  if (!p.next_w) return;
  float sx = 0.0f;
#pragma unroll
  for (int e = 0; e < CPT; ++e) sx = fmaf(xv[e], xv[e], sx);
  for (int i = tid + 256 * CPT; i < n; i += 256) sx = fmaf(xr[i], xr[i], sx);  // (written by this thread above)
  const float rx = 1.0f / sqrtf(block_sum_256(sx, red) * inv_n + p.eps);
#pragma unroll
  for (int e = 0; e < CPT; ++e) {
    const int i = tid + 256 * e;
    if (i < n) {
      const float o = xv[e] * rx * wn[e];
      if (p.h) p.h[r * n + i] = o;
      if (p.h16) p.h16[r * n + i] = f2bf(o);
    }
  }
  for (int i = tid + 256 * CPT; i < n; i += 256) {
    const float o = xr[i] * rx * p.next_w[i];
    if (p.h) p.h[r * n + i] = o;
    if (p.h16) p.h16[r * n + i] = f2bf(o);
  }
}

}  // namespace lgs

extern "C" int lgs_embed_streams(const int* tokens, const void* table, int w_f32, float scale, float* x, int T, int W,
                                 int vocab, int streams, hipStream_t stream) {
  LGA_CHECK_ARG(tokens && table && x && T > 0 && W > 0 && vocab > 0, "lgs_embed_streams: bad arguments");
  LGA_CHECK_ARG(streams >= 1 && streams <= lgs::kMaxStreams, "lgs_embed_streams: 1 to 8 streams");
  if (w_f32) lgs::embed_streams_kernel<true><<<T, 256, 0, stream>>>(tokens, table, scale, x, W, streams);
  else lgs::embed_streams_kernel<false><<<T, 256, 0, stream>>>(tokens, table, scale, x, W, streams);
  LGA_LAUNCH_RETURN();
}

extern "C" int lgs_streams_step(float* x, const float* y, const float* mix, const float* out, const float* in,
                                const float* norm_w, float* h, void* h_bf16, float eps, int T, int W, int streams,
                                hipStream_t stream) {
  LGA_CHECK_ARG(x && T > 0 && W > 0, "lgs_streams_step: bad arguments");
  LGA_CHECK_ARG(streams >= 1 && streams <= lgs::kMaxStreams, "lgs_streams_step: 1 to 8 streams");
  LGA_CHECK_ARG(!y || (mix && out), "lgs_streams_step: a write-back needs the mix matrix and the output weights");
  LGA_CHECK_ARG(!in || h, "lgs_streams_step: a read needs a result buffer");
  LGA_CHECK_ARG(norm_w || !h_bf16, "lgs_streams_step: the bf16 copy is made by the norm");
  LGA_CHECK_ARG(y || in, "lgs_streams_step: nothing to do");
  lgs::StreamArgs p{x, y, mix, out, in, norm_w, h, (uint16_t*)h_bf16, eps, W, streams};
  bool done;
  if (streams == 1) done = lgs::streams_step_reg<1>(p, T, stream);
  else if (streams == 2) done = lgs::streams_step_reg<2>(p, T, stream);
  else if (streams <= 4) done = lgs::streams_step_reg<4>(p, T, stream);
  else done = lgs::streams_step_reg<8>(p, T, stream);
  if (!done) lgs::streams_step_kernel<<<T, 256, 0, stream>>>(p);  // wide rows: column blocks one after the other
  LGA_LAUNCH_RETURN();
}

extern "C" int lgs_sandwich_step(float* x, const float* y0, const float* w0, const float* y1, const float* w1,
                                 float coef, const float* post_w, const float* next_w, float* h, void* h_bf16, float eps,
                                 int rows, int n, hipStream_t stream) {
  LGA_CHECK_ARG(x && rows > 0 && n > 0, "lgs_sandwich_step: bad arguments");
  LGA_CHECK_ARG(!y0 || post_w, "lgs_sandwich_step: a sublayer's output needs the output norm's weight");
  LGA_CHECK_ARG(y0 || !y1, "lgs_sandwich_step: a second branch without a first");
  LGA_CHECK_ARG(y0 || next_w, "lgs_sandwich_step: nothing to do");
  LGA_CHECK_ARG(!next_w || h || h_bf16, "lgs_sandwich_step: the next input needs a place");
  lgs::SandwichArgs p{x, y0, w0, y1, w1, coef, post_w, next_w, h, (uint16_t*)h_bf16, eps, n};
  if (n <= 1024) lgs::sandwich_step_kernel<4><<<rows, 256, 0, stream>>>(p);
  else if (n <= 2048) lgs::sandwich_step_kernel<8><<<rows, 256, 0, stream>>>(p);
  else lgs::sandwich_step_kernel<16><<<rows, 256, 0, stream>>>(p);
  LGA_LAUNCH_RETURN();
}
