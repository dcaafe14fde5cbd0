// Shared declarations of liblitgpt_seq.so: the kernels of the layered models (retention, latent-, differential-,
// sink- and rotary attention, state-space, delta-rule and gated linear-attention mixers, gated and ungated
// feed-forwards, sparse experts, per-layer token inputs) over an fp32 residual stream.
//
// Conventions: activations are fp32 in memory in both precisions. A weight matrix is [out][in], either bf16 (raw
// uint16; the activation operand of a product is then rounded to bf16 and the sum is fp32: the matrix-core
// convention) or fp32 (everything fp32, plain FMA). Norm weights, decays, sinks and rotary frequencies are fp32.
// A step is a packed batch: the tokens of all its sequences lie row after row; per token an int32 cache slot and
// position, per sequence its first row, slot and first position. Nothing is allocated or synchronised here, every
// launch goes to the caller's stream, so a step can be captured into a HIP graph.
#pragma once

#include "common.h"

namespace lgs {
using namespace lga;

enum Act { kActNone = 0, kActRelu2 = 1, kActGeluTanh = 2, kActSilu = 3, kActSigmoid = 4 };

__device__ __forceinline__ float gelu_tanh_f(float z) {
  return 0.5f * z * (1.0f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}
__device__ __forceinline__ float sigmoid_f(float z) { return 1.0f / (1.0f + expf(-z)); }
__device__ __forceinline__ float act_f(int kind, float z) {
  switch (kind) {
    case kActRelu2: { const float r = fmaxf(z, 0.0f); return r * r; }
    case kActGeluTanh: return gelu_tanh_f(z);
    case kActSilu: return z * sigmoid_f(z);
    case kActSigmoid: return sigmoid_f(z);
    default: return z;
  }
}

// weight element i of a bf16 (WF32 = false) or fp32 (true) array
template <bool WF32>
__device__ __forceinline__ float wload(const void* w, size_t i) {
  return WF32 ? ((const float*)w)[i] : bf2f(((const uint16_t*)w)[i]);
}
// the activation operand of a product: rounded to bf16 beside bf16 weights, as stored beside fp32 weights
template <bool WF32>
__device__ __forceinline__ float aop(float v) { return WF32 ? v : round_bf(v); }

// eight consecutive weights starting at element i (i % 8 == 0, 16-byte aligned rows): one 16-byte load for bf16
template <bool WF32>
__device__ __forceinline__ void wload8(const void* w, size_t i, float* o) {
  if (WF32) {
    const float4 a = *(const float4*)((const float*)w + i), b = *(const float4*)((const float*)w + i + 4);
    o[0] = a.x, o[1] = a.y, o[2] = a.z, o[3] = a.w, o[4] = b.x, o[5] = b.y, o[6] = b.z, o[7] = b.w;
  } else {
    const uint4 a = *(const uint4*)((const uint16_t*)w + i);
    o[0] = bflo(a.x), o[1] = bfhi(a.x), o[2] = bflo(a.y), o[3] = bfhi(a.y);
    o[4] = bflo(a.z), o[5] = bfhi(a.z), o[6] = bflo(a.w), o[7] = bfhi(a.w);
  }
}
// the product of one row of a small second map with its `rank` inputs x (already rounded as the weights' precision
// asks, in LDS or registers' reach): w row i holds rank weights; rank % 8 == 0 takes 16-byte loads
template <bool WF32>
__device__ __forceinline__ float lowrank_dot(const void* w, size_t i, const float* x, int rank) {
  float acc = 0.0f;
  if ((rank & 7) == 0) {
    for (int r = 0; r < rank; r += 8) {
      float u[8];
      wload8<WF32>(w, i * rank + r, u);
#pragma unroll
      for (int e = 0; e < 8; ++e) acc = fmaf(x[r + e], u[e], acc);
    }
  } else {
    for (int r = 0; r < rank; ++r) acc = fmaf(x[r], wload<WF32>(w, i * rank + r), acc);
  }
  return acc;
}

// sum over the 256 threads of a workgroup (4 waves); `red` holds 4 floats; every thread gets the sum
__device__ __forceinline__ float block_sum_256(float v, float* red) {
  v = wave_sum(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  return (red[0] + red[1]) + (red[2] + red[3]);
}

}  // namespace lgs
