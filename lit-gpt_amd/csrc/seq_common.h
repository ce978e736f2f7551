// Shared declarations of liblitgpt_seq.so: the kernels of the layered models (retention and latent-attention
// mixers, gated feed-forwards, sparse experts, per-layer token inputs) over an fp32 residual stream.
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

// sum over the 256 threads of a workgroup (4 waves); `red` holds 4 floats; every thread gets the sum
__device__ __forceinline__ float block_sum_256(float v, float* red) {
  v = wave_sum(v);
  __syncthreads();
  if ((threadIdx.x & 63) == 0) red[threadIdx.x >> 6] = v;
  __syncthreads();
  return (red[0] + red[1]) + (red[2] + red[3]);
}

}  // namespace lgs
