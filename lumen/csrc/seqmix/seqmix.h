// Shared pieces of the sequence-mixing kernels (hybrid models): dtype dispatch and the fp32
// scalar functions every kernel here uses.  All arithmetic is fp32; 16-bit types only appear at
// loads and stores.  Launchers are `extern "C"`, take raw pointers and a stream, never allocate
// or synchronise (safe under hipGraph capture) and return hipGetLastError().
#pragma once
#include "../kernels/common.h"

namespace lumen {

__device__ __forceinline__ float sigmoid_f(float x) { return 1.f / (1.f + expf(-x)); }
__device__ __forceinline__ float silu_f(float x) { return x / (1.f + expf(-x)); }
__device__ __forceinline__ float gelu_tanh_f(float z) {
  return 0.5f * z * (1.f + tanhf(0.7978845608028654f * (z + 0.044715f * z * z * z)));
}
__device__ __forceinline__ float dyt_f(float x, float alpha, float w, float b) {
  return tanhf(alpha * x) * w + b;
}

// four consecutive elements as one vector access (16 bytes of fp32, 8 bytes of a 16-bit type)
template <typename T> __device__ __forceinline__ void load4(const T* __restrict__ p, float (&o)[4]) {
  const uint2 raw = *reinterpret_cast<const uint2*>(p);
  const T* e = reinterpret_cast<const T*>(&raw);
#pragma unroll
  for (int j = 0; j < 4; ++j) o[j] = to_f32(e[j]);
}
template <> __device__ __forceinline__ void load4<float>(const float* __restrict__ p, float (&o)[4]) {
  const float4 a = *reinterpret_cast<const float4*>(p);
  o[0] = a.x; o[1] = a.y; o[2] = a.z; o[3] = a.w;
}
template <typename T> __device__ __forceinline__ void store4(T* __restrict__ p, const float (&v)[4]) {
  *reinterpret_cast<uint2*>(p) = make_uint2(pk2<T>(v[0], v[1]), pk2<T>(v[2], v[3]));
}
template <> __device__ __forceinline__ void store4<float>(float* __restrict__ p, const float (&v)[4]) {
  *reinterpret_cast<float4*>(p) = make_float4(v[0], v[1], v[2], v[3]);
}

}  // namespace lumen

// run `CALL(T)` with T = float / fp16 / bf16 for dtype code `dt`
#define SM_DISPATCH(dt, CALL)                          \
  switch (dt) {                                        \
    case lumen::kF32: { CALL(float); break; }          \
    case lumen::kF16: { CALL(lumen::fp16); break; }    \
    case lumen::kBF16: { CALL(lumen::bf16); break; }   \
    default: return hipErrorInvalidValue;              \
  }
