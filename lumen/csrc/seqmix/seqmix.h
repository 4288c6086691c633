// Shared pieces of the sequence-mixing kernels (hybrid models): dtype dispatch and the fp32
// scalar functions every kernel here uses.  All arithmetic is fp32; 16-bit types only appear at
// loads and stores.  Launchers are `extern "C"`, take raw pointers and a stream, never allocate
// or synchronise (safe under hipGraph capture) and return hipGetLastError().
#pragma once
#include "../kernels/common.h"

namespace lumen {

__device__ __forceinline__ float sigmoid_f(float x) { return 1.f / (1.f + expf(-x)); }
__device__ __forceinline__ float silu_f(float x) { return x / (1.f + expf(-x)); }
__device__ __forceinline__ float dyt_f(float x, float alpha, float w, float b) {
  return tanhf(alpha * x) * w + b;
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
