// Mixture-of-experts helpers around the two stacked library GEMMs of a hybrid layer's
// feed-forward:
//   sm_route_topk  router logits [T, E] fp32 -> dense routing weights [T, E] fp32 (softmax over
//                  the row's `top` largest logits at their places, zero elsewhere).  One wave per
//                  row: each lane keeps E / 64 logits in registers, `top` rounds of a wave-wide
//                  arg-max (ties: lowest index).
//   sm_gated_act   act(gate) * up over stacked [gate | up] blocks (act: SiLU, ReLU or tanh-GELU),
//                  expert e's block scaled by the row's routing weight; fp32 math.
//   sm_write_k     rows of the key projection into the paged key cache by slot.
#include "seqmix.h"

using namespace lumen;

namespace {

constexpr int kMaxPerLane = 16;   // experts <= 1024

// the gate's activation: 0 SiLU, 1 ReLU, 2 tanh-GELU
__device__ __forceinline__ float gate_act(float g, int act) {
  return act == 0 ? silu_f(g) : act == 1 ? fmaxf(g, 0.f) : gelu_tanh_f(g);
}

__global__ void __launch_bounds__(256)
route_topk_kernel(const float* __restrict__ z, float* __restrict__ out, int T, int E, int top) {
  const int lane = threadIdx.x & 63;
  const int row = blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (row >= T) return;
  const float* zr = z + (long long)row * E;
  float val[kMaxPerLane];
  unsigned sel = 0;
#pragma unroll
  for (int q = 0; q < kMaxPerLane; ++q) {
    const int e = lane + 64 * q;
    val[q] = e < E ? zr[e] : -INFINITY;
  }
  float m0 = 0.f, den = 0.f;
  for (int it = 0; it < top; ++it) {
    float bv = -INFINITY;
    int bi = 0x7fffffff;
#pragma unroll
    for (int q = 0; q < kMaxPerLane; ++q) {
      const int e = lane + 64 * q;
      if (e < E && !((sel >> q) & 1u) && (val[q] > bv || (val[q] == bv && e < bi))) {
        bv = val[q];
        bi = e;
      }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) {
      const float ov = __shfl_xor(bv, o, 64);
      const int oi = __shfl_xor(bi, o, 64);
      if (ov > bv || (ov == bv && oi < bi)) { bv = ov; bi = oi; }
    }
    if (bi == 0x7fffffff) break;         // fewer than `top` finite candidates
    if (it == 0) m0 = bv;
    den += expf(bv - m0);
    if ((bi & 63) == lane) sel |= 1u << (bi >> 6);
  }
  float* orow = out + (long long)row * E;
#pragma unroll
  for (int q = 0; q < kMaxPerLane; ++q) {
    const int e = lane + 64 * q;
    if (e < E) orow[e] = ((sel >> q) & 1u) ? expf(val[q] - m0) / den : 0.f;
  }
}

template <typename T>
__global__ void gated_act_kernel(const T* __restrict__ gu, const float* __restrict__ wts,
                                 T* __restrict__ out, int Tn, int E, int ff, int ffs,
                                 int act) {
  const int in_w = E * 2 * ff + 2 * ffs, out_w = E * ff + ffs;
  const long long n = (long long)Tn * out_w;
  for (long long i = blockIdx.x * (long long)blockDim.x + threadIdx.x; i < n;
       i += (long long)gridDim.x * blockDim.x) {
    const int t = (int)(i / out_w), c = (int)(i % out_w);
    const T* row = gu + (long long)t * in_w;
    float g, u, w = 1.f;
    if (c < E * ff) {
      const int e = c / ff, q = c % ff;
      w = wts[(long long)t * E + e];
      g = to_f32(row[e * 2 * ff + q]);
      u = to_f32(row[e * 2 * ff + ff + q]);
    } else {
      const int q = c - E * ff;
      g = to_f32(row[E * 2 * ff + q]);
      u = to_f32(row[E * 2 * ff + ffs + q]);
    }
    out[i] = from_f32<T>(w == 0.f ? 0.f : gate_act(g, act) * u * w);
  }
}

// eight outputs per thread (16-byte accesses): every block size a multiple of 8, 16-bit dtypes
template <typename T>
__global__ void __launch_bounds__(256)
gated_act_v8(const T* __restrict__ gu, const float* __restrict__ wts, T* __restrict__ out, int Tn,
             int E, int ff, int ffs, int act) {
  const int in_w = E * 2 * ff + 2 * ffs, out_w = E * ff + ffs;
  const int c = 8 * (blockIdx.x * 256 + threadIdx.x);
  if (c >= out_w) return;
  int e = -1, goff, uoff;
  if (c < E * ff) {
    e = c / ff;
    goff = e * 2 * ff + (c - e * ff);
    uoff = goff + ff;
  } else {
    goff = E * 2 * ff + (c - E * ff);
    uoff = goff + ffs;
  }
  for (int t = blockIdx.y; t < Tn; t += gridDim.y) {
    const T* row = gu + (long long)t * in_w;
    const float w = e >= 0 ? wts[(long long)t * E + e] : 1.f;
    float g[8], u[8], o[8];
    if (w == 0.f) {
#pragma unroll
      for (int j = 0; j < 8; ++j) o[j] = 0.f;
    } else {
      load8<T>(row + goff, g);
      load8<T>(row + uoff, u);
#pragma unroll
      for (int j = 0; j < 8; ++j) o[j] = gate_act(g[j], act) * u[j] * w;
    }
    store8<T>(out + (long long)t * out_w + c, o);
  }
}

template <typename T>
__global__ void write_k_kernel(const T* __restrict__ k, long long ld, T* __restrict__ cache,
                               const long long* __restrict__ slots, int Tn, int GD) {
  const long long n = (long long)Tn * GD;
  for (long long i = blockIdx.x * (long long)blockDim.x + threadIdx.x; i < n;
       i += (long long)gridDim.x * blockDim.x) {
    const int t = (int)(i / GD), c = (int)(i % GD);
    const long long s = slots[t];
    if (s >= 0) cache[s * GD + c] = k[(long long)t * ld + c];
  }
}

inline int grid_for(long long n, int block = 256) {
  long long g = (n + block - 1) / block;
  return (int)(g < 1 ? 1 : (g > 65536 ? 65536 : g));
}

}  // namespace

extern "C" {

hipError_t sm_route_topk(const float* z, float* out, int T, int E, int top, hipStream_t st) {
  if (T == 0) return hipSuccess;
  if (E < 1 || E > 64 * kMaxPerLane || top < 1 || top > E) return hipErrorInvalidValue;
  route_topk_kernel<<<(T + 3) / 4, 256, 0, st>>>(z, out, T, E, top);
  return hipGetLastError();
}

hipError_t sm_gated_act(int dt, const void* gu, const float* wts, void* out, int T, int E, int ff,
                        int ffs, int act, hipStream_t st) {
  const long long n = (long long)T * (E * ff + ffs);
  if (n == 0) return hipSuccess;
  if (E > 0 && wts == nullptr) return hipErrorInvalidValue;
  if (ff % 8 == 0 && ffs % 8 == 0 && (dt == kBF16 || dt == kF16)) {
    const dim3 grid(((E * ff + ffs) / 8 + 255) / 256, T < 65535 ? T : 65535);
    if (dt == kBF16)
      gated_act_v8<bf16><<<grid, 256, 0, st>>>((const bf16*)gu, wts, (bf16*)out, T, E, ff, ffs,
                                                 act);
    else
      gated_act_v8<fp16><<<grid, 256, 0, st>>>((const fp16*)gu, wts, (fp16*)out, T, E, ff, ffs,
                                                 act);
    return hipGetLastError();
  }
#define CALL(TT) gated_act_kernel<TT><<<grid_for(n), 256, 0, st>>>((const TT*)gu, wts, (TT*)out, T, E, ff, ffs, act)
  SM_DISPATCH(dt, CALL)
#undef CALL
  return hipGetLastError();
}

hipError_t sm_write_k(int dt, const void* k, long long ld, void* cache, const long long* slots,
                      int T, int GD, hipStream_t st) {
  if ((long long)T * GD == 0) return hipSuccess;
#define CALL(TT) write_k_kernel<TT><<<grid_for((long long)T * GD), 256, 0, st>>>((const TT*)k, ld, (TT*)cache, slots, T, GD)
  SM_DISPATCH(dt, CALL)
#undef CALL
  return hipGetLastError();
}

}  // extern "C"
