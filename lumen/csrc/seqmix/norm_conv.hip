// Dynamic Tanh norms of the hybrid stack, fused with what surrounds them:
//   sm_dyt           out = DyT(x)                              (final norm on the scored rows)
//   sm_dyt_residual  x += DyT_post(y);  h = DyT_pre(x)         (fp32 residual stream, in place)
//   sm_dyt_canon     out_t = h_t + sum_j cw[:, j] h_(t-taps+1+j), h = DyT(x), rows before a
//                    segment's first row taken from the per-slot tail (zero below position 0)
//   sm_canon_tail    the tail moves on to the segment's last taps - 1 normed rows
//   sm_token_shift   out[s] = h + (h_prev - h) * mu[s], h_prev the previous row of the sequence
//   sm_shift_tail    prev[slot] = the segment's last row
// All are memory-bound passes.  When the width is a multiple of 4 a thread owns FOUR consecutive
// channels (16-byte fp32 / 8-byte 16-bit accesses), rows come from the grid's y dimension (no
// index division), per-channel constants are loaded once per thread; the convolution walks a
// strip of rows with the last taps - 1 normed rows in registers, so every tanh is computed once
// (plus the strip's halo).  Other widths take the one-element-per-thread kernels.
#include "seqmix.h"

using namespace lumen;

namespace {

constexpr int kMaxTaps = 16;

template <typename TI, typename TO>
__global__ void dyt_kernel(const TI* __restrict__ x, const float* __restrict__ w,
                           const float* __restrict__ b, const float* __restrict__ alpha,
                           TO* __restrict__ out, long long n, int W) {
  const float a = *alpha;
  for (long long i = blockIdx.x * (long long)blockDim.x + threadIdx.x; i < n;
       i += (long long)gridDim.x * blockDim.x) {
    const int c = (int)(i % W);
    out[i] = from_f32<TO>(dyt_f(to_f32(x[i]), a, w[c], b[c]));
  }
}

template <typename TY, typename TH>
__global__ void dyt_residual_kernel(float* __restrict__ x, const TY* __restrict__ y,
                                    const float* __restrict__ pw, const float* __restrict__ pb,
                                    const float* __restrict__ pa, TH* __restrict__ h,
                                    const float* __restrict__ w2, const float* __restrict__ b2,
                                    const float* __restrict__ a2, long long n, int W) {
  const float ap = *pa;
  const float an = h ? *a2 : 0.f;
  for (long long i = blockIdx.x * (long long)blockDim.x + threadIdx.x; i < n;
       i += (long long)gridDim.x * blockDim.x) {
    const int c = (int)(i % W);
    const float v = x[i] + dyt_f(to_f32(y[i]), ap, pw[c], pb[c]);
    x[i] = v;
    if (h) h[i] = from_f32<TH>(dyt_f(v, an, w2[c], b2[c]));
  }
}

template <typename TO>
__global__ void dyt_canon_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                 const float* __restrict__ b, const float* __restrict__ alpha,
                                 const float* __restrict__ cw, const float* __restrict__ tail,
                                 TO* __restrict__ out, const int* __restrict__ cu,
                                 const int* __restrict__ slot, const int* __restrict__ start,
                                 const int* __restrict__ row_seg, int T, int W, int taps) {
  const float a = *alpha;
  const int K = taps - 1;
  const long long n = (long long)T * W;
  for (long long i = blockIdx.x * (long long)blockDim.x + threadIdx.x; i < n;
       i += (long long)gridDim.x * blockDim.x) {
    const int t = (int)(i / W), c = (int)(i % W);
    const int sg = row_seg[t];
    const int local = t - cu[sg];
    const int p0 = start[sg];
    const float wc = w[c], bc = b[c];
    const float hc = dyt_f(x[i], a, wc, bc);
    float acc = cw[(long long)c * taps + K] * hc;
    for (int d = 1; d <= K; ++d) {            // the row d positions back
      const int src = local - d;
      float hv = 0.f;
      if (src >= 0) {
        hv = dyt_f(x[i - (long long)d * W], a, wc, bc);
      } else if (p0 + src >= 0) {
        hv = tail[((long long)slot[sg] * K + (K + src)) * W + c];
      }
      acc += cw[(long long)c * taps + (K - d)] * hv;
    }
    out[i] = from_f32<TO>(hc + acc);
  }
}

__global__ void canon_tail_kernel(const float* __restrict__ x, const float* __restrict__ w,
                                  const float* __restrict__ b, const float* __restrict__ alpha,
                                  float* __restrict__ tail, const int* __restrict__ cu,
                                  const int* __restrict__ slot, const int* __restrict__ start,
                                  int S, int W, int taps) {
  const float a = *alpha;
  const int K = taps - 1;
  const long long n = (long long)S * W;
  for (long long i = blockIdx.x * (long long)blockDim.x + threadIdx.x; i < n;
       i += (long long)gridDim.x * blockDim.x) {
    const int sg = (int)(i / W), c = (int)(i % W);
    const int r0 = cu[sg], L = cu[sg + 1] - r0;
    if (L <= 0) continue;
    const int p0 = start[sg];
    float* tp = tail + (long long)slot[sg] * K * W + c;
    float old[kMaxTaps];
#pragma unroll
    for (int k = 0; k < kMaxTaps; ++k) old[k] = k < K ? tp[(long long)k * W] : 0.f;
    for (int k = 0; k < K; ++k) {             // new tail row k is local row L - K + k
      const int src = L - K + k;
      float hv = 0.f;
      if (src >= 0) {
        hv = dyt_f(x[(long long)(r0 + src) * W + c], a, w[c], b[c]);
      } else if (p0 + src >= 0) {
        float o = 0.f;
#pragma unroll
        for (int q = 0; q < kMaxTaps; ++q) o = (q == k + L) ? old[q] : o;
        hv = o;
      }
      tp[(long long)k * W] = hv;
    }
  }
}

template <typename T>
__global__ void token_shift_kernel(const T* __restrict__ h, const float* __restrict__ mu,
                                   const float* __restrict__ prev, T* __restrict__ out,
                                   const int* __restrict__ cu, const int* __restrict__ slot,
                                   const int* __restrict__ start, const int* __restrict__ row_seg,
                                   int Tn, int W, int nmix) {
  const long long n = (long long)Tn * W;
  for (long long i = blockIdx.x * (long long)blockDim.x + threadIdx.x; i < n;
       i += (long long)gridDim.x * blockDim.x) {
    const int t = (int)(i / W), c = (int)(i % W);
    const int sg = row_seg[t];
    const float hv = to_f32(h[i]);
    float pv = 0.f;
    if (t > cu[sg]) pv = to_f32(h[i - W]);
    else if (start[sg] > 0) pv = prev[(long long)slot[sg] * W + c];
    const float d = pv - hv;
    for (int s = 0; s < nmix; ++s)
      out[(long long)s * n + i] = from_f32<T>(hv + d * mu[(long long)s * W + c]);
  }
}

template <typename T>
__global__ void shift_tail_kernel(const T* __restrict__ h, float* __restrict__ prev,
                                  const int* __restrict__ cu, const int* __restrict__ slot, int S,
                                  int W) {
  const long long n = (long long)S * W;
  for (long long i = blockIdx.x * (long long)blockDim.x + threadIdx.x; i < n;
       i += (long long)gridDim.x * blockDim.x) {
    const int sg = (int)(i / W), c = (int)(i % W);
    const int last = cu[sg + 1] - 1;
    if (last < cu[sg]) continue;
    prev[(long long)slot[sg] * W + c] = to_f32(h[(long long)last * W + c]);
  }
}

// ---- four channels per thread ------------------------------------------------------------------
template <typename TY, typename TH>
__global__ void __launch_bounds__(256)
dyt_residual_v4(float* __restrict__ x, const TY* __restrict__ y, const float* __restrict__ pw,
                const float* __restrict__ pb, const float* __restrict__ pa, TH* __restrict__ h,
                const float* __restrict__ w2, const float* __restrict__ b2,
                const float* __restrict__ a2, int T, int W) {
  const int c = 4 * (blockIdx.x * 256 + threadIdx.x);
  if (c >= W) return;
  const float ap = *pa, an = h ? *a2 : 0.f;
  float w1[4], b1[4], wn[4] = {0, 0, 0, 0}, bn[4] = {0, 0, 0, 0};
  load4<float>(pw + c, w1);
  load4<float>(pb + c, b1);
  if (h) { load4<float>(w2 + c, wn); load4<float>(b2 + c, bn); }
  for (int t = blockIdx.y; t < T; t += gridDim.y) {
    const long long i = (long long)t * W + c;
    float xv[4], yv[4], hv[4];
    load4<float>(x + i, xv);
    load4<TY>(y + i, yv);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      xv[j] += dyt_f(yv[j], ap, w1[j], b1[j]);
      hv[j] = dyt_f(xv[j], an, wn[j], bn[j]);
    }
    store4<float>(x + i, xv);
    if (h) store4<TH>(h + i, hv);
  }
}

constexpr int kStrip = 16;   // rows per workgroup of the convolution

template <typename TO, int TAPS>
__global__ void __launch_bounds__(64)
dyt_canon_v4(const float* __restrict__ x, const float* __restrict__ w, const float* __restrict__ b,
             const float* __restrict__ alpha, const float* __restrict__ cw,
             const float* __restrict__ tail, TO* __restrict__ out, const int* __restrict__ cu,
             const int* __restrict__ slot, const int* __restrict__ start,
             const int* __restrict__ row_seg, int T, int W) {
  constexpr int K = TAPS - 1;
  const int c = 4 * (blockIdx.x * 64 + threadIdx.x);
  if (c >= W) return;
  const float a = *alpha;
  float wv[4], bv[4], cwv[4][TAPS];
  load4<float>(w + c, wv);
  load4<float>(b + c, bv);
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int q = 0; q < TAPS; ++q) cwv[j][q] = cw[(long long)(c + j) * TAPS + q];
  float win[K > 0 ? K : 1][4];        // win[d - 1]: the normed row d positions back
  const int r0 = blockIdx.y * kStrip, r1 = min(T, r0 + kStrip);
  int cur = -1;
  for (int t = r0; t < r1; ++t) {
    const int sg = row_seg[t];
    const long long i = (long long)t * W + c;
    if (sg != cur) {                   // strip start or a new segment: rebuild the window
      cur = sg;
      const int local = t - cu[sg], p0 = start[sg];
#pragma unroll
      for (int d = 1; d <= K; ++d) {
        const int src = local - d;
        float hv[4] = {0.f, 0.f, 0.f, 0.f};
        if (src >= 0) {
          load4<float>(x + i - (long long)d * W, hv);
#pragma unroll
          for (int j = 0; j < 4; ++j) hv[j] = dyt_f(hv[j], a, wv[j], bv[j]);
        } else if (p0 + src >= 0) {
          load4<float>(tail + ((long long)slot[sg] * K + (K + src)) * W + c, hv);
        }
#pragma unroll
        for (int j = 0; j < 4; ++j) win[d - 1][j] = hv[j];
      }
    }
    float hc[4], o[4];
    load4<float>(x + i, hc);
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      hc[j] = dyt_f(hc[j], a, wv[j], bv[j]);
      float acc = cwv[j][K] * hc[j];
#pragma unroll
      for (int d = 1; d <= K; ++d) acc += cwv[j][K - d] * win[d - 1][j];
      o[j] = hc[j] + acc;
    }
    store4<TO>(out + i, o);
#pragma unroll
    for (int d = K; d >= 2; --d)
#pragma unroll
      for (int j = 0; j < 4; ++j) win[d - 1][j] = win[d - 2][j];
    if (K > 0) {
#pragma unroll
      for (int j = 0; j < 4; ++j) win[0][j] = hc[j];
    }
  }
}

template <typename T>
__global__ void __launch_bounds__(256)
token_shift_v4(const T* __restrict__ h, const float* __restrict__ mu, const float* __restrict__ prev,
               T* __restrict__ out, const int* __restrict__ cu, const int* __restrict__ slot,
               const int* __restrict__ start, const int* __restrict__ row_seg, int Tn, int W,
               int nmix) {
  const int c = 4 * (blockIdx.x * 256 + threadIdx.x);
  if (c >= W) return;
  const long long n = (long long)Tn * W;
  for (int t = blockIdx.y; t < Tn; t += gridDim.y) {
    const int sg = row_seg[t];
    const long long i = (long long)t * W + c;
    float hv[4], pv[4] = {0.f, 0.f, 0.f, 0.f};
    load4<T>(h + i, hv);
    if (t > cu[sg]) load4<T>(h + i - W, pv);
    else if (start[sg] > 0) load4<float>(prev + (long long)slot[sg] * W + c, pv);
    for (int s = 0; s < nmix; ++s) {
      float m4[4], o[4];
      load4<float>(mu + (long long)s * W + c, m4);
#pragma unroll
      for (int j = 0; j < 4; ++j) o[j] = hv[j] + (pv[j] - hv[j]) * m4[j];
      store4<T>(out + (long long)s * n + i, o);
    }
  }
}

inline int grid_for(long long n, int block = 256) {
  long long g = (n + block - 1) / block;
  return (int)(g < 1 ? 1 : (g > 65536 ? 65536 : g));
}

}  // namespace

extern "C" {

hipError_t sm_dyt(int dt_in, int dt_out, const void* x, const float* w, const float* b,
                  const float* alpha, void* out, int rows, int W, hipStream_t st) {
  const long long n = (long long)rows * W;
  if (n == 0) return hipSuccess;
  if (dt_in != kF32) return hipErrorInvalidValue;
#define CALL(T) dyt_kernel<float, T><<<grid_for(n), 256, 0, st>>>((const float*)x, w, b, alpha, (T*)out, n, W)
  SM_DISPATCH(dt_out, CALL)
#undef CALL
  return hipGetLastError();
}

hipError_t sm_dyt_residual(int dt_y, int dt_h, float* x, const void* y, const float* pw,
                           const float* pb, const float* pa, void* h, const float* w2,
                           const float* b2, const float* a2, int T, int W, hipStream_t st) {
  const long long n = (long long)T * W;
  if (n == 0) return hipSuccess;
  if (h && dt_h != dt_y) return hipErrorInvalidValue;
  if (W % 4 == 0) {
    const dim3 grid((W / 4 + 255) / 256, T < 65535 ? T : 65535);
#define CALL(TT) dyt_residual_v4<TT, TT><<<grid, 256, 0, st>>>(x, (const TT*)y, pw, pb, pa, (TT*)h, w2, b2, a2, T, W)
    SM_DISPATCH(dt_y, CALL)
#undef CALL
    return hipGetLastError();
  }
#define CALL(TT) dyt_residual_kernel<TT, TT><<<grid_for(n), 256, 0, st>>>(x, (const TT*)y, pw, pb, pa, (TT*)h, w2, b2, a2, n, W)
  SM_DISPATCH(dt_y, CALL)
#undef CALL
  return hipGetLastError();
}

hipError_t sm_dyt_canon(int dt, const float* x, const float* w, const float* b, const float* alpha,
                        const float* cw, const float* tail, void* out, const int* cu,
                        const int* slot, const int* start, const int* row_seg, int T, int W,
                        int taps, hipStream_t st) {
  if ((long long)T * W == 0) return hipSuccess;
  if (taps < 1 || taps > kMaxTaps) return hipErrorInvalidValue;
  if (W % 4 == 0 && taps <= 8) {
    const dim3 grid((W / 4 + 63) / 64, (T + kStrip - 1) / kStrip);
#define GO(TT, TP) dyt_canon_v4<TT, TP><<<grid, 64, 0, st>>>(x, w, b, alpha, cw, tail, (TT*)out, cu, slot, start, row_seg, T, W)
#define CALL(TT)                                                                     \
    switch (taps) {                                                                  \
      case 1: GO(TT, 1); break; case 2: GO(TT, 2); break; case 3: GO(TT, 3); break;  \
      case 4: GO(TT, 4); break; case 5: GO(TT, 5); break; case 6: GO(TT, 6); break;  \
      case 7: GO(TT, 7); break; default: GO(TT, 8); break;                           \
    }
    SM_DISPATCH(dt, CALL)
#undef CALL
#undef GO
    return hipGetLastError();
  }
#define CALL(TT) dyt_canon_kernel<TT><<<grid_for((long long)T * W), 256, 0, st>>>(x, w, b, alpha, cw, tail, (TT*)out, cu, slot, start, row_seg, T, W, taps)
  SM_DISPATCH(dt, CALL)
#undef CALL
  return hipGetLastError();
}

hipError_t sm_canon_tail(const float* x, const float* w, const float* b, const float* alpha,
                         float* tail, const int* cu, const int* slot, const int* start, int S,
                         int W, int taps, hipStream_t st) {
  if ((long long)S * W == 0 || taps <= 1) return hipSuccess;
  if (taps > kMaxTaps) return hipErrorInvalidValue;
  canon_tail_kernel<<<grid_for((long long)S * W), 256, 0, st>>>(x, w, b, alpha, tail, cu, slot,
                                                                 start, S, W, taps);
  return hipGetLastError();
}

hipError_t sm_token_shift(int dt, const void* h, const float* mu, const float* prev, void* out,
                          const int* cu, const int* slot, const int* start, const int* row_seg,
                          int T, int W, int nmix, hipStream_t st) {
  if ((long long)T * W == 0) return hipSuccess;
  if (W % 4 == 0) {
    const dim3 grid((W / 4 + 255) / 256, T < 65535 ? T : 65535);
#define CALL(TT) token_shift_v4<TT><<<grid, 256, 0, st>>>((const TT*)h, mu, prev, (TT*)out, cu, slot, start, row_seg, T, W, nmix)
    SM_DISPATCH(dt, CALL)
#undef CALL
    return hipGetLastError();
  }
#define CALL(TT) token_shift_kernel<TT><<<grid_for((long long)T * W), 256, 0, st>>>((const TT*)h, mu, prev, (TT*)out, cu, slot, start, row_seg, T, W, nmix)
  SM_DISPATCH(dt, CALL)
#undef CALL
  return hipGetLastError();
}

hipError_t sm_shift_tail(int dt, const void* h, float* prev, const int* cu, const int* slot, int S,
                         int W, hipStream_t st) {
  if ((long long)S * W == 0) return hipSuccess;
#define CALL(TT) shift_tail_kernel<TT><<<grid_for((long long)S * W), 256, 0, st>>>((const TT*)h, prev, cu, slot, S, W)
  SM_DISPATCH(dt, CALL)
#undef CALL
  return hipGetLastError();
}

}  // extern "C"
