// RMS norms in groups, fused with what surrounds them:
//   sm_group_rms   v = x / sqrt(mean_g(x^2) + eps) * w, the row split into `groups` equal
//                  consecutive parts that are each divided by their OWN root mean square
//                  (groups = 1: the ordinary RMS norm).  Without a residual the result is stored
//                  in the output dtype; with one, the fp32 residual row takes it in place,
//                  res += v, and -- optionally -- the new row is also stored rounded to the model
//                  dtype (the input of the next sublayer's GEMMs).
//   sm_gate_rows   out[t, d] = gelu_tanh(z[t, d]) * table[token[t], col0 + d]: a slice of a
//                  per-token embedding row gated by a projection of the stream.
// One workgroup of four waves per row.  With four or more groups a wave owns a group (and walks
// the groups four at a time); with fewer, 4 / groups waves share one and add their partial sums in
// a fixed order, so the result never depends on timing.  Sums, roots and products are fp32.
#include "seqmix.h"

using namespace lumen;

namespace {

template <typename TI, typename TO, bool VEC>
__global__ void __launch_bounds__(256)
group_rms_kernel(const TI* __restrict__ x, long long ldx, const float* __restrict__ w,
                 float* __restrict__ res, TO* __restrict__ out, long long ldo, int W, int groups,
                 float eps) {
  const int r = blockIdx.x, lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
  const int gs = W / groups;
  const int wpg = groups >= 4 ? 1 : groups == 1 ? 4 : groups == 2 ? 2 : 1;   // waves per group
  const int per_pass = 4 / wpg;
  const int slot = wv / wpg, sub = wv % wpg;
  const TI* xr = x + (long long)r * ldx;
  __shared__ float s_part[4];
  constexpr int V = VEC ? 4 : 1;
  for (int g0 = 0; g0 < groups; g0 += per_pass) {
    const int g = g0 + slot;
    const bool on = g < groups && slot < per_pass;
    float ss = 0.f;
    if (on) {
      for (int c = (sub * 64 + lane) * V; c < gs; c += wpg * 64 * V) {
        if (VEC) {
          float v[4];
          load4<TI>(xr + g * gs + c, v);
          ss += v[0] * v[0] + v[1] * v[1] + v[2] * v[2] + v[3] * v[3];
        } else {
          const float v = to_f32(xr[g * gs + c]);
          ss += v * v;
        }
      }
    }
    ss = wave_sum(ss);
    if (lane == 0) s_part[wv] = ss;
    __syncthreads();
    if (on) {
      float tot = 0.f;
      for (int k = 0; k < wpg; ++k) tot += s_part[slot * wpg + k];
      const float inv = 1.f / sqrtf(tot / (float)gs + eps);
      for (int c = (sub * 64 + lane) * V; c < gs; c += wpg * 64 * V) {
        const int col = g * gs + c;
        if (VEC) {
          float v[4], ww[4];
          load4<TI>(xr + col, v);
          load4<float>(w + col, ww);
#pragma unroll
          for (int e = 0; e < 4; ++e) v[e] = v[e] * inv * ww[e];
          if (res) {
            float a[4];
            load4<float>(res + (long long)r * W + col, a);
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] += a[e];
            store4<float>(res + (long long)r * W + col, v);
          }
          if (out) store4<TO>(out + (long long)r * ldo + col, v);
        } else {
          float v = to_f32(xr[col]) * inv * w[col];
          if (res) {
            v += res[(long long)r * W + col];
            res[(long long)r * W + col] = v;
          }
          if (out) out[(long long)r * ldo + col] = from_f32<TO>(v);
        }
      }
    }
    __syncthreads();
  }
}

template <typename T>
__global__ void gate_rows_kernel(const T* __restrict__ z, long long ldz, const T* __restrict__ table,
                                 long long ldt, const long long* __restrict__ tokens, int col0,
                                 int dim, T* __restrict__ out, long long n) {
  for (long long i = blockIdx.x * (long long)blockDim.x + threadIdx.x; i < n;
       i += (long long)gridDim.x * blockDim.x) {
    const long long t = i / dim;
    const int d = (int)(i % dim);
    const float e = to_f32(table[tokens[t] * ldt + col0 + d]);
    out[i] = from_f32<T>(gelu_tanh_f(to_f32(z[t * ldz + d])) * e);
  }
}

template <typename TI, typename TO>
hipError_t launch_rms(const void* x, long long ldx, const float* w, float* res, void* out,
                      long long ldo, int rows, int W, int groups, float eps, hipStream_t st) {
  const int gs = W / groups;
  const bool vec = gs % 4 == 0 && ldx % 4 == 0 && ldo % 4 == 0 &&
                   ((uintptr_t)x % 16 == 0) && ((uintptr_t)out % 16 == 0);
  if (vec)
    group_rms_kernel<TI, TO, true><<<rows, 256, 0, st>>>((const TI*)x, ldx, w, res, (TO*)out, ldo,
                                                         W, groups, eps);
  else
    group_rms_kernel<TI, TO, false><<<rows, 256, 0, st>>>((const TI*)x, ldx, w, res, (TO*)out, ldo,
                                                          W, groups, eps);
  return hipGetLastError();
}

inline int grid_for(long long n, int block = 256) {
  const long long g = (n + block - 1) / block;
  return (int)(g < 1 ? 1 : g > 65535 ? 65535 : g);
}

}  // namespace

extern "C" {

// x [rows, W] (row stride ldx) in dtype dt_in (fp32 or the model dtype); out (nullable when res
// is given) [rows, W] (row stride ldo) in dtype dt_out; res (nullable) fp32 [rows, W] contiguous.
hipError_t sm_group_rms(int dt_in, int dt_out, const void* x, long long ldx, const float* w,
                        float* res, void* out, long long ldo, int rows, int W, int groups,
                        float eps, hipStream_t st) {
  if (rows == 0) return hipSuccess;
  if (groups < 1 || W % groups != 0 || (!res && !out)) return hipErrorInvalidValue;
#define CALL_O(TO)                                                                              \
  {                                                                                             \
    if (dt_in == kF32) return launch_rms<float, TO>(x, ldx, w, res, out, ldo, rows, W, groups,  \
                                                    eps, st);                                   \
    if (dt_in == kBF16) return launch_rms<bf16, TO>(x, ldx, w, res, out, ldo, rows, W, groups,  \
                                                    eps, st);                                   \
    if (dt_in == kF16) return launch_rms<fp16, TO>(x, ldx, w, res, out, ldo, rows, W, groups,   \
                                                   eps, st);                                    \
    return hipErrorInvalidValue;                                                                \
  }
  SM_DISPATCH(dt_out, CALL_O)
#undef CALL_O
  return hipGetLastError();
}

hipError_t sm_gate_rows(int dt, const void* z, long long ldz, const void* table, long long ldt,
                        const long long* tokens, int col0, int dim, void* out, int T,
                        hipStream_t st) {
  const long long n = (long long)T * dim;
  if (n == 0) return hipSuccess;
#define CALL(TT) gate_rows_kernel<TT><<<grid_for(n), 256, 0, st>>>((const TT*)z, ldz, (const TT*)table, ldt, tokens, col0, dim, (TT*)out, n)
  SM_DISPATCH(dt, CALL)
#undef CALL
  return hipGetLastError();
}

}  // extern "C"
