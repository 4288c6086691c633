// Linear-recurrence scans with a matrix state per (sequence, head): RWKV-style `wkv` and the
// generalised delta rule.  One workgroup per (segment, head).  The state S [key channel i, value
// channel j] lives in registers for the whole segment: KS adjacent lanes share column j, each
// holding KT consecutive key channels of it, so the rank-one updates are private FMAs and the
// two reductions over i (the read-out S^T r, and the delta rule's u^T S) are KT FMAs plus
// log2(KS) lane exchanges inside the lane group:
//     wkv    o_j = sum_i r_i S_ij + v_j sum_i r_i u_i k_i ;   S_ij <- w_i S_ij + k_i v_j
//     delta  c_j = sum_i un_i S_ij ;  S_ij <- w_i S_ij - (a_i un_i) c_j + k_i v_j ;  o_j = sum_i r_i S_ij
// Splitting the key channels over lanes (rather than one lane per column) gives head size 128
// eight waves per workgroup instead of two and a quarter of the serial FMA chain per token.
// The per-token vectors over the key channel (r, k, decay, removal) are the same for every
// column: a batch of TB tokens is staged in LDS (fp32; decays, sigmoids and the unit key computed
// while staging) and read back as 16-byte broadcasts; each lane group's slice is padded by four
// floats so the KS slices of a wave fall into different banks.  The read-outs of the batch are
// then normalised per head (RMS over the value channels), scaled by the channel weight and the
// output gate, and stored in the compute dtype.  Sequential in time by construction: parallelism
// is segments x heads workgroups, which fills the chip for decode batches and mixed steps; a
// single long prompt runs on `heads` workgroups (the chunk-parallel matrix form is the known
// faster shape for that case).
// State in HBM: [slot, head, i, j] fp32; a segment starting at position 0 starts from zero.
#include "seqmix.h"

using namespace lumen;

namespace {

constexpr int TB = 8;   // tokens staged per batch

template <typename T, int KT, int KS, bool DELTA>
__global__ void __launch_bounds__(1024)
scan_kernel(const T* __restrict__ r, long long ldr, const T* __restrict__ k, long long ldk,
            const T* __restrict__ v, long long ldv, const T* __restrict__ wl, long long ldw,
            const T* __restrict__ al, long long lda, const T* __restrict__ gl, long long ldg,
            const float* __restrict__ w0, const float* __restrict__ ub,  // u (wkv) / a bias (delta)
            const float* __restrict__ normw, float* __restrict__ state, T* __restrict__ out,
            long long ldo, const int* __restrict__ cu, const int* __restrict__ slot,
            const int* __restrict__ start, int H, int D, float eps, float decay_scale,
            float key_eps) {
  constexpr int DK = KT * KS;          // padded key size
  constexpr int LS = KT + 4;           // LDS stride of one lane group's slice
  const int sg = blockIdx.x, hd = blockIdx.y;
  const int r0 = cu[sg], L = cu[sg + 1] - r0;
  if (L <= 0) return;
  const int tid = threadIdx.x, NT = blockDim.x;
  const int j = tid / KS, p = tid % KS;
  const bool active = j < D;
  const int col = hd * D;
  __shared__ __align__(16) float s_r[TB * KS * LS], s_k[TB * KS * LS], s_w[TB * KS * LS],
      s_x[TB * KS * LS];                                   // s_x: u (wkv) / a * un (delta)
  __shared__ __align__(16) float s_un[DELTA ? TB * KS * LS : 4];
  __shared__ float s_o[TB][DK];
  __shared__ float s_tok[TB];   // wkv: sum_i r_i u_i k_i ; delta: 1 / sqrt(sum k^2 + eps)
  auto at = [](int tb, int i) { return (tb * KS + i / KT) * LS + i % KT; };

  float S[KT];
  float* sp = state + ((long long)slot[sg] * H + hd) * D * D;
  const bool fresh = start[sg] == 0;
#pragma unroll
  for (int ii = 0; ii < KT; ++ii) {
    const int i = p * KT + ii;
    S[ii] = (!fresh && active && i < D) ? sp[(long long)i * D + j] : 0.f;
  }

  for (int t0 = 0; t0 < L; t0 += TB) {
    const int nb = min(TB, L - t0);
    // ---- stage the batch's key-channel vectors (zero-padded to DK) ----
    for (int idx = tid; idx < nb * DK; idx += NT) {
      const int tb = idx / DK, i = idx % DK;
      const long long row = r0 + t0 + tb;
      float rv = 0.f, kv = 0.f, wv = 0.f, xv = 0.f;
      if (i < D) {
        rv = to_f32(r[row * ldr + col + i]);
        kv = to_f32(k[row * ldk + col + i]);
        const float z = to_f32(wl[row * ldw + col + i]) + w0[col + i];
        if (DELTA) {
          wv = expf(-decay_scale * sigmoid_f(z));
          xv = sigmoid_f(to_f32(al[row * lda + col + i]) + ub[col + i]);
        } else {
          wv = expf(-expf(z));
          xv = ub[col + i];
        }
      }
      const int a = at(tb, i);
      s_r[a] = rv; s_k[a] = kv; s_w[a] = wv; s_x[a] = xv;
    }
    __syncthreads();
    {                                   // per-token scalars: one wave per token
      const int lane = tid & 63, wv_ = tid >> 6, nw = NT >> 6;
      for (int tb = wv_; tb < nb; tb += nw) {
        float acc = 0.f;
        for (int i = lane; i < D; i += 64) {
          const int a = at(tb, i);
          acc += DELTA ? s_k[a] * s_k[a] : s_r[a] * s_x[a] * s_k[a];
        }
        acc = wave_sum(acc);
        if (lane == 0) s_tok[tb] = DELTA ? 1.f / sqrtf(acc + key_eps) : acc;
      }
    }
    __syncthreads();
    if (DELTA) {
      for (int idx = tid; idx < nb * DK; idx += NT) {
        const int tb = idx / DK, a = at(tb, idx % DK);
        const float un = s_k[a] * s_tok[tb];
        s_un[a] = un;
        s_x[a] *= un;
      }
      __syncthreads();
    }
    // ---- the recurrence over the batch (lane group of column j, slice p) ----
    if (active) {
      for (int tb = 0; tb < nb; ++tb) {
        const float vj = to_f32(v[(long long)(r0 + t0 + tb) * ldv + col + j]);
        const int base = (tb * KS + p) * LS;
        float o = 0.f;
        if (DELTA) {
          float c = 0.f;
#pragma unroll
          for (int ii = 0; ii < KT; ii += 4) {
            const float4 u4 = *reinterpret_cast<const float4*>(&s_un[base + ii]);
            c += u4.x * S[ii] + u4.y * S[ii + 1] + u4.z * S[ii + 2] + u4.w * S[ii + 3];
          }
#pragma unroll
          for (int m = 1; m < KS; m <<= 1) c += __shfl_xor(c, m, 64);
#pragma unroll
          for (int ii = 0; ii < KT; ii += 4) {
            const float4 w4 = *reinterpret_cast<const float4*>(&s_w[base + ii]);
            const float4 x4 = *reinterpret_cast<const float4*>(&s_x[base + ii]);
            const float4 k4 = *reinterpret_cast<const float4*>(&s_k[base + ii]);
            const float4 r4 = *reinterpret_cast<const float4*>(&s_r[base + ii]);
            S[ii] = w4.x * S[ii] - x4.x * c + k4.x * vj;
            S[ii + 1] = w4.y * S[ii + 1] - x4.y * c + k4.y * vj;
            S[ii + 2] = w4.z * S[ii + 2] - x4.z * c + k4.z * vj;
            S[ii + 3] = w4.w * S[ii + 3] - x4.w * c + k4.w * vj;
            o += r4.x * S[ii] + r4.y * S[ii + 1] + r4.z * S[ii + 2] + r4.w * S[ii + 3];
          }
        } else {
#pragma unroll
          for (int ii = 0; ii < KT; ii += 4) {
            const float4 w4 = *reinterpret_cast<const float4*>(&s_w[base + ii]);
            const float4 k4 = *reinterpret_cast<const float4*>(&s_k[base + ii]);
            const float4 r4 = *reinterpret_cast<const float4*>(&s_r[base + ii]);
            o += r4.x * S[ii] + r4.y * S[ii + 1] + r4.z * S[ii + 2] + r4.w * S[ii + 3];
            S[ii] = w4.x * S[ii] + k4.x * vj;
            S[ii + 1] = w4.y * S[ii + 1] + k4.y * vj;
            S[ii + 2] = w4.z * S[ii + 2] + k4.z * vj;
            S[ii + 3] = w4.w * S[ii + 3] + k4.w * vj;
          }
        }
#pragma unroll
        for (int m = 1; m < KS; m <<= 1) o += __shfl_xor(o, m, 64);
        if (!DELTA) o += s_tok[tb] * vj;
        if (p == 0) s_o[tb][j] = o;
      }
    }
    __syncthreads();
    // ---- per-head RMS norm, channel weight, output gate: one wave per token ----
    const int lane = tid & 63, wv_ = tid >> 6, nw = NT >> 6;
    for (int tb = wv_; tb < nb; tb += nw) {
      float ss = 0.f;
      for (int c = lane; c < D; c += 64) ss += s_o[tb][c] * s_o[tb][c];
      ss = wave_sum(ss);
      const float rs = 1.f / sqrtf(ss / D + eps);
      const long long row = r0 + t0 + tb;
      for (int c = lane; c < D; c += 64) {
        const float g = to_f32(gl[row * ldg + col + c]);
        const float gate = DELTA ? sigmoid_f(g) : silu_f(g);
        out[row * ldo + col + c] = from_f32<T>(s_o[tb][c] * rs * normw[col + c] * gate);
      }
    }
    __syncthreads();
  }
  if (active) {
#pragma unroll
    for (int ii = 0; ii < KT; ++ii) {
      const int i = p * KT + ii;
      if (i < D) sp[(long long)i * D + j] = S[ii];
    }
  }
}

template <typename T, bool DELTA>
hipError_t launch_scan(const void* r, long long ldr, const void* k, long long ldk, const void* v,
                       long long ldv, const void* wl, long long ldw, const void* al,
                       long long lda, const void* gl, long long ldg, const float* w0,
                       const float* ub, const float* normw, float* state, void* out,
                       long long ldo, const int* cu, const int* slot, const int* start, int S,
                       int H, int D, float eps, float decay_scale, float key_eps,
                       hipStream_t st) {
  if (S == 0) return hipSuccess;
  if (D < 1 || D > 256) return hipErrorInvalidValue;
  const dim3 grid(S, H);
#define GO(KT, KS)                                                                               \
  scan_kernel<T, KT, KS, DELTA><<<grid, ((D * KS + 63) / 64) * 64, 0, st>>>(                     \
      (const T*)r, ldr, (const T*)k, ldk, (const T*)v, ldv, (const T*)wl, ldw, (const T*)al, lda, \
      (const T*)gl, ldg, w0, ub, normw, state, (T*)out, ldo, cu, slot, start, H, D, eps,         \
      decay_scale, key_eps)
  if (D <= 32) GO(16, 2);
  else if (D <= 64) GO(16, 4);
  else if (D <= 128) GO(32, 4);
  else GO(64, 4);
#undef GO
  return hipGetLastError();
}

}  // namespace

extern "C" {

hipError_t sm_wkv(int dt, const void* r, long long ldr, const void* k, long long ldk,
                  const void* v, long long ldv, const void* wl, long long ldw, const void* g,
                  long long ldg, const float* w0, const float* u, const float* normw,
                  float* state, void* out, long long ldo, const int* cu, const int* slot,
                  const int* start, int S, int H, int D, float eps, hipStream_t st) {
#define CALL(T) return launch_scan<T, false>(r, ldr, k, ldk, v, ldv, wl, ldw, nullptr, 0, g, ldg, w0, u, normw, state, out, ldo, cu, slot, start, S, H, D, eps, 0.f, 0.f, st)
  SM_DISPATCH(dt, CALL)
#undef CALL
  return hipSuccess;
}

hipError_t sm_gdelta(int dt, const void* r, long long ldr, const void* k, long long ldk,
                     const void* v, long long ldv, const void* wl, long long ldw, const void* al,
                     long long lda, const void* gl, long long ldg, const float* w0,
                     const float* a_b, const float* normw, float* state, void* out,
                     long long ldo, const int* cu, const int* slot, const int* start, int S,
                     int H, int D, float eps, float decay_scale, float key_eps, hipStream_t st) {
#define CALL(T) return launch_scan<T, true>(r, ldr, k, ldk, v, ldv, wl, ldw, al, lda, gl, ldg, w0, a_b, normw, state, out, ldo, cu, slot, start, S, H, D, eps, decay_scale, key_eps, st)
  SM_DISPATCH(dt, CALL)
#undef CALL
  return hipSuccess;
}

}  // extern "C"
