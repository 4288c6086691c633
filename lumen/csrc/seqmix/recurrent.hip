// Linear-recurrence scans with a matrix state per (sequence, head): RWKV-style `wkv` and the
// generalised delta rule.  One workgroup per (segment, head); thread j owns COLUMN j of the
// state S [key channel i, value channel j] in registers (DK fp32 values), so the rank-one
// updates and the read-out S^T r are private FMAs with no cross-lane traffic:
//     wkv    o_j = sum_i r_i S_ij + v_j sum_i r_i u_i k_i ;   S_ij <- w_i S_ij + k_i v_j
//     delta  c_j = sum_i un_i S_ij ;  S_ij <- w_i S_ij - (a_i un_i) c_j + k_i v_j ;  o_j = sum_i r_i S_ij
// The per-token vectors over the key channel (r, k, decay, removal) are the same for every
// thread: a batch of TB tokens is staged in LDS (fp32, decays / sigmoids / the unit key computed
// while staging) and read back as broadcasts.  The read-outs of the batch are then normalised
// per head (RMS over the value channels), scaled by the channel weight and the output gate, and
// stored in the compute dtype.  Sequential in time by construction: parallelism is segments x
// heads workgroups, which fills the chip for decode batches and mixed steps; a single long
// prompt runs on `heads` workgroups (the chunk-parallel matrix form is the known faster shape
// for that case).
// State in HBM: [slot, head, i, j] fp32; a segment starting at position 0 starts from zero.
#include "seqmix.h"

using namespace lumen;

namespace {

constexpr int TB = 8;   // tokens staged per batch

template <typename T, int DK, bool DELTA>
__global__ void __launch_bounds__(256)
scan_kernel(const T* __restrict__ r, long long ldr, const T* __restrict__ k, long long ldk,
            const T* __restrict__ v, long long ldv, const T* __restrict__ wl, long long ldw,
            const T* __restrict__ al, long long lda, const T* __restrict__ gl, long long ldg,
            const float* __restrict__ w0, const float* __restrict__ ub,  // u (wkv) / a bias (delta)
            const float* __restrict__ normw, float* __restrict__ state, T* __restrict__ out,
            long long ldo, const int* __restrict__ cu, const int* __restrict__ slot,
            const int* __restrict__ start, int H, int D, float eps, float decay_scale,
            float key_eps) {
  const int sg = blockIdx.x, hd = blockIdx.y;
  const int r0 = cu[sg], L = cu[sg + 1] - r0;
  if (L <= 0) return;
  const int j = threadIdx.x, NT = blockDim.x;
  const int col = hd * D;
  __shared__ float s_r[TB][DK], s_k[TB][DK], s_w[TB][DK], s_x[TB][DK];  // s_x: a*un (delta)
  __shared__ float s_un[DELTA ? TB : 1][DELTA ? DK : 1];
  __shared__ float s_o[TB][DK];
  __shared__ float s_tok[TB];   // wkv: sum_i r_i u_i k_i ; delta: 1 / sqrt(sum k^2 + eps)

  float S[DK];
  float* sp = state + ((long long)slot[sg] * H + hd) * D * D;
  const bool fresh = start[sg] == 0;
#pragma unroll
  for (int i = 0; i < DK; ++i)
    S[i] = (!fresh && i < D && j < D) ? sp[(long long)i * D + j] : 0.f;

  for (int t0 = 0; t0 < L; t0 += TB) {
    const int nb = min(TB, L - t0);
    // ---- stage the batch's key-channel vectors (zero-padded to DK) ----
    for (int idx = j; idx < nb * DK; idx += NT) {
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
      s_r[tb][i] = rv; s_k[tb][i] = kv; s_w[tb][i] = wv; s_x[tb][i] = xv;
    }
    __syncthreads();
    if (j < nb) {                       // per-token scalars, one thread each
      float acc = 0.f;
      for (int i = 0; i < D; ++i)
        acc += DELTA ? s_k[j][i] * s_k[j][i] : s_r[j][i] * s_x[j][i] * s_k[j][i];
      s_tok[j] = DELTA ? 1.f / sqrtf(acc + key_eps) : acc;
    }
    __syncthreads();
    if (DELTA) {
      for (int idx = j; idx < nb * DK; idx += NT) {
        const int tb = idx / DK, i = idx % DK;
        const float un = s_k[tb][i] * s_tok[tb];
        s_un[tb][i] = un;
        s_x[tb][i] *= un;
      }
      __syncthreads();
    }
    // ---- the recurrence over the batch (thread j: column j) ----
    if (j < D) {
      for (int tb = 0; tb < nb; ++tb) {
        const float vj = to_f32(v[(long long)(r0 + t0 + tb) * ldv + col + j]);
        float o = 0.f;
        if (DELTA) {
          float c = 0.f;
#pragma unroll
          for (int i = 0; i < DK; ++i) c += s_un[tb][i] * S[i];
#pragma unroll
          for (int i = 0; i < DK; ++i) {
            S[i] = s_w[tb][i] * S[i] - s_x[tb][i] * c + s_k[tb][i] * vj;
            o += s_r[tb][i] * S[i];
          }
        } else {
#pragma unroll
          for (int i = 0; i < DK; ++i) {
            o += s_r[tb][i] * S[i];
            S[i] = s_w[tb][i] * S[i] + s_k[tb][i] * vj;
          }
          o += s_tok[tb] * vj;
        }
        s_o[tb][j] = o;
      }
    }
    __syncthreads();
    // ---- per-head RMS norm, channel weight, output gate: one wave per token ----
    const int lane = j & 63, wv_ = j >> 6, nw = NT >> 6;
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
  if (j < D) {
#pragma unroll
    for (int i = 0; i < DK; ++i)
      if (i < D) sp[(long long)i * D + j] = S[i];
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
  const int nt = ((D + 63) / 64) * 64;
#define GO(DK)                                                                                   \
  scan_kernel<T, DK, DELTA><<<grid, nt, 0, st>>>(                                                \
      (const T*)r, ldr, (const T*)k, ldk, (const T*)v, ldv, (const T*)wl, ldw, (const T*)al, lda, \
      (const T*)gl, ldg, w0, ub, normw, state, (T*)out, ldo, cu, slot, start, H, D, eps,         \
      decay_scale, key_eps)
  if (D <= 32) GO(32);
  else if (D <= 64) GO(64);
  else if (D <= 128) GO(128);
  else GO(256);
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
