// Attention of the hybrid stack over a paged cache of un-normalised keys that double as values:
//   score(i, j) = scale * (q_i / rms(q_i)) . (k_j / rms(k_j)),   j <= i, same chunk as i
//   p_j = exp(s_j) / (sink + sum_j' exp(s_j')),   o_i = sum_j p_j k_j
// `chunk` > 0 restricts row i to keys with j / chunk == i / chunk (positions in the sequence);
// `sink` adds a key of score 0 that carries no value, i.e. the running softmax starts from
// (max 0, denominator 1) instead of (-inf, 0).
//
// One wave per (row, query head), for prefill chunks and decode rows alike (a row is a row: its
// position and its segment's block table say which keys it sees, so the result cannot depend on
// how the step was cut).  Keys are visited 64 at a time: lane l scores key j0 + l -- the dot
// product and the key's sum of squares come from the same 16-byte loads -- then the wave takes
// the tile's max and sum (online softmax), and for the value pass lane l owns channels l, l + 64,
// ... of the output and walks the tile's keys (coalesced rows).  Scores, norms and the softmax
// are fp32.  The mask bounds a row's keys by `chunk`, so decode reads at most chunk keys and a
// split over the keys is not needed.
#include "seqmix.h"

using namespace lumen;

namespace {

constexpr int kMaxD = 256;

template <typename T>
__global__ void __launch_bounds__(64)
chunk_attn_kernel(const T* __restrict__ q, long long ldq, const T* __restrict__ cache,
                  T* __restrict__ out, const int* __restrict__ tables, int maxb,
                  const int* __restrict__ row_seg, const int* __restrict__ positions, int H, int G,
                  int D, int bs, float scale, float eps, int chunk, int sink) {
  const int t = blockIdx.x, hd = blockIdx.y, lane = threadIdx.x;
  const int g = hd / (H / G);
  const int pos = positions[t];
  const int* tbl = tables + (long long)row_seg[t] * maxb;
  const int lo = chunk > 0 ? (pos / chunk) * chunk : 0;
  __shared__ float s_q[kMaxD];
  __shared__ float s_p[64];
  __shared__ long long s_row[64];

  float ss = 0.f;
  for (int d = lane; d < D; d += 64) {
    const float v = to_f32(q[(long long)t * ldq + hd * D + d]);
    s_q[d] = v;
    ss += v * v;
  }
  ss = wave_sum(ss);
  const float qn = scale / sqrtf(ss / D + eps);
  __syncthreads();

  float m = sink ? 0.f : -INFINITY, l = sink ? 1.f : 0.f;
  float acc[kMaxD / 64] = {0.f, 0.f, 0.f, 0.f};
  const bool vec = (D % 8) == 0;
  for (int j0 = lo; j0 <= pos; j0 += 64) {
    const int j = j0 + lane;
    const bool valid = j <= pos;
    float s = -INFINITY;
    long long rowoff = 0;
    if (valid) {
      rowoff = (((long long)tbl[j / bs] * bs + j % bs) * G + g) * D;
      const T* kp = cache + rowoff;
      float dot = 0.f, k2 = 0.f;
      if (vec) {
        for (int d = 0; d < D; d += 8) {
          float kv[8];
          load8<T>(kp + d, kv);
#pragma unroll
          for (int e = 0; e < 8; ++e) { dot += s_q[d + e] * kv[e]; k2 += kv[e] * kv[e]; }
        }
      } else {
        for (int d = 0; d < D; ++d) {
          const float kv = to_f32(kp[d]);
          dot += s_q[d] * kv;
          k2 += kv * kv;
        }
      }
      s = dot * qn / sqrtf(k2 / D + eps);
    }
    const float mn = fmaxf(m, wave_max(s));
    const float p = valid ? expf(s - mn) : 0.f;
    const float corr = expf(m - mn);       // m = -inf only before the first tile without a sink
    l = l * corr + wave_sum(p);
    m = mn;
    s_p[lane] = p;
    s_row[lane] = rowoff;
    __syncthreads();
    const int nk = min(64, pos - j0 + 1);
#pragma unroll
    for (int c = 0; c < kMaxD / 64; ++c) acc[c] *= corr;
    for (int jj = 0; jj < nk; ++jj) {
      const float pj = s_p[jj];
      const T* kp = cache + s_row[jj];
#pragma unroll
      for (int c = 0; c < kMaxD / 64; ++c) {
        const int d = lane + 64 * c;
        if (d < D) acc[c] += pj * to_f32(kp[d]);
      }
    }
    __syncthreads();
  }
  const float inv = 1.f / l;
#pragma unroll
  for (int c = 0; c < kMaxD / 64; ++c) {
    const int d = lane + 64 * c;
    if (d < D) out[((long long)t * H + hd) * D + d] = from_f32<T>(acc[c] * inv);
  }
}

}  // namespace

extern "C" {

hipError_t sm_chunk_attn(int dt, const void* q, long long ldq, const void* cache, void* out,
                         const int* tables, int maxb, const int* row_seg, const int* positions,
                         int T, int H, int G, int D, int bs, float scale, float eps, int chunk,
                         int sink, hipStream_t st) {
  if (T == 0) return hipSuccess;
  if (D < 1 || D > kMaxD || G < 1 || H % G || bs < 1 || chunk < 0) return hipErrorInvalidValue;
  const dim3 grid(T, H);
#define CALL(TT) chunk_attn_kernel<TT><<<grid, 64, 0, st>>>((const TT*)q, ldq, (const TT*)cache, (TT*)out, tables, maxb, row_seg, positions, H, G, D, bs, scale, eps, chunk, sink)
  SM_DISPATCH(dt, CALL)
#undef CALL
  return hipGetLastError();
}

}  // extern "C"
