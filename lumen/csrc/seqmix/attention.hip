// Attention of the hybrid stack over a paged cache of un-normalised keys that double as values:
//   score(i, j) = scale * (q_i / rms(q_i)) . (k_j / rms(k_j)),   j <= i, same chunk as i
//   p_j = exp(s_j) / (sink + sum_j' exp(s_j')),   o_i = sum_j p_j k_j
// `chunk` > 0 restricts row i to keys with j / chunk == i / chunk (positions in the sequence);
// `sink` adds a key of score 0 that carries no value, i.e. the running softmax starts from
// (max 0, denominator 1) instead of (-inf, 0).
//
// Four waves per (row, query head), for prefill chunks and decode rows alike (a row is a row: its
// position and its segment's block table say which keys it sees, so the result cannot depend on
// how the step was cut).  The waves take the 64-key tiles in turn; within a tile lane l scores key j0 + l -- the dot
// product and the key's sum of squares come from the same 16-byte loads -- then the wave takes
// the tile's max and sum (online softmax), and for the value pass lane l owns channels l, l + 64,
// ... of the output and walks the tile's keys (coalesced rows).  Scores, norms and the softmax
// are fp32.  The mask bounds a row's keys by `chunk`, so decode reads at most chunk keys and a
// split over the keys is not needed.
#include "seqmix.h"

using namespace lumen;

namespace {

constexpr int kMaxD = 256;

constexpr int kRowWaves = 4;   // waves per (row, head): each takes every fourth 64-key tile

template <typename T>
__global__ void __launch_bounds__(64 * kRowWaves)
chunk_attn_kernel(const T* __restrict__ q, long long ldq, const T* __restrict__ cache,
                  T* __restrict__ out, const int* __restrict__ tables, int maxb,
                  const int* __restrict__ row_seg, const int* __restrict__ positions, int H, int G,
                  int D, int bs, float scale, float eps, int chunk, int sink) {
  const int t = blockIdx.x, hd = blockIdx.y, lane = threadIdx.x & 63, w = threadIdx.x >> 6;
  const int g = hd / (H / G);
  const int pos = positions[t];
  const int* tbl = tables + (long long)row_seg[t] * maxb;
  const int lo = chunk > 0 ? (pos / chunk) * chunk : 0;
  __shared__ float s_q[kMaxD];
  __shared__ float s_p[kRowWaves][64];
  __shared__ long long s_row[kRowWaves][64];
  __shared__ float s_acc[kRowWaves][kMaxD];
  __shared__ float s_m[kRowWaves], s_l[kRowWaves];

  float ss = 0.f;
  for (int d = lane; d < D; d += 64) {
    const float v = to_f32(q[(long long)t * ldq + hd * D + d]);
    if (w == 0) s_q[d] = v;
    ss += v * v;
  }
  ss = wave_sum(ss);
  const float qn = scale / sqrtf(ss / D + eps);
  __syncthreads();

  // every wave keeps its own running (max, sum, accumulator) over its tiles; wave 0 starts from
  // the sink, the others from nothing, and the partial results are merged at the end
  float m = (sink && w == 0) ? 0.f : -INFINITY, l = (sink && w == 0) ? 1.f : 0.f;
  float acc[kMaxD / 64] = {0.f, 0.f, 0.f, 0.f};
  float acc8[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
  const bool vec = (D % 8) == 0;
  const int lpk = vec ? D / 8 : 64, kpi = 64 / lpk;   // lanes per key row, keys per step
  const int grp = lane / lpk, part = lane % lpk;
  for (int j0 = lo + 64 * w; j0 <= pos; j0 += 64 * kRowWaves) {
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
    const float mn = fmaxf(m, wave_max(s));       // finite: the tile's first key is valid
    const float p = valid ? expf(s - mn) : 0.f;
    const float corr = expf(m - mn);
    l = l * corr + wave_sum(p);
    m = mn;
    s_p[w][lane] = p;
    s_row[w][lane] = rowoff;
    __builtin_amdgcn_wave_barrier();
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
    const int nk = min(64, pos - j0 + 1);
    if (vec) {
      // value pass, 16 bytes per lane: lpk = D / 8 lanes cover one key row, 64 / lpk keys per
      // step; a lane accumulates its 8 channels over the keys of its group, the groups are
      // summed once at the end
#pragma unroll
      for (int e = 0; e < 8; ++e) acc8[e] *= corr;
      if (grp < kpi) {
        for (int jj = grp; jj < nk; jj += kpi) {
          const float pj = s_p[w][jj];
          float kv[8];
          load8<T>(cache + s_row[w][jj] + 8 * part, kv);
#pragma unroll
          for (int e = 0; e < 8; ++e) acc8[e] += pj * kv[e];
        }
      }
    } else {
#pragma unroll
      for (int c = 0; c < kMaxD / 64; ++c) acc[c] *= corr;
      for (int jj = 0; jj < nk; ++jj) {
        const float pj = s_p[w][jj];
        const T* kp = cache + s_row[w][jj];
#pragma unroll
        for (int c = 0; c < kMaxD / 64; ++c) {
          const int d = lane + 64 * c;
          if (d < D) acc[c] += pj * to_f32(kp[d]);
        }
      }
    }
    __builtin_amdgcn_wave_barrier();
  }
  if (vec) {
    // sum the key groups of this wave: every group adds its channels into s_acc[w] in turn
    for (int d = lane; d < D; d += 64) s_acc[w][d] = 0.f;
    for (int gq = 0; gq < kpi; ++gq) {
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      if (grp == gq) {
#pragma unroll
        for (int e = 0; e < 8; ++e) s_acc[w][8 * part + e] += acc8[e];
      }
    }
  } else {
#pragma unroll
    for (int c = 0; c < kMaxD / 64; ++c) {
      const int d = lane + 64 * c;
      if (d < D) s_acc[w][d] = acc[c];
    }
  }
  if (lane == 0) { s_m[w] = m; s_l[w] = l; }
  __syncthreads();
  if (w == 0) {
    float mt = -INFINITY;
#pragma unroll
    for (int x = 0; x < kRowWaves; ++x) mt = fmaxf(mt, s_m[x]);
    float lt = 0.f, f[kRowWaves];
#pragma unroll
    for (int x = 0; x < kRowWaves; ++x) {
      f[x] = s_m[x] == -INFINITY ? 0.f : expf(s_m[x] - mt);
      lt += s_l[x] * f[x];
    }
    const float inv = 1.f / lt;
    for (int d = lane; d < D; d += 64) {
      float o = 0.f;
#pragma unroll
      for (int x = 0; x < kRowWaves; ++x) o += s_acc[x][d] * f[x];
      out[((long long)t * H + hd) * D + d] = from_f32<T>(o * inv);
    }
  }
}

// ---- prefill tiles on the matrix cores (16-bit dtypes, D a multiple of 32) ---------------------
// A workgroup of NW waves takes 32 * NW consecutive rows of ONE segment and one query head; the
// keys the tile can see (from the first row's chunk start to the last row's position) are
// visited 32 at a time, staged in LDS twice (row-major for the scores, transposed for the value
// pass) and shared by the waves.  Per wave (32 queries) and key tile, with v_mfma_f32_32x32x16:
//   S^T = K Q^T      keys on the accumulator rows, queries on the columns (lane & 31): a lane
//                    owns ONE query, so its running max / sum / correction are plain scalars;
//                    q and k enter un-normalised (exactly as projected) and the two RMS factors
//                    multiply the fp32 score (k's sum of squares comes from the operand the lane
//                    loads anyway);
//   O^T += V^T P^T   the accumulator registers 8s .. 8s+7 of S^T are keys {16s + 4hi + 0..3,
//                    16s + 8 + 4hi + 0..3}: exactly one k = 16 operand when the transposed key
//                    image is read in that order, so P goes from registers to the next product
//                    without touching LDS.  P is split into a 16-bit head and a 16-bit remainder
//                    (two products), which keeps ~16 mantissa bits of the fp32 weights.
// Accumulator layout of the 32x32 products: lane l, register 4j + i = row 8j + 4(l >> 5) + i,
// column l & 31; operand lanes hold k = 8(l >> 5) + 0..7.
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef __bf16 bf16x8v __attribute__((ext_vector_type(8)));
typedef _Float16 f16x8v __attribute__((ext_vector_type(8)));

template <typename T> struct Mma32;
template <> struct Mma32<bf16> {
  static __device__ __forceinline__ f32x16 run(uint4 a, uint4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8v, a),
                                                   __builtin_bit_cast(bf16x8v, b), c, 0, 0, 0);
  }
};
template <> struct Mma32<fp16> {
  static __device__ __forceinline__ f32x16 run(uint4 a, uint4 b, f32x16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8v, a),
                                                  __builtin_bit_cast(f16x8v, b), c, 0, 0, 0);
  }
};

// the two halves of a packed 16-bit pair as fp32 (bf16: a shift and a mask)
template <typename T> __device__ __forceinline__ void unpack2(unsigned v, float& a, float& b);
template <> __device__ __forceinline__ void unpack2<bf16>(unsigned v, float& a, float& b) {
  a = __uint_as_float(v << 16);
  b = __uint_as_float(v & 0xffff0000u);
}
template <> __device__ __forceinline__ void unpack2<fp16>(unsigned v, float& a, float& b) {
  const lumen_f16x2 h = __builtin_bit_cast(lumen_f16x2, v);
  a = static_cast<float>(h[0]);
  b = static_cast<float>(h[1]);
}

template <typename T>
__device__ __forceinline__ float sumsq8(uint4 v) {
  const unsigned w[4] = {v.x, v.y, v.z, v.w};
  float s = 0.f;
#pragma unroll
  for (int x = 0; x < 4; ++x) {
    float a, b;
    unpack2<T>(w[x], a, b);
    s += a * a + b * b;
  }
  return s;
}

// (register budget: three waves per SIMD up to head size 128 -- 168 VGPRs, no scratch -- two
// above; left to itself the compiler takes > 300 registers and runs one wave per SIMD, which
// measured slower than the staging it was meant to speed up)
template <typename T, int D, int NW>
__global__ void __launch_bounds__(64 * NW) __attribute__((amdgpu_waves_per_eu(D <= 128 ? 3 : 2)))
tile_attn_kernel(const T* __restrict__ q, long long ldq, const T* __restrict__ cache,
                 T* __restrict__ out, const int* __restrict__ tables, int maxb,
                 const int* __restrict__ tiles, const int* __restrict__ cu,
                 const int* __restrict__ start, int H, int G, int bs, float scale, float eps,
                 int chunk, int sink) {
  constexpr int QT = 32 * NW, LK = D + 8, LT = 40, NV = D / 8;
  __shared__ __align__(16) T s_k[32 * LK];    // key tile, row-major
  __shared__ __align__(16) T s_t[D * LT];     // key tile, transposed [d][key]
  __shared__ float s_kn[32];                  // 1 / rms of the tile's keys (power-of-two D / 8)
  constexpr int kTbl = 512;                   // block-table entries of the visible keys, in LDS
  __shared__ int s_tbl[kTbl];
  constexpr bool kStagedNorm = (NV & (NV - 1)) == 0 && NV <= 64;
  const int tid = threadIdx.x, lane = tid & 63, w = tid >> 6, c = lane & 31, hi = lane >> 5;
  const int hd = blockIdx.y, g = hd / (H / G);
  // tiles are listed in row order, so later tiles see more keys: issue them first
  const int tix = gridDim.x - 1 - blockIdx.x;
  const int sg = tiles[2 * tix], row0 = tiles[2 * tix + 1];
  const int seg_r0 = cu[sg], p0 = start[sg];
  const int nrows = min(QT, cu[sg + 1] - row0);
  const int* tbl = tables + (long long)sg * maxb;

  const bool qv = 32 * w + c < nrows;
  const int qrow = row0 + 32 * w + c;
  const int pos = qv ? p0 + (qrow - seg_r0) : -1;
  const int lo = (chunk > 0 && qv) ? (pos / chunk) * chunk : 0;
  uint4 qreg[D / 16];
  float q2 = 0.f;
#pragma unroll
  for (int kk = 0; kk < D / 16; ++kk) {
    qreg[kk] = qv ? *reinterpret_cast<const uint4*>(q + (long long)qrow * ldq + hd * D + 16 * kk + 8 * hi)
                  : make_uint4(0, 0, 0, 0);
    q2 += sumsq8<T>(qreg[kk]);
  }
  q2 += __shfl_xor(q2, 32, 64);
  const float qn = scale / sqrtf(q2 / D + eps);

  const int pos_first = p0 + (row0 - seg_r0), kend = pos_first + nrows - 1;
  const int kbeg = chunk > 0 ? (pos_first / chunk) * chunk : 0;
  const bool wave_on = 32 * w < nrows;
  const int wpos_min = pos_first + 32 * w, wpos_max = min(kend, wpos_min + 31);
  const int wlo_min = chunk > 0 ? (wpos_min / chunk) * chunk : 0;

  // the block ids of the keys this tile can see, so that a key's address never waits for a
  // table load (entries beyond kTbl, i.e. very long chunks, are read from global memory)
  const int b_first = kbeg / bs, b_count = kend / bs - b_first + 1;
  for (int i = tid; i < min(b_count, kTbl); i += 64 * NW) s_tbl[i] = tbl[b_first + i];
  const int bshift = (bs & (bs - 1)) == 0 ? __ffs(bs) - 1 : -1;
  __syncthreads();

  float m = sink ? 0.f : -INFINITY, l = sink ? 1.f : 0.f;
  f32x16 O[D / 32];
#pragma unroll
  for (int db = 0; db < D / 32; ++db)
#pragma unroll
    for (int r = 0; r < 16; ++r) O[db][r] = 0.f;

  // staging: one item = 4 consecutive keys x 8 channels (four 16-byte loads); the row-major
  // image takes them as they are, the transposed image takes eight 8-byte stores of 4 keys each
  // (transposed in registers).  The next tile's loads are issued before this tile's products, so
  // their latency hides behind the matrix work.
  constexpr int NT = 64 * NW, ITEMS = (D + NT - 1) / NT;
  uint4 pre[ITEMS][4];
  auto prefetch = [&](int k0) {
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) {
      const int item = tid + it * NT;
      if (item < D) {
        const int kq = item / NV, part = item % NV;
#pragma unroll
        for (int x = 0; x < 4; ++x) {
          const int j = k0 + 4 * kq + x;
          pre[it][x] = make_uint4(0, 0, 0, 0);
          if (j <= kend) {
            const int jb = bshift >= 0 ? j >> bshift : j / bs, jo = j - jb * bs;
            const int bi = jb - b_first;
            const int blk = bi < kTbl ? s_tbl[bi] : tbl[jb];
            const long long off = (((long long)blk * bs + jo) * G + g) * D;
            pre[it][x] = *reinterpret_cast<const uint4*>(cache + off + 8 * part);
          }
        }
      }
    }
  };
  auto commit = [&]() {
#pragma unroll
    for (int it = 0; it < ITEMS; ++it) {
      const int item = tid + it * NT;
      if (item < D) {
        const int kq = item / NV, part = item % NV;
#pragma unroll
        for (int x = 0; x < 4; ++x)
          *reinterpret_cast<uint4*>(&s_k[(4 * kq + x) * LK + 8 * part]) = pre[it][x];
        if (kStagedNorm) {   // the NV lanes of a key quad are adjacent: sum their partial squares
#pragma unroll
          for (int x = 0; x < 4; ++x) {
            float k2 = sumsq8<T>(pre[it][x]);
#pragma unroll
            for (int o = 1; o < NV; o <<= 1) k2 += __shfl_xor(k2, o, 64);
            if (part == 0) s_kn[4 * kq + x] = 1.f / sqrtf(k2 / D + eps);
          }
        }
        const unsigned w0[4] = {pre[it][0].x, pre[it][0].y, pre[it][0].z, pre[it][0].w};
        const unsigned w1[4] = {pre[it][1].x, pre[it][1].y, pre[it][1].z, pre[it][1].w};
        const unsigned w2[4] = {pre[it][2].x, pre[it][2].y, pre[it][2].z, pre[it][2].w};
        const unsigned w3[4] = {pre[it][3].x, pre[it][3].y, pre[it][3].z, pre[it][3].w};
#pragma unroll
        for (int mm = 0; mm < 4; ++mm) {     // word mm holds channels 2mm (low half), 2mm + 1
          // the key quads of a row are permuted by the row's group of 8 (all rows a lane
          // writes share it): lanes that differ in `part` land in different banks
          T* t0 = &s_t[(8 * part + 2 * mm) * LT + 4 * (kq ^ (part & 7))];
          *reinterpret_cast<uint2*>(t0) = make_uint2((w0[mm] & 0xffffu) | (w1[mm] << 16),
                                                     (w2[mm] & 0xffffu) | (w3[mm] << 16));
          *reinterpret_cast<uint2*>(t0 + LT) = make_uint2(
              (w0[mm] >> 16) | (w1[mm] & 0xffff0000u), (w2[mm] >> 16) | (w3[mm] & 0xffff0000u));
        }
      }
    }
  };

  prefetch(kbeg);
  for (int k0 = kbeg; k0 <= kend; k0 += 32) {
    __syncthreads();                       // the previous tile has been consumed
    commit();
    __syncthreads();
    if (k0 + 32 <= kend) prefetch(k0 + 32);
    if (!wave_on || k0 > wpos_max || k0 + 31 < wlo_min) continue;   // nothing this wave may see

    f32x16 acc;
#pragma unroll
    for (int r = 0; r < 16; ++r) acc[r] = 0.f;
    float k2 = 0.f;
#pragma unroll
    for (int kk = 0; kk < D / 16; ++kk) {
      const uint4 a = *reinterpret_cast<const uint4*>(&s_k[c * LK + 16 * kk + 8 * hi]);
      if (!kStagedNorm) k2 += sumsq8<T>(a);
      acc = Mma32<T>::run(a, qreg[kk], acc);
    }
    float kn = 0.f;                                      // of key k0 + c (other head sizes)
    if (!kStagedNorm) {
      k2 += __shfl_xor(k2, 32, 64);
      kn = 1.f / sqrtf(k2 / D + eps);
    }
    // a tile every query of the wave sees whole needs no mask
    const bool whole = k0 >= (chunk > 0 ? (wpos_max / chunk) * chunk : 0) && k0 + 31 <= wpos_min &&
                       32 * w + 31 < nrows;
    float sc[16];
    float mloc = -INFINITY;
#pragma unroll
    for (int r = 0; r < 16; ++r) {
      const int keyr = 8 * (r >> 2) + 4 * hi + (r & 3);
      const float knr = kStagedNorm ? s_kn[keyr] : __shfl(kn, keyr, 64);
      sc[r] = acc[r] * qn * knr;
    }
    if (!whole) {
#pragma unroll
      for (int r = 0; r < 16; ++r) {
        const int j = k0 + 8 * (r >> 2) + 4 * hi + (r & 3);
        sc[r] = (j >= lo && j <= pos) ? sc[r] : -INFINITY;
      }
    }
#pragma unroll
    for (int r = 0; r < 16; ++r) mloc = fmaxf(mloc, sc[r]);
    mloc = fmaxf(mloc, __shfl_xor(mloc, 32, 64));
    const float mn = fmaxf(m, mloc);
    const float ms = mn == -INFINITY ? 0.f : mn;
    // (v_exp_f32: this kernel serves 16-bit dtypes only, the weights are rounded to ~16 bits)
    const float corr = __expf(m - ms);
    float psum = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) { sc[r] = __expf(sc[r] - ms); psum += sc[r]; }
    psum += __shfl_xor(psum, 32, 64);
    l = l * corr + psum;
    m = mn;
    if (__any(corr != 1.f)) {              // the running max moved for some query of the wave
#pragma unroll
      for (int db = 0; db < D / 32; ++db)
#pragma unroll
        for (int r = 0; r < 16; ++r) O[db][r] *= corr;
    }
#pragma unroll
    for (int s2 = 0; s2 < 2; ++s2) {
      unsigned ph[4], pl[4];
#pragma unroll
      for (int x = 0; x < 4; ++x) {
        const float a0 = sc[8 * s2 + 2 * x], a1 = sc[8 * s2 + 2 * x + 1];
        ph[x] = pk2<T>(a0, a1);                      // one packed conversion
        float h0, h1;
        unpack2<T>(ph[x], h0, h1);
        pl[x] = pk2<T>(a0 - h0, a1 - h1);
      }
      const uint4 bh = make_uint4(ph[0], ph[1], ph[2], ph[3]);
      const uint4 bl = make_uint4(pl[0], pl[1], pl[2], pl[3]);
#pragma unroll
      for (int db = 0; db < D / 32; ++db) {
        const int row = 32 * db + c, sw = (row >> 3) & 7;     // undo the store's permutation
        const T* tp = &s_t[row * LT];
        const uint2 a0 = *reinterpret_cast<const uint2*>(tp + 4 * ((4 * s2 + hi) ^ sw));
        const uint2 a1 = *reinterpret_cast<const uint2*>(tp + 4 * ((4 * s2 + 2 + hi) ^ sw));
        const uint4 a = make_uint4(a0.x, a0.y, a1.x, a1.y);
        O[db] = Mma32<T>::run(a, bh, O[db]);
        O[db] = Mma32<T>::run(a, bl, O[db]);
      }
    }
  }
  if (qv) {
    const float inv = 1.f / l;
    T* op = out + ((long long)qrow * H + hd) * D;
#pragma unroll
    for (int db = 0; db < D / 32; ++db)
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int d = 32 * db + 8 * j + 4 * hi;
        const unsigned x0 = pk2<T>(O[db][4 * j] * inv, O[db][4 * j + 1] * inv);
        const unsigned x1 = pk2<T>(O[db][4 * j + 2] * inv, O[db][4 * j + 3] * inv);
        *reinterpret_cast<uint2*>(op + d) = make_uint2(x0, x1);
      }
  }
}

template <typename T>
hipError_t launch_tiles(const void* q, long long ldq, const void* cache, void* out,
                        const int* tables, int maxb, const int* tiles, int ntiles, const int* cu,
                        const int* start, int H, int G, int D, int bs, float scale, float eps,
                        int chunk, int sink, int tile_rows, hipStream_t st) {
  const dim3 grid(ntiles, H);
#define GO(DD)                                                                                   \
  if (tile_rows == 128)                                                                          \
    tile_attn_kernel<T, DD, 4><<<grid, 256, 0, st>>>((const T*)q, ldq, (const T*)cache, (T*)out, \
                                                     tables, maxb, tiles, cu, start, H, G, bs,   \
                                                     scale, eps, chunk, sink);                   \
  else                                                                                           \
    tile_attn_kernel<T, DD, 2><<<grid, 128, 0, st>>>((const T*)q, ldq, (const T*)cache, (T*)out, \
                                                     tables, maxb, tiles, cu, start, H, G, bs,   \
                                                     scale, eps, chunk, sink)
  switch (D) {
    case 32: GO(32); break;
    case 64: GO(64); break;
    case 96: GO(96); break;
    case 128: GO(128); break;
    case 192: GO(192); break;
    case 256: GO(256); break;
    default: return hipErrorInvalidValue;
  }
#undef GO
  return hipGetLastError();
}

}  // namespace

extern "C" {

// 1 when sm_chunk_attn_tiles has a kernel for this dtype / head size
int sm_chunk_attn_tiles_ok(int dt, int D) {
  return (dt == kBF16 || dt == kF16) &&
         (D == 32 || D == 64 || D == 96 || D == 128 || D == 192 || D == 256);
}

// tiles: [ntiles, 2] int32 (segment, first row); every tile covers up to tile_rows (64 or 128)
// rows of its segment
hipError_t sm_chunk_attn_tiles(int dt, const void* q, long long ldq, const void* cache, void* out,
                               const int* tables, int maxb, const int* tiles, int ntiles,
                               const int* cu, const int* start, int H, int G, int D, int bs,
                               float scale, float eps, int chunk, int sink, int tile_rows,
                               hipStream_t st) {
  if (ntiles == 0) return hipSuccess;
  if (G < 1 || H % G || bs < 1 || chunk < 0 || (ldq % 8) != 0) return hipErrorInvalidValue;
  if (tile_rows != 64 && tile_rows != 128) return hipErrorInvalidValue;
  if (dt == kBF16)
    return launch_tiles<bf16>(q, ldq, cache, out, tables, maxb, tiles, ntiles, cu, start, H, G, D,
                              bs, scale, eps, chunk, sink, tile_rows, st);
  if (dt == kF16)
    return launch_tiles<fp16>(q, ldq, cache, out, tables, maxb, tiles, ntiles, cu, start, H, G, D,
                              bs, scale, eps, chunk, sink, tile_rows, st);
  return hipErrorInvalidValue;
}

hipError_t sm_chunk_attn(int dt, const void* q, long long ldq, const void* cache, void* out,
                         const int* tables, int maxb, const int* row_seg, const int* positions,
                         int T, int H, int G, int D, int bs, float scale, float eps, int chunk,
                         int sink, hipStream_t st) {
  if (T == 0) return hipSuccess;
  if (D < 1 || D > kMaxD || G < 1 || H % G || bs < 1 || chunk < 0) return hipErrorInvalidValue;
  const dim3 grid(T, H);
#define CALL(TT) chunk_attn_kernel<TT><<<grid, 64 * kRowWaves, 0, st>>>((const TT*)q, ldq, (const TT*)cache, (TT*)out, tables, maxb, row_seg, positions, H, G, D, bs, scale, eps, chunk, sink)
  SM_DISPATCH(dt, CALL)
#undef CALL
  return hipGetLastError();
}

}  // extern "C"
