// Decode attention: one new query token per sequence against the whole key/value cache,
// the branch of the reference adapter that calls flash_attn_func with a single query
// (moba/wrapper.py:76-82).  Full attention (every cached key is visible), grouped-query
// heads handled in place, softmax scale supplied by the caller.
//
// HBM-bound: K and V of the cache are read exactly once, 16 bytes per lane.  The key range
// of a (batch, kv head) is cut into splits, one workgroup each; a 16-lane group owns one
// key at a time (8 head dimensions per lane), so a wave streams 4 keys per load.  All
// REP query heads of the kv head are served from the same loads.  Each lane group keeps
// its own online softmax state; groups, waves and finally splits are combined with the
// usual log-sum-exp algebra (the running maximum moves lazily, so the common step is
// p = exp2(s - m); acc += p * v).
//
//   decode_partial_kernel   part_o[b, hq, split, :] (normalised, fp32), part_lse (log2 domain)
//   decode_merge_kernel     out[b, hq, :]
#include "common.h"

namespace moba {

constexpr int kDecodeMaxSplits = 128;

// sum over the 16 lanes of a DPP row, delivered to all of them, without LDS traffic:
// row mirror (i <-> 15-i), half-row mirror (i <-> 7-i), then the two quad permutations
template <int CTRL>
__device__ __forceinline__ float dpp_move(float x) {
  return __builtin_bit_cast(float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, x), CTRL, 0xF, 0xF, true));
}
__device__ __forceinline__ float sum_row16(float x) {
  x += dpp_move<0x140>(x);  // row_mirror
  x += dpp_move<0x141>(x);  // row_half_mirror
  x += dpp_move<0xB1>(x);   // quad_perm [1,0,3,2]
  x += dpp_move<0x4E>(x);   // quad_perm [2,3,0,1]
  return x;
}

template <class E, int REP>
__global__ __launch_bounds__(256) void decode_partial_kernel(
    const typename E::elem* __restrict__ q, const typename E::elem* __restrict__ k,
    const typename E::elem* __restrict__ v, float* __restrict__ part_o, float* __restrict__ part_lse, int Hkv,
    int Skv, int64_t q_stride_b, int64_t q_stride_h, int64_t kv_stride_b, int64_t kv_stride_h, int keys_per_split,
    int nsplit, float scale_log2) {
  MOBA_ELEM_TYPES(E)
  __shared__ float red_o[4][REP][kHeadDim];
  __shared__ float red_m[4][REP], red_l[4][REP];
  const int split = blockIdx.x, hkv = blockIdx.y, b = blockIdx.z;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int g = lane >> 4, c = lane & 15;
  const int key_lo = split * keys_per_split;
  const int key_hi = min(Skv, key_lo + keys_per_split);

  float qf[REP][8];
#pragma unroll
  for (int r = 0; r < REP; ++r) {
    const elem8 x = *reinterpret_cast<const elem8*>(q + b * q_stride_b + (int64_t)(hkv * REP + r) * q_stride_h + 8 * c);
#pragma unroll
    for (int e = 0; e < 8; ++e) qf[r][e] = (float)x[e] * scale_log2;
  }
  float m[REP], l[REP], acc[REP][8];
#pragma unroll
  for (int r = 0; r < REP; ++r) {
    m[r] = -1e30f;  // finite: exp2(m - m_new) stays defined before the first key
    l[r] = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[r][e] = 0.f;
  }
  const elem* kb = k + b * kv_stride_b + (int64_t)hkv * kv_stride_h + 8 * c;
  const elem* vb = v + b * kv_stride_b + (int64_t)hkv * kv_stride_h + 8 * c;

  // 16 keys per workgroup step (4 waves x 4 lane groups), kUnroll steps (8 row loads per lane) in flight
  constexpr int kUnroll = 4;
  for (int key0 = key_lo + 4 * wave + g; key0 < key_hi; key0 += 16 * kUnroll) {
    elem8 kf[kUnroll], vf[kUnroll];
    bool ok[kUnroll];
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      const int key = key0 + 16 * u;
      ok[u] = key < key_hi;
      const int64_t off = (int64_t)(ok[u] ? key : key_lo) * kHeadDim;
      kf[u] = __builtin_nontemporal_load(reinterpret_cast<const elem8*>(kb + off));
      vf[u] = __builtin_nontemporal_load(reinterpret_cast<const elem8*>(vb + off));
    }
#pragma unroll
    for (int u = 0; u < kUnroll; ++u) {
      float s[REP];
#pragma unroll
      for (int r = 0; r < REP; ++r) {
        float d = 0.f;
#pragma unroll
        for (int e = 0; e < 8; ++e) d += qf[r][e] * (float)kf[u][e];
        d = sum_row16(d);
        s[r] = ok[u] ? d : -INFINITY;
      }
      bool grow = false;
#pragma unroll
      for (int r = 0; r < REP; ++r) grow |= s[r] > m[r];
      if (__any(grow)) {  // rare once the maximum has settled
#pragma unroll
        for (int r = 0; r < REP; ++r) {
          const float m_new = fmaxf(m[r], s[r]);
          const float alpha = fast_exp2(m[r] - m_new);
          m[r] = m_new;
          l[r] *= alpha;
#pragma unroll
          for (int e = 0; e < 8; ++e) acc[r][e] *= alpha;
        }
      }
#pragma unroll
      for (int r = 0; r < REP; ++r) {
        const float p = fast_exp2(s[r] - m[r]);
        l[r] += p;
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[r][e] += p * (float)vf[u][e];
      }
    }
  }

  // combine the four lane groups of the wave, then the four waves
#pragma unroll
  for (int r = 0; r < REP; ++r) {
#pragma unroll
    for (int o = 16; o <= 32; o <<= 1) {
      const float m_o = __shfl_xor(m[r], o, 64);
      const float l_o = __shfl_xor(l[r], o, 64);
      const float m_new = fmaxf(m[r], m_o);
      const float a = fast_exp2(m[r] - m_new), a_o = fast_exp2(m_o - m_new);
      l[r] = l[r] * a + l_o * a_o;
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[r][e] = acc[r][e] * a + __shfl_xor(acc[r][e], o, 64) * a_o;
      m[r] = m_new;
    }
    if (g == 0) {
#pragma unroll
      for (int e = 0; e < 8; ++e) red_o[wave][r][8 * c + e] = acc[r][e];
      if (c == 0) {
        red_m[wave][r] = m[r];
        red_l[wave][r] = l[r];
      }
    }
  }
  __syncthreads();
  for (int i = threadIdx.x; i < REP * kHeadDim; i += 256) {
    const int r = i / kHeadDim, d = i % kHeadDim;
    float mm = red_m[0][r];
#pragma unroll
    for (int w = 1; w < 4; ++w) mm = fmaxf(mm, red_m[w][r]);
    float ll = 0.f, oo = 0.f;
#pragma unroll
    for (int w = 0; w < 4; ++w) {
      const float a = fast_exp2(red_m[w][r] - mm);
      ll += red_l[w][r] * a;
      oo += red_o[w][r][d] * a;
    }
    const int64_t row = ((int64_t)b * Hkv * REP + hkv * REP + r) * nsplit + split;
    // a split without keys cannot occur (the host sizes the splits), so ll > 0
    part_o[row * kHeadDim + d] = oo / ll;
    if (d == 0) part_lse[row] = mm + fast_log2(ll);
  }
}

// One workgroup per (batch, query head): four waves take a quarter of the splits each, a lane owns
// two head dimensions; the four partial sums meet in LDS.
template <class E>
__global__ __launch_bounds__(256) void decode_merge_kernel(const float* __restrict__ part_o,
                                                           const float* __restrict__ part_lse,
                                                           typename E::elem* __restrict__ out, int nsplit) {
  typedef typename E::elem elem;
  __shared__ float red[4][kHeadDim];
  __shared__ float red_l[4];
  const int64_t row = blockIdx.x;  // b * Hq + hq
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const float* pl = part_lse + row * nsplit;
  float mm = -INFINITY;
  for (int i = lane; i < nsplit; i += 64) mm = fmaxf(mm, pl[i]);
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) mm = fmaxf(mm, __shfl_xor(mm, o, 64));
  float ll = 0.f, o0 = 0.f, o1 = 0.f;
  const float* po = part_o + row * nsplit * kHeadDim + 2 * lane;
  for (int i = wave; i < nsplit; i += 4) {
    const float w = fast_exp2(pl[i] - mm);
    const float2 x = *reinterpret_cast<const float2*>(po + (int64_t)i * kHeadDim);
    ll += w;
    o0 += w * x.x;
    o1 += w * x.y;
  }
  red[wave][2 * lane] = o0;
  red[wave][2 * lane + 1] = o1;
  if (lane == 0) red_l[wave] = ll;
  __syncthreads();
  if (threadIdx.x < kHeadDim) {
    const int d = threadIdx.x;
    const float l4 = red_l[0] + red_l[1] + red_l[2] + red_l[3];
    out[row * kHeadDim + d] = (elem)((red[0][d] + red[1][d] + red[2][d] + red[3][d]) / l4);
  }
}

}  // namespace moba

using namespace moba;

// Number of key splits the kernels will use for this problem: the caller sizes
// part_o [B*Hq*splits, D] fp32 and part_lse [B*Hq*splits] fp32 with it.
static int decode_split(int B, int Hkv, int Skv, int* keys_per_split) {
  const int64_t groups = (int64_t)B * Hkv;
  int64_t want = (1024 + groups - 1) / groups;        // enough workgroups to fill 256 CUs several times
  const int64_t by_len = (Skv + 255) / 256;           // at least 256 keys per split
  if (want > by_len) want = by_len;
  if (want > kDecodeMaxSplits) want = kDecodeMaxSplits;
  if (want < 1) want = 1;
  const int per = (int)((Skv + want - 1) / want);
  *keys_per_split = per;
  return (Skv + per - 1) / per;                        // no empty split
}

extern "C" int moba_decode_splits(int B, int Hkv, int Skv) {
  if (B <= 0 || Hkv <= 0 || Skv <= 0) return 0;
  int per;
  return decode_split(B, Hkv, Skv, &per);
}

template <class E, int REP>
static void launch_decode(const void* q, const void* k, const void* v, void* out, float* part_o, float* part_lse,
                          int B, int Hkv, int Skv, int64_t qsb, int64_t qsh, int64_t kvsb, int64_t kvsh, int nsplit,
                          int per, float scale_log2, hipStream_t st) {
  typedef typename E::elem elem;
  hipLaunchKernelGGL((decode_partial_kernel<E, REP>), dim3(nsplit, Hkv, B), dim3(256), 0, st, (const elem*)q,
                     (const elem*)k, (const elem*)v, part_o, part_lse, Hkv, Skv, qsb, qsh, kvsb, kvsh, per, nsplit,
                     scale_log2);
  hipLaunchKernelGGL(decode_merge_kernel<E>, dim3((unsigned)(B * Hkv * REP)), dim3(256), 0, st,
                     (const float*)part_o, (const float*)part_lse, (elem*)out, nsplit);
}

// q [B, H, D] (strides q_stride_b, q_stride_h in elements, D contiguous); k, v [B, Hkv, Skv, D]
// (strides kv_stride_b, kv_stride_h; a key row is D contiguous elements and rows are D apart);
// out [B, H, D] contiguous.  H / Hkv must be 1, 2, 4 or 8.
extern "C" int moba_decode(const void* q, const void* k, const void* v, void* out, float* part_o, float* part_lse,
                           int B, int H, int Hkv, int Skv, int D, int64_t q_stride_b, int64_t q_stride_h,
                           int64_t kv_stride_b, int64_t kv_stride_h, float scale, int dtype, void* stream) {
  LaunchCheck launch_check;
  if (!q || !k || !v || !out || !part_o || !part_lse) return MOBA_ERR_ARG;
  if (B <= 0 || H <= 0 || Hkv <= 0 || Skv <= 0 || H % Hkv != 0 || B > 65535 || Hkv > 65535) return MOBA_ERR_ARG;
  if (D != kHeadDim || (dtype != MOBA_DTYPE_BF16 && dtype != MOBA_DTYPE_F16)) return MOBA_ERR_UNSUPPORTED;
  if (((uintptr_t)q & 15) || ((uintptr_t)k & 15) || ((uintptr_t)v & 15)) return MOBA_ERR_ARG;
  if ((q_stride_b | q_stride_h | kv_stride_b | kv_stride_h) & 7) return MOBA_ERR_ARG;  // 16-byte loads
  const int rep = H / Hkv;
  int per;
  const int nsplit = decode_split(B, Hkv, Skv, &per);
  const float sl2 = scale * 1.4426950408889634f;
  hipStream_t st = (hipStream_t)stream;
#define MOBA_DECODE(EL, R)                                                                                      \
  launch_decode<EL, R>(q, k, v, out, part_o, part_lse, B, Hkv, Skv, q_stride_b, q_stride_h, kv_stride_b,       \
                       kv_stride_h, nsplit, per, sl2, st)
#define MOBA_DECODE_REP(EL)                 \
  switch (rep) {                            \
    case 1: MOBA_DECODE(EL, 1); break;      \
    case 2: MOBA_DECODE(EL, 2); break;      \
    case 4: MOBA_DECODE(EL, 4); break;      \
    case 8: MOBA_DECODE(EL, 8); break;      \
    default: return MOBA_ERR_UNSUPPORTED;   \
  }
  if (dtype == MOBA_DTYPE_F16) { MOBA_DECODE_REP(F16) } else { MOBA_DECODE_REP(Bf16) }
#undef MOBA_DECODE_REP
#undef MOBA_DECODE
  return launch_check.result();
}
