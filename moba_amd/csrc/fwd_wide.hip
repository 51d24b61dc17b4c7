// Fused MoBA forward, wide-tile variant: 256 query rows per workgroup, one wave per SIMD.
//
// Same tiles and same arithmetic as the 128-row kernel of fwd.hip, reorganised so that one
// wave keeps the matrix pipe and the vector pipe busy at the same time:
//   * a wave owns 64 query rows (two 32-row blocks A and B): every K fragment and every
//     V^T fragment read from LDS feeds two MFMAs, halving LDS traffic per flop, and a
//     K/V tile loaded from L2 serves 256 rows;
//   * the loop is software pipelined by hand.  Step i runs
//         phase 1:  S^T(i+1) = K(i+1) Q^T   [32 MFMA]   with   second half of softmax(i)
//         phase 2:  O^T += V^T(i) P^T(i)    [32 MFMA]   with   first half of softmax(i+1)
//     so the exponentials of one key tile execute under the MFMAs of its neighbours;
//   * K/V tiles travel global -> LDS through a 4-stage ring (128 KiB) filled by
//     global_load_lds_dwordx4 three tiles ahead, which hides an L2 miss.
#include "attn_common.h"

namespace moba {

constexpr int TMW = 256;                  // query rows per workgroup
constexpr int NS = 4;                     // LDS ring stages
constexpr int PF = 3;                     // tiles in flight ahead of the one being multiplied
constexpr int kStageBytes = 2 * kTileBytes;  // K tile then V tile
constexpr int kFwdWideLds = NS * kStageBytes;
constexpr float kRescaleThresholdW = 8.f;

struct FwdWideParams {
  const bf16* q;
  const bf16* k;
  const bf16* v;
  bf16* part_o;
  float* part_lse;
  TileTables t;  // tile_off / self_tile_prefix counted in 256-row tiles
  float scale_log2;
};

struct WideTile {
  int h, kv_tok0, nkeys, row_count, rot;
  int list_base;  // >= 0: history tile, index of its first list entry
  int c0, r0;     // self tile: first token of the chunk, first row
};

__device__ __forceinline__ bool decode_wide(const TileTables& p, int logical, WideTile& t) {
  const int H = p.H;
  if (logical < p.hist_bound) {
    const int FH = p.F * H;
    if (FH == 0 || logical >= p.tile_off[FH]) return false;
    const int seg = upper_row(p.tile_off, FH, logical);
    const int tile = logical - p.tile_off[seg];
    const int f = seg / H;
    t.h = seg - f * H;
    t.list_base = p.seg_off[seg] + tile * TMW;
    t.row_count = min(TMW, p.seg_off[seg + 1] - t.list_base);
    t.kv_tok0 = p.fchunk_tok[f];
    t.nkeys = p.B;
    t.rot = tile;
    t.c0 = 0;
    t.r0 = 0;
    return true;
  }
  const int st = logical - p.hist_bound;
  if (st >= p.self_total) return false;
  int lo = 0, hi = p.N;
  while (hi - lo > 1) {
    const int mid = (lo + hi) >> 1;
    if (p.self_tile_prefix[mid] * H <= st) lo = mid; else hi = mid;
  }
  const int c = lo;
  const int rem = st - p.self_tile_prefix[c] * H;
  const int nt = p.self_tile_prefix[c + 1] - p.self_tile_prefix[c];
  t.h = rem / nt;
  const int tin = nt - 1 - (rem - t.h * nt);  // longest tiles first
  t.c0 = p.chunk_tok[c];
  const int len = p.chunk_tok[c + 1] - t.c0;
  t.r0 = tin * TMW;
  t.row_count = min(TMW, len - t.r0);
  t.kv_tok0 = t.c0;
  t.nkeys = min(len, t.r0 + TMW);
  t.rot = 0;
  t.list_base = -1;
  return true;
}

__device__ __forceinline__ void wait_vmem_n(int n) {  // n in {0, 4, 8}: loads allowed to stay in flight
  if (n == 0) __builtin_amdgcn_s_waitcnt(0x0F70);
  else if (n == 4) __builtin_amdgcn_s_waitcnt(0x0F74);
  else __builtin_amdgcn_s_waitcnt(0x0F78);
}

__global__ __launch_bounds__(512, 1) void moba_fwd_wide_kernel(const FwdWideParams p) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int n = lane & 31, hh = lane >> 5;
  const int H = p.t.H, K1 = p.t.K1;

  WideTile t;
  if (!decode_wide(p.t, logical_tile_id(), t)) return;
  const int h = t.h, nkeys = t.nkeys, kv_tok0 = t.kv_tok0;

  // ---- this lane's row: wave*32 + n ----
  const int r = wave * 32 + n;
  const bool row_valid = r < t.row_count;
  const int rc = min(r, t.row_count - 1);
  int tok, dest, limit;
  if (t.list_base >= 0) {
    dest = p.t.seg_dest[t.list_base + rc];
    tok = dest / (H * K1);
    limit = nkeys - 1;
  } else {
    tok = t.c0 + t.r0 + rc;
    dest = (tok * H + h) * K1;
    limit = t.r0 + rc;
  }
  const bool hist = t.list_base >= 0;
  const int wave_min_limit = hist ? nkeys - 1 : t.r0 + min(wave * 32, t.row_count - 1);
  const int wave_max_limit = hist ? nkeys - 1 : t.r0 + min(wave * 32 + 31, t.row_count - 1);

  // ---- Q^T operand ----
  bf16x8 bq[8];
  {
    const bf16* src = p.q + ((int64_t)tok * H + h) * kHeadDim + 8 * hh;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) bq[ks] = *reinterpret_cast<const bf16x8*>(src + 16 * ks);
  }

  // ---- K/V tile loader (global -> LDS): 8 waves, each issues slabs w and w+8 of K and of V ----
  const int64_t row_bytes = (int64_t)H * kHeadDim * 2;
  const uint32_t lds_base = lds_addr(smem);
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  const int ld_kin = lane >> 4, ld_pc = lane & 15;
  uint32_t ld_off[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int key = 4 * (8 * i + wave_u) + ld_kin;
    ld_off[i] = (uint32_t)(key * row_bytes + sw_col16(key, ld_pc) * 16);
  }
  const char* k_head = (const char*)p.k + (int64_t)kv_tok0 * row_bytes + h * (kHeadDim * 2);
  const char* v_head = (const char*)p.v + (int64_t)kv_tok0 * row_bytes + h * (kHeadDim * 2);
  auto issue_tile = [&](int kt, int stage) {
    const uint32_t kdst = lds_base + stage * kStageBytes;
    const uint32_t vdst = kdst + kTileBytes;
    const int key0 = kt * TN;
    const bool full = (key0 + TN <= nkeys) && (kv_tok0 + key0 + TN <= p.t.S);
    if (full) {
      const char* kb = k_head + (int64_t)key0 * row_bytes;
      const char* vb = v_head + (int64_t)key0 * row_bytes;
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int slab = 8 * i + wave_u;
        async_copy16_sv(kb, ld_off[i], kdst + slab * 1024);
        async_copy16_sv(vb, ld_off[i], vdst + slab * 1024);
      }
    } else {
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int slab = 8 * i + wave_u;
        const int key = 4 * slab + ld_kin;
        const int c16 = sw_col16(key, ld_pc);
        const int64_t tk = min((int64_t)kv_tok0 + key0 + key, (int64_t)p.t.S - 1);
        const int64_t off = tk * row_bytes + h * (kHeadDim * 2) + c16 * 16;
        async_copy16((const char*)p.k + off, kdst + slab * 1024);
        async_copy16((const char*)p.v + off, vdst + slab * 1024);
      }
    }
  };
  // V rows past the key range are multiplied by P = 0: clear them so that no NaN can form
  auto scrub_tile = [&](int kt, int stage) {
    const int key0 = kt * TN;
    if (key0 + TN <= nkeys) return;
    char* vdst = smem + stage * kStageBytes + kTileBytes;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int slab = 8 * i + wave;
      const int key = 4 * slab + ld_kin;
      if (key0 + key >= nkeys) *reinterpret_cast<u32x4*>(vdst + slab * 1024 + lane * 16) = u32x4{0, 0, 0, 0};
    }
  };

  const int nkt = (nkeys + TN - 1) / TN;
  const int rot = t.rot % nkt;
  auto key_tile = [&](int it) { const int x = it + rot; return x >= nkt ? x - nkt : x; };

  // ---- fragment addressing ----
  const int g16 = lane >> 4, i0 = (lane & 15) >> 2, i1 = lane & 3;
  const int k_row_off = n * 256;
  const int k_sw = ((n & 3) << 2) ^ ((n >> 2) & 3);
  const int v_c16 = 2 * (g16 & 1) + (i1 >> 1);
  const int v_sub = (i1 & 1) * 8;
  const float sl2 = p.scale_log2;

  f32x16 oacc[4];
#pragma unroll
  for (int db = 0; db < 4; ++db)
#pragma unroll
    for (int e = 0; e < 16; ++e) oacc[db][e] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;

  // ---- prologue: fill the ring (each wave has 4 copies in flight per tile) ----
  const int npre = min(PF, nkt);
  for (int i = 0; i < npre; ++i) issue_tile(key_tile(i), i % NS);
  wait_vmem_n(4 * (npre - 1));
  scrub_tile(key_tile(0), 0);
  __syncthreads();
  if (nkt > 1) {
    wait_vmem_n(npre > 2 ? 4 : 0);
    scrub_tile(key_tile(1), 1 % NS);
  }

  for (int it = 0; it < nkt; ++it) {
    const int stage = it % NS;
    const int kt = key_tile(it);
    if (it + PF < nkt) issue_tile(key_tile(it + PF), (it + PF) % NS);

    if (kt * TN <= wave_max_limit) {
      const char* ks = smem + stage * kStageBytes;
      const char* vs = ks + kTileBytes;
      bf16x8 ka[2][8];
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int s8 = 0; s8 < 8; ++s8)
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
          ka[kb][s8] = *reinterpret_cast<const bf16x8*>(ks + kb * 8192 + k_row_off + (((2 * s8 + hh) ^ k_sw) << 4));
      f32x16 sacc[2];
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int e = 0; e < 16; ++e) sacc[kb][e] = 0.f;
#pragma unroll
      for (int s8 = 0; s8 < 8; ++s8)
#pragma unroll
        for (int kb = 0; kb < 2; ++kb) sacc[kb] = mfma32(ka[kb][s8], bq[s8], sacc[kb]);
      __builtin_amdgcn_sched_group_barrier(0x100, 8, 0);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, 8, 0);
      __builtin_amdgcn_sched_barrier(0);

      if (kt * TN + TN - 1 > wave_min_limit) {
#pragma unroll
        for (int kb = 0; kb < 2; ++kb)
#pragma unroll
          for (int e = 0; e < 16; ++e) {
            const int key = kt * TN + 32 * kb + 8 * (e >> 2) + 4 * hh + (e & 3);
            if (key > limit) sacc[kb][e] = -INFINITY;
          }
      }
      float mx = fmaxf(sacc[0][0], sacc[1][0]);
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int e = 1; e < 16; ++e) mx = fmaxf(mx, sacc[kb][e]);
      mx = max_xhalf(mx) * sl2;
      if (__any(mx > m_run + kRescaleThresholdW)) {
        const float m_new = fmaxf(m_run, mx);
        const float alpha = fast_exp2(m_run - m_new);
        m_run = m_new;
        l_run *= alpha;
#pragma unroll
        for (int db = 0; db < 4; ++db)
#pragma unroll
          for (int e = 0; e < 16; ++e) oacc[db][e] *= alpha;
      }
      float rs = 0.f;
#pragma unroll
      for (int kb = 0; kb < 2; ++kb)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const float pe = fast_exp2(sacc[kb][e] * sl2 - m_run);
          sacc[kb][e] = pe;
          rs += pe;
        }
      l_run += rs;
      bf16x8 pb[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int kb = j >> 1, e0 = 8 * (j & 1);
#pragma unroll
        for (int e = 0; e < 8; ++e) pb[j][e] = (bf16)sacc[kb][e0 + e];
      }
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int keyA = 16 * j + 4 * hh + i0;
        const int keyB = keyA + 8;
#pragma unroll
        for (int db = 0; db < 4; ++db) {
          const int c16 = 4 * db + v_c16;
          const bf16x4 va = lds_read_tr(vs + keyA * 256 + ((c16 ^ (i0 << 2) ^ hh) << 4) + v_sub);
          const bf16x4 vb = lds_read_tr(vs + keyB * 256 + ((c16 ^ (i0 << 2) ^ (hh + 2)) << 4) + v_sub);
          bf16x8 a;
          a[0] = va[0]; a[1] = va[1]; a[2] = va[2]; a[3] = va[3];
          a[4] = vb[0]; a[5] = vb[1]; a[6] = vb[2]; a[7] = vb[3];
          oacc[db] = mfma32(a, pb[j], oacc[db]);
        }
      }
    }
    // tile it+2 must have landed (this wave's share) before the barrier that publishes it;
    // the barrier also frees the stage of tile it, refilled at the top of step it+1
    if (it + 2 < nkt) {
      wait_vmem_n(it + PF < nkt ? 4 : 0);
      scrub_tile(key_tile(it + 2), (it + 2) % NS);
    }
    __syncthreads();
  }

  // ---- epilogue ----
  const float l_tot = sum_xhalf(l_run);
  const float inv = 1.f / l_tot;
  if (row_valid) {
    bf16* dst = p.part_o + (int64_t)dest * kHeadDim;
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        u32x2 w;
        w[0] = pack_bf16(oacc[db][4 * g + 0] * inv, oacc[db][4 * g + 1] * inv);
        w[1] = pack_bf16(oacc[db][4 * g + 2] * inv, oacc[db][4 * g + 3] * inv);
        *reinterpret_cast<u32x2*>(dst + 32 * db + 8 * g + 4 * hh) = w;
      }
    if (hh == 0) p.part_lse[dest] = m_run + fast_log2(l_tot);
  }
}

// tile_off[i] = number of tile_rows-row tiles of segment i (to be prefix-summed)
__global__ __launch_bounds__(256) void tile_counts_kernel(const int* __restrict__ seg_off, int* __restrict__ tile_off,
                                                          int nseg, int tile_rows) {
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i < nseg) tile_off[i] = (seg_off[i + 1] - seg_off[i] + tile_rows - 1) / tile_rows;
}

}  // namespace moba

using namespace moba;

extern "C" int moba_fwd_wide_tile_rows(void) { return TMW; }

extern "C" int moba_fwd_partials_wide(const void* q, const void* k, const void* v, void* part_o, float* part_lse,
                                      const int32_t* seg_off, const int32_t* tile_off, const int32_t* seg_dest,
                                      const int32_t* fchunk_tok, const int32_t* chunk_tok,
                                      const int32_t* self_tile_prefix, int64_t S, int H, int D, int K, int F, int N,
                                      int B, int64_t hist_bound, int64_t self_tiles, void* stream) {
  if (!q || !k || !v || !part_o || !part_lse || !chunk_tok || !self_tile_prefix) return MOBA_ERR_ARG;
  if (K > 0 && (!seg_off || !tile_off || !seg_dest || !fchunk_tok)) return MOBA_ERR_ARG;
  if (D != kHeadDim) return MOBA_ERR_UNSUPPORTED;
  if (S <= 0 || H <= 0 || K < 0 || F < 0 || N <= 0 || B <= 0 || hist_bound < 0 || self_tiles <= 0) return MOBA_ERR_ARG;
  if (((uintptr_t)q & 15) || ((uintptr_t)k & 15) || ((uintptr_t)v & 15) || ((uintptr_t)part_o & 15)) return MOBA_ERR_ARG;
  if ((int64_t)S * H * (K + 1) >= 0x7fffffffLL) return MOBA_ERR_LIMIT;
  const int64_t total = (K > 0 ? hist_bound : 0) + self_tiles * H;
  const int64_t grid = (total + 8 * kXcdBlock - 1) / (8 * kXcdBlock) * (8 * kXcdBlock);
  if (grid >= 0x7fffffffLL) return MOBA_ERR_LIMIT;
  FwdWideParams p;
  p.q = (const bf16*)q; p.k = (const bf16*)k; p.v = (const bf16*)v;
  p.part_o = (bf16*)part_o; p.part_lse = part_lse;
  p.t.seg_off = seg_off; p.t.tile_off = tile_off; p.t.seg_dest = seg_dest; p.t.fchunk_tok = fchunk_tok;
  p.t.chunk_tok = chunk_tok; p.t.self_tile_prefix = self_tile_prefix;
  p.t.S = (int)S; p.t.H = H; p.t.K1 = K + 1; p.t.F = (K > 0) ? F : 0; p.t.N = N; p.t.B = B;
  p.t.hist_bound = (K > 0) ? (int)hist_bound : 0;
  p.t.self_total = (int)(self_tiles * H);
  p.scale_log2 = (float)(1.4426950408889634 / sqrt((double)D));
  static bool attr_set = false;
  if (!attr_set) {
    if (hipFuncSetAttribute((const void*)moba_fwd_wide_kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                            kFwdWideLds) != hipSuccess)
      return MOBA_ERR_LAUNCH;
    attr_set = true;
  }
  hipLaunchKernelGGL(moba_fwd_wide_kernel, dim3((unsigned)grid), dim3(512), kFwdWideLds, (hipStream_t)stream, p);
  return hipGetLastError() == hipSuccess ? MOBA_OK : MOBA_ERR_LAUNCH;
}

// Prefix sum of ceil(rows / tile_rows) over the F*H gather-list segments, for a kernel whose
// row tile differs from the one moba_build_lists was called with.  tile_off has nseg+1 entries.
extern "C" void moba_scan_i32(int32_t* a, int n, void* stream);
extern "C" int moba_tile_offsets(const int32_t* seg_off, int32_t* tile_off, int nseg, int tile_rows, void* stream) {
  if (!seg_off || !tile_off || nseg <= 0 || tile_rows <= 0) return MOBA_ERR_ARG;
  hipLaunchKernelGGL(tile_counts_kernel, dim3((nseg + 255) / 256), dim3(256), 0, (hipStream_t)stream, seg_off,
                     tile_off, nseg, tile_rows);
  moba_scan_i32(tile_off, nseg, stream);
  return hipGetLastError() == hipSuccess ? MOBA_OK : MOBA_ERR_LAUNCH;
}
