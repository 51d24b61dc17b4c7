// Fused MoBA forward for gfx950.
//
// One kernel covers both kinds of work, as tiles of 128 query rows of one head:
//   history tile : 128 rows of the gather list of segment (filtered chunk f, head h),
//                  against the B keys of chunk f, no mask
//   self tile    : 128 consecutive rows of one chunk against the keys of the same
//                  chunk up to the diagonal (causal); with the chunk table set to whole
//                  sequences this is plain causal attention (the k <= 0 case)
// Each tile runs a flash-style loop over 64-key tiles: K and V tiles are staged in LDS
// (double buffered, bank-conflict-free swizzles), S^T = K Q^T and O^T += V^T P^T use
// v_mfma_f32_32x32x16_bf16 with the query index in the lane dimension, so a row's
// softmax statistics live in one lane pair; V^T fragments come from ds_read_b64_tr_b16.
// A tile writes a normalised partial output (bf16) and its log2-sum-exp into the
// row's slot; the merge kernel combines the K+1 slots of every (token, head).
//
// Algorithmic work: 4*D flops per attended (query, key) pair; the bound is the bf16
// MFMA rate.  Compulsory HBM traffic is q, k, v once, the partials once each way.
#include "attn_common.h"

namespace moba {

constexpr int kFwdLds = 4 * kTileBytes;  // K[2], V[2]

struct FwdParams {
  const bf16* q;
  const bf16* k;
  const bf16* v;
  bf16* part_o;     // [S*H*K1, D]
  float* part_lse;  // [S*H*K1], log2 domain
  TileTables t;
  float scale_log2;  // D^-0.5 * log2(e)
};

constexpr float kRescaleThreshold = 8.f;  // log2 units: the running max may lag the true max by this much

__global__ __launch_bounds__(256, 2) void moba_fwd_kernel(const FwdParams p) {
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int n = lane & 31, hh = lane >> 5;
  const int H = p.t.H;

  Tile t;
  const int r = wave * 32 + n;
  if (!decode_tile(p.t, logical_tile_id(), wave, r, t)) return;
  const int h = t.h, nkeys = t.nkeys, kv_tok0 = t.kv_tok0, limit = t.limit;
  const bool row_valid = r < t.row_count;

  // ---- Q^T operand: lane (n, hh) holds q[tok][16*ks + 8*hh .. +7] ----
  bf16x8 bq[8];
  {
    const bf16* src = p.q + ((int64_t)t.tok * H + h) * kHeadDim + 8 * hh;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) bq[ks] = *reinterpret_cast<const bf16x8*>(src + 16 * ks);
  }

  // ---- K/V tile loader: global -> LDS without passing through registers.
  // A wave copy fills 1 KiB = 4 keys x 16 columns of 16 bytes; wave w issues slabs
  // w, w+4, w+8, w+12 of K and of V.  Lane i lands at slab + 16*i, so the lane picks the
  // global column whose swizzled LDS position is i.
  const int64_t row_bytes = (int64_t)H * kHeadDim * 2;
  const uint32_t lds_base = lds_addr(smem);
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  const int ld_kin = lane >> 4;  // key within the slab
  const int ld_pc = lane & 15;   // physical 16-byte column
  // per-lane byte offset of the lane's 16 bytes inside a 64-key tile, for each of the 4 slabs
  uint32_t ld_off[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int key = 4 * (4 * i + wave_u) + ld_kin;
    ld_off[i] = (uint32_t)(key * row_bytes + sw_col16(key, ld_pc) * 16);  // the swizzle is an involution
  }
  const char* k_head = (const char*)p.k + (int64_t)kv_tok0 * row_bytes + h * (kHeadDim * 2);
  const char* v_head = (const char*)p.v + (int64_t)kv_tok0 * row_bytes + h * (kHeadDim * 2);
  auto issue_tile = [&](int kt, int buf) {
    const uint32_t kdst = lds_base + buf * kTileBytes;
    const uint32_t vdst = lds_base + (2 + buf) * kTileBytes;
    const int key0 = kt * TN;
    const bool full = (key0 + TN <= nkeys) && (kv_tok0 + key0 + TN <= p.t.S);
    if (full) {  // uniform tile base in SGPRs + constant per-lane offsets: no address arithmetic
      const char* kb = k_head + (int64_t)key0 * row_bytes;
      const char* vb = v_head + (int64_t)key0 * row_bytes;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int slab = 4 * i + wave_u;
        async_copy16_sv(kb, ld_off[i], kdst + slab * 1024);
        async_copy16_sv(vb, ld_off[i], vdst + slab * 1024);
      }
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int slab = 4 * i + wave_u;
        const int key = 4 * slab + ld_kin;  // key within the tile
        const int c16 = sw_col16(key, ld_pc);
        const int64_t tk = min((int64_t)kv_tok0 + key0 + key, (int64_t)p.t.S - 1);
        const int64_t off = tk * row_bytes + h * (kHeadDim * 2) + c16 * 16;
        async_copy16((const char*)p.k + off, kdst + slab * 1024);
        async_copy16((const char*)p.v + off, vdst + slab * 1024);
      }
    }
  };
  // rows of V past the end of the key range must not reach the MFMA (0 * NaN): clear them
  auto scrub_tile = [&](int kt, int buf) {
    const int key0 = kt * TN;
    if (key0 + TN <= nkeys) return;
    char* vdst = smem + (2 + buf) * kTileBytes;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int slab = 4 * i + wave;
      const int key = 4 * slab + ld_kin;
      if (key0 + key >= nkeys) *reinterpret_cast<u32x4*>(vdst + slab * 1024 + lane * 16) = u32x4{0, 0, 0, 0};
    }
  };

  // Tiles that run side by side on an XCD work on the same chunk; starting each at a
  // different key tile spreads their first touches of the chunk over all of it, instead of
  // every workgroup waiting on the same cache miss at every step.
  const int nkt = (nkeys + TN - 1) / TN;
  const int rot = t.rot % nkt;
  auto key_tile = [&](int it) { const int x = it + rot; return x >= nkt ? x - nkt : x; };
  issue_tile(key_tile(0), 0);
  wait_vmem();
  scrub_tile(key_tile(0), 0);
  __syncthreads();

  f32x16 oacc[4];
#pragma unroll
  for (int db = 0; db < 4; ++db)
#pragma unroll
    for (int e = 0; e < 16; ++e) oacc[db][e] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;
  const float sl2 = p.scale_log2;

  // per-lane pieces of the fragment addresses
  const int g16 = lane >> 4, i0 = (lane & 15) >> 2, i1 = lane & 3;
  // K row fragment: row 32*kb + n, column 2*s8 + hh
  const int k_row_off = n * 256;
  const int k_sw = ((n & 3) << 2) ^ ((n >> 2) & 3);
  // V^T quad read: rows 16*j + 4*hh + i0 (+8), 8 bytes at d = 32*db + 16*(g16&1) + 4*i1
  const int v_c16 = 2 * (g16 & 1) + (i1 >> 1);
  const int v_sub = (i1 & 1) * 8;

  for (int it = 0; it < nkt; ++it) {
    const int buf = it & 1;
    const bool has_next = it + 1 < nkt;
    const int kt = key_tile(it);
    if (has_next) issue_tile(key_tile(it + 1), buf ^ 1);

    if (kt * TN <= t.wave_max_limit) {  // wave-uniform: skip tiles entirely above the diagonal
      const char* ks = smem + buf * kTileBytes;
      const char* vs = smem + (2 + buf) * kTileBytes;
      // S^T (keys x queries), two 32-key blocks: fetch all K fragments, then two
      // interleaved accumulation chains
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
      // 8 fragment reads ahead, then reads and MFMAs in step
      __builtin_amdgcn_sched_group_barrier(0x100, 8, 0);
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
        __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
      }
      __builtin_amdgcn_sched_group_barrier(0x008, 8, 0);
      __builtin_amdgcn_sched_barrier(0);

      if (kt * TN + TN - 1 > t.wave_min_limit) {
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
      // lazy running max: move it only when the tile max exceeds it by the threshold
      if (__any(mx > m_run + kRescaleThreshold)) {
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
      // P^T operand for the four 16-key steps
      bf16x8 pb[4];
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int kb = j >> 1, e0 = 8 * (j & 1);
#pragma unroll
        for (int e = 0; e < 8; ++e) pb[j][e] = (bf16)sacc[kb][e0 + e];
      }
      // O^T += V^T P^T
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        const int keyA = 16 * j + 4 * hh + i0;  // keyA & 3 == i0, (keyA >> 2) & 3 == hh
        const int keyB = keyA + 8;              // (keyB >> 2) & 3 == hh + 2
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
    if (has_next) {
      wait_vmem();
      scrub_tile(key_tile(it + 1), buf ^ 1);
    }
    __syncthreads();
  }

  // ---- epilogue: normalise, write the partial ----
  const float l_tot = sum_xhalf(l_run);
  const float inv = 1.f / l_tot;
  if (row_valid) {
    bf16* dst = p.part_o + (int64_t)t.dest * kHeadDim;
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        u32x2 w;
        w[0] = pack_bf16(oacc[db][4 * g + 0] * inv, oacc[db][4 * g + 1] * inv);
        w[1] = pack_bf16(oacc[db][4 * g + 2] * inv, oacc[db][4 * g + 3] * inv);
        *reinterpret_cast<u32x2*>(dst + 32 * db + 8 * g + 4 * hh) = w;
      }
    if (hh == 0) p.part_lse[t.dest] = m_run + fast_log2(l_tot);
  }
}

// Combine the K1 slots of each (token, head): slot 0 is the self part, slot 1+j the
// j-th selected history chunk (present iff sel[row, j] >= 0).  16 lanes per row.
__global__ __launch_bounds__(256) void moba_merge_kernel(const bf16* __restrict__ part_o,
                                                         const float* __restrict__ part_lse,
                                                         const int* __restrict__ sel, bf16* __restrict__ out,
                                                         float* __restrict__ lse, int64_t rows, int K1) {
  const int64_t row = (int64_t)blockIdx.x * 16 + (threadIdx.x >> 4);
  if (row >= rows) return;
  const int c8 = threadIdx.x & 15;
  const int K = K1 - 1;
  const float* pl = part_lse + row * K1;
  const int* ps = sel + row * K;
  float mx = pl[0];
  for (int j = 0; j < K; ++j)
    if (ps[j] >= 0) mx = fmaxf(mx, pl[1 + j]);
  float acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = 0.f;
  float wsum = 0.f;
  const bf16* po = part_o + row * K1 * kHeadDim + c8 * 8;
  for (int j = 0; j < K1; ++j) {
    if (j > 0 && ps[j - 1] < 0) continue;
    const float w = fast_exp2(pl[j] - mx);
    wsum += w;
    const bf16x8 x = *reinterpret_cast<const bf16x8*>(po + (int64_t)j * kHeadDim);
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] += w * (float)x[e];
  }
  const float inv = 1.f / wsum;
  bf16x8 o;
#pragma unroll
  for (int e = 0; e < 8; ++e) o[e] = (bf16)(acc[e] * inv);
  *reinterpret_cast<bf16x8*>(out + row * kHeadDim + c8 * 8) = o;
  if (c8 == 0) lse[row] = (mx + fast_log2(wsum)) * 0.6931471805599453f;
}

}  // namespace moba

using namespace moba;

extern "C" int moba_fwd_tile_rows(void) { return TM; }

// hist_bound: any upper bound on the number of history tiles (floor(M/128) + F*H is one).
extern "C" int moba_fwd_partials(const void* q, const void* k, const void* v, void* part_o, float* part_lse,
                                 const int32_t* seg_off, const int32_t* tile_off, const int32_t* seg_dest,
                                 const int32_t* fchunk_tok, const int32_t* chunk_tok,
                                 const int32_t* self_tile_prefix, int64_t S, int H, int D, int K, int F, int N, int B,
                                 int64_t hist_bound, int64_t self_tiles, void* stream) {
  if (!q || !k || !v || !part_o || !part_lse || !chunk_tok || !self_tile_prefix) return MOBA_ERR_ARG;
  if (K > 0 && (!seg_off || !tile_off || !seg_dest || !fchunk_tok)) return MOBA_ERR_ARG;
  if (D != kHeadDim) return MOBA_ERR_UNSUPPORTED;
  if (S <= 0 || H <= 0 || K < 0 || F < 0 || N <= 0 || B <= 0 || hist_bound < 0 || self_tiles <= 0) return MOBA_ERR_ARG;
  if (((uintptr_t)q & 15) || ((uintptr_t)k & 15) || ((uintptr_t)v & 15) || ((uintptr_t)part_o & 15)) return MOBA_ERR_ARG;
  if ((int64_t)S * H * (K + 1) >= 0x7fffffffLL) return MOBA_ERR_LIMIT;
  const int64_t total = (K > 0 ? hist_bound : 0) + self_tiles * H;
  const int64_t grid = (total + 8 * kXcdBlock - 1) / (8 * kXcdBlock) * (8 * kXcdBlock);
  if (grid >= 0x7fffffffLL) return MOBA_ERR_LIMIT;
  FwdParams p;
  p.q = (const bf16*)q; p.k = (const bf16*)k; p.v = (const bf16*)v;
  p.part_o = (bf16*)part_o; p.part_lse = part_lse;
  p.t.seg_off = seg_off; p.t.tile_off = tile_off; p.t.seg_dest = seg_dest; p.t.fchunk_tok = fchunk_tok;
  p.t.chunk_tok = chunk_tok; p.t.self_tile_prefix = self_tile_prefix;
  p.t.S = (int)S; p.t.H = H; p.t.K1 = K + 1; p.t.F = (K > 0) ? F : 0; p.t.N = N; p.t.B = B;
  p.t.hist_bound = (K > 0) ? (int)hist_bound : 0;
  p.t.self_total = (int)(self_tiles * H);
  p.scale_log2 = (float)(1.4426950408889634 / sqrt((double)D));
  hipStream_t st = (hipStream_t)stream;
  static bool attr_set = false;
  if (!attr_set) {
    if (hipFuncSetAttribute((const void*)moba_fwd_kernel, hipFuncAttributeMaxDynamicSharedMemorySize, kFwdLds) !=
        hipSuccess)
      return MOBA_ERR_LAUNCH;
    attr_set = true;
  }
  hipLaunchKernelGGL(moba_fwd_kernel, dim3((unsigned)grid), dim3(256), kFwdLds, st, p);
  return hipGetLastError() == hipSuccess ? MOBA_OK : MOBA_ERR_LAUNCH;
}

extern "C" int moba_fwd_merge(const void* part_o, const float* part_lse, const int32_t* sel, void* out, float* lse,
                              int64_t S, int H, int D, int K, void* stream) {
  if (!part_o || !part_lse || !out || !lse || (K > 0 && !sel)) return MOBA_ERR_ARG;
  if (D != kHeadDim) return MOBA_ERR_UNSUPPORTED;
  if (S <= 0 || H <= 0 || K < 0 || ((uintptr_t)part_o & 15) || ((uintptr_t)out & 15)) return MOBA_ERR_ARG;
  const int64_t rows = S * H;
  hipLaunchKernelGGL(moba_merge_kernel, dim3((unsigned)((rows + 15) / 16)), dim3(256), 0, (hipStream_t)stream,
                     (const bf16*)part_o, part_lse, sel, (bf16*)out, lse, rows, K + 1);
  return hipGetLastError() == hipSuccess ? MOBA_OK : MOBA_ERR_LAUNCH;
}

// Whole attention stage: partial attentions of every tile, then the merge.
extern "C" int moba_fwd(const void* q, const void* k, const void* v, void* part_o, float* part_lse,
                        const int32_t* sel, const int32_t* seg_off, const int32_t* tile_off,
                        const int32_t* seg_dest, const int32_t* fchunk_tok, const int32_t* chunk_tok,
                        const int32_t* self_tile_prefix, void* out, float* lse, int64_t S, int H, int D, int K,
                        int F, int N, int B, int64_t hist_bound, int64_t self_tiles, void* stream) {
  int rc = moba_fwd_partials(q, k, v, part_o, part_lse, seg_off, tile_off, seg_dest, fchunk_tok, chunk_tok,
                             self_tile_prefix, S, H, D, K, F, N, B, hist_bound, self_tiles, stream);
  if (rc != MOBA_OK) return rc;
  return moba_fwd_merge(part_o, part_lse, sel, out, lse, S, H, D, K, stream);
}
