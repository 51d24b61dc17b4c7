// Varlen gather lists: for every (filtered chunk f, head h) the ascending list of
// query tokens that selected it, as a counting sort keyed by (f, h) that is stable
// in the token index -- integer work, no copy of q or kv.
//
//   pass 1  count    one workgroup per (query chunk, head): how many of its tokens
//                    picked each earlier chunk of the sequence -> cnt[(f, h, query chunk)]
//   pass 2  scan     exclusive prefix sum of cnt in (f, h, query chunk) order: that is
//                    the list position of the first such token, because query chunks
//                    of a sequence are visited in ascending token order
//   pass 3  fill     same decomposition as pass 1; inside a workgroup the four waves own
//                    consecutive quarters of the chunk, and inside a 64-token batch
//                    the rank of a token among those with the same pick comes from a
//                    64-bit lane mask built with LDS atomics (order independent)
//   pass 4  segment offsets and per-segment tile counts, then their prefix sum
//
// List entries are destination rows of the partial-result buffers:
// dest = (token * H + h) * (K + 1) + 1 + slot, from which the token is recovered by
// one division.
#include "common.h"

namespace moba {

__device__ __forceinline__ int cnt_index(const int* __restrict__ pair_off, int f, int h, int H, int crel) {
  const int p0 = pair_off[f];
  const int nq = pair_off[f + 1] - p0;
  return p0 * H + h * nq + crel;
}

template <int NT>  // threads per workgroup
__global__ __launch_bounds__(NT) void lists_count_kernel(
    const int* __restrict__ sel, const int* __restrict__ chunk_tok, const int* __restrict__ chunk_fb,
    const int* __restrict__ chunk_local, const int* __restrict__ pair_off, int* __restrict__ cnt, int H, int K,
    int dense_local) {
  extern __shared__ int lds[];
  const int cq = blockIdx.x, h = blockIdx.y;
  const int c = chunk_local[cq];
  if (c == 0) return;
  const int fb = chunk_fb[cq];
  if (c <= dense_local) {  // a chunk of a dense prefix: its tokens have no list entries, its counts are zero
    for (int i = threadIdx.x; i < c; i += NT) cnt[cnt_index(pair_off, fb + i, h, H, c - i - 1)] = 0;
    return;
  }
  const int t0 = chunk_tok[cq], t1 = chunk_tok[cq + 1];
  for (int i = threadIdx.x; i < c; i += NT) lds[i] = 0;
  __syncthreads();
  for (int s = t0 + threadIdx.x; s < t1; s += NT) {
    const int* src = sel + ((int64_t)s * H + h) * K;
    for (int j = 0; j < K; ++j) {
      const int i = src[j] - fb;
      if ((unsigned)i < (unsigned)c) atomicAdd(&lds[i], 1);
    }
  }
  __syncthreads();
  for (int i = threadIdx.x; i < c; i += NT) cnt[cnt_index(pair_off, fb + i, h, H, c - i - 1)] = lds[i];
}

// the lanes of a wave see each other's LDS writes: a wave's LDS instructions execute in the order issued, so only
// the compiler has to be held to that order
__device__ __forceinline__ void wave_lds_sync() {
  __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
  __builtin_amdgcn_wave_barrier();
  __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
}

// KC: compile-time bound on K (a lane keeps its token's picks in registers); NW: waves of the workgroup, which
// own consecutive NW-ths of the chunk.  base_of() returns the scanned count array, in global memory or in LDS;
// it is called by the whole workgroup once the first loads of the picks are under way (it may synchronise).
template <int KC, int NW, class BaseFn>
__device__ __forceinline__ void lists_fill_body(
    const int* __restrict__ sel, const int* __restrict__ chunk_tok, const int* __restrict__ chunk_fb,
    const int* __restrict__ chunk_local, const int* __restrict__ pair_off, BaseFn base_of,
    int* __restrict__ seg_dest, int H, int K, int dense_local, int* lds) {
  const int cq = blockIdx.x, h = blockIdx.y;
  const int c_real = chunk_local[cq];
  const int c = c_real > dense_local ? c_real : 0;  // (no list entries from a chunk of a dense prefix)
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  int* pos = lds;                                             // [NW][c] running list position per wave
  unsigned* bits = reinterpret_cast<unsigned*>(lds + NW * c);  // [NW][c][2] lanes of the batch that picked i
  const int fb = chunk_fb[cq];
  const int t0 = chunk_tok[cq], t1 = chunk_tok[cq + 1];
  const int qlen = (t1 - t0 + NW - 1) / NW;
  const int w0 = min(t1, t0 + wave * qlen), w1 = min(t1, w0 + qlen);
  const int K1 = K + 1;
  // candidate index of each pick of this lane's token in a batch of 64, -1 when it is not a list entry
  auto load_picks = [&](int bi, int (&pick)[KC]) {
    const int s = w0 + bi * 64 + lane;
    const bool active = s < w1;
    const int* src = sel + ((int64_t)(active ? s : t0) * H + h) * K;
#pragma unroll
    for (int j = 0; j < KC; ++j) {
      pick[j] = -1;
      if (j < K) {
        const int i = src[j] - fb;
        if (active && (unsigned)i < (unsigned)c) pick[j] = i;
      }
    }
  };
  constexpr int kKept = 2;  // the picks of the first batches stay in registers from the counting pass on
  int kept[kKept][KC];
#pragma unroll
  for (int bi = 0; bi < kKept; ++bi) load_picks(bi, kept[bi]);
  const int* base = base_of();
  if (c == 0) return;  // (the whole workgroup)
  for (int i = threadIdx.x; i < NW * c; i += NW * 64) {
    pos[i] = 0;
    bits[2 * i] = 0;
    bits[2 * i + 1] = 0;
  }
  __syncthreads();
  const int nbatch = (qlen + 63) / 64;  // same for all waves
  // per-wave counts
  for (int bi = 0; bi < nbatch; ++bi) {
    int pick[KC];
    if (bi < kKept) {
#pragma unroll
      for (int j = 0; j < KC; ++j) pick[j] = bi == 0 ? kept[0][j] : kept[1][j];
    } else {
      load_picks(bi, pick);
    }
#pragma unroll
    for (int j = 0; j < KC; ++j)
      if (pick[j] >= 0) atomicAdd(&pos[wave * c + pick[j]], 1);
  }
  __syncthreads();
  // counts -> start positions: global base of (f, h, this query chunk) plus the earlier waves
  for (int i = threadIdx.x; i < c; i += NW * 64) {
    int run = base[cnt_index(pair_off, fb + i, h, H, c - i - 1)];
#pragma unroll
    for (int w = 0; w < NW; ++w) {
      const int n = pos[w * c + i];
      pos[w * c + i] = run;
      run += n;
    }
  }
  __syncthreads();
  // from here on a wave works on its own positions and lane masks only
  int* wpos = pos + wave * c;
  unsigned* wbits = bits + 2 * wave * c;
  const uint64_t below = (lane == 0) ? 0ull : (~0ull >> (64 - lane));
  for (int bi = 0; bi < nbatch; ++bi) {
    const int s = w0 + bi * 64 + lane;
    int pick[KC];
    if (bi < kKept) {
#pragma unroll
      for (int j = 0; j < KC; ++j) pick[j] = bi == 0 ? kept[0][j] : kept[1][j];
    } else {
      load_picks(bi, pick);
    }
#pragma unroll
    for (int j = 0; j < KC; ++j)
      if (pick[j] >= 0) atomicOr(&wbits[2 * pick[j] + (lane >> 5)], 1u << (lane & 31));
    wave_lds_sync();
#pragma unroll
    for (int j = 0; j < KC; ++j) {
      if (pick[j] >= 0) {
        const int i = pick[j];
        const uint64_t m = (uint64_t)wbits[2 * i] | ((uint64_t)wbits[2 * i + 1] << 32);
        const int rank = __popcll(m & below);
        seg_dest[wpos[i] + rank] = (s * H + h) * K1 + 1 + j;
      }
    }
    wave_lds_sync();
#pragma unroll
    for (int j = 0; j < KC; ++j) {
      if (pick[j] >= 0) {
        const int i = pick[j];
        const uint64_t m = (uint64_t)wbits[2 * i] | ((uint64_t)wbits[2 * i + 1] << 32);
        if ((m & below) == 0) {  // the first lane of this pick closes the batch for it
          wpos[i] += __popcll(m);
          wbits[2 * i] = 0;
          wbits[2 * i + 1] = 0;
        }
      }
    }
    wave_lds_sync();
  }
}

// NW waves per (query chunk, head): 4, or 16 for long chunks -- a wave walks its share of the chunk in batches of
// 64 tokens with three LDS round trips each, so the kernel's time is the number of batches per wave times that
// latency unless many waves are resident to hide it
template <int KC, int NW>
__global__ __launch_bounds__(NW * 64) void lists_fill_kernel(
    const int* __restrict__ sel, const int* __restrict__ chunk_tok, const int* __restrict__ chunk_fb,
    const int* __restrict__ chunk_local, const int* __restrict__ pair_off, const int* __restrict__ base,
    int* __restrict__ seg_dest, int H, int K, int dense_local) {
  extern __shared__ int lds[];
  lists_fill_body<KC, NW>(sel, chunk_tok, chunk_fb, chunk_local, pair_off, [&] { return base; }, seg_dest, H, K,
                          dense_local, lds);
}

// exclusive prefix sum of a[0..n) in place, total stored at a[n]; one workgroup.
__global__ __launch_bounds__(1024) void scan_kernel(int* __restrict__ a, int n) {
  __shared__ int wsum[16];
  __shared__ int carry_s;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  if (tid == 0) carry_s = 0;
  __syncthreads();
  for (int base = 0; base < n; base += 4096) {
    const int i0 = base + tid * 4;
    int v[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = (i0 + e < n) ? a[i0 + e] : 0;
    const int tsum = v[0] + v[1] + v[2] + v[3];
    int inc = tsum;  // inclusive scan across the wave
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const int t = __shfl_up(inc, o, 64);
      if (lane >= o) inc += t;
    }
    if (lane == 63) wsum[wave] = inc;
    __syncthreads();
    int woff = 0, total = 0;
#pragma unroll
    for (int w = 0; w < 16; ++w) {
      const int x = wsum[w];
      if (w < wave) woff += x;
      total += x;
    }
    const int carry = carry_s;
    int run = carry + woff + inc - tsum;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      if (i0 + e < n) a[i0 + e] = run;
      run += v[e];
    }
    __syncthreads();
    if (tid == 0) carry_s = carry + total;
    __syncthreads();
  }
  if (tid == 0) a[n] = carry_s;
}

// per (f, h): list start and number of row tiles
__global__ __launch_bounds__(256) void lists_segments_kernel(const int* __restrict__ base,
                                                             const int* __restrict__ pair_off,
                                                             int* __restrict__ seg_off, int* __restrict__ tile_off,
                                                             int F, int H, int tile_rows) {
  const int fh = blockIdx.x * 256 + threadIdx.x;
  if (fh > F * H) return;
  if (fh == F * H) {
    seg_off[fh] = base[pair_off[F] * H];
    return;
  }
  const int f = fh / H, h = fh % H;
  const int p0 = pair_off[f];
  const int nq = pair_off[f + 1] - p0;
  const int start = base[p0 * H + h * nq];
  const int end = base[p0 * H + (h + 1) * nq];
  seg_off[fh] = start;
  tile_off[fh] = (end - start + tile_rows - 1) / tile_rows;
}

// number of row tiles per (f, h) from the list starts
__global__ __launch_bounds__(256) void lists_tile_counts_kernel(const int* __restrict__ seg_off,
                                                                int* __restrict__ tile_off, int FH, int tile_rows) {
  const int fh = blockIdx.x * 256 + threadIdx.x;
  if (fh < FH) tile_off[fh] = (seg_off[fh + 1] - seg_off[fh] + tile_rows - 1) / tile_rows;
}

// segment of every history tile id below `bound` (-1 past the last tile): the attention
// kernels then find their tile with one load instead of a search in tile_off
__global__ __launch_bounds__(256) void lists_tile_seg_kernel(const int* __restrict__ tile_off,
                                                             int* __restrict__ tile_seg, int FH, int bound) {
  const int t = blockIdx.x * 256 + threadIdx.x;
  if (t >= bound) return;
  tile_seg[t] = t < tile_off[FH] ? upper_row(tile_off, FH, t) : -1;
}

// Few segments and few tiles: what lists_segments_kernel (or lists_tile_counts_kernel, when `base` is null and
// seg_off is given), the scan of the tile counts and lists_tile_seg_kernel do, in one workgroup with the counts
// in LDS -- three dependent launches of a few microseconds each are most of the list stage of a small problem.
constexpr int kTailMaxSegments = 4096, kTailMaxTiles = 16384;
// (off: kTailMaxSegments + 1 ints of LDS, wsum: 16; `base` may point into LDS)
__device__ __forceinline__ void lists_tail_body(const int* base, const int* __restrict__ pair_off,
                                                int* __restrict__ seg_off, int* __restrict__ tile_off,
                                                int* __restrict__ tile_seg, int F, int H, int tile_rows, int bound,
                                                int* off, int* wsum) {
  const int FH = F * H, tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  // this thread's four consecutive segments: list starts (written out when they come from the counts), tile counts
  int v[4];
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int fh = tid * 4 + e;
    v[e] = 0;
    if (fh < FH) {
      int start, end;
      if (base) {
        const int f = fh / H, h = fh % H;
        const int p0 = pair_off[f];
        const int nq = pair_off[f + 1] - p0;
        start = base[p0 * H + h * nq];
        end = base[p0 * H + (h + 1) * nq];
        seg_off[fh] = start;
      } else {
        start = seg_off[fh];
        end = seg_off[fh + 1];
      }
      v[e] = (end - start + tile_rows - 1) / tile_rows;
    } else if (fh == FH && base) {
      seg_off[fh] = base[pair_off[F] * H];
    }
  }
  const int tsum = v[0] + v[1] + v[2] + v[3];
  int inc = tsum;  // inclusive scan across the wave, then across the waves
#pragma unroll
  for (int o = 1; o < 64; o <<= 1) {
    const int t = __shfl_up(inc, o, 64);
    if (lane >= o) inc += t;
  }
  if (lane == 63) wsum[wave] = inc;
  __syncthreads();
  int woff = 0, total = 0;
#pragma unroll
  for (int w = 0; w < 16; ++w) {
    const int x = wsum[w];
    if (w < wave) woff += x;
    total += x;
  }
  int run = woff + inc - tsum;
#pragma unroll
  for (int e = 0; e < 4; ++e) {
    const int fh = tid * 4 + e;
    if (fh < FH) {
      off[fh] = run;
      tile_off[fh] = run;
    }
    run += v[e];
  }
  if (tid == 0) {
    off[FH] = total;
    tile_off[FH] = total;
  }
  __syncthreads();
  for (int t = tid; t < bound; t += 1024) {
    int seg = -1;
    if (t < total) {
      int lo = 0, hi = FH;  // off[lo] <= t < off[hi]
      while (hi - lo > 1) {
        const int mid = (lo + hi) >> 1;
        if (off[mid] <= t) lo = mid; else hi = mid;
      }
      seg = lo;
    }
    tile_seg[t] = seg;
  }
}

__global__ __launch_bounds__(1024) void lists_tail_kernel(const int* __restrict__ base, const int* __restrict__ pair_off,
                                                          int* __restrict__ seg_off, int* __restrict__ tile_off,
                                                          int* __restrict__ tile_seg, int F, int H, int tile_rows,
                                                          int bound) {
  __shared__ int off[kTailMaxSegments + 1];
  __shared__ int wsum[16];
  lists_tail_body(base, pair_off, seg_off, tile_off, tile_seg, F, H, tile_rows, bound, off, wsum);
}

// Small problems (few counts, few segments, few tiles, few workgroups): the scan, the fill and the tail in one
// launch.  Every workgroup scans the whole count array for itself into LDS (cheaper than a launch that does it
// once); workgroups (cq < N, h) fill their part of the lists with 16 waves, workgroup (N, 0) writes the segment and
// tile tables, which depend on the scanned counts only.
constexpr int kFusedMaxCounts = 4096, kFusedMaxCand = 128;
template <int KC>
__global__ __launch_bounds__(1024) void lists_fill_tail_kernel(
    const int* __restrict__ sel, const int* __restrict__ chunk_tok, const int* __restrict__ chunk_fb,
    const int* __restrict__ chunk_local, const int* __restrict__ pair_off, const int* __restrict__ cnt,
    int* __restrict__ seg_dest, int* __restrict__ seg_off, int* __restrict__ tile_off, int* __restrict__ tile_seg,
    int N, int H, int K, int F, int PH, int tile_rows, int bound, int tile_rows_b, int* __restrict__ tile_off_b,
    int* __restrict__ tile_seg_b, int bound_b, int dense_local) {
  __shared__ int sbase[kFusedMaxCounts + 1];
  // the tail's tile starts, or the fill's positions and lane masks: 16 waves x 3 ints per candidate chunk
  __shared__ int off[kFusedMaxCand * 48 > kTailMaxSegments + 1 ? kFusedMaxCand * 48 : kTailMaxSegments + 1];
  __shared__ int wsum[16];
  if (blockIdx.x == N && blockIdx.y != 0) return;
  auto scanned_counts = [&]() -> const int* {
    const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
    const int i0 = tid * 4;
    int v[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) v[e] = (i0 + e < PH) ? cnt[i0 + e] : 0;
    const int tsum = v[0] + v[1] + v[2] + v[3];
    int inc = tsum;
#pragma unroll
    for (int o = 1; o < 64; o <<= 1) {
      const int t = __shfl_up(inc, o, 64);
      if (lane >= o) inc += t;
    }
    if (lane == 63) wsum[wave] = inc;
    __syncthreads();
    int woff = 0, total = 0;
#pragma unroll
    for (int w = 0; w < 16; ++w) {
      const int x = wsum[w];
      if (w < wave) woff += x;
      total += x;
    }
    int run = woff + inc - tsum;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
      if (i0 + e < PH) sbase[i0 + e] = run;
      run += v[e];
    }
    if (tid == 0) sbase[PH] = total;
    __syncthreads();
    return sbase;
  };
  if (blockIdx.x == N) {
    const int* base = scanned_counts();
    lists_tail_body(base, pair_off, seg_off, tile_off, tile_seg, F, H, tile_rows, bound, off, wsum);
    if (tile_off_b) {  // the same lists cut into tiles of another height (the backward kernels')
      __syncthreads();
      lists_tail_body(base, pair_off, seg_off, tile_off_b, tile_seg_b, F, H, tile_rows_b, bound_b, off, wsum);
    }
  } else
    lists_fill_body<KC, 16>(sel, chunk_tok, chunk_fb, chunk_local, pair_off, scanned_counts, seg_dest, H, K,
                            dense_local, off);
}

}  // namespace moba

using namespace moba;

static void launch_tile_tables(const int32_t* seg_off, int32_t* tile_off, int32_t* tile_seg, int H, int F,
                               int tile_rows, int64_t hist_bound, hipStream_t st) {
  if ((int64_t)F * H < kTailMaxSegments && hist_bound <= kTailMaxTiles) {
    hipLaunchKernelGGL(lists_tail_kernel, dim3(1), dim3(1024), 0, st, (const int*)nullptr, (const int*)nullptr,
                       const_cast<int*>(seg_off), tile_off, tile_seg, F, H, tile_rows, (int)hist_bound);
    return;
  }
  hipLaunchKernelGGL(lists_tile_counts_kernel, dim3((F * H + 255) / 256), dim3(256), 0, st, seg_off, tile_off, F * H,
                     tile_rows);
  hipLaunchKernelGGL(scan_kernel, dim3(1), dim3(1024), 0, st, tile_off, F * H);
  hipLaunchKernelGGL(lists_tile_seg_kernel, dim3((unsigned)((hist_bound + 255) / 256)), dim3(256), 0, st,
                     (const int*)tile_off, tile_seg, F * H, (int)hist_bound);
}

// Limits: chunks per sequence minus one (cmax) is bounded by the LDS the fill pass
// needs, 12 bytes per wave and candidate chunk (4 waves up to 3413 chunks, one wave up to 13653).
extern "C" int moba_build_lists(const int32_t* sel, const int32_t* chunk_tok, const int32_t* chunk_fb,
                                const int32_t* chunk_local, const int32_t* pair_off, int32_t* cnt,
                                int32_t* seg_off, int32_t* tile_off, int32_t* seg_dest, int32_t* tile_seg,
                                int64_t S, int H, int K, int N, int F, int P, int cmax, int tile_rows,
                                int64_t hist_bound, int counted, int tile_rows_b, int32_t* tile_off_b,
                                int32_t* tile_seg_b, int64_t hist_bound_b, int dense_local, void* stream) {
  LaunchCheck launch_check;
  if (!sel || !chunk_tok || !chunk_fb || !chunk_local || !pair_off || !cnt || !seg_off || !tile_off || !seg_dest ||
      !tile_seg)
    return MOBA_ERR_ARG;
  if (hist_bound <= 0 || hist_bound >= 0x7fffffffLL) return MOBA_ERR_ARG;
  if (tile_off_b && (!tile_seg_b || tile_rows_b <= 0 || hist_bound_b <= 0 || hist_bound_b >= 0x7fffffffLL))
    return MOBA_ERR_ARG;
  if (S <= 0 || H <= 0 || K <= 0 || N <= 0 || F <= 0 || P <= 0 || cmax <= 0 || tile_rows <= 0) return MOBA_ERR_ARG;
  if (dense_local < 0 || dense_local > K) return MOBA_ERR_ARG;
  if ((int64_t)S * H * (K + 1) >= 0x7fffffffLL || (int64_t)P * H >= 0x7fffffffLL) return MOBA_ERR_LIMIT;
  if (H > 65535 || (size_t)cmax * 12 > 160 * 1024) return MOBA_ERR_LIMIT;
  hipStream_t st = (hipStream_t)stream;
  dim3 grid(N, H);
  const bool small_tail = (int64_t)F * H < kTailMaxSegments && hist_bound <= kTailMaxTiles;
  if (small_tail && (int64_t)P * H <= kFusedMaxCounts && cmax <= kFusedMaxCand && (int64_t)N * H <= 512 && K <= 16 &&
      (!tile_off_b || hist_bound_b <= kTailMaxTiles)) {
    if (!counted)
      hipLaunchKernelGGL(lists_count_kernel<1024>, grid, dim3(1024), (size_t)cmax * 4, st, sel, chunk_tok, chunk_fb,
                         chunk_local, pair_off, cnt, H, K, dense_local);
#define MOBA_FILL_TAIL(KC)                                                                                       \
  hipLaunchKernelGGL(lists_fill_tail_kernel<KC>, dim3(N + 1, H), dim3(1024), 0, st, sel, chunk_tok, chunk_fb,    \
                     chunk_local, pair_off, (const int*)cnt, seg_dest, seg_off, tile_off, tile_seg, N, H, K, F,  \
                     P * H, tile_rows, (int)hist_bound, tile_rows_b, tile_off_b, tile_seg_b, (int)hist_bound_b,     \
                     dense_local)
    if (K <= 4) MOBA_FILL_TAIL(4);
    else MOBA_FILL_TAIL(16);
#undef MOBA_FILL_TAIL
    return launch_check.result();
  }
  if (!counted)
    hipLaunchKernelGGL(lists_count_kernel<256>, grid, dim3(256), (size_t)cmax * 4, st, sel, chunk_tok, chunk_fb,
                       chunk_local, pair_off, cnt, H, K, dense_local);
  hipLaunchKernelGGL(scan_kernel, dim3(1), dim3(1024), 0, st, cnt, P * H);
  // more than 64 KiB of dynamic LDS has to be asked for explicitly
  // (LDS: 12 bytes per wave and candidate chunk)
  const bool wide = S / N >= 1024 && (size_t)cmax * 192 <= 64 * 1024;  // long chunks: 16 waves per (chunk, head)
#define MOBA_FILL(KC)                                                                                          \
  {                                                                                                            \
    if (wide) {                                                                                                \
      hipLaunchKernelGGL((lists_fill_kernel<KC, 16>), grid, dim3(1024), (size_t)cmax * 192, st, sel, chunk_tok, \
                         chunk_fb, chunk_local, pair_off, (const int*)cnt, seg_dest, H, K, dense_local);       \
    } else if ((size_t)cmax * 48 <= 160 * 1024) {                                                              \
      if ((size_t)cmax * 48 > 64 * 1024 &&                                                                     \
          hipFuncSetAttribute((const void*)lists_fill_kernel<KC, 4>, hipFuncAttributeMaxDynamicSharedMemorySize, \
                              (int)((size_t)cmax * 48)) != hipSuccess)                                         \
        return MOBA_ERR_LAUNCH;                                                                                \
      hipLaunchKernelGGL((lists_fill_kernel<KC, 4>), grid, dim3(256), (size_t)cmax * 48, st, sel, chunk_tok,   \
                         chunk_fb, chunk_local, pair_off, (const int*)cnt, seg_dest, H, K, dense_local);       \
    } else { /* very many chunks per sequence: one wave, so that its tables still fit */                       \
      if (hipFuncSetAttribute((const void*)lists_fill_kernel<KC, 1>, hipFuncAttributeMaxDynamicSharedMemorySize, \
                              (int)((size_t)cmax * 12)) != hipSuccess)                                         \
        return MOBA_ERR_LAUNCH;                                                                                \
      hipLaunchKernelGGL((lists_fill_kernel<KC, 1>), grid, dim3(64), (size_t)cmax * 12, st, sel, chunk_tok,    \
                         chunk_fb, chunk_local, pair_off, (const int*)cnt, seg_dest, H, K, dense_local);       \
    }                                                                                                          \
  }
  if (K <= 4) MOBA_FILL(4)
  else if (K <= 16) MOBA_FILL(16)
  else if (K <= 64) MOBA_FILL(64)
  else return MOBA_ERR_LIMIT;
#undef MOBA_FILL
  if (small_tail) {
    hipLaunchKernelGGL(lists_tail_kernel, dim3(1), dim3(1024), 0, st, (const int*)cnt, pair_off, seg_off, tile_off,
                       tile_seg, F, H, tile_rows, (int)hist_bound);
  } else {
    hipLaunchKernelGGL(lists_segments_kernel, dim3((F * H + 1 + 255) / 256), dim3(256), 0, st, (const int*)cnt,
                       pair_off, seg_off, tile_off, F, H, tile_rows);
    hipLaunchKernelGGL(scan_kernel, dim3(1), dim3(1024), 0, st, tile_off, F * H);
    hipLaunchKernelGGL(lists_tile_seg_kernel, dim3((unsigned)((hist_bound + 255) / 256)), dim3(256), 0, st,
                       (const int*)tile_off, tile_seg, F * H, (int)hist_bound);
  }
  if (tile_off_b) launch_tile_tables(seg_off, tile_off_b, tile_seg_b, H, F, tile_rows_b, hist_bound_b, st);
  return launch_check.result();
}

// The tile tables alone, for another number of rows per tile, from the list starts moba_build_lists wrote
// (the forward and the backward kernels cut the same lists into tiles of different heights).
extern "C" int moba_tile_tables(const int32_t* seg_off, int32_t* tile_off, int32_t* tile_seg, int H, int F,
                                int tile_rows, int64_t hist_bound, void* stream) {
  LaunchCheck launch_check;
  if (!seg_off || !tile_off || !tile_seg) return MOBA_ERR_ARG;
  if (H <= 0 || F <= 0 || tile_rows <= 0 || hist_bound <= 0 || hist_bound >= 0x7fffffffLL) return MOBA_ERR_ARG;
  if ((int64_t)F * H >= 0x7fffffffLL) return MOBA_ERR_LIMIT;
  launch_tile_tables(seg_off, tile_off, tile_seg, H, F, tile_rows, hist_bound, (hipStream_t)stream);
  return launch_check.result();
}
