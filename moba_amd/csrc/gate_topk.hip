// Parameter-less gate and causal top-k.
//
// score(s, h, f) = <q[s,h,:], kbar[f,h,:]> in fp32 (bf16 x bf16 products are exact in
// fp32; the MFMA accumulates them in fp32).  A token s in the c-th chunk of its
// sequence may pick among the c earlier chunks of the same sequence, whose
// filtered-chunk ids are [fb, fb + c) with fb the first filtered id of the
// sequence.  The K best are kept; ties go to the lower chunk id; a -inf or NaN
// score is never picked.  Output sel[s, h, 0..K) holds filtered-chunk ids in
// descending score order, -1 padded.  With dense_local = d > 0 the tokens of the
// chunks 0..d of every sequence (which would pick every earlier chunk) get no picks
// at all: the attention kernels serve them through one causal pass over the prefix.
//
// One wave handles 64 consecutive tokens of one head: the score tile
// (32 chunks x 64 tokens) is two 32x32x16 MFMA accumulators, staged through LDS
// so that each lane then owns one token and runs an insertion top-k held in
// registers.  Scores never reach HBM (except through the optional debug output).
#include "common.h"

namespace moba {

template <int KMAX>
struct TopK {
  float val[KMAX];
  int idx[KMAX];
  __device__ __forceinline__ void init() {
#pragma unroll
    for (int j = 0; j < KMAX; ++j) {
      val[j] = -INFINITY;
      idx[j] = -1;
    }
  }
  // keep the list sorted by descending value; an equal value stays behind the
  // entries already present, so among equal scores the lower id (seen first) wins
  // (the values are in descending order, so the new entry j is the median of the old entries j - 1 and j and of
  // x: one instruction; inside the test x is a number)
  __device__ __forceinline__ void push(float x, int id) {
    if (x > val[KMAX - 1]) {
#pragma unroll
      for (int j = KMAX - 1; j >= 1; --j) {
        const bool shift = x > val[j - 1];
        const bool here = x > val[j];
        idx[j] = shift ? idx[j - 1] : (here ? id : idx[j]);
        val[j] = __builtin_amdgcn_fmed3f(val[j - 1], val[j], x);
      }
      idx[0] = x > val[0] ? id : idx[0];
      val[0] = fmaxf(val[0], x);
    }
  }
};

// locate the sequence of token s: largest b with cu[b] <= s
__device__ __forceinline__ int find_seq(const int* __restrict__ cu, int nseq, int s) {
  return upper_row(cu, nseq, s);
}

// (up to 12 picks the kernel is held to the registers of three waves per SIMD: it is bound by its vector
// instructions, which the waves of a SIMD issue in turn while others wait for memory, LDS and barriers)
template <class E, int KMAX>
__global__ __launch_bounds__(256, KMAX <= 12 ? 3 : 1) void gate_topk_kernel(
    const typename E::elem* __restrict__ q, const typename E::elem* __restrict__ kbar, const int* __restrict__ cu_seqlens,
    const int* __restrict__ seq_fbase, int* __restrict__ sel, float* __restrict__ scores_out,
    int S, int H, int Hkv, int nseq, int F, int B, int K, int64_t q_tok_stride, int64_t q_head_stride,
    int batch_rows, int64_t q_batch_stride, const int* __restrict__ pair_off, int* __restrict__ cnt, int dense_local) {
  MOBA_ELEM_TYPES(E)
  __shared__ float sc[4][64][33];
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int n = lane & 31, hh = lane >> 5;
  const int tok0 = blockIdx.x * 64;
  const int h = blockIdx.y * 4 + wave;
  const bool head_ok = h < H;
  const int hc = head_ok ? h : H - 1;

  // this lane's own token (selection phase)
  const int s = tok0 + lane;
  int fb = 0, c = 0;
  if (s < S) {
    const int b = find_seq(cu_seqlens, nseq, s);
    fb = seq_fbase[b];
    c = (s - cu_seqlens[b]) / B;
    // a token of a dense prefix attends all its earlier chunks through the causal self path: no picks, no counts
    if (c <= dense_local) c = 0;
  }
  // union of the candidate ranges of the 64 tokens (identical for the 4 waves)
  int flo = c > 0 ? fb : 0x7fffffff;
  int fhi = c > 0 ? fb + c : 0;
#pragma unroll
  for (int o = 32; o >= 1; o >>= 1) {
    flo = min(flo, __shfl_xor(flo, o, 64));
    fhi = max(fhi, __shfl_xor(fhi, o, 64));
  }

  TopK<KMAX> top;
  top.init();

  if (fhi > 0) {  // wave-uniform (and block-uniform)
    // Q^T operand: lane (n, hh) holds q[token n (+32)][16*ks + 8*hh .. +7]
    elem8 bq[2][8];
#pragma unroll
    for (int qb = 0; qb < 2; ++qb) {
      const int tok = min(tok0 + 32 * qb + n, S - 1);
      const int be = batch_rows ? tok / batch_rows : 0;  // batch entry of the token in a batched layout
      const elem* src = q + (be * q_batch_stride + (tok - be * batch_rows) * q_tok_stride + hc * q_head_stride) + 8 * hh;
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) bq[qb][ks] = *reinterpret_cast<const elem8*>(src + 16 * ks);
    }
    for (int f0 = flo; f0 < fhi; f0 += 32) {
      const int fr = min(f0 + n, F - 1);
      const elem* src = kbar + ((int64_t)fr * Hkv + hc / (H / Hkv)) * kHeadDim + 8 * hh;
      f32x16 acc0 = {0}, acc1 = {0};
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) {
        const elem8 a = *reinterpret_cast<const elem8*>(src + 16 * ks);
        acc0 = mfma32(a, bq[0][ks], acc0);
        acc1 = mfma32(a, bq[1][ks], acc1);
      }
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int ch = 8 * (e >> 2) + 4 * hh + (e & 3);
        sc[wave][n][ch] = acc0[e];
        sc[wave][32 + n][ch] = acc1[e];
      }
      __syncthreads();
      if (f0 == flo || scores_out) {  // (uniform) the first candidates: every one of them enters the list
#pragma unroll 4
        for (int j = 0; j < 32; ++j) {
          const int f = f0 + j;
          const float x = sc[wave][lane][j];
          const bool valid = (f >= fb) && (f < fb + c);
          if (valid) {
            top.push(x, f);
            if (scores_out && head_ok) scores_out[((int64_t)s * H + h) * F + f] = x;
          }
        }
      } else {
        // Later candidates: few beat the worst entry a lane's list holds by now (it only rises), so the lanes
        // first mark those that do, then insert them in ascending order, one per pass, until no lane has any
        // left -- a handful of insertions per 32 candidates instead of 32.
        const float worst = top.val[KMAX - 1];
        uint32_t beat = 0;
#pragma unroll 8
        for (int j = 0; j < 32; ++j) {
          const int f = f0 + j;
          const bool valid = (f >= fb) && (f < fb + c);
          beat |= (valid && sc[wave][lane][j] > worst) ? 1u << j : 0u;
        }
        while (__ballot(beat != 0)) {  // (wave-uniform)
          if (beat) {
            const int j = __ffs(beat) - 1;
            beat &= beat - 1;
            top.push(sc[wave][lane][j], f0 + j);
          }
        }
      }
      __syncthreads();
    }
  }
  // The four waves hold the lists of four consecutive heads of the same 64 tokens: K ints per (token, head) that
  // lie 4K ints in a row per token in sel.  Through LDS, so that the workgroup stores those runs with consecutive
  // lanes on consecutive ints (a lane storing its own K ints touches a cache line for 4K bytes of it).
  __syncthreads();  // (the score tile is read out)
  int* stage = reinterpret_cast<int*>(&sc[0][0][0]);  // [64 tokens][4 heads][K]
  if (4 * 64 * K <= (int)(sizeof(sc) / sizeof(int))) {  // (uniform; K <= 33)
#pragma unroll
    for (int j = 0; j < KMAX; ++j)
      if (j < K) stage[(lane * 4 + wave) * K + j] = top.idx[j];
    __syncthreads();
    const int run = 4 * K;                       // ints per token in this workgroup's four heads
    const int heads_here = min(4, H - blockIdx.y * 4);
    for (int i = threadIdx.x; i < 64 * run; i += 256) {
      const int tk = i / run, w = i - tk * run;  // token of the tile, int within its run
      if (tok0 + tk < S && w < heads_here * K)
        sel[((int64_t)(tok0 + tk) * H + blockIdx.y * 4) * K + w] = stage[i];
    }
  } else if (s < S && head_ok) {
    int* dst = sel + ((int64_t)s * H + h) * K;
#pragma unroll
    for (int j = 0; j < KMAX; ++j)
      if (j < K) dst[j] = top.idx[j];
  }
  // The gather lists' counts as a by-product: how many tokens of a (query chunk, head) picked each earlier chunk,
  // added into cnt[(chunk, head, query chunk)] (integer sums: the order of the additions does not matter).  A
  // wave's 64 tokens lie in one query chunk, or in a few: one pass per chunk, through a histogram in LDS.
  if (!cnt) return;
  __syncthreads();  // (the staged lists are stored)
  constexpr int kHist = (int)(sizeof(sc) / sizeof(int)) / 4;
  int* hist = reinterpret_cast<int*>(&sc[0][0][0]) + wave * kHist;
  const bool counts = head_ok && s < S && c > 0;
  uint64_t todo = __ballot(counts);
  while (todo) {  // (wave-uniform)
    const int leader = __ffsll((unsigned long long)todo) - 1;
    const int cc = __shfl(c, leader, 64), cfb = __shfl(fb, leader, 64);
    const bool mine = counts && c == cc && fb == cfb;
    for (int w0 = 0; w0 < cc; w0 += kHist) {
      const int wn = min(kHist, cc - w0);
      for (int i = lane; i < wn; i += 64) hist[i] = 0;
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      if (mine) {
#pragma unroll
        for (int j = 0; j < KMAX; ++j) {
          const int i = (j < K && top.idx[j] >= 0) ? top.idx[j] - cfb - w0 : -1;
          if ((unsigned)i < (unsigned)wn) atomicAdd(&hist[i], 1);
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      for (int i = lane; i < wn; i += 64) {
        const int n = hist[i];
        if (n) {
          const int f = cfb + w0 + i;
          const int q0 = pair_off[f], nq = pair_off[f + 1] - q0;
          atomicAdd(&cnt[q0 * H + h * nq + (cc - (w0 + i) - 1)], n);
        }
      }
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
    }
    todo &= ~__ballot(mine);
  }
}

// Selection alone, on scores supplied by the caller ([S, H, F] fp32, -inf where a
// chunk is not a valid candidate).  Same insertion routine as the fused kernel.
template <int KMAX>
__global__ __launch_bounds__(256) void topk_from_scores_kernel(const float* __restrict__ scores,
                                                               int* __restrict__ sel, int64_t rows, int F, int K) {
  const int64_t r = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (r >= rows) return;
  TopK<KMAX> top;
  top.init();
  const float* src = scores + r * F;
  for (int f = 0; f < F; ++f) top.push(src[f], f);
  int* dst = sel + r * K;
#pragma unroll
  for (int j = 0; j < KMAX; ++j)
    if (j < K) dst[j] = top.idx[j];
}

}  // namespace moba

using namespace moba;

#define MOBA_DISPATCH_K(K, CALL)            \
  if ((K) <= 2) { CALL(2); }                \
  else if ((K) <= 4) { CALL(4); }           \
  else if ((K) <= 8) { CALL(8); }           \
  else if ((K) <= 12) { CALL(12); }         \
  else if ((K) <= 16) { CALL(16); }         \
  else if ((K) <= 32) { CALL(32); }         \
  else if ((K) <= 64) { CALL(64); }         \
  else return MOBA_ERR_LIMIT;

extern "C" int moba_gate_topk(const void* q, const void* kbar, const int32_t* cu_seqlens, const int32_t* seq_fbase,
                              int32_t* sel, float* scores_out, const int32_t* pair_off, int32_t* cnt, int64_t S, int H,
                              int Hkv, int D, int nseq, int F, int B, int K, int dense_local, const int64_t* strides,
                              int dtype, void* stream) {
  LaunchCheck launch_check;
  if (!q || !kbar || !cu_seqlens || !seq_fbase || !sel || (cnt && !pair_off)) return MOBA_ERR_ARG;
  if (Hkv <= 0 || H % Hkv != 0) return MOBA_ERR_ARG;
  if (dtype != MOBA_DTYPE_BF16 && dtype != MOBA_DTYPE_F16) return MOBA_ERR_UNSUPPORTED;
  if (S <= 0 || S > 0x7fffffff - 64 || H <= 0 || nseq <= 0 || F <= 0 || B <= 0 || K <= 0) return MOBA_ERR_ARG;
  if (dense_local < 0 || dense_local > K) return MOBA_ERR_ARG;
  if (D != kHeadDim) return MOBA_ERR_UNSUPPORTED;
  if (((uintptr_t)q & 15) || ((uintptr_t)kbar & 15)) return MOBA_ERR_ARG;
  // strides (elements): {q token, q head, ., ., rows per batch entry, q batch, .}; null = packed [S, H, 128]
  const int64_t qts = strides ? strides[0] : (int64_t)H * kHeadDim, qhs = strides ? strides[1] : kHeadDim;
  if (strides && (strides[4] < 0 || strides[4] > 0x7fffffffLL)) return MOBA_ERR_ARG;  // (before it is narrowed)
  const int qbr = strides ? (int)strides[4] : 0;
  const int64_t qbs = strides ? strides[5] : 0;
  if (qts <= 0 || qhs <= 0 || (qts & 7) || (qhs & 7)) return MOBA_ERR_ARG;
  if (qbr < 0 || (qbr > 0 && (qbs <= 0 || (qbs & 7)))) return MOBA_ERR_ARG;
  dim3 grid((unsigned)((S + 63) / 64), (unsigned)((H + 3) / 4));
  hipStream_t st = (hipStream_t)stream;
#define CALL(KM)                                                                                               \
  if (dtype == MOBA_DTYPE_F16)                                                                                 \
    hipLaunchKernelGGL((gate_topk_kernel<F16, KM>), grid, dim3(256), 0, st, (const f16*)q, (const f16*)kbar,   \
                       cu_seqlens, seq_fbase, sel, scores_out, (int)S, H, Hkv, nseq, F, B, K, qts, qhs, qbr, qbs, \
                       pair_off, cnt, dense_local);                                                            \
  else                                                                                                         \
    hipLaunchKernelGGL((gate_topk_kernel<Bf16, KM>), grid, dim3(256), 0, st, (const bf16*)q, (const bf16*)kbar, \
                       cu_seqlens, seq_fbase, sel, scores_out, (int)S, H, Hkv, nseq, F, B, K, qts, qhs, qbr, qbs, \
                       pair_off, cnt, dense_local)
  MOBA_DISPATCH_K(K, CALL)
#undef CALL
  return launch_check.result();
}

extern "C" int moba_topk_from_scores(const float* scores, int32_t* sel, int64_t S, int H, int F, int K,
                                     void* stream) {
  LaunchCheck launch_check;
  if (!scores || !sel || S <= 0 || H <= 0 || F <= 0 || K <= 0) return MOBA_ERR_ARG;
  const int64_t rows = S * H;
  dim3 grid((unsigned)((rows + 255) / 256));
  hipStream_t st = (hipStream_t)stream;
#define CALL(KM) \
  hipLaunchKernelGGL(topk_from_scores_kernel<KM>, grid, dim3(256), 0, st, scores, sel, rows, F, K)
  MOBA_DISPATCH_K(K, CALL)
#undef CALL
  return launch_check.result();
}
