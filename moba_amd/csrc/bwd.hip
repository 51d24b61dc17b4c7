// MoBA backward for gfx950: dq, dk, dv of the attention over the fixed sparse pattern.
//
// With P = exp(scale * q k^T - LSE) (the global softmax probability, LSE from the
// forward), delta = rowsum(dO * O) and dS = P * (dO V^T - delta):
//     dV = P^T dO        dK = scale * dS^T Q        dQ = scale * dS K
// Nothing is differentiated through the gate.  The result is deterministic: no
// floating-point atomics, every output element is produced by one workgroup in a
// fixed order.
//
//   bwd_delta_kernel     delta[token, head]
//   bwd_dq_kernel        row-tile major, same tiling as the forward: each tile (128
//                        query rows x the keys of one chunk) writes its partial dQ, scaled
//                        and rounded to the element type, into the row's slot;
//                        bwd_dq_reduce_kernel sums the K+1 slots in fp32
//   bwd_dkv_kernel       key-tile major: a workgroup owns 128 keys of (chunk, head) and
//                        walks first the causal rows of the same chunk, then the gather
//                        list of rows that selected the chunk; dK/dV accumulate in
//                        registers and are written once
//
// All matrix products use v_mfma_f32_32x32x16_bf16; transposed operands come from
// ds_read_b64_tr_b16.  Algorithmic work: 10*D flops per attended (query, key) pair
// (the recomputation of S and dO V^T in both kernels adds 4*D on top).
#include <type_traits>

#include "attn_common.h"

namespace moba {

constexpr float kLog2e = 1.4426950408889634f;
constexpr int TQ = 64;                                  // query rows per step of the dK/dV kernel
constexpr int kDqIdSlot = 4 * kTileBytes;                // after K[2], V[2]: the tile id wave 0 drew
constexpr int kBwdDqLds = kDqIdSlot + 16;
constexpr int kQStage = 2 * TQ * kHeadDim * 2 + 2 * TQ * 4;  // Q tile, dO tile, lse, delta
constexpr int kDkvStages = 3;
constexpr int kDkvIdSlot = kDkvStages * kQStage;  // where wave 0 hands the tile id it drew to the other waves
constexpr int kBwdDkvLds = kDkvIdSlot + 16;

template <class E>
struct BwdParams {
  const typename E::elem* q;
  const typename E::elem* k;
  const typename E::elem* v;
  const typename E::elem* dout;
  const float* lse;    // [S*H] natural log
  const float* delta;  // [S*H]
  const float* lse2;   // [S*H] lse in the log2 domain
  typename E::elem* part_dq;  // [S*H*K1, D]: per-slot dQ in the element type
  typename E::elem* dq;       // [S*H, D]: where the tiles of chunks without history slots (TileTables::chunk_direct) write
  typename E::elem* dk;
  typename E::elem* dv;
  const int* chunk_fid;  // [N] filtered id of a chunk, -1 for the last chunk of a sequence
  // The key tiles of the dK/dV kernel: TM keys of one chunk and key/value head.  The rows that attend them
  // causally run from the tile's first key to chunk_self_end (the end of the chunk, or of the dense prefix the
  // chunk belongs to); the rows beyond come from the chunk's gather list.
  const int* kv_chunk_tok;    // [N+1] first token of every chunk
  const int* kv_tile_prefix;  // [N+1] prefix sum of ceil(chunk length / TM)
  const int* kv_tile_chunk;   // [kv_tile_prefix[N]] chunk of every such tile
  const int* chunk_self_end;  // [N]
  int kv_total;               // kv_tile_prefix[N] * Hkv
  TileTables t;
  float scale_log2;
  float scale;
  uint32_t hk_magic;  // n / (H*K1) == (n * hk_magic) >> hk_shift for every n < 2^31
  uint32_t hk_shift;
  int* queues;        // [16] tile counters, one per XCD, of the dQ kernel and of the dK/dV kernel; zero at the start
  // Small problems: every key tile of the dK/dV kernel is cut into dkv_split parts (its rows' stages in equal
  // shares) that run as tiles of their own and leave fp32 sums in part_dkv [tiles * dkv_split][2][128][128],
  // which bwd_dkv_reduce_kernel adds up in a fixed order.  dkv_split = 1: whole tiles, dk and dv written directly.
  float* part_dkv;
  int dkv_split;
  // 3: eight queues, one per XCD (tiles that share rows or keys run behind one L2); 0: one queue for all, for a
  // problem of few tiles per workgroup, whose ids come longest tile first: whoever is free takes the longest left
  int queues_log2;
};

// which 128-key tile of which key/value head: the forward's self-tile enumeration over the chunks and Hkv heads
struct KvTile {
  int c, hkv, key0, c0, len;  // chunk, key/value head, first key inside the chunk, first token and length of the chunk
  int self_len;               // the rows that attend the chunk's keys causally end this far behind c0 (>= len)
};
template <class E>
__device__ __forceinline__ KvTile decode_kv_tile(const BwdParams<E>& p, int st) {
  const int Hkv = p.t.Hkv;
  KvTile t;
  t.c = p.kv_tile_chunk[st / Hkv];
  const int rem = st - p.kv_tile_prefix[t.c] * Hkv;
  const int nt = p.kv_tile_prefix[t.c + 1] - p.kv_tile_prefix[t.c];
  t.hkv = rem / nt;
  t.key0 = (rem - t.hkv * nt) * TM;
  t.c0 = p.kv_chunk_tok[t.c];
  t.len = p.kv_chunk_tok[t.c + 1] - t.c0;
  t.self_len = p.chunk_self_end[t.c] - t.c0;
  return t;
}

template <class E>
__global__ __launch_bounds__(256) void bwd_delta_kernel(const typename E::elem* __restrict__ dout,
                                                        const typename E::elem* __restrict__ out,
                                                        const float* __restrict__ lse, float* __restrict__ delta,
                                                        float* __restrict__ lse2, int64_t rows,
                                                        int* __restrict__ queues) {
  MOBA_ELEM_TYPES(E)
  // the 16 tile counters of the two kernels that follow start at zero (here: one launch less than a kernel of its
  // own, and, unlike a memset, safe to record into a graph)
  if (blockIdx.x == 0 && threadIdx.x < 16) queues[threadIdx.x] = 0;
  const int64_t row = (int64_t)blockIdx.x * 16 + (threadIdx.x >> 4);
  const int c8 = threadIdx.x & 15;
  float acc = 0.f;
  if (row < rows) {
    const elem8 a = *reinterpret_cast<const elem8*>(dout + row * kHeadDim + c8 * 8);
    const elem8 b = *reinterpret_cast<const elem8*>(out + row * kHeadDim + c8 * 8);
#pragma unroll
    for (int e = 0; e < 8; ++e) acc += (float)a[e] * (float)b[e];
  }
#pragma unroll
  for (int o = 8; o >= 1; o >>= 1) acc += __shfl_xor(acc, o, 64);
  if (row < rows && c8 == 0) {
    delta[row] = acc;
    lse2[row] = lse[row] * kLog2e;
  }
}

// ------------------------------------------------------------------------------------ dQ
template <class E>
__global__ __launch_bounds__(256, 2) void bwd_dq_kernel(const BwdParams<E> p) {
  MOBA_ELEM_TYPES(E)
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int n = lane & 31, hh = lane >> 5;
  const int H = p.t.H;

  // The workgroups (two per CU, all resident) draw their tiles from eight queues, one per XCD: queue x
  // hands out the ids (8i + x) * kXcdBlock + j in order, so that the tiles in flight on an XCD are
  // consecutive ids (tiles that share a K/V chunk behind one L2), and a workgroup whose queue is empty
  // goes on with the next XCD's: the XCDs differ in speed by a few percent and finish together this way.
  // The draw for the next tile is in flight while the current one is computed.
  const int ql = p.queues_log2, qmask = (1 << ql) - 1;  // eight queues, or one for a problem of few tiles
  int queue = blockIdx.x & qmask, empty_queues = 0;
  int drawn_next = 0;  // thread 0: the counter value drawn for the next tile
  // (With few tiles per workgroup a tile drawn ahead is a tile that waits for its holder while other workgroups
  // run out of work: the draw is made when the tile is due then, two microseconds that nothing hides.)
  const bool draw_ahead = !p.t.self_first;
  if (tid == 0 && draw_ahead)
    drawn_next = __hip_atomic_fetch_add(p.queues + queue, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  while (true) {
  __syncthreads();  // the previous tile is done with LDS, and every wave has read the previous draw
  if (tid == 0) {
    if (!draw_ahead)
      drawn_next = __hip_atomic_fetch_add(p.queues + queue, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    *reinterpret_cast<int*>(smem + kDqIdSlot) = drawn_next;
  }
  __syncthreads();
  const int drawn = __builtin_amdgcn_readfirstlane(*reinterpret_cast<const int*>(smem + kDqIdSlot));
  const int64_t id = (((int64_t)(drawn / kXcdBlock) << ql) + queue) * kXcdBlock + (drawn % kXcdBlock);
  const int ks = p.t.key_split_log2;
  const bool past_end = id >= ((int64_t)p.t.hist_bound << ks) + p.t.self_total;
  if (past_end) {
    queue = (queue + 1) & qmask;
    if (++empty_queues > qmask) break;
  } else {
    empty_queues = 0;
  }
  if (tid == 0 && draw_ahead)
    drawn_next = __hip_atomic_fetch_add(p.queues + queue, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  if (past_end) continue;

  Tile t;
  const int r = wave * 32 + n;
  // With few tiles per workgroup (self_first) the self tiles take the first ids -- the longest of them are as
  // long as a history tile, and drawn last they would run alone at the end -- and the keys of a history tile
  // are cut into 1 << ks parts that are tiles of their own, each with slot rows of its own for its partial dQ
  // (part g of a slot row lies g * part_stride rows behind part 0; bwd_dq_reduce_kernel adds them up).
  int logical = (int)id, key_part = 0;
  if (p.t.self_first) {
    if (logical < p.t.self_total) {
      logical += p.t.hist_bound;
    } else {
      logical -= p.t.self_total;
      key_part = logical & ((1 << ks) - 1);
      logical >>= ks;
    }
  }
  if (!decode_tile_head(p.t, logical, t)) continue;  // an unused id below hist_bound
  if (t.base >= 0) {
    t.nkeys >>= ks;
    t.kv_tok0 += key_part * t.nkeys;
  }
  decode_tile_rows(p.t, wave, r, t);
  t.dest += key_part * p.t.part_stride;
  const int h = t.h, nkeys = t.nkeys, kv_tok0 = t.kv_tok0, limit = t.limit;
  const bool row_valid = r < t.row_count;

  elem8 bq[8], bdo[8];
  {
    const int64_t off = ((int64_t)t.tok * H + h) * kHeadDim + 8 * hh;
    const elem* qsrc = reinterpret_cast<const elem*>((const char*)p.q + q_tok_bytes(p.t, t.tok) + h * p.t.q_head_b) + 8 * hh;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      bq[ks] = *reinterpret_cast<const elem8*>(qsrc + 16 * ks);
      bdo[ks] = *reinterpret_cast<const elem8*>(p.dout + off + 16 * ks);
    }
  }
  const float lse2 = p.lse[(int64_t)t.tok * H + h] * kLog2e;
  const float dl = p.delta[(int64_t)t.tok * H + h];

  const int hkv = h / p.t.rep;                                // key/value head of this query head
  const int64_t row_bytes = p.t.kv_tok_b;                     // from one K or V token to the next
  const uint32_t lds_base = lds_addr(smem);
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  const int ld_kin = lane >> 4, ld_pc = lane & 15;
  uint32_t ld_off[4];  // per-lane byte offset of its 16 bytes inside a full tile (slab 4*i + wave)
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int key = 4 * (4 * i + wave_u) + ld_kin;
    ld_off[i] = (uint32_t)(key * row_bytes + sw_col16(key, ld_pc) * 16);
  }
  const int64_t kv_off = kv_tok_bytes(p.t, kv_tok0) + hkv * p.t.kv_head_b;
  const char* k_head = (const char*)p.k + kv_off;
  const char* v_head = (const char*)p.v + kv_off;
  auto issue_tile = [&](int kt, int buf) __attribute__((always_inline)) {
    const uint32_t kdst = lds_base + buf * kTileBytes;
    const uint32_t vdst = lds_base + (2 + buf) * kTileBytes;
    const int key0 = kt * TN;
    const bool full = key0 + TN <= nkeys;  // (the keys of a tile all belong to one chunk, hence to one sequence)
    if (full) {  // uniform tile base in SGPRs + constant per-lane offsets: no address arithmetic
      const char* kb_ = k_head + (int64_t)key0 * row_bytes;
      const char* vb_ = v_head + (int64_t)key0 * row_bytes;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        async_copy16_sv(kb_, ld_off[i], kdst + (4 * i + wave_u) * 1024);
        async_copy16_sv(vb_, ld_off[i], vdst + (4 * i + wave_u) * 1024);
      }
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int slab = 4 * i + wave_u;
        const int key = 4 * slab + ld_kin;
        const int c16 = sw_col16(key, ld_pc);
        // (keys past the end of the range: the last key again -- their rows are cleared after they land)
        const int64_t off = (int64_t)min(key0 + key, nkeys - 1) * row_bytes + c16 * 16;
        async_copy16(k_head + off, kdst + slab * 1024);
        async_copy16(v_head + off, vdst + slab * 1024);
      }
    }
  };
  // rows past the key range are multiplied by dS = 0: clear them so that no NaN can form
  auto scrub_tile = [&](int kt, int buf) {
    const int key0 = kt * TN;
    if (key0 + TN <= nkeys) return;
    char* kdst = smem + buf * kTileBytes;
    char* vdst = smem + (2 + buf) * kTileBytes;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int slab = 4 * i + wave;
      const int key = 4 * slab + ld_kin;
      if (key0 + key >= nkeys) {
        *reinterpret_cast<u32x4*>(kdst + slab * 1024 + lane * 16) = u32x4{0, 0, 0, 0};
        *reinterpret_cast<u32x4*>(vdst + slab * 1024 + lane * 16) = u32x4{0, 0, 0, 0};
      }
    }
  };

  const int nkt = (nkeys + TN - 1) / TN;
  // history tiles may visit their key tiles in any order: co-resident tiles of one chunk start
  // at different key tiles so that they do not all ask for the same lines at the same time
  const int rot = t.rot % nkt;
  auto key_tile = [&](int it) __attribute__((always_inline)) { const int x = it + rot; return x >= nkt ? x - nkt : x; };
  issue_tile(key_tile(0), 0);
  wait_vmem();
  scrub_tile(key_tile(0), 0);
  __syncthreads();

  f32x16 dqacc[4];
#pragma unroll
  for (int db = 0; db < 4; ++db)
#pragma unroll
    for (int e = 0; e < 16; ++e) dqacc[db][e] = 0.f;
  const float sl2 = p.scale_log2;

  // Per-lane LDS byte addresses of the fragments inside K stage 0 (numbers, not pointers into smem: a read's
  // address is then one register plus an immediate for stage, key block and V, with no base left to add):
  // row fragments (key 32*kb + n, 16-byte column 2*s8 + hh) and transposed quads (keys 32*kb + 16*j2 + 4*hh +
  // i0 and + 8, 8 bytes at d = 32*db + 16*(g16&1) + 4*i1).
  const int g16 = lane >> 4, i0 = (lane & 15) >> 2, i1 = lane & 3;
  uint32_t foff[8], toffA[4], toffB[4];
  {
    const int row_sw = ((n & 3) << 2) ^ ((n >> 2) & 3);
#pragma unroll
    for (int s8 = 0; s8 < 8; ++s8) {
      foff[s8] = lds_base + n * 256 + (((2 * s8 + hh) ^ row_sw) << 4);
      asm volatile("" : "+v"(foff[s8]));  // finished addresses, kept as they are
    }
    const int tr_c16 = 2 * (g16 & 1) + (i1 >> 1);
    const int tr_sub = (i1 & 1) * 8;
#pragma unroll
    for (int db = 0; db < 4; ++db) {
      const int c16 = 4 * db + tr_c16;
      toffA[db] = lds_base + (4 * hh + i0) * 256 + ((c16 ^ (i0 << 2) ^ hh) << 4) + tr_sub;
      toffB[db] = lds_base + (4 * hh + i0 + 8) * 256 + ((c16 ^ (i0 << 2) ^ (hh + 2)) << 4) + tr_sub;
      asm volatile("" : "+v"(toffA[db]));
      asm volatile("" : "+v"(toffB[db]));
    }
  }

  // one key tile; buf_c: its LDS stage, a constant in the two copies of the loop body
  auto key_tile_body = [&](int it, auto buf_c) __attribute__((always_inline)) {
    constexpr int buf = decltype(buf_c)::value;
    const int kt = key_tile(it);
    const bool has_next = it + 1 < nkt;
    if (has_next) issue_tile(key_tile(it + 1), buf ^ 1);

    if (kt * TN <= t.wave_max_limit) {
      constexpr uint32_t ks = buf * kTileBytes;         // K stage, relative to stage 0
      constexpr uint32_t vs = (2 + buf) * kTileBytes;   // V stage
      const bool masked = kt * TN + TN - 1 > t.wave_min_limit;
#pragma unroll
      for (int kb = 0; kb < 2; ++kb) {
        // S^T and (dO V^T)^T for 32 keys x 32 queries: two independent MFMA chains
        elem8 ka[8], va[8];
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int s8 = 0; s8 < 8; ++s8) {
          ka[s8] = *lds_ptr<const elem8>(foff[s8] + (ks + kb * 8192));
          va[s8] = *lds_ptr<const elem8>(foff[s8] + (vs + kb * 8192));
        }
        f32x16 sacc, dpacc;
#pragma unroll
        for (int e = 0; e < 16; ++e) { sacc[e] = 0.f; dpacc[e] = 0.f; }
#pragma unroll
        for (int s8 = 0; s8 < 8; ++s8) {
          sacc = mfma32(ka[s8], bq[s8], sacc);
          dpacc = mfma32(va[s8], bdo[s8], dpacc);
        }
        // 8 fragment reads ahead, then reads and MFMAs in step (bounded register use)
        __builtin_amdgcn_sched_group_barrier(0x100, 8, 0);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);
          __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
        }
        __builtin_amdgcn_sched_group_barrier(0x008, 8, 0);
        __builtin_amdgcn_sched_barrier(0);
        // the first K^T operands of the dQ product travel while the exponentials run
        elem4 tr[8][2];
        auto issue_tr = [&](int idx) __attribute__((always_inline)) {
          const int j2 = idx >> 2, db = idx & 3;
          tr[idx][0] = lds_read_tr<elem4>(toffA[db] + (ks + 16 * (2 * kb + j2) * 256));
          tr[idx][1] = lds_read_tr<elem4>(toffB[db] + (ks + 16 * (2 * kb + j2) * 256));
        };
#pragma unroll
        for (int idx = 0; idx < 4; ++idx) issue_tr(idx);
        __builtin_amdgcn_sched_barrier(0);
        if (masked) {
#pragma unroll
          for (int e = 0; e < 16; ++e) {
            const int key = kt * TN + 32 * kb + 8 * (e >> 2) + 4 * hh + (e & 3);
            if (key > limit) sacc[e] = -INFINITY;
          }
        }
        elem8 dsb[2];
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const float pe = fast_exp2(sacc[e] * sl2 - lse2);
          dsb[e >> 3][e & 7] = (elem)(pe * (dpacc[e] - dl));
        }
        __builtin_amdgcn_sched_barrier(0);
        // dQ^T += K^T dS^T
#pragma unroll
        for (int idx = 0; idx < 8; ++idx) {
          if (idx + 4 < 8) issue_tr(idx + 4);
          elem8 a;
          a[0] = tr[idx][0][0]; a[1] = tr[idx][0][1]; a[2] = tr[idx][0][2]; a[3] = tr[idx][0][3];
          a[4] = tr[idx][1][0]; a[5] = tr[idx][1][1]; a[6] = tr[idx][1][2]; a[7] = tr[idx][1][3];
          dqacc[idx & 3] = mfma32(a, dsb[idx >> 2], dqacc[idx & 3]);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
    if (has_next) {
      wait_vmem();
      scrub_tile(key_tile(it + 1), buf ^ 1);
    }
    __syncthreads();
  };
  {
    int it = 0;
    for (; it + 1 < nkt; it += 2) {
      key_tile_body(it, std::integral_constant<int, 0>{});
      key_tile_body(it + 1, std::integral_constant<int, 1>{});
    }
    if (it < nkt) key_tile_body(it, std::integral_constant<int, 0>{});
  }

  // The accumulators hold dQ^T (a lane owns 4-element pieces of one row).  The partial is rounded to the
  // element type, as the per-chunk dQ that flash-attn returns to the reference is, and goes through this
  // wave's 8 KiB of LDS (free since the barrier that ended the last key tile) so that it leaves as whole
  // 256-byte rows, four per store instruction.
  {
    char* stage = smem + wave_u * 8192;
    char* wrow = stage + n * 256 + 8 * hh;
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        u32x2 w;
        // (scaled before the rounding: a partial then overflows fp16 only where dQ itself would)
        w[0] = pack2<E>(dqacc[db][4 * g + 0] * p.scale, dqacc[db][4 * g + 1] * p.scale);
        w[1] = pack2<E>(dqacc[db][4 * g + 2] * p.scale, dqacc[db][4 * g + 3] * p.scale);
        // elements 32*db + 8*g + 4*hh .. +3 of row n: 16-byte column 4*db + g, swizzled by the row
        *reinterpret_cast<u32x2*>(wrow + (((4 * db + g) ^ (n & 15)) << 4)) = w;
      }
    const int c16 = lane & 15;
    const int rows_here = t.row_count - wave_u * 32;  // rows of this wave that exist
    // (a tile of a chunk without history slots holds the whole dQ of its rows: nothing to add it to)
    elem* const dq_base = t.direct ? p.dq : p.part_dq;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      const int row = 4 * i + (lane >> 4);
      const int dest = __shfl(t.dest, row, 64);
      const u32x4 x = *reinterpret_cast<const u32x4*>(stage + row * 256 + ((c16 ^ (row & 15)) << 4));
      if (row < rows_here) *reinterpret_cast<u32x4*>(dq_base + (int64_t)dest * kHeadDim + c16 * 8) = x;
    }
  }
  }  // tiles
}

// dq[row] = sum over the row's valid slots of part_dq (in fp32); 16 lanes per row.  With token ranges (mrg_start /
// mrg_prefix, as in the forward's merge) only the rows of those tokens, `rows` counting them: the dQ kernel wrote
// the others itself.
template <class E>
__global__ __launch_bounds__(256) void bwd_dq_reduce_kernel(const typename E::elem* __restrict__ part_dq,
                                                            const int* __restrict__ sel,
                                                            typename E::elem* __restrict__ dq, int64_t rows, int K1,
                                                            int parts, int64_t all_rows,
                                                            const int* __restrict__ mrg_start,
                                                            const int* __restrict__ mrg_prefix, int nranges, int H) {
  MOBA_ELEM_TYPES(E)
  const int64_t row_raw = (int64_t)blockIdx.x * 16 + (threadIdx.x >> 4);
  const bool row_ok = row_raw < rows;
  int64_t row = row_ok ? row_raw : rows - 1;  // whole 16-lane groups stay active for the shuffles
  if (mrg_start) {
    const int t = (int)(row / H), h = (int)(row - (int64_t)t * H);
    const int b = upper_row(mrg_prefix, nranges, t);
    row = (int64_t)(mrg_start[b] + (t - mrg_prefix[b])) * H + h;
  }
  const int c8 = threadIdx.x & 15;
  const int K = K1 - 1;
  const int* ps = sel + row * K;
  float acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = 0.f;
  const elem* src = part_dq + row * K1 * kHeadDim + c8 * 8;
  // lane c8 fetches the presence of slot j0 + c8; absent slots are redirected to slot 0 and
  // multiplied by 0, so the loads of eight slots are unconditional and in flight together.
  // With parts, slot v of the parts * K1 is slot v % K1 of part v / K1, rows * K1 slot rows behind the part
  // before (an int: the buffer holds fewer than 2^31 slot rows); the self slot exists in part 0 only.
  const int nvirt = parts * K1;
  const int part_rows = (int)(all_rows * K1);
  if (nvirt <= 8) {  // (uniform)
    // Few slots: all are requested at once, before the picks that say which are present have arrived -- one
    // round trip instead of two.  (An absent slot's bytes are whatever the buffer holds: dropped by selection.)
    elem8 a[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int part = parts == 1 ? 0 : u / K1, j = u - part * K1;
      if (u < nvirt)
        a[u] = __builtin_nontemporal_load(reinterpret_cast<const elem8*>(src + (int64_t)(part * part_rows + j) * kHeadDim));
    }
    const int part = parts == 1 ? 0 : c8 / K1, j = c8 - part * K1;
    const bool ok = c8 < nvirt && (j == 0 ? part == 0 : ps[j - 1] >= 0);
    const float present = ok ? 1.f : 0.f;
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      if (u >= nvirt) break;
      const float w = __shfl(present, u, 16);
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] += w > 0.f ? (float)a[u][e] : 0.f;
    }
    if (!row_ok) return;
    elem8 o;
#pragma unroll
    for (int e = 0; e < 8; ++e) o[e] = (elem)acc[e];
    *reinterpret_cast<elem8*>(dq + row * kHeadDim + c8 * 8) = o;
    return;
  }
  for (int j0 = 0; j0 < nvirt; j0 += 16) {
    const int v = j0 + c8;
    const int part = parts == 1 ? 0 : v / K1, j = v - part * K1;
    const bool ok = v < nvirt && (j == 0 ? part == 0 : ps[j - 1] >= 0);
    const float present = ok ? 1.f : 0.f;
    const int at = ok ? part * part_rows + j : 0;
    const int nslot = min(16, nvirt - j0);
    for (int u0 = 0; u0 < nslot; u0 += 8) {
      elem8 a[8];
      float w[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        w[u] = __shfl(present, u0 + u, 16);
        const int jj = parts == 1 ? (w[u] > 0.f ? j0 + u0 + u : 0) : __shfl(at, u0 + u, 16);
        if (u0 + u < nslot)  // uniform: no loads for slots that do not exist
          a[u] = __builtin_nontemporal_load(reinterpret_cast<const elem8*>(src + (int64_t)jj * kHeadDim));
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        if (u0 + u >= nslot) break;
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] += w[u] * (float)a[u][e];
      }
    }
  }
  if (!row_ok) return;
  elem8 o;
#pragma unroll
  for (int e = 0; e < 8; ++e) o[e] = (elem)acc[e];
  *reinterpret_cast<elem8*>(dq + row * kHeadDim + c8 * 8) = o;
}

// ------------------------------------------------------------------------------------ dK, dV
// kBatched: q is a batched layout (rows of different batch entries are not an affine function of the token);
// the common case has no division and no branch in the address of a gathered Q row.
template <class E, bool kBatched>
__global__ __launch_bounds__(256, 1) void bwd_dkv_kernel(const BwdParams<E> p) {
  MOBA_ELEM_TYPES(E)
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int n = lane & 31, hh = lane >> 5;
  const int H = p.t.H, K1 = p.t.K1, Hkv = p.t.Hkv, rep = p.t.rep;

  // The workgroups (one per CU, all resident) draw their tiles from eight queues, one per XCD: queue x
  // hands out the ids (8i + x) * kXcdBlock + j in order -- consecutive ids, i.e. key tiles of one
  // (chunk, head) that gather the same Q and dO rows, run side by side behind one L2 -- and a workgroup whose
  // queue is empty goes on with the next XCD's, so that the XCDs, which differ in speed by a few percent,
  // finish together.  A tile runs for about a millisecond: the draw (one atomic, two barriers) is free.
  const int ql = p.queues_log2, qmask = (1 << ql) - 1;
  int queue = blockIdx.x & qmask, empty_queues = 0;
  while (true) {
  __syncthreads();  // every wave is done with the LDS of the previous tile and has read the previous draw
  if (tid == 0)
    *reinterpret_cast<int*>(smem + kDkvIdSlot) =
        __hip_atomic_fetch_add(p.queues + 8 + queue, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  __syncthreads();
  const int drawn = __builtin_amdgcn_readfirstlane(*reinterpret_cast<const int*>(smem + kDkvIdSlot));
  const int64_t id = (((int64_t)(drawn / kXcdBlock) << ql) + queue) * kXcdBlock + (drawn % kXcdBlock);
  const int split = p.dkv_split;
  if (id >= (int64_t)p.kv_total * split) {
    queue = (queue + 1) & qmask;
    if (++empty_queues > qmask) break;
    continue;
  }
  empty_queues = 0;
  // ---- which part of which 128-key tile (consecutive ids: the parts of one tile) ----
  const int unit = (int)id;
  const int part = unit % split;
  const KvTile kt = decode_kv_tile(p, unit / split);
  const int c = kt.c, hkv = kt.hkv, c0 = kt.c0, len = kt.len, key0 = kt.key0;
  const int mykey = key0 + wave * 32 + n;        // position inside the chunk
  const bool key_valid = mykey < len;

  // ---- the rows that attend these keys: the causal rows (of the chunk, or of its dense prefix), then the gather list ----
  const int self_rows = kt.self_len - key0;      // chunk positions key0 .. self_len-1
  const int nself = (self_rows + TQ - 1) / TQ;
  const int fid = (p.chunk_fid && K1 > 1) ? p.chunk_fid[c] : -1;
  // the query heads of this key/value head are walked one after the other; per head:
  int h = hkv * rep, list_base = 0, list_rows = 0, ntile = nself;
  auto select_head = [&](int hq) __attribute__((always_inline)) {
    h = hq;
    list_base = 0;
    list_rows = 0;
    if (fid >= 0) {
      list_base = p.t.seg_off[fid * H + hq];
      list_rows = p.t.seg_off[fid * H + hq + 1] - list_base;
    }
    ntile = nself + (list_rows + TQ - 1) / TQ;
  };

  // ---- K^T and V^T operands of this lane's key: [16*ks + 8*hh .. +7] ----
  elem8 bk[8], bv[8];
  {
    const int64_t off = kv_tok_bytes(p.t, c0) + min(mykey, len - 1) * p.t.kv_tok_b + hkv * p.t.kv_head_b + 16 * hh;  // bytes
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      bk[ks] = *reinterpret_cast<const elem8*>((const char*)p.k + off + 32 * ks);
      bv[ks] = *reinterpret_cast<const elem8*>((const char*)p.v + off + 32 * ks);
    }
  }

  // ---- stage loader: TQ rows of Q and dO (16 KiB each) + lse + delta ----
  const uint32_t lds_base = lds_addr(smem);
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  const int ld_rin = lane >> 4, ld_pc = lane & 15;
  // Row lookups run one stage ahead of the copies: fetch_rows(qi) starts the load of the gather-list entries of
  // stage qi (self stages need none), prepare_stage(qi) turns them into tokens.  Rows past the end repeat the last
  // row.  A lane looks up row `lane` of the stage (the row whose lse and delta it copies); the 16 rows whose Q and
  // dO this wave copies, 4*(4*i + wave) + lane/16 for i < 4, are among those 64: their tokens come from the
  // lanes that hold them (ds_bpermute), one lookup and one division per lane and stage instead of five.
  int raw = 0;
  auto fetch_rows = [&](int qi) __attribute__((always_inline)) {
    if (qi < nself || qi >= ntile) return;
    raw = p.t.seg_dest[list_base + min((qi - nself) * TQ + lane, list_rows - 1)];
  };
  const int row_src_lane4 = (4 * wave_u + ld_rin) * 4;  // 4 x the lane that holds row 4*(4*0 + wave) + lane/16
  uint64_t q_lane_base = 0, do_lane_base = 0;  // this lane's 16 bytes in token 0's row of q and dO, head h
  auto set_lane_bases = [&]() __attribute__((always_inline)) {
    const int c16 = ld_pc ^ (ld_rin << 2) ^ (wave_u & 3);  // sw_col16(4*slab + ld_rin, ld_pc) for slab = 4*i + wave
    q_lane_base = (uint64_t)p.q + (uint64_t)((int64_t)h * p.t.q_head_b + c16 * 16);
    do_lane_base = (uint64_t)p.dout + (uint64_t)(h * (kHeadDim * 2) + c16 * 16);
  };
  int toks[5];  // tokens of the rows of the stage whose copies are being issued
  auto prepare_stage = [&](int qi) __attribute__((always_inline)) {
    // (a list entry is (token*H + h)*K1 + 1 + slot with H*K1 >= 2: the quotient by H*K1 is the high word of the
    // product with the magic number, shifted; exact for entries below 2^31)
    toks[4] = qi < nself ? c0 + key0 + min(qi * TQ + lane, self_rows - 1)
                         : (int)(__umulhi((uint32_t)raw, p.hk_magic) >> (p.hk_shift - 32));
#pragma unroll
    for (int i = 0; i < 4; ++i) toks[i] = __builtin_amdgcn_ds_bpermute(row_src_lane4 + 64 * i, toks[4]);
  };
  // part g of the 8 row copies of a stage (slab g/2 of Q for even g, of dO for odd g); the last part also
  // brings the softmax statistics.  A copy instruction occupies the wave for tens of cycles while the
  // address unit takes its 64 lanes, so the parts are issued one at a time between MFMAs, not in a burst.
  // The 16 bytes a lane copies lie at the same place in every row it copies (the swizzled column of row
  // 4*slab + lane/16 depends on the slab only through slab % 4, which is the wave): with that place added to
  // the head's base once per head, the address of a copy is one multiply-add of the row's token (tokens and
  // token strides fit 32 bits).
  auto issue_part = [&](int g, int buf) __attribute__((always_inline)) {
    const uint32_t qdst = lds_base + buf * kQStage;
    const int i = g >> 1;
    const int slab = 4 * i + wave_u;
    if ((g & 1) == 0) {
      if constexpr (kBatched)
        async_copy16((const char*)q_lane_base + q_tok_bytes(p.t, toks[i]), qdst + slab * 1024);
      else
        async_copy16((const char*)(q_lane_base + (uint64_t)(uint32_t)toks[i] * (uint32_t)p.t.q_tok_b), qdst + slab * 1024);
    } else {
      async_copy16((const char*)(do_lane_base + (uint64_t)(uint32_t)toks[i] * (uint32_t)(H * kHeadDim * 2)),
                   qdst + TQ * kHeadDim * 2 + slab * 1024);
    }
    if (g == 7 && wave_u < 2) {
      const float* src = (wave_u == 0 ? p.lse2 : p.delta) + ((int64_t)toks[4] * H + h);
      async_copy4(src, qdst + 2 * TQ * kHeadDim * 2 + wave_u * (TQ * 4));
    }
  };
  auto issue_stage = [&](int qi, int buf) __attribute__((always_inline)) {
    prepare_stage(qi);
#pragma unroll
    for (int g = 0; g < 8; ++g) issue_part(g, buf);
  };
  auto no_dma = [](int) __attribute__((always_inline)) {};

  f32x16 dkacc[4], dvacc[4];
#pragma unroll
  for (int db = 0; db < 4; ++db)
#pragma unroll
    for (int e = 0; e < 16; ++e) { dkacc[db][e] = 0.f; dvacc[db][e] = 0.f; }
  const float sl2 = p.scale_log2;

  const int g16 = lane >> 4, i0 = (lane & 15) >> 2, i1 = lane & 3;
  const int row_off = n * 256;
  const int row_sw = ((n & 3) << 2) ^ ((n >> 2) & 3);
  const int tr_c16 = 2 * (g16 & 1) + (i1 >> 1);
  const int tr_sub = (i1 & 1) * 8;

  // The loop is software pipelined over blocks of 32 query rows (two per stage):
  //   phase A of block b: the 16 MFMAs of S and dO V^T of block b+1, one per slot, each slot
  //                       also holding the exponential of one element of block b -- MFMA and
  //                       VALU pipes busy together;
  //   phase B of block b: dV^T += dO^T P and dK^T += Q^T dS (16 MFMAs fed by transposed LDS
  //                       reads), while the row fragments and softmax statistics that the
  //                       next phase A needs are fetched from LDS.
  // Three LDS stages and one barrier per stage: at the barrier after phase A of the first
  // block of stage s every wave is past stage s-1, whose buffer then takes stage s+2, and the
  // copies of stage s+1 (issued one stage earlier) have landed.
#define MOBA_PIN(x) asm volatile("" : "+v"(x))
  elem8 qa[8], oa[8];  // row fragments of the block whose S comes next
  f32x4 l4[4], d4[4];   // log2-LSE and delta of the rows of the block whose P comes next
  auto load_frags = [&](const char* qs, int qb) __attribute__((always_inline)) {
    const char* os = qs + TQ * kHeadDim * 2;
#pragma unroll
    for (int s8 = 0; s8 < 8; ++s8) {
      const int o = qb * 8192 + row_off + (((2 * s8 + hh) ^ row_sw) << 4);
      qa[s8] = *reinterpret_cast<const elem8*>(qs + o);
      oa[s8] = *reinterpret_cast<const elem8*>(os + o);
    }
  };
  auto load_stats = [&](const char* qs, int qb) __attribute__((always_inline)) {
    const float* lse_s = reinterpret_cast<const float*>(qs + 2 * TQ * kHeadDim * 2);
    const float* del_s = lse_s + TQ;
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      l4[g] = *reinterpret_cast<const f32x4*>(lse_s + 32 * qb + 8 * g + 4 * hh);
      d4[g] = *reinterpret_cast<const f32x4*>(del_s + 32 * qb + 8 * g + 4 * hh);
    }
  };
  // S and dO V^T from qa/oa into (s_next, dp_next); P and dS of (s_cur, dp_cur) with l4/d4.
  // Block rows are 32*qb + 8g + 4hh + r; `rows_ok` rows of the stage are real, self stages are causal.
  auto phase_a = [&](f32x16& s_next, f32x16& dp_next, const f32x16& s_cur, const f32x16& dp_cur, auto masked_c,
                     int qb, int rows_ok, bool is_self, int qpos0, elem8 (&pb)[2], elem8 (&dsb)[2], auto dma)
                     __attribute__((always_inline)) {
    __builtin_amdgcn_sched_barrier(0);
    // The product of element e is formed in the slot of element e+1: an exponential followed at once by
    // an instruction that uses it costs an idle issue cycle.
    float pe[16], ds[16], sx[16], dx[16];
#pragma unroll
    for (int k = 0; k < 16; k += 2) {
      const int s8 = k >> 1;
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        if (u == 0) mfma32_into_vgprs(s_next, qa[s8], bk[s8], s8 == 0);
        else        mfma32_into_vgprs(dp_next, oa[s8], bv[s8], s8 == 0);
        const int e = k + u, g = e >> 2, rr = e & 3;
        // (the inputs of an element are taken up one slot before the element's own: without the pins the
        // scale-and-subtract of all sixteen elements runs ahead of the first MFMA of the phase, with the matrix
        // pipe idle meanwhile; a pin right in front of its use costs a wait state)
        if (e == 0) {
          sx[0] = s_cur[0];
          MOBA_PIN(sx[0]);
        }
        if (e + 1 < 16) {
          sx[e + 1] = s_cur[e + 1];
          MOBA_PIN(sx[e + 1]);
        }
        dx[e] = dp_cur[e];
        MOBA_PIN(dx[e]);
        pe[e] = fast_exp2(sx[e] * sl2 - l4[g][rr]);
        if (e > 0) {
          ds[e - 1] = pe[e - 1] * (dx[e - 1] - d4[(e - 1) >> 2][(e - 1) & 3]);
          MOBA_PIN(ds[e - 1]);
        }
        if constexpr (decltype(masked_c)::value) {
          const int row = 32 * qb + 8 * g + 4 * hh + rr;
          const bool ok = (row < rows_ok) && (!is_self || qpos0 + row >= mykey);
          pe[e] = ok ? pe[e] : 0.f;
        }
        MOBA_PIN(pe[e]);
        __builtin_amdgcn_sched_barrier(0);
      }
      pb[k >> 3][k & 7] = (elem)pe[k];
      pb[k >> 3][(k & 7) + 1] = (elem)pe[k + 1];
      if (k > 0) {
        dsb[(k - 2) >> 3][(k - 2) & 7] = (elem)ds[k - 2];
        dsb[(k - 2) >> 3][((k - 2) & 7) + 1] = (elem)ds[k - 1];
      }
      dma(k >> 1);  // one global -> LDS copy (or nothing) per pair of MFMAs
      __builtin_amdgcn_sched_barrier(0);
    }
    ds[15] = pe[15] * (dx[15] - d4[3][3]);
    dsb[1][6] = (elem)ds[14];
    dsb[1][7] = (elem)ds[15];
    __builtin_amdgcn_sched_barrier(0);
  };
  // accumulate block (qs, qb); meanwhile fetch the fragments of (qs_f, qb_f) and the statistics of (qs_s, qb_s).
  // Eight slots of two MFMAs; the four transposed reads of a slot are issued two slots ahead (an LDS read takes
  // longer than a slot), the 24 prefetch reads ride along, three per slot.
  auto phase_b = [&](const char* qs, int qb, const elem8 (&pb)[2], const elem8 (&dsb)[2], const char* qs_f, int qb_f,
                     const char* qs_s, int qb_s) __attribute__((always_inline)) {
    const char* os = qs + TQ * kHeadDim * 2;
    const char* os_f = qs_f + TQ * kHeadDim * 2;
    const float* lse_s = reinterpret_cast<const float*>(qs_s + 2 * TQ * kHeadDim * 2);
    const float* del_s = lse_s + TQ;
    elem4 ring[3][4];
    auto issue = [&](int idx, int r) __attribute__((always_inline)) {
      const int j2 = idx >> 2, db = idx & 3;
      const int rowA = 32 * qb + 16 * j2 + 4 * hh + i0;
      const int rowB = rowA + 8;
      const int c16 = 4 * db + tr_c16;
      const int offA = rowA * 256 + ((c16 ^ (i0 << 2) ^ hh) << 4) + tr_sub;
      const int offB = rowB * 256 + ((c16 ^ (i0 << 2) ^ (hh + 2)) << 4) + tr_sub;
      ring[r][0] = lds_read_tr<elem4>(os + offA);
      ring[r][1] = lds_read_tr<elem4>(os + offB);
      ring[r][2] = lds_read_tr<elem4>(qs + offA);
      ring[r][3] = lds_read_tr<elem4>(qs + offB);
    };
    __builtin_amdgcn_sched_barrier(0);
    issue(0, 0);
    issue(1, 1);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int idx = 0; idx < 8; ++idx) {
      const int r = idx % 3;
      if (idx + 2 < 8) issue(idx + 2, (idx + 2) % 3);
      // prefetches: statistics in the first four slots, two row fragments in every slot
      if (idx < 4) {
        l4[idx] = *reinterpret_cast<const f32x4*>(lse_s + 32 * qb_s + 8 * idx + 4 * hh);
        d4[idx] = *reinterpret_cast<const f32x4*>(del_s + 32 * qb_s + 8 * idx + 4 * hh);
      }
      {
        const int o = qb_f * 8192 + row_off + (((2 * idx + hh) ^ row_sw) << 4);
        qa[idx] = *reinterpret_cast<const elem8*>(qs_f + o);
        oa[idx] = *reinterpret_cast<const elem8*>(os_f + o);
      }
      elem8 ao, aq;
      ao[0] = ring[r][0][0]; ao[1] = ring[r][0][1]; ao[2] = ring[r][0][2]; ao[3] = ring[r][0][3];
      ao[4] = ring[r][1][0]; ao[5] = ring[r][1][1]; ao[6] = ring[r][1][2]; ao[7] = ring[r][1][3];
      aq[0] = ring[r][2][0]; aq[1] = ring[r][2][1]; aq[2] = ring[r][2][2]; aq[3] = ring[r][2][3];
      aq[4] = ring[r][3][0]; aq[5] = ring[r][3][1]; aq[6] = ring[r][3][2]; aq[7] = ring[r][3][3];
      const int j2 = idx >> 2, db = idx & 3;
      dvacc[db] = mfma32(ao, pb[j2], dvacc[db]);
      dkacc[db] = mfma32(aq, dsb[j2], dkacc[db]);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  for (int hq = hkv * rep; hq < (hkv + 1) * rep; ++hq) {
  select_head(hq);
  // this part's share of the head's stages
  const int q_first = (int)((int64_t)ntile * part / split), q_end = (int)((int64_t)ntile * (part + 1) / split);
  if (q_end == q_first) continue;  // (uniform)
  set_lane_bases();
  __syncthreads();  // every wave is done with the LDS stages of the previous head
  raw = 0;
  fetch_rows(q_first);
  issue_stage(q_first, 0);
  fetch_rows(q_first + 1);
  wait_vmem();
  __syncthreads();
  if (q_end - q_first > 1) issue_stage(q_first + 1, 1);
  fetch_rows(q_first + 2);

  // S of block 0 (a phase A whose softmax half works on zeros and is discarded)
  f32x16 sA, dA, sB, dB;
  {
    elem8 pb[2], dsb[2];
#pragma unroll
    for (int e = 0; e < 16; ++e) { sB[e] = 0.f; dB[e] = 0.f; }
#pragma unroll
    for (int g = 0; g < 4; ++g) { l4[g] = f32x4{0.f, 0.f, 0.f, 0.f}; d4[g] = l4[g]; }
    load_frags(smem, 0);
    phase_a(sA, dA, sB, dB, std::false_type{}, 0, 0, false, 0, pb, dsb, no_dma);
    load_stats(smem, 0);
    load_frags(smem, 1);
  }
  int buf = 0;
  for (int qi = q_first; qi < q_end; ++qi) {
    const char* qs = smem + buf * kQStage;
    const int buf1 = buf == 2 ? 0 : buf + 1;
    const int buf2 = buf1 == 2 ? 0 : buf1 + 1;
    const bool has_next = qi + 1 < q_end;
    const bool is_self = qi < nself;
    // number of real rows in this stage, and for self stages the chunk position of row 0
    const int rows_here = is_self ? min(TQ, self_rows - qi * TQ) : min(TQ, list_rows - (qi - nself) * TQ);
    const int qpos0 = key0 + qi * TQ;  // only meaningful for self stages
    // causal masking can only bite while the stage's first row is before the wave's last key
    const bool masked = (rows_here < TQ) || (is_self && qpos0 < key0 + wave * 32 + 31);
    // the block after the last one is the last one again: its S is computed and dropped
    const char* qs_next = has_next ? smem + buf1 * kQStage : qs;
    elem8 pb[2], dsb[2];

    if (masked) phase_a(sB, dB, sA, dA, std::true_type{}, 0, rows_here, is_self, qpos0, pb, dsb, no_dma);
    else        phase_a(sB, dB, sA, dA, std::false_type{}, 0, rows_here, is_self, qpos0, pb, dsb, no_dma);

    if (has_next) wait_vmem();
    __syncthreads();
    // the copies of stage qi+2 go out one at a time inside the next phase A
    // (past the last stage the copies go on, into buffers that nobody reads, with the rows of the last
    // lookup: the stage loop then has no branch around any of them)
    prepare_stage(qi + 2);
    fetch_rows(qi + 3);

    phase_b(qs, 0, pb, dsb, qs_next, 0, qs, 1);
    auto dma = [&](int g) __attribute__((always_inline)) { issue_part(g, buf2); };
    if (masked) phase_a(sA, dA, sB, dB, std::true_type{}, 1, rows_here, is_self, qpos0, pb, dsb, dma);
    else        phase_a(sA, dA, sB, dB, std::false_type{}, 1, rows_here, is_self, qpos0, pb, dsb, dma);
    phase_b(qs, 1, pb, dsb, qs_next, 1, qs_next, 0);
    buf = buf1;
  }
  // The last phase A left an S and a dO V^T that nobody reads: their registers may be reused at once on the way
  // out of the loop, and the compiler puts no wait states behind the hand-issued MFMAs that wrote them.
  asm volatile("s_nop 15");
  wait_vmem();  // (the copies past the last stage: nothing may be on its way into LDS when the workgroup ends)
  }  // query heads

  if (split > 1) {
    // this part's sums, unscaled, in fp32: [dk, dv][key of the tile][128]
    float* dst = p.part_dkv + (int64_t)unit * (2 * TM * kHeadDim) + (wave * 32 + n) * kHeadDim + 4 * hh;
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        *reinterpret_cast<f32x4*>(dst + 32 * db + 8 * g) =
            f32x4{dkacc[db][4 * g + 0], dkacc[db][4 * g + 1], dkacc[db][4 * g + 2], dkacc[db][4 * g + 3]};
        *reinterpret_cast<f32x4*>(dst + TM * kHeadDim + 32 * db + 8 * g) =
            f32x4{dvacc[db][4 * g + 0], dvacc[db][4 * g + 1], dvacc[db][4 * g + 2], dvacc[db][4 * g + 3]};
      }
  } else if (key_valid) {
    const int64_t off = ((int64_t)(c0 + mykey) * Hkv + hkv) * kHeadDim;
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        u32x2 wk, wv;
        wk[0] = pack2<E>(dkacc[db][4 * g + 0] * p.scale, dkacc[db][4 * g + 1] * p.scale);
        wk[1] = pack2<E>(dkacc[db][4 * g + 2] * p.scale, dkacc[db][4 * g + 3] * p.scale);
        wv[0] = pack2<E>(dvacc[db][4 * g + 0], dvacc[db][4 * g + 1]);
        wv[1] = pack2<E>(dvacc[db][4 * g + 2], dvacc[db][4 * g + 3]);
        *reinterpret_cast<u32x2*>(p.dk + off + 32 * db + 8 * g + 4 * hh) = wk;
        *reinterpret_cast<u32x2*>(p.dv + off + 32 * db + 8 * g + 4 * hh) = wv;
      }
  }
  }  // tiles
#undef MOBA_PIN
}

// dk, dv of the 128-key tiles from the fp32 sums of their parts, added in the order of the parts.
// Sixteen workgroups per tile; a thread owns four consecutive elements of one key (coalesced 16-byte loads).
template <class E>
__global__ __launch_bounds__(256) void bwd_dkv_reduce_kernel(const BwdParams<E> p) {
  MOBA_ELEM_TYPES(E)
  const int tile = blockIdx.x >> 4;
  const KvTile kt = decode_kv_tile(p, tile);
  const int in_tile = (blockIdx.x & 15) * 256 + threadIdx.x;  // 128 keys x 32 groups of four elements
  const int key = in_tile >> 5, d = (in_tile & 31) * 4;
  if (kt.key0 + key >= kt.len) return;
  const int split = p.dkv_split;
  const float* src = p.part_dkv + (int64_t)tile * split * (2 * TM * kHeadDim) + key * kHeadDim + d;
  f32x4 sk = {0.f, 0.f, 0.f, 0.f}, sv = sk;
  for (int r = 0; r < split; ++r) {
    const float* s = src + (int64_t)r * (2 * TM * kHeadDim);
    sk += *reinterpret_cast<const f32x4*>(s);
    sv += *reinterpret_cast<const f32x4*>(s + TM * kHeadDim);
  }
  const int64_t off = ((int64_t)(kt.c0 + kt.key0 + key) * p.t.Hkv + kt.hkv) * kHeadDim + d;
  u32x2 wk, wv;
  wk[0] = pack2<E>(sk[0] * p.scale, sk[1] * p.scale);
  wk[1] = pack2<E>(sk[2] * p.scale, sk[3] * p.scale);
  wv[0] = pack2<E>(sv[0], sv[1]);
  wv[1] = pack2<E>(sv[2], sv[3]);
  *reinterpret_cast<u32x2*>(p.dk + off) = wk;
  *reinterpret_cast<u32x2*>(p.dv + off) = wv;
}

}  // namespace moba

using namespace moba;

template <class E>
static int launch_bwd(const void* dout, const void* q, const void* k, const void* v, const void* out, const float* lse,
                      const int32_t* sel, const int32_t* chunk_fid, const int32_t* kv_chunk_tok,
                      const int32_t* kv_tile_prefix, const int32_t* kv_tile_chunk, const int32_t* chunk_self_end,
                      int kv_total, const int32_t* mrg_start, const int32_t* mrg_prefix, int nranges,
                      int64_t merge_tokens, float* delta, void* part_dq, void* dq, void* dk, void* dv, const TileTables& t, int64_t S, int H, int D, int K, float softmax_scale, int64_t grid_q,
                      int64_t grid_kv, int* queues, float* part_dkv, int dkv_split, hipStream_t st) {
  LaunchCheck launch_check;
  typedef typename E::elem elem;
  BwdParams<E> p;
  p.q = (const elem*)q; p.k = (const elem*)k; p.v = (const elem*)v; p.dout = (const elem*)dout;
  p.lse = lse; p.delta = delta; p.lse2 = delta + S * H; p.part_dq = (elem*)part_dq; p.dk = (elem*)dk; p.dv = (elem*)dv;
  p.dq = (elem*)dq;
  p.chunk_fid = chunk_fid;
  p.kv_chunk_tok = kv_chunk_tok; p.kv_tile_prefix = kv_tile_prefix; p.kv_tile_chunk = kv_tile_chunk;
  p.chunk_self_end = chunk_self_end; p.kv_total = kv_total;
  p.queues = queues;
  p.part_dkv = part_dkv;
  p.dkv_split = dkv_split;
  p.queues_log2 = t.self_first ? 0 : 3;
  p.t = t;
  p.scale = softmax_scale > 0.f ? softmax_scale : (float)(1.0 / sqrt((double)D));
  p.scale_log2 = softmax_scale > 0.f ? (float)(1.4426950408889634 * (double)softmax_scale)
                                     : (float)(1.4426950408889634 / sqrt((double)D));
  // division by H*K1 as a multiplication: with s = 31 + ceil(log2 d) and m = floor(2^s / d) + 1 the
  // error m*d - 2^s is at most d <= 2^(s-31), so n*m >> s is the exact quotient for n < 2^31; m < 2^32
  const uint64_t hk = (uint64_t)H * (K + 1);
  uint32_t lg = 1;  // (at least 1: the kernels take the product's high word and shift by hk_shift - 32; a list entry
                    // exists only with K >= 1, hence H*K1 >= 2)
  while ((1ull << lg) < hk) ++lg;
  p.hk_shift = 31 + lg;
  p.hk_magic = (uint32_t)((1ull << p.hk_shift) / hk + 1);

  static bool allowed_dq[kMaxDevices], allowed_dkv[2][kMaxDevices];  // one set per element type
  const bool batched = t.batch_rows != 0;
  if (!allow_dynamic_lds((const void*)bwd_dq_kernel<E>, kBwdDqLds, allowed_dq) ||
      !(batched ? allow_dynamic_lds((const void*)bwd_dkv_kernel<E, true>, kBwdDkvLds, allowed_dkv[1])
                : allow_dynamic_lds((const void*)bwd_dkv_kernel<E, false>, kBwdDkvLds, allowed_dkv[0])))
    return MOBA_ERR_LAUNCH;
  const int64_t rows = S * H;
  hipLaunchKernelGGL(bwd_delta_kernel<E>, dim3((unsigned)((rows + 15) / 16)), dim3(256), 0, st, (const elem*)dout,
                     (const elem*)out, lse, delta, delta + S * H, rows, queues);
  hipLaunchKernelGGL(bwd_dq_kernel<E>, dim3((unsigned)grid_q), dim3(256), kBwdDqLds, st, p);
  if (merge_tokens > 0) {  // (0: the dQ kernel wrote every row itself)
    const int64_t sum_rows = merge_tokens * H;
    hipLaunchKernelGGL(bwd_dq_reduce_kernel<E>, dim3((unsigned)((sum_rows + 15) / 16)), dim3(256), 0, st,
                       (const elem*)part_dq, sel, (elem*)dq, sum_rows, K + 1, 1 << t.key_split_log2, rows, mrg_start,
                       mrg_prefix, nranges, H);
  }
  if (batched) hipLaunchKernelGGL((bwd_dkv_kernel<E, true>), dim3((unsigned)grid_kv), dim3(256), kBwdDkvLds, st, p);
  else hipLaunchKernelGGL((bwd_dkv_kernel<E, false>), dim3((unsigned)grid_kv), dim3(256), kBwdDkvLds, st, p);
  if (dkv_split > 1)
    hipLaunchKernelGGL(bwd_dkv_reduce_kernel<E>, dim3((unsigned)p.kv_total * 16), dim3(256), 0, st, p);
  return launch_check.result();
}

extern "C" int moba_bwd_tile_rows(void) { return TM; }

// Parts per key tile of the dK/dV kernel.  With fewer tiles than two per compute unit the tiles of the first
// chunks of a sequence, whose gather lists are the longest, set the kernel's time while most of the chip is
// idle: they are cut into parts then (at most 4: every part leaves 128 KiB of fp32 sums to be added up).
// Problems below 4096 tokens are too short for the parts' extra traffic to pay.
static int dkv_split_for(int64_t S, int64_t tiles) {
  const int cus = resident_compute_units();
  if (cus <= 0 || tiles <= 0 || tiles >= 2 * (int64_t)cus || S < 4096) return 1;
  const int64_t r = (3 * (int64_t)cus + tiles - 1) / tiles;
  return (int)(r < 1 ? 1 : (r > 4 ? 4 : r));
}

extern "C" size_t moba_bwd_dkv_scratch_bytes(int64_t S, int Hkv, int64_t kv_tiles) {
  if (S <= 0 || Hkv <= 0 || kv_tiles <= 0) return 0;
  const int64_t tiles = kv_tiles * Hkv;
  const int split = dkv_split_for(S, tiles);
  return split > 1 ? (size_t)tiles * split * (2 * TM * kHeadDim) * sizeof(float) : 0;
}

// Parts per history tile of the dQ kernel (a power of two).  With fewer tiles than workgroup slots to fill a few
// times over, a tile of 128 rows x B keys is too coarse a unit: the kernel's time is then two such tiles in a row
// on some workgroups while others idle.  Every part keeps at least 512 keys; part_dq grows by the same factor.
extern "C" int moba_bwd_dq_key_split(int64_t S, int H, int K, int B, int64_t hist_bound, int64_t self_tiles) {
  const int cus = resident_compute_units();
  if (cus <= 0 || S <= 0 || H <= 0 || K <= 0 || B <= 0 || hist_bound <= 0 || self_tiles <= 0) return 1;
  const int64_t slots = 2 * (((int64_t)cus + 7) / 8 * 8), own = self_tiles * H;
  int split = 1;
  while (split < 8 && B % (64 * 2 * split) == 0 && B / (2 * split) >= 512 &&
         own + hist_bound * 2 * split <= 3 * slots && S * H * (K + 1) * 2 * split < 0x7fffffffLL)
    split *= 2;
  return split;
}

extern "C" int moba_bwd(const void* dout, const void* q, const void* k, const void* v, const void* out,
                        const float* lse, const int32_t* sel, const int32_t* seg_off, const int32_t* tile_off,
                        const int32_t* seg_dest, const int32_t* fchunk_tok, const int32_t* chunk_tok,
                        const int32_t* self_tile_prefix, const int32_t* tile_seg, const int32_t* self_tile_chunk,
                        const int32_t* chunk_fid, const int32_t* kv_chunk_tok, const int32_t* kv_tile_prefix,
                        const int32_t* kv_tile_chunk, const int32_t* chunk_self_end, const int32_t* chunk_direct,
                        const int32_t* mrg_start, const int32_t* mrg_prefix, int nranges, int64_t merge_tokens,
                        float* delta, void* part_dq,
                        void* dq, void* dk, void* dv, int64_t S, int H, int Hkv, int D, int K, int F, int N, int B,
                        int64_t hist_bound, int64_t self_tiles, int64_t kv_tiles, int dq_key_split, const int64_t* strides,
                        int32_t* queues, void* dkv_scratch, int64_t dkv_scratch_bytes, float softmax_scale, int dtype,
                        void* stream) {
  if (!dout || !q || !k || !v || !out || !lse || !chunk_tok || !self_tile_prefix || !self_tile_chunk || !delta ||
      !part_dq || !dq || !dk || !dv || !queues || !kv_chunk_tok || !kv_tile_prefix || !kv_tile_chunk || !chunk_self_end)
    return MOBA_ERR_ARG;
  if (K > 0 && (!sel || !seg_off || !tile_off || !seg_dest || !fchunk_tok || !chunk_fid || !tile_seg))
    return MOBA_ERR_ARG;
  if (D != kHeadDim || (dtype != MOBA_DTYPE_BF16 && dtype != MOBA_DTYPE_F16)) return MOBA_ERR_UNSUPPORTED;
  if (S <= 0 || H <= 0 || K < 0 || F < 0 || N <= 0 || B <= 0 || hist_bound < 0 || self_tiles <= 0 || kv_tiles <= 0)
    return MOBA_ERR_ARG;
  if (Hkv <= 0 || H % Hkv != 0) return MOBA_ERR_ARG;
  // (direct rows and the token ranges of the sum over the slots come together: both, or neither and every token)
  if (chunk_direct ? (!mrg_start || !mrg_prefix || nranges <= 0 || merge_tokens < 0 || merge_tokens > S)
                   : (mrg_start || mrg_prefix || merge_tokens != S))
    return MOBA_ERR_ARG;
  const void* ptrs[] = {dout, q, k, v, out, part_dq, dq, dk, dv};
  for (const void* x : ptrs)
    if ((uintptr_t)x & 15) return MOBA_ERR_ARG;
  if (dq_key_split < 1 || dq_key_split > 8 || (dq_key_split & (dq_key_split - 1))) return MOBA_ERR_ARG;
  if (dq_key_split > 1 && (K == 0 || B % (64 * dq_key_split) != 0)) return MOBA_ERR_ARG;
  if ((int64_t)S * H * (K + 1) * dq_key_split >= 0x7fffffffLL) return MOBA_ERR_LIMIT;
  const int64_t total_q = (K > 0 ? hist_bound * dq_key_split : 0) + self_tiles * H;
  // the dK/dV kernel: one workgroup per CU, resident, drawing its tiles from the queues
  const int cus = resident_compute_units();
  if (cus <= 0) return MOBA_ERR_LAUNCH;
  const int64_t grid_kv = ((int64_t)cus + 7) / 8 * 8;
  const int64_t grid_q = 2 * grid_kv;  // the dQ kernel fits two workgroups on a CU
  if (total_q >= 0x7fffffffLL) return MOBA_ERR_LIMIT;
  TileTables t;
  t.seg_off = seg_off; t.tile_off = tile_off; t.seg_dest = seg_dest; t.fchunk_tok = fchunk_tok;
  t.chunk_tok = chunk_tok; t.self_tile_prefix = self_tile_prefix;
  t.tile_seg = tile_seg; t.self_tile_chunk = self_tile_chunk;
  t.S = (int)S; t.H = H; t.K1 = K + 1; t.F = (K > 0) ? F : 0; t.N = N; t.B = B;
  t.Hkv = Hkv; t.rep = H / Hkv;
  t.hist_bound = (K > 0) ? (int)hist_bound : 0;
  t.self_total = (int)(self_tiles * H);
  if (!set_layout(t, strides)) return MOBA_ERR_ARG;
  // the dQ kernel's order of tiles and its parts per history tile (the dK/dV kernel has parts of its own)
  t.self_first = dq_key_split > 1 || total_q < 8 * grid_q;
  while ((1 << t.key_split_log2) < dq_key_split) ++t.key_split_log2;
  t.part_stride = (int)(S * H * (K + 1));
  t.chunk_direct = chunk_direct;
  // the key tiles are cut into parts only if the caller brought the scratch for their sums
  const int64_t kv_total = kv_tiles * Hkv;
  int dkv_split = dkv_split_for(S, kv_total);
  if (dkv_split > 1 && (!dkv_scratch || ((uintptr_t)dkv_scratch & 15) ||
                        dkv_scratch_bytes < (int64_t)(kv_total * dkv_split * (2 * TM * kHeadDim) * sizeof(float))))
    dkv_split = 1;
  if (kv_total * dkv_split >= 0x7fffffffLL) return MOBA_ERR_LIMIT;
  hipStream_t st = (hipStream_t)stream;
  return dtype == MOBA_DTYPE_F16
             ? launch_bwd<F16>(dout, q, k, v, out, lse, sel, chunk_fid, kv_chunk_tok, kv_tile_prefix, kv_tile_chunk,
                               chunk_self_end, (int)kv_total, mrg_start, mrg_prefix, nranges, merge_tokens, delta, part_dq, dq, dk, dv,
                                t, S, H, D, K,
                               softmax_scale, grid_q, grid_kv, queues, (float*)dkv_scratch, dkv_split, st)
             : launch_bwd<Bf16>(dout, q, k, v, out, lse, sel, chunk_fid, kv_chunk_tok, kv_tile_prefix, kv_tile_chunk,
                                chunk_self_end, (int)kv_total, mrg_start, mrg_prefix, nranges, merge_tokens, delta, part_dq, dq, dk, dv,
                                t, S, H, D, K,
                                softmax_scale, grid_q, grid_kv, queues, (float*)dkv_scratch, dkv_split, st);
}
