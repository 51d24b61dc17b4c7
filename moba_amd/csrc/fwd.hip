// Fused MoBA forward for gfx950.
//
// One kernel covers both kinds of work, as tiles of 256 query rows of one head (eight waves of 32 rows:
// one workgroup per CU, so that a K/V tile is copied into the CU's LDS once for 256 rows -- the copies
// global -> LDS are the second largest cost of the kernel after the matrix instructions):
//   history tile : 256 rows of the gather list of segment (filtered chunk f, head h),
//                  against the B keys of chunk f, no mask
//   self tile    : 256 consecutive rows of one chunk against the keys of the same
//                  chunk up to the diagonal (causal); with the chunk table set to whole
//                  sequences this is plain causal attention (the k <= 0 case)
// Each tile runs a flash-style loop over 64-key tiles: K and V tiles are staged in LDS
// (a ring of three stages, bank-conflict-free swizzles), S^T = K Q^T and O^T += V^T P^T use
// v_mfma_f32_32x32x16_bf16 with the query index in the lane dimension, so a row's
// softmax statistics live in one lane pair; V^T fragments come from ds_read_b64_tr_b16.
// A tile writes a normalised partial output (bf16) and its log2-sum-exp into the
// row's slot; the merge kernel combines the K+1 slots of every (token, head).
//
// Algorithmic work: 4*D flops per attended (query, key) pair; the bound is the bf16
// MFMA rate.  Compulsory HBM traffic is q, k, v once, the partials once each way.
#include <cstddef>
#include <type_traits>
#include "attn_common.h"

namespace moba {

// LDS: three K stages, three V stages (a ring: key tile t lives in stage t % 3), then 256 bytes per wave for the
// gather-list entries of the next tile's rows, then the slot through which wave 0 hands the tile id it drew to
// the other waves
constexpr int kFwdWaves = 8;
constexpr int kFwdStages = 3;
constexpr int kFwdVBase = kFwdStages * kTileBytes;
constexpr int kFwdEntries = 2 * kFwdStages * kTileBytes, kFwdIdSlot = kFwdEntries + kFwdWaves * 256;
constexpr int kFwdRedoWord = kFwdIdSlot + 8;  // set by a wave whose rows left the range of the fixed-reference softmax
constexpr int kFwdLds = kFwdIdSlot + 16;

template <class E>
struct FwdParams {
  const typename E::elem* q;
  const typename E::elem* k;
  const typename E::elem* v;
  typename E::elem* part_o;  // [S*H*K1, D]
  float* part_lse;  // [S*H*K1], log2 domain
  typename E::elem* out;     // [S*H, D]: where the tiles of chunks without history slots (TileTables::chunk_direct) write
  float* lse;                // [S*H], natural log
  TileTables t;
  float scale_log2;  // D^-0.5 * log2(e)
  int* queues;       // [8] tile counters, one per XCD, zero when the kernel starts
  int* redo;         // [1 + tiles] count and ids of the tiles to be computed again (see kFixedRef); count zero at the start
};

constexpr float kRescaleThreshold = 8.f;  // log2 units: the running max may lag the true max by this much
// Fixed-reference softmax: a row's sum of exponentials (relative to the row maximum of the tile's first key
// block) at or beyond this, or not a number, sends the tile to the kernel that tracks the maximum; so does an
// accumulator of the row that is not finite (a probability beyond the element type's range -- 2^16 for fp16 --
// or products with large |v| that left fp32).
constexpr float kFixedRefMaxSum = 0x1p96f;

// how a workgroup comes by its tiles
enum : int {
  kTilePerGroup = 0,  // one tile, the id from the workgroup id (small problems)
  kTilesQueued = 1,   // resident workgroups drawing ids from the per-XCD queues
  kTilesListed = 2,   // resident workgroups walking the list FwdParams::redo
};

// The loop is software pipelined by hand at the granularity of a 32-key block u:
//     phase 1:  S^T(u+1)      8 MFMA   with   exponentials 8..15 of block u, packing of P(u)
//     phase 2:  O^T += V^T P^T(u)  8 MFMA   with   row max of block u+1 and its exponentials 0..7
// so the vector work of one block executes under the MFMAs of its neighbours, and the
// fragment reads from LDS run a few MFMAs ahead.
//
// K and V tiles (64 keys) travel through a ring of three LDS stages; every wave copies an eighth of each tile.
// One barrier per key tile, at its top: a wave first waits for its own copies of tile t+1 (issued a whole tile
// earlier), and once all eight waves have passed the barrier tile t+1 is complete in LDS and nobody reads tile
// t-1 any more, so its stage takes tile t+2.
// kMode: resident workgroups that draw tiles from the queues (large problems), or one tile per workgroup,
// the id from the workgroup id: with few tiles the queue protocol's start-up and wind-down (three passes
// to fill the look-ahead, eight empty draws to know that nothing is left) would dominate.
// kFixedRef (queued): the softmax of a tile is taken relative to one fixed reference per row, the row
// maximum of the tile's first 32-key block, instead of a running maximum.  A bf16 probability has the
// exponent range of fp32, so later scores may exceed the reference by almost 2^7 before anything overflows
// (an fp16 probability: by 2^4 = 16 powers of two, still far more than scores of one row differ in practice):
// the per-block row maximum, its exchange between the lane halves, the comparison with the running maximum
// and the rescale branch all go (22 of 88 vector instructions per key block).  A row that leaves the safe
// range -- its sum of exponentials beyond 2^96, or an accumulator that is not finite because a probability
// overflowed the element type -- marks its tile in FwdParams::redo, and the kTilesListed kernel, which tracks
// the maximum, computes those tiles again.  (A probability below the element type's smallest number is lost
// either way; relative to the first block's maximum fewer are than relative to the true one.)
template <class E, int kMode, bool kFixedRef>
__global__ __launch_bounds__(512, 2) void moba_fwd_kernel(const FwdParams<E> p) {
  MOBA_ELEM_TYPES(E)
  constexpr bool kQueued = kMode == kTilesQueued;
  static_assert(!kFixedRef || kQueued, "the fixed reference comes with the queued tiles' redo list");
  extern __shared__ __attribute__((aligned(16))) char smem[];
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63;
  const int n = lane & 31, hh = lane >> 5;
  const int H = p.t.H;

  // The workgroups (two per CU, all resident) draw tiles from eight queues, one per XCD: queue x hands
  // out the ids (8i + x) * kQueueRun + j in order, so that the tiles in flight on an XCD are consecutive ids
  // -- tiles that share a K/V chunk behind one L2 -- and an XCD that runs ahead (they differ by a few
  // percent) goes on with the next queue when its own is empty.  A tile's description takes dependent
  // lookups: the id (an atomic), the big table, the small tables, the gather-list entry of every row.
  // They run three, two and one tile ahead of the tile being computed, each issued at one tile switch
  // and used at the next; the entries travel global -> LDS, so nothing of this occupies vector registers.
  const int r = wave * 32 + n;
  Tile t, t1;              // the tile being computed; the next one (its row entries on their way to LDS)
  int id1 = -1, code1 = kTileUnused;   // id and first lookup of the next tile
  TileHeadEntries head1 = {0, 0, 0, 0, 0};  // its small-table entries
  int id2 = -1, code2 = kTileUnused;   // id and first lookup of the tile after next
  int id3 = -1;                        // id of the tile after that, as drawn
  int queue = blockIdx.x & 7, empty_queues = 0;
  t.row_count = 0; t.nkeys = 0; t.base = -1; t.direct = 0; t1 = t;   // row_count 0: not a tile; nkeys < 0: no tiles left
  int h = 0, nkeys = 0, kv_tok0 = 0, hkv = 0;
  int min_limit = 0;       // smallest row limit of the wave's 32 rows
  bool row_valid = false;
  int limit = 0;           // this lane's row attends keys <= limit
  elem8 bq[8];

  // ---- K/V tile loader: global -> LDS without passing through registers.
  // A wave copy fills 1 KiB = 4 keys x 16 columns of 16 bytes; wave w issues slabs w and w+8 of the
  // tile's 16.  Lane i lands at slab + 16*i, so the lane picks the global column whose swizzled LDS
  // position is i.  LDS: K stages at 0, 16, 32 KiB, V stages at 48, 64, 80 KiB.
  const int64_t row_bytes = p.t.kv_tok_b;                        // from one K or V token to the next
  const uint32_t lds_base = lds_addr(smem);
  const int wave_u = __builtin_amdgcn_readfirstlane(wave);
  const int ld_kin = lane >> 4;  // key within the slab
  const int ld_pc = lane & 15;   // physical 16-byte column
  uint32_t ld_off[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int key = 4 * (8 * i + wave_u) + ld_kin;
    ld_off[i] = (uint32_t)(key * row_bytes + sw_col16(key, ld_pc) * 16);  // the swizzle is an involution
  }
  const char* k_head = nullptr;  // key 0 of the current tile's key range, this tile's key/value head
  const char* v_head = nullptr;
  auto issue = [&](const char* head, int kt, uint32_t dst) __attribute__((always_inline)) {
    const int key0 = kt * TN;
    const bool full = key0 + TN <= nkeys;  // (the keys of a tile all belong to one chunk, hence to one sequence)
    if (full) {  // uniform tile base in SGPRs + constant per-lane offsets: no address arithmetic
      const char* base = head + (int64_t)key0 * row_bytes;
#pragma unroll
      for (int i = 0; i < 2; ++i) async_copy16_sv(base, ld_off[i], dst + (8 * i + wave_u) * 1024);
    } else {
      // (rare path: its per-lane constants are derived here, from a value the compiler cannot trace, so
      // that they are not computed ahead of the tile loop and carried through it in registers)
      int kin = ld_kin;
      asm volatile("" : "+v"(kin));
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int slab = 8 * i + wave_u;
        const int key = 4 * slab + kin;
        // (keys past the end of the range: the last key again -- their scores are masked, their V rows cleared)
        async_copy16(head + (int64_t)min(key0 + key, nkeys - 1) * row_bytes + sw_col16(key, ld_pc) * 16, dst + slab * 1024);
      }
    }
  };
  auto issue_k = [&](int kt, int stage) __attribute__((always_inline)) { issue(k_head, kt, lds_base + stage * kTileBytes); };
  auto issue_v = [&](int kt, int stage) __attribute__((always_inline)) { issue(v_head, kt, lds_base + kFwdVBase + stage * kTileBytes); };
  // rows of V past the end of the key range must not reach the MFMA (0 * NaN): clear them
  auto scrub_v = [&](int kt, int stage) __attribute__((always_inline)) {
    const int key0 = kt * TN;
    if (key0 + TN <= nkeys) return;
    char* vdst = smem + kFwdVBase + stage * kTileBytes;
    int ln = lane;  // rare path: see the remark in the loader
    asm volatile("" : "+v"(ln));
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int slab = 8 * i + wave_u;
      const int key = 4 * slab + (ln >> 4);
      if (key0 + key >= nkeys) *reinterpret_cast<u32x4*>(vdst + slab * 1024 + ln * 16) = u32x4{0, 0, 0, 0};
    }
  };
  // Tiles that run side by side on an XCD work on the same chunk; starting each at a
  // different key tile spreads their first touches of the chunk over all of it.
  int nkt = 1, rot = 0;
  auto key_tile = [&](int it) __attribute__((always_inline)) { const int x = it + rot; return x >= nkt ? x - nkt : x; };

  // ---- fragment addressing: per-lane LDS byte addresses inside a tile (numbers, not pointers into smem:
  // the address of a read is then one register plus an immediate, with no base left to add) ----
  const int g16 = lane >> 4, i0 = (lane & 15) >> 2, i1 = lane & 3;
  // K row fragment (row 32*kb + n, 16-byte column 2*s8 + hh)
  uint32_t koff[8];
  {
    const int k_sw = ((n & 3) << 2) ^ ((n >> 2) & 3);
#pragma unroll
    for (int s8 = 0; s8 < 8; ++s8) koff[s8] = lds_base + n * 256 + (((2 * s8 + hh) ^ k_sw) << 4);
  }
  // V^T quads: rows 32*kb + 16*j2 + 4*hh + i0 (A) and +8 (B), 8 bytes at d = 32*db + 16*(g16&1) + 4*i1
  // (addresses inside V stage 0: the immediate of a read spans 64 KiB, not the whole ring)
  uint32_t voffA[4], voffB[4];
  {
    const int v_c16 = 2 * (g16 & 1) + (i1 >> 1);
    const int v_sub = (i1 & 1) * 8;
#pragma unroll
    for (int db = 0; db < 4; ++db) {
      const int c16 = 4 * db + v_c16;
      voffA[db] = lds_base + kFwdVBase + (4 * hh + i0) * 256 + ((c16 ^ (i0 << 2) ^ hh) << 4) + v_sub;
      voffB[db] = lds_base + kFwdVBase + (4 * hh + i0 + 8) * 256 + ((c16 ^ (i0 << 2) ^ (hh + 2)) << 4) + v_sub;
      // finished addresses, kept as they are: the compiler otherwise holds their summands and adds them
      // again at every use (eight additions per key block)
      asm volatile("" : "+v"(voffA[db]));
      asm volatile("" : "+v"(voffB[db]));
    }
  }
  auto k_frag = [&](int tile_off, int kb, int s8) __attribute__((always_inline)) {
    return *lds_ptr<const elem8>(koff[s8] + (uint32_t)(tile_off + kb * 8192));
  };
  auto v_frag = [&](int tile_off, int kb, int j2, int db) __attribute__((always_inline)) {
    const elem4 va = lds_read_tr<elem4>(voffA[db] + (uint32_t)(tile_off + (32 * kb + 16 * j2) * 256));
    const elem4 vb = lds_read_tr<elem4>(voffB[db] + (uint32_t)(tile_off + (32 * kb + 16 * j2) * 256));
    elem8 a;
    a[0] = va[0]; a[1] = va[1]; a[2] = va[2]; a[3] = va[3];
    a[4] = vb[0]; a[5] = vb[1]; a[6] = vb[2]; a[7] = vb[3];
    return a;
  };

  f32x16 oacc[4];
#pragma unroll
  for (int db = 0; db < 4; ++db)
#pragma unroll
    for (int e = 0; e < 16; ++e) oacc[db][e] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;
  const float sl2 = p.scale_log2;

  // mask of a key block starting at key0 (causal diagonal / end of the key range)
  auto mask_block = [&](f32x16& s, int key0) __attribute__((always_inline)) {
#pragma unroll
    for (int e = 0; e < 16; ++e)
      if (key0 + 8 * (e >> 2) + 4 * hh + (e & 3) > limit) s[e] = -INFINITY;
  };
  // running-max update for a block with row max mx (already scaled): returns the factor for older terms
  auto update_max = [&](float mx) __attribute__((always_inline)) {
    const float m_new = (mx > m_run + kRescaleThreshold) ? fmaxf(m_run, mx) : m_run;
    const float alpha = fast_exp2(m_run - m_new);
    m_run = m_new;
    return alpha;
  };
// keeps a value, and therefore the instructions that produce it, at this point of the program
#define MOBA_PIN(x) asm volatile("" : "+v"(x))


  bool have_partial = false;  // the accumulators hold a finished tile whose partial is not written yet
  // The drawn id travels through one of two LDS words, alternating per pass: a pass without a tile has no
  // barrier after the waves read the word, so wave 0 may already be writing the next pass's id -- into the
  // other word.  The word of pass i is rewritten in pass i + 2, behind the barrier of pass i + 1.
  int id_word = 0;
  int dest_done = 0, rows_done = 0, id_done = 0;
  bool valid_done = false, direct_done = false;  // (direct: the tile's rows go straight to the outputs)
  int list_pos = blockIdx.x;  // kTilesListed: position in the list of the next tile
  int key_part = 0;           // kTilePerGroup: which part of a history tile's keys this workgroup takes
  if constexpr (kFixedRef) {
    if (tid == 0) *reinterpret_cast<int*>(smem + kFwdRedoWord) = 0;  // first read many barriers from here
  }
  // The finished tile's partial: normalise, write.  The accumulators hold O^T (a lane owns 4-element pieces of
  // one row); the rows go through 4 KiB of LDS per wave, half a row at a time, so that they leave as 128-byte
  // pieces of rows, eight rows per store instruction, instead of 8-byte pieces of 32 rows.  The 4 KiB lie in the
  // third K and V stages, which take their next copies only behind the barrier of the next tile's first key
  // tile: the first two stages are already receiving the next tile's keys and values while this runs.
  auto write_partial = [&]() __attribute__((always_inline)) {
    const FwdParams<E> pn = kernarg_now<FwdParams<E>>(0);
    int ln = lane;  // taken afresh: none of the addresses below is computed ahead of the tile loop
    asm volatile("" : "+v"(ln));
    const int en = ln & 31, ehh = ln >> 5;
    const float l_tot = sum_xhalf(l_run);
    const float inv = 1.f / l_tot;
    if constexpr (kFixedRef) {
      // compared as bit patterns (the file is compiled without NaN semantics): infinities, every NaN and
      // negative sums all read as "too large"; the largest magnitude among the row's accumulators likewise
      uint32_t worst = 0;
#pragma unroll
      for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int e = 0; e < 16; ++e) worst = max(worst, __builtin_bit_cast(uint32_t, oacc[db][e]) & 0x7fffffffu);
      const bool bad = valid_done && (__builtin_bit_cast(uint32_t, l_tot) >= __builtin_bit_cast(uint32_t, kFixedRefMaxSum) ||
                                      worst >= 0x7f800000u);
      if (__any(bad) && ln == 0) *reinterpret_cast<volatile int*>(smem + kFwdRedoWord) = 1;
    }
    char* stage = smem + (wave_u < 4 ? 2 * kTileBytes + wave_u * 4096 : kFwdVBase + 2 * kTileBytes + (wave_u - 4) * 4096);
    char* wrow = stage + en * 128 + 8 * ehh;
    const int wsw = (en >> 1) & 7;  // rows 128 bytes apart: the 16-byte column is swizzled by the row pair
    // a tile of a chunk without history slots writes the operator's outputs (natural-log LSE), any other its slot row
    elem* const o_base = direct_done ? pn.out : pn.part_o;
    if (valid_done && ehh == 0) {
      const float l2 = m_run + fast_log2(l_tot);
      if (direct_done) pn.lse[dest_done] = l2 * 0.6931471805599453f;
      else pn.part_lse[dest_done] = l2;
    }
    const int c16 = ln & 7;
    int dest[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) dest[i] = __shfl(dest_done, 8 * i + (ln >> 3), 64);
#pragma unroll
    for (int half = 0; half < 2; ++half) {
#pragma unroll
      for (int d2 = 0; d2 < 2; ++d2)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int db = 2 * half + d2;
          u32x2 w;
          w[0] = pack2<E>(oacc[db][4 * g + 0] * inv, oacc[db][4 * g + 1] * inv);
          w[1] = pack2<E>(oacc[db][4 * g + 2] * inv, oacc[db][4 * g + 3] * inv);
          // elements 32*db + 8*g + 4*hh .. +3 of row n: 16-byte column 4*d2 + g of this half
          *reinterpret_cast<u32x2*>(wrow + (((4 * d2 + g) ^ wsw) << 4)) = w;
        }
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int row = 8 * i + (ln >> 3);
        const u32x4 x = *reinterpret_cast<const u32x4*>(stage + row * 128 + ((c16 ^ ((row >> 1) & 7)) << 4));
        if (row < rows_done) *reinterpret_cast<u32x4*>(o_base + (int64_t)dest[i] * kHeadDim + 64 * half + c16 * 8) = x;
      }
    }
  };
  // a tile of the fixed-reference kernel whose rows left the safe range (marked in LDS by the waves that wrote
  // its partial; call behind a barrier that follows those writes) enters the list of tiles to compute again
  auto list_for_redo = [&]() __attribute__((always_inline)) {
    if constexpr (kFixedRef) {
      if (tid == 0 && *reinterpret_cast<volatile int*>(smem + kFwdRedoWord) != 0) {
        const FwdParams<E> pn = kernarg_now<FwdParams<E>>(0);
        *reinterpret_cast<volatile int*>(smem + kFwdRedoWord) = 0;
        const int at = __hip_atomic_fetch_add(pn.redo, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        pn.redo[1 + at] = id_done;
      }
    }
  };
  // Queued tiles: the Q rows of the next tile are requested while the current tile still computes -- between
  // the two steps of its last key tile, the first point at which the registers of the Q^T operand are free
  // (the last step forms no S^T) -- so that they travel under the last matrix instructions and the partial's
  // stores.  The next tile's row entries have been in LDS since this tile's first key tile; its rows are decoded
  // here.  On every pass, from row 0 when no tile follows: the operand carries no value around the loop.
  auto prefetch_q = [&]() __attribute__((always_inline)) {
    if constexpr (kQueued) {
      const FwdParams<E> pn = kernarg_now<FwdParams<E>>(0);
      int tx = threadIdx.x;  // taken afresh
      asm volatile("" : "+v"(tx));
      const int er = (tx >> 6) * 32 + (tx & 31);
      wait_vmem();  // (the entries' copy; nothing else of this wave is in flight here)
      int q_tok = 0, q_head = 0;
      if (t1.row_count > 0) {
        const int entry = *reinterpret_cast<const int*>(smem + kFwdEntries + 4 * tx);
        decode_tile_rows(pn.t, tx >> 6, er, entry, t1);
        q_tok = t1.tok;
        q_head = t1.h;
      }
      const elem* src = reinterpret_cast<const elem*>((const char*)pn.q + q_tok_bytes(pn.t, q_tok) + q_head * pn.t.q_head_b) + 8 * (tx >> 5 & 1);
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) bq[ks] = *reinterpret_cast<const elem8*>(src + 16 * ks);
    }
  };
  while (true) {
  // ================= tile switch =================
  // The next tile's first copies and loads are issued before the finished tile's partial is written: they
  // travel while the partial is normalised and stored.
  if constexpr (kMode == kTilePerGroup) {
    if (have_partial) {
      write_partial();
      return;
    }
  }
  int drawn = 0;  // wave 0, lane 0: the value of the queue's counter
  {
    const FwdParams<E> pn = kernarg_now<FwdParams<E>>(0);
    int tx = threadIdx.x;  // taken afresh, as above
    asm volatile("" : "+v"(tx));
    const int er = (tx >> 6) * 32 + (tx & 31);
    if constexpr (kQueued) {
      t = t1;  // the next tile becomes the current one: its rows' gather-list entries are in LDS by now
    } else if constexpr (kMode == kTilesListed) {
      t.row_count = 0;
      t.nkeys = -1;  // unless there is another tile in the list
      if (list_pos < pn.redo[0]) {  // (uniform; the count is final: the kernel that wrote it has ended)
        const int listed = pn.redo[1 + list_pos];
        list_pos += gridDim.x;
        if (!decode_tile_head(pn.t, listed, t, kFwdTileRows)) t.nkeys = -1;  // (cannot happen: listed ids are tiles)
      }
    } else {
      // the parts of the history tiles (hist_bound << ks ids, the part in the low bits) and the self tiles,
      // whichever kind takes longer first: workgroups start in the order of their ids
      int logical = logical_tile_id(pn.t.xcd_block_log2);
      const int ks = pn.t.key_split_log2;
      const int parts_end = pn.t.hist_bound << ks;
      int hist_part = pn.t.self_first ? logical - pn.t.self_total : (logical < parts_end ? logical : -1);
      if (hist_part >= parts_end) return;
      if (hist_part >= 0) {
        key_part = hist_part & ((1 << ks) - 1);
        logical = hist_part >> ks;
      } else {
        logical = pn.t.hist_bound + (pn.t.self_first ? logical : logical - parts_end);
      }
      if (!decode_tile_head(pn.t, logical, t, kFwdTileRows)) return;
      if (t.base >= 0) {  // this part's share of the chunk's keys
        t.nkeys >>= ks;
        t.kv_tok0 += key_part * t.nkeys;
      }
    }
    int q_tok = 0, q_head = 0;  // token and head of this lane's query row
    if (t.row_count > 0) {
      // the wave-uniform half of the description is enough to start the first copies: the first two K
      // and V tiles (global -> LDS)
      h = t.h; nkeys = t.nkeys; kv_tok0 = t.kv_tok0;
      hkv = h / pn.t.rep;  // key/value head of this query head
      const int64_t kv_off = kv_tok_bytes(pn.t, kv_tok0) + hkv * pn.t.kv_head_b;
      k_head = (const char*)pn.k + kv_off;
      v_head = (const char*)pn.v + kv_off;
      nkt = (nkeys + TN - 1) / TN;
      rot = t.rot % nkt;
      issue_k(key_tile(0), 0);
      issue_v(key_tile(0), 0);
      if (nkt > 1) {
        issue_k(key_tile(1), 1);
        issue_v(key_tile(1), 1);
      }

      // the per-row half (queued: decoded when the Q rows were requested, see prefetch_q), then the Q rows
      if constexpr (!kQueued) {
        decode_tile_rows(pn.t, tx >> 6, er, decode_tile_row_entry(pn.t, er, t), t);
        if constexpr (kMode == kTilePerGroup) t.dest += key_part * pn.t.part_stride;  // (part 0 for a self tile)
      }
      limit = t.limit;
      min_limit = __builtin_amdgcn_readfirstlane(t.wave_min_limit);
      row_valid = er < t.row_count;
      q_tok = t.tok;
      q_head = h;
    }
    if constexpr (!kQueued) {
      // Q^T operand: lane (n, hh) holds q[tok][16*ks + 8*hh .. +7]
      // (loaded on every pass, from row 0 when there is no tile, so that the operand carries no value from one
      // pass of the loop to the next)
      const elem* src = reinterpret_cast<const elem*>((const char*)pn.q + q_tok_bytes(pn.t, q_tok) + q_head * pn.t.q_head_b) + 8 * (tx >> 5 & 1);
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) bq[ks] = *reinterpret_cast<const elem8*>(src + 16 * ks);
    }
    if constexpr (kQueued) {
      // look-ahead: small-table lookups of the tile after (their results are taken up behind the partial's
      // stores), big-table lookup of the one after that, a new id
      id1 = id2;
      code1 = code2;
      head1 = tile_head_entries(pn.t, id1, code1);
      id2 = id3;
      code2 = decode_tile_code(pn.t, id2);
      if (tx == 0) drawn = __hip_atomic_fetch_add(pn.queues + queue, 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
  }
  if (have_partial) write_partial();
  if constexpr (kQueued) {
    const TileTables tt = kernarg_now<TileTables>(offsetof(FwdParams<E>, t));
    if (!decode_tile_head(tt, id1, code1, head1, t1, kFwdTileRows)) t1.nkeys = (code1 == kTilePastEnd) ? -1 : 0;
  }
  // (on every pass, so that the accumulators carry no value from one pass of the loop to the next)
#pragma unroll
  for (int db = 0; db < 4; ++db)
#pragma unroll
    for (int e = 0; e < 16; ++e) oacc[db][e] = 0.f;
  m_run = -INFINITY;
  l_run = 0.f;
  if (t.nkeys < 0) {  // (uniform) no tiles left
    if constexpr (kFixedRef) {
      __syncthreads();
      list_for_redo();
    }
    break;
  }
  // every copy of this wave has landed, and wave 0 has its draw
  wait_vmem();
  if constexpr (kQueued) {
    if (tid == 0) *reinterpret_cast<int*>(smem + kFwdIdSlot + 4 * id_word) = drawn;
  }
  if (t.row_count > 0) {
    scrub_v(key_tile(0), 0);
    if (nkt > 1) scrub_v(key_tile(1), 1);
  }
  __syncthreads();
  list_for_redo();  // (the finished tile's id is still in id_done)
  if constexpr (kQueued) {
    // the id drawn: queue `queue` counts the ids (8i + queue) * kQueueRun + j; past the last tile the
    // workgroup moves to the next queue, and after eight empty queues in a row there is nothing left
    const TileTables tt = kernarg_now<TileTables>(offsetof(FwdParams<E>, t));
    const int j = __builtin_amdgcn_readfirstlane(*reinterpret_cast<const int*>(smem + kFwdIdSlot + 4 * id_word));
    id_word ^= 1;
    const int64_t id = ((int64_t)(j / kQueueRun) * 8 + queue) * kQueueRun + (j % kQueueRun);
    if (id < (int64_t)tt.hist_bound + tt.self_total) {
      id3 = (int)id;
      empty_queues = 0;
    } else {
      queue = (queue + 1) & 7;
      ++empty_queues;
      id3 = empty_queues >= 8 ? 0x7fffffff : -1;   // past the end / no tile this time
    }
    // the entries of the next tile's rows start their way to LDS (its small-table lookups were issued
    // at the switch, a few thousand cycles ago)
    int tx = threadIdx.x;
    asm volatile("" : "+v"(tx));
    if (t1.row_count > 0 && t1.base >= 0) {
      const int er = (tx >> 6) * 32 + (tx & 31);
      async_copy4(tt.seg_dest + t1.base + min(er, t1.row_count - 1), lds_base + kFwdEntries + wave_u * 256);
    }
  }
  have_partial = t.row_count > 0;
  if (!have_partial) {
    prefetch_q();
    continue;
  }
  dest_done = t.dest;
  direct_done = t.direct != 0;
  id_done = t.id;
  valid_done = row_valid;
  rows_done = t.row_count - wave_u * 32;  // rows of this wave that exist

  f32x16 s0, s1;   // S^T, then P^T, of the current and the next key block
  elem8 pb[2];    // P^T operand of the current block: elements 0..7 and 8..15
  constexpr int kPre = 4;
  elem8 kpre[kPre > 0 ? kPre : 1];  // the first K fragments of the next step's S^T, read one step ahead
  {
#pragma unroll
    for (int e = 0; e < 16; ++e) s0[e] = 0.f;
#pragma unroll
    for (int s8 = 0; s8 < 8; ++s8) s0 = mfma32(k_frag(0, 0, s8), bq[s8], s0);
    if (key_tile(0) * TN + 31 > min_limit) mask_block(s0, key_tile(0) * TN);
    float mx = s0[0];
#pragma unroll
    for (int e = 1; e < 16; ++e) mx = fmaxf(mx, s0[e]);
    // the row maximum of the first block: where the running maximum starts, or the tile's fixed reference
    // (every row has a key in this block: key 0 of a causal tile, any key of a history tile)
    if constexpr (kFixedRef) m_run = max_xhalf(mx) * sl2;
    else update_max(max_xhalf(mx) * sl2);  // nothing accumulated yet: the factor is not needed
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const float pe = fast_exp2(s0[e] * sl2 - m_run);
      l_run += pe;
      pb[0][e] = (elem)pe;
    }
#pragma unroll
    for (int i = 0; i < kPre; ++i) kpre[i] = k_frag(0, 1, i);
  }

  // One pipeline step on key block (tile it, block kb).  sc: its S^T with the running max decided
  // and elements 0..7 already exponentiated into pb[0].  sn receives S^T of the next block.
  // kn/vs: LDS byte offsets (compile-time) of the K tile of the next block and the V tile of this block.  Each of the 16 slots is one MFMA
  // plus a share of the vector work; the pins and scheduling barriers keep that order.
  auto step = [&](f32x16& sc, f32x16& sn, int kn, int nkb, int next_key0, auto has_next_c, bool masked, int vs,
                  int kb, bool pre, int pre_kn, int pre_kb) __attribute__((always_inline)) {
    constexpr bool has_next = decltype(has_next_c)::value;
    // ---- phase 1: S^T of the next block under exponentials 8..15 of this block ----
    // (its first K fragments were read during phase 2 of the step before: kpre)
    elem8 ka[8];
    elem8 va[8];
    float pf[8];
    float rs = 0.f;
    if constexpr (has_next) {
#pragma unroll
      for (int i = 0; i < kPre; ++i) ka[i] = kpre[i];
#pragma unroll
      for (int i = kPre; i < 4; ++i) ka[i] = k_frag(kn, nkb, i);
    }
#pragma unroll
    for (int s8 = 0; s8 < 8; ++s8) {
      if constexpr (has_next) {
        if (s8 + 4 < 8) ka[s8 + 4] = k_frag(kn, nkb, s8 + 4);
        if (s8 == 0) {
#pragma unroll
          for (int e = 0; e < 16; ++e) sn[e] = 0.f;
        }
        sn = mfma32(ka[s8], bq[s8], sn);
      }
      pf[s8] = fast_exp2(sc[8 + s8] * sl2 - m_run);
      if (s8 > 0) rs += pf[s8 - 1];  // one slot late: an instruction that uses a fresh exponential waits a cycle
      MOBA_PIN(pf[s8]);
      MOBA_PIN(rs);
      if (s8 >= 4 && s8 < 6) {  // first V^T fragments of phase 2, four slots before their MFMAs
        va[2 * (s8 - 4)] = v_frag(vs, kb, 0, 2 * (s8 - 4));
        va[2 * (s8 - 4) + 1] = v_frag(vs, kb, 0, 2 * (s8 - 4) + 1);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    l_run += rs + pf[7];
#pragma unroll
    for (int e = 0; e < 8; ++e) pb[1][e] = (elem)pf[e];

    // ---- phase 2: O^T += V^T P^T of this block under the row max and exponentials 0..7 of the next ----
    if constexpr (has_next) {
      if (masked) mask_block(sn, next_key0);
    }
    float pg[8];
    if constexpr (kFixedRef) {
      // no row maximum: the eight exponentials spread over slots 1..7 (slot 0 is left to the packing above
      // and to the last S^T MFMA's result), each sum one slot behind its exponential
      float rn = 0.f;
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        const int j2 = k >> 2, db = k & 3;
        if (k + 4 < 8) va[k + 4] = v_frag(vs, kb, 1, db);
        if (k >= 8 - kPre && pre) kpre[k - (8 - kPre)] = k_frag(pre_kn, pre_kb, k - (8 - kPre));  // for the next step
        oacc[db] = mfma32(va[k], pb[j2], oacc[db]);
        if constexpr (has_next) {
          if (k == 1) {
            pg[0] = fast_exp2(sn[0] * sl2 - m_run);
            pg[1] = fast_exp2(sn[1] * sl2 - m_run);
            MOBA_PIN(pg[0]);
            MOBA_PIN(pg[1]);
          } else if (k >= 2) {
            pg[k] = fast_exp2(sn[k] * sl2 - m_run);
            rn = (k == 2) ? pg[0] + pg[1] : rn + pg[k - 1];
            MOBA_PIN(pg[k]);
            MOBA_PIN(rn);
          }
        }
        __builtin_amdgcn_sched_barrier(0);
      }
      if constexpr (has_next) {
        l_run += rn + pg[7];
#pragma unroll
        for (int e = 0; e < 8; ++e) pb[0][e] = (elem)pg[e];
      }
    } else {
    float mx = -INFINITY, alpha = 1.f, rn = 0.f;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
      const int j2 = k >> 2, db = k & 3;
      if (k + 4 < 8) va[k + 4] = v_frag(vs, kb, 1, db);
      if (k >= 8 - kPre && pre) kpre[k - (8 - kPre)] = k_frag(pre_kn, pre_kb, k - (8 - kPre));  // for the next step
      oacc[db] = mfma32(va[k], pb[j2], oacc[db]);
      if constexpr (has_next) {
        if (k == 1) {
          mx = fmaxf(fmaxf(sn[0], sn[1]), fmaxf(sn[2], sn[3]));
          mx = fmaxf(mx, fmaxf(fmaxf(sn[4], sn[5]), fmaxf(sn[6], sn[7])));
          MOBA_PIN(mx);
        } else if (k == 2) {
          mx = fmaxf(mx, fmaxf(fmaxf(sn[8], sn[9]), fmaxf(sn[10], sn[11])));
          mx = fmaxf(mx, fmaxf(fmaxf(sn[12], sn[13]), fmaxf(sn[14], sn[15])));
          MOBA_PIN(mx);
        } else if (k == 3) {
          alpha = update_max(max_xhalf(mx) * sl2);
          MOBA_PIN(alpha);
        } else if (k >= 4) {
#pragma unroll
          for (int e = 2 * (k - 4); e < 2 * (k - 4) + 2; ++e) {
            pg[e] = fast_exp2(sn[e] * sl2 - m_run);
            rn += pg[e];
            MOBA_PIN(pg[e]);
          }
          MOBA_PIN(rn);
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    if constexpr (has_next) {
      if (__any(alpha != 1.f)) {  // rare: the running max moved
#pragma unroll
        for (int db = 0; db < 4; ++db)
#pragma unroll
          for (int e = 0; e < 16; ++e) oacc[db][e] *= alpha;
      }
      l_run = l_run * alpha + rn;
#pragma unroll
      for (int e = 0; e < 8; ++e) pb[0][e] = (elem)pg[e];
    }
    }
  };

  // st: LDS stage of this key tile (it % 3): a constant in the three copies of the hot loop, so that every
  // LDS address is a per-lane register plus an immediate, a number in the copies that finish a query tile.
  auto tile_body = [&](int it, auto st_c, auto more_c) __attribute__((always_inline)) {
    const int st = static_cast<int>(st_c);
    constexpr bool more = decltype(more_c)::value;  // a key tile follows this one
    const int st1 = (st + 1) % kFwdStages, st2 = (st + 2) % kFwdStages;
    const int kcur = st * kTileBytes, knext = st1 * kTileBytes, vcur = st * kTileBytes;
    const int key0 = key_tile(it) * TN;
    const int key0n = more ? key_tile(it + 1) * TN : 0;
    // the mask is needed once a key block reaches past the smallest row limit of the wave
    const bool mask_a = key0 + 63 > min_limit;
    const bool mask_b = more && (key0n + 31 > min_limit);
    if constexpr (more) {
      wait_vmem();
      scrub_v(key_tile(it + 1), st1);
      __syncthreads();
      if (it + 2 < nkt) {
        issue_k(key_tile(it + 2), st2);
        issue_v(key_tile(it + 2), st2);
      }
    }
    step(s0, s1, kcur, 1, key0 + 32, std::true_type{}, mask_a, vcur, 0, more, knext, 0);
    if constexpr (!more) prefetch_q();
    step(s1, s0, knext, 0, key0n, more_c, mask_b, vcur, 1, more, knext, 1);
  };
  using St0 = std::integral_constant<int, 0>;
  using St1 = std::integral_constant<int, 1>;
  using St2 = std::integral_constant<int, 2>;
  // Three copies of the body, one per stage, make the hot loop.  The up to two key tiles left before the
  // last one, and the last one (no tile follows it), run through a fourth and a fifth copy that take the
  // stage as a number: with more copies, or a loop with several exits, the compiler's register allocation
  // degrades for the whole kernel (a thousand bytes of spills).
  int it = 0;
  for (; it + 3 < nkt; it += 3) {
    tile_body(it, St0{}, std::true_type{});
    tile_body(it + 1, St1{}, std::true_type{});
    tile_body(it + 2, St2{}, std::true_type{});
  }
  for (; it + 1 < nkt; ++it) {
    int st = it % kFwdStages;
    asm volatile("" : "+s"(st));  // a number, not one of three constants
    tile_body(it, st, std::true_type{});
  }
  {
    int st = it % kFwdStages;
    asm volatile("" : "+s"(st));
    tile_body(it, st, std::false_type{});
  }
  __syncthreads();  // every wave has read its last fragments: the stages may take the partial's rows
  }  // tiles
#undef MOBA_PIN
}

// The merge of a row with at most NV slots (parts included), by the row's 16 lanes: the slots' partials are
// requested at once, before the statistics that say which are present have arrived -- one round trip instead of
// two.  (An absent slot's bytes are whatever the buffer holds; they are dropped by selection, not multiplied by
// a zero weight.)  Slots are accumulated in ascending order, as in the general form below.  For up to 8 slots:
// with 16 in registers too few waves fit a compute unit, and the kernel takes three times as long.
template <class E, int NV>
__device__ __forceinline__ void merge_few_slots(const typename E::elem* __restrict__ po, const float* __restrict__ pl,
                                                const int* __restrict__ ps, typename E::elem* __restrict__ out,
                                                float* __restrict__ lse, int64_t row, bool row_ok, int c8, int K1,
                                                int parts, int nvirt, int part_rows) {
  MOBA_ELEM_TYPES(E)
  elem8 x[NV];
#pragma unroll
  for (int u = 0; u < NV; ++u) {
    const int part = parts == 1 ? 0 : u / K1, j = u - part * K1;
    if (u < nvirt)
      x[u] = __builtin_nontemporal_load(reinterpret_cast<const elem8*>(po + (int64_t)(part * part_rows + j) * kHeadDim));
  }
  const int part = parts == 1 ? 0 : c8 / K1, j = c8 - part * K1;
  const bool ok = c8 < nvirt && (j == 0 ? part == 0 : ps[j - 1] >= 0);
  const float l = ok ? pl[(int64_t)part * part_rows + j] : -INFINITY;
  float mx = l;
#pragma unroll
  for (int o = 8; o >= 1; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 16));
  const float wl = ok ? fast_exp2(l - mx) : 0.f;
  float acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = 0.f;
  float wsum = 0.f;
#pragma unroll
  for (int u = 0; u < NV; ++u) {
    if (u >= nvirt) break;
    const float w = __shfl(wl, u, 16);
    wsum += w;
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] += w > 0.f ? w * (float)x[u][e] : 0.f;
  }
  if (!row_ok) return;
  const float inv = 1.f / wsum;
  elem8 o;
#pragma unroll
  for (int e = 0; e < 8; ++e) o[e] = (elem)(acc[e] * inv);
  __builtin_nontemporal_store(o, reinterpret_cast<elem8*>(out + row * kHeadDim + c8 * 8));
  if (c8 == 0) lse[row] = (mx + fast_log2(wsum)) * 0.6931471805599453f;
}

// Combine the K1 slots of each (token, head): slot 0 is the self part, slot 1+j the
// j-th selected history chunk (present iff sel[row, j] >= 0).  16 lanes per row.
// With token ranges (mrg_start / mrg_prefix [nranges(+1)]: range b holds the tokens mrg_start[b] + i for
// i < mrg_prefix[b+1] - mrg_prefix[b]) only the rows of those tokens are merged, `rows` counting them: the others
// were written by the attention kernel itself.  Null: every row of [0, rows).
template <class E>
__global__ __launch_bounds__(256) void moba_merge_kernel(const typename E::elem* __restrict__ part_o,
                                                         const float* __restrict__ part_lse,
                                                         const int* __restrict__ sel, typename E::elem* __restrict__ out,
                                                         float* __restrict__ lse, int64_t rows, int K1, int parts,
                                                         int64_t all_rows, const int* __restrict__ mrg_start,
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
  const float* pl = part_lse + row * K1;
  const int* ps = sel + row * K;
  const elem* po = part_o + row * K1 * kHeadDim + c8 * 8;  // the self slot: always written
  // Lane c8 of the row's group fetches the LSE and the presence of slot j0 + c8, so the slot
  // statistics cost one round trip per 16 slots; weights travel by lane shuffles.  Absent slots
  // are redirected to the self slot with weight 0, so the partial-output loads are unconditional and
  // eight of them are in flight together.  Slots are accumulated in ascending order.
  // With `parts` > 1 the history slots hold `parts` partials each (the forward cut the chunks' keys): those of
  // part g lie rows * K1 slot rows behind those of part g - 1; the self slot has part 0 only.
  // The parts are slots like any other: slot v of the parts * K1 is slot v % K1 of part v / K1, at slot row
  // (v / K1) * rows * K1 + v % K1 of the row's first (an int: the buffers hold fewer than 2^31 slot rows).
  const int nvirt = parts * K1;
  const int part_rows = (int)(all_rows * K1);
  if (nvirt <= 8) {  // (uniform)
    merge_few_slots<E, 8>(po, pl, ps, out, lse, row, row_ok, c8, K1, parts, nvirt, part_rows);
    return;
  }
  float mx = -INFINITY;
  for (int v0 = 0; v0 < nvirt; v0 += 16) {
    const int v = v0 + c8;
    const int part = parts == 1 ? 0 : v / K1, j = v - part * K1;
    const bool ok = v < nvirt && (j == 0 ? part == 0 : ps[j - 1] >= 0);
    const float l = ok ? pl[(int64_t)part * part_rows + j] : -INFINITY;
    mx = fmaxf(mx, l);
  }
#pragma unroll
  for (int o = 8; o >= 1; o >>= 1) mx = fmaxf(mx, __shfl_xor(mx, o, 16));
  float acc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = 0.f;
  float wsum = 0.f;
  for (int v0 = 0; v0 < nvirt; v0 += 16) {
    const int v = v0 + c8;
    const int part = parts == 1 ? 0 : v / K1, j = v - part * K1;
    const bool ok = v < nvirt && (j == 0 ? part == 0 : ps[j - 1] >= 0);
    const int at = part * part_rows + j;  // (0, the self slot, for a slot that is absent)
    const float wl = ok ? fast_exp2(pl[(int64_t)part * part_rows + j] - mx) : 0.f;
    const int at_ok = ok ? at : 0;
    const int nslot = min(16, nvirt - v0);
    for (int u0 = 0; u0 < nslot; u0 += 8) {
      elem8 x[8];
      float w[8];
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        w[u] = __shfl(wl, u0 + u, 16);           // 0 for slots past the last too (their lanes computed ok = false)
        const int where = parts == 1 ? (w[u] > 0.f ? v0 + u0 + u : 0) : __shfl(at_ok, u0 + u, 16);
        if (u0 + u < nslot)                      // uniform: no loads for slots that do not exist
          x[u] = __builtin_nontemporal_load(reinterpret_cast<const elem8*>(po + (int64_t)where * kHeadDim));
      }
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        if (u0 + u >= nslot) break;
        wsum += w[u];
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] += w[u] * (float)x[u][e];
      }
    }
  }
  if (!row_ok) return;
  const float inv = 1.f / wsum;
  elem8 o;
#pragma unroll
  for (int e = 0; e < 8; ++e) o[e] = (elem)(acc[e] * inv);
  __builtin_nontemporal_store(o, reinterpret_cast<elem8*>(out + row * kHeadDim + c8 * 8));
  if (c8 == 0) lse[row] = (mx + fast_log2(wsum)) * 0.6931471805599453f;
}

}  // namespace moba

using namespace moba;

extern "C" int moba_fwd_tile_rows(void) { return kFwdTileRows; }

constexpr int kMaxKeySplit = 8;
// workgroups of the forward kernel: resident ones drawing from the queues (> 0), or one per tile id (< 0, see
// moba_fwd_partials)
static int fwd_xcd_block_log2(int64_t total) {  // runs of at most an eighth of an XCD's share of the ids
  int b = 0;
  while (b < 6 && (128LL << b) <= total) ++b;
  return b;
}
static int64_t fwd_grid(int64_t total, int cus) {
  int64_t grid = ((int64_t)cus + 7) / 8 * 8;
  if (total < 8 * grid) {
    const int64_t run = 8LL << fwd_xcd_block_log2(total);
    grid = -((total + run - 1) / run * run);
  }
  return grid;
}
// Whether moba_fwd_partials would run a problem of this many tiles with resident workgroups that draw their tiles
// from the queues (1) or with one workgroup per tile (0).  A caller that may plan a batch with or without dense
// prefixes asks this for the plan with them: their long causal tiles pay only in the first form.
extern "C" int moba_fwd_is_queued(int64_t hist_bound, int64_t self_tiles, int H) {
  const int cus = resident_compute_units();
  if (cus <= 0 || hist_bound < 0 || self_tiles < 0 || H <= 0) return 0;
  return fwd_grid(hist_bound + self_tiles * H, cus) > 0 ? 1 : 0;
}

// Into how many parts moba_fwd_partials should cut the keys of every history tile: 1 unless the problem is so
// small that whole tiles leave compute units idle at the end (a tile of 256 rows x 2048 keys takes 65 us, and
// workgroups start in the order of their ids, not where the work is); then the largest power of two that
// keeps 512 keys per part (a part costs 4 us of its own) and the number of tiles within three per unit.
extern "C" int moba_fwd_key_split(int64_t S, int H, int K, int B, int64_t hist_bound, int64_t self_tiles) {
  if (S <= 0 || H <= 0 || K <= 0 || B <= 0 || hist_bound <= 0 || self_tiles <= 0) return 1;
  const int cus = resident_compute_units();
  if (cus <= 0) return 1;
  const int64_t own = self_tiles * H;
  int split = 1;
  while (split < kMaxKeySplit && B % (TN * 2 * split) == 0 && B / (2 * split) >= 512 &&
         hist_bound * 2 * split + own <= 3 * (int64_t)cus && S * H * (K + 1) * 2 * split < 0x7fffffffLL)
    split *= 2;
  return split;
}

template <class E>
static int launch_partials(const void* q, const void* k, const void* v, void* part_o, float* part_lse, void* out,
                           float* lse, const TileTables& t, int D, float softmax_scale, int64_t grid, int* queues,
                           int* redo, hipStream_t st) {
  LaunchCheck launch_check;
  FwdParams<E> p;
  p.q = (const typename E::elem*)q; p.k = (const typename E::elem*)k; p.v = (const typename E::elem*)v;
  p.part_o = (typename E::elem*)part_o; p.part_lse = part_lse;
  p.out = (typename E::elem*)out; p.lse = lse;
  p.t = t;
  p.scale_log2 = softmax_scale > 0.f ? (float)(1.4426950408889634 * (double)softmax_scale)
                                     : (float)(1.4426950408889634 / sqrt((double)D));
  p.queues = queues;
  p.redo = redo;
  static bool allowed[4][kMaxDevices];  // one set of arrays per element type
  if (grid > 0) {  // resident workgroups drawing from the queues
    hipLaunchKernelGGL(zero_queues_kernel, dim3(1), dim3(8), 0, st, queues, redo);  // a kernel, not a memset: graph safe
    {
      if (redo) {
        // fixed-reference softmax, then the tiles it could not serve (normally none) with the tracked maximum
        if (!allow_dynamic_lds((const void*)moba_fwd_kernel<E, kTilesQueued, true>, kFwdLds, allowed[2]) ||
            !allow_dynamic_lds((const void*)moba_fwd_kernel<E, kTilesListed, false>, kFwdLds, allowed[3]))
          return MOBA_ERR_LAUNCH;
        hipLaunchKernelGGL((moba_fwd_kernel<E, kTilesQueued, true>), dim3((unsigned)grid), dim3(512), kFwdLds, st, p);
        hipLaunchKernelGGL((moba_fwd_kernel<E, kTilesListed, false>), dim3((unsigned)grid), dim3(512), kFwdLds, st, p);
        return launch_check.result();
      }
    }
    if (!allow_dynamic_lds((const void*)moba_fwd_kernel<E, kTilesQueued, false>, kFwdLds, allowed[1])) return MOBA_ERR_LAUNCH;
    hipLaunchKernelGGL((moba_fwd_kernel<E, kTilesQueued, false>), dim3((unsigned)grid), dim3(512), kFwdLds, st, p);
  } else {         // one workgroup per tile id
    if (!allow_dynamic_lds((const void*)moba_fwd_kernel<E, kTilePerGroup, false>, kFwdLds, allowed[0])) return MOBA_ERR_LAUNCH;
    hipLaunchKernelGGL((moba_fwd_kernel<E, kTilePerGroup, false>), dim3((unsigned)-grid), dim3(512), kFwdLds, st, p);
  }
  return launch_check.result();
}

// hist_bound: any upper bound on the number of history tiles (floor(M/128) + F*H is one).
extern "C" int moba_fwd_partials(const void* q, const void* k, const void* v, void* part_o, float* part_lse,
                                 const int32_t* seg_off, const int32_t* tile_off, const int32_t* seg_dest,
                                 const int32_t* fchunk_tok, const int32_t* chunk_tok,
                                 const int32_t* self_tile_prefix, const int32_t* tile_seg,
                                 const int32_t* self_tile_chunk, const int32_t* chunk_direct, void* out, float* lse,
                                 int64_t S, int H, int Hkv, int D, int K, int F,
                                 int N, int B, int64_t hist_bound, int64_t self_tiles, int key_split,
                                 const int64_t* strides, int32_t* queues, int32_t* redo, float softmax_scale,
                                 int dtype, int self_tile_skip, int64_t q_tok_shift, void* stream) {
  if (!q || !k || !v || !part_o || !part_lse || !chunk_tok || !self_tile_prefix || !self_tile_chunk || !queues)
    return MOBA_ERR_ARG;
  if (chunk_direct && (!out || !lse || ((uintptr_t)out & 15))) return MOBA_ERR_ARG;
  // queries that are the tail of their sequence: plain causal attention whose rows all go straight to the outputs
  if (self_tile_skip < 0 || q_tok_shift < 0 || q_tok_shift > (int64_t)self_tile_skip * kFwdTileRows) return MOBA_ERR_ARG;
  if (self_tile_skip > 0 && (K != 0 || !chunk_direct || (strides && strides[4] != 0))) return MOBA_ERR_ARG;
  if (Hkv <= 0 || H % Hkv != 0) return MOBA_ERR_ARG;
  if (K > 0 && (!seg_off || !tile_off || !seg_dest || !fchunk_tok || !tile_seg)) return MOBA_ERR_ARG;
  if (D != kHeadDim || (dtype != MOBA_DTYPE_BF16 && dtype != MOBA_DTYPE_F16)) return MOBA_ERR_UNSUPPORTED;
  if (S <= 0 || H <= 0 || K < 0 || F < 0 || N <= 0 || B <= 0 || hist_bound < 0 || self_tiles <= 0) return MOBA_ERR_ARG;
  if (((uintptr_t)q & 15) || ((uintptr_t)k & 15) || ((uintptr_t)v & 15) || ((uintptr_t)part_o & 15)) return MOBA_ERR_ARG;
  int key_split_log2 = 0;
  while ((1 << key_split_log2) < key_split) ++key_split_log2;
  if (key_split < 1 || key_split > kMaxKeySplit || (1 << key_split_log2) != key_split) return MOBA_ERR_ARG;
  if (K == 0) key_split = 1, key_split_log2 = 0;  // (no history tiles: nothing to cut)
  if ((int64_t)S * H * (K + 1) * key_split >= 0x7fffffffLL) return MOBA_ERR_LIMIT;
  const int64_t total = (K > 0 ? hist_bound * key_split : 0) + self_tiles * H;
  if (total >= 0x7fffffffLL) return MOBA_ERR_LIMIT;
  // one workgroup of eight waves per CU (what the kernel's registers allow), all resident at once and drawing
  // tiles from the queues; a multiple of 8 so that every XCD starts on its own queue with as many
  const int cus = resident_compute_units();
  if (cus <= 0) return MOBA_ERR_LAUNCH;
  // with fewer than a few tiles per resident workgroup the queues do not pay: one workgroup per id then
  // (a negative grid tells the launcher)
  const int64_t grid = fwd_grid(total, cus);
  // the parts are tiles of the one-workgroup-per-id form only, whole key tiles each
  if (key_split > 1 && (grid > 0 || B % (TN * key_split) != 0)) return MOBA_ERR_ARG;
  TileTables t;
  t.seg_off = seg_off; t.tile_off = tile_off; t.seg_dest = seg_dest; t.fchunk_tok = fchunk_tok;
  t.chunk_tok = chunk_tok; t.self_tile_prefix = self_tile_prefix;
  t.tile_seg = tile_seg; t.self_tile_chunk = self_tile_chunk;
  t.S = (int)S; t.H = H; t.K1 = K + 1; t.F = (K > 0) ? F : 0; t.N = N; t.B = B;
  t.Hkv = Hkv; t.rep = H / Hkv;
  t.hist_bound = (K > 0) ? (int)hist_bound : 0;
  t.self_total = (int)(self_tiles * H);
  if (!set_layout(t, strides)) return MOBA_ERR_ARG;
  t.key_split_log2 = key_split_log2;
  t.part_stride = (int)(S * H * (K + 1));
  t.xcd_block_log2 = fwd_xcd_block_log2(total);
  t.self_first = key_split > 1;
  t.chunk_direct = chunk_direct;
  t.self_skip = self_tile_skip; t.q_shift = (int)q_tok_shift;
  hipStream_t st = (hipStream_t)stream;
  return dtype == MOBA_DTYPE_F16
             ? launch_partials<F16>(q, k, v, part_o, part_lse, out, lse, t, D, softmax_scale, grid, queues, redo, st)
             : launch_partials<Bf16>(q, k, v, part_o, part_lse, out, lse, t, D, softmax_scale, grid, queues, redo, st);
}

// mrg_start [nranges], mrg_prefix [nranges + 1], merge_tokens = mrg_prefix[nranges]: the tokens to merge, for a
// caller whose attention call wrote the other tokens' rows itself (chunk_direct); null, null, 0, S: every token.
extern "C" int moba_fwd_merge(const void* part_o, const float* part_lse, const int32_t* sel, void* out, float* lse,
                              int64_t S, int H, int D, int K, int key_split, const int32_t* mrg_start,
                              const int32_t* mrg_prefix, int nranges, int64_t merge_tokens, int dtype, void* stream) {
  LaunchCheck launch_check;
  if (!part_o || !part_lse || !out || !lse || (K > 0 && !sel)) return MOBA_ERR_ARG;
  if (key_split < 1 || key_split > kMaxKeySplit) return MOBA_ERR_ARG;
  if (K == 0) key_split = 1;
  if (D != kHeadDim || (dtype != MOBA_DTYPE_BF16 && dtype != MOBA_DTYPE_F16)) return MOBA_ERR_UNSUPPORTED;
  if (S <= 0 || H <= 0 || K < 0 || ((uintptr_t)part_o & 15) || ((uintptr_t)out & 15)) return MOBA_ERR_ARG;
  if (mrg_start ? (!mrg_prefix || nranges <= 0 || merge_tokens < 0 || merge_tokens > S)
                : (mrg_prefix || merge_tokens != S))
    return MOBA_ERR_ARG;
  if (merge_tokens == 0) return MOBA_OK;  // every row was written by the attention kernel
  const int64_t rows = merge_tokens * H;
  const dim3 grid((unsigned)((rows + 15) / 16));
  if (dtype == MOBA_DTYPE_F16)
    hipLaunchKernelGGL(moba_merge_kernel<F16>, grid, dim3(256), 0, (hipStream_t)stream, (const f16*)part_o, part_lse,
                       sel, (f16*)out, lse, rows, K + 1, key_split, S * H, mrg_start, mrg_prefix, nranges, H);
  else
    hipLaunchKernelGGL(moba_merge_kernel<Bf16>, grid, dim3(256), 0, (hipStream_t)stream, (const bf16*)part_o,
                       part_lse, sel, (bf16*)out, lse, rows, K + 1, key_split, S * H, mrg_start, mrg_prefix, nranges, H);
  return launch_check.result();
}

// Whole attention stage: partial attentions of every tile, then the merge.
extern "C" int moba_fwd(const void* q, const void* k, const void* v, void* part_o, float* part_lse,
                        const int32_t* sel, const int32_t* seg_off, const int32_t* tile_off,
                        const int32_t* seg_dest, const int32_t* fchunk_tok, const int32_t* chunk_tok,
                        const int32_t* self_tile_prefix, const int32_t* tile_seg, const int32_t* self_tile_chunk,
                        const int32_t* chunk_direct, const int32_t* mrg_start, const int32_t* mrg_prefix, int nranges,
                        int64_t merge_tokens, void* out, float* lse, int64_t S, int H, int Hkv, int D, int K, int F,
                        int N, int B, int64_t hist_bound, int64_t self_tiles, int key_split, const int64_t* strides,
                        int32_t* queues, int32_t* redo, float softmax_scale, int dtype, void* stream) {
  if (!out || !lse) return MOBA_ERR_ARG;
  // (direct rows and the merge's token ranges come together: either both or neither)
  if ((chunk_direct != nullptr) != (mrg_start != nullptr)) return MOBA_ERR_ARG;
  int rc = moba_fwd_partials(q, k, v, part_o, part_lse, seg_off, tile_off, seg_dest, fchunk_tok, chunk_tok,
                             self_tile_prefix, tile_seg, self_tile_chunk, chunk_direct, out, lse, S, H, Hkv, D, K, F, N,
                             B, hist_bound, self_tiles, key_split, strides, queues, redo, softmax_scale, dtype, 0, 0,
                             stream);
  if (rc != MOBA_OK) return rc;
  return moba_fwd_merge(part_o, part_lse, sel, out, lse, S, H, D, K, key_split, mrg_start, mrg_prefix, nranges,
                        merge_tokens, dtype, stream);
}
