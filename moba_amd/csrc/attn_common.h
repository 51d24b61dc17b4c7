// Pieces shared by the forward and backward attention kernels: the tile tables, the
// decoding of a workgroup id into a tile of query rows, LDS swizzles and the
// asynchronous global -> LDS copy.
#pragma once
#include "common.h"

namespace moba {

constexpr int TM = 128;  // query rows per workgroup of the backward kernels (32 per wave)
constexpr int kFwdTileRows = 256;  // ... and of the forward kernel (8 waves)
constexpr int TN = 64;   // keys per inner iteration
constexpr int kTileBytes = TN * kHeadDim * 2;
constexpr int kXcdBlock = 64;  // consecutive logical tiles that share an XCD (one workgroup per tile id)
// The same for kernels whose resident workgroups draw ids from per-XCD queues.  Longer runs there: an id is
// computed a few tiles after it was drawn, by workgroups whose speeds differ, so the ids in flight on an XCD
// span about two of its 64 slots' worth; with runs of 256 they still mostly belong to one K/V chunk.
constexpr int kQueueRun = 256;

// Index tables that define the tiles of one call.
struct TileTables {
  const int* seg_off;           // [F*H+1] list start of segment (f, h)
  const int* tile_off;          // [F*H+1] prefix sum of row tiles per segment
  const int* seg_dest;          // [M] (token*H + h)*K1 + 1 + slot
  const int* fchunk_tok;        // [F] first token of filtered chunk f
  const int* chunk_tok;         // [N+1] first token of every chunk
  const int* self_tile_prefix;  // [N+1] prefix sum of row tiles per chunk
  const int* tile_seg;          // [hist_bound] segment (f*H + h) of every history tile, -1 past the last one
  const int* self_tile_chunk;   // [self_tile_prefix[N]] chunk of every per-head self tile
  // [N] or null: 1 for a chunk whose rows have no history slots at all (the first attention chunk of a sequence).
  // The forward kernel writes the result of such a chunk's self tiles straight into the operator's outputs: there
  // is nothing to merge it with.  Null (the backward): every tile writes its slot row.
  const int* chunk_direct;
  int S, H, K1, F, N, B;
  int Hkv, rep;                 // key/value heads and query heads per key/value head (H = Hkv * rep)
  int hist_bound;               // logical tile ids below it are history tiles
  int self_total;               // self_tile_prefix[N] * H
  // byte strides of q[token][head][:] and of k, v[token][kv head][:] (k and v share theirs); the
  // 128 elements of a (token, head) are contiguous
  int64_t q_tok_b, q_head_b, kv_tok_b, kv_head_b;
  // batched layouts ([batch, heads, tokens, dim] tensors seen as packed tokens): token t lies in batch entry
  // t / batch_rows at position t % batch_rows; batch_rows = 0 for one affine range of tokens
  int batch_rows;
  int64_t q_batch_b, kv_batch_b;
  // forward, one workgroup per tile id only: every history tile is cut into 1 << key_split_log2 parts along its
  // keys, each a tile of its own whose partial goes to slot row `dest + part * part_stride` (0, 0 elsewhere)
  int key_split_log2, part_stride;
  int xcd_block_log2;  // ... ids reach the XCDs in runs of 1 << xcd_block_log2
  int self_first;      // ... the self tiles take the first ids (they are the longer ones once the history tiles are cut)
  // Queries that are the tail of their sequence (new tokens against a key/value cache): the first self_skip row
  // tiles of every chunk do not exist -- self_tile_prefix counts the others -- and q and the directly written
  // outputs hold the rows from token q_shift on (q_shift <= self_skip * rows per tile).  0, 0: every row exists.
  int self_skip, q_shift;
};

// byte offset of the row of token `tok` (without the head term) in q and in k, v
__device__ __forceinline__ int64_t q_tok_bytes(const TileTables& t, int tok) {
  tok = max(tok - t.q_shift, 0);  // (q holds the rows from q_shift on; row 0 stands in where there is no tile)
  if (t.batch_rows == 0) return (int64_t)tok * t.q_tok_b;
  const int b = tok / t.batch_rows;
  return (int64_t)b * t.q_batch_b + (int64_t)(tok - b * t.batch_rows) * t.q_tok_b;
}
__device__ __forceinline__ int64_t kv_tok_bytes(const TileTables& t, int tok) {
  if (t.batch_rows == 0) return (int64_t)tok * t.kv_tok_b;
  const int b = tok / t.batch_rows;
  return (int64_t)b * t.kv_batch_b + (int64_t)(tok - b * t.batch_rows) * t.kv_tok_b;
}

// strides: {q token, q head, k/v token, k/v head, rows per batch entry, q batch, k/v batch} in elements
// (seven entries; the last three are 0 for one affine range of tokens), or null for packed [S, H, 128] /
// [S, Hkv, 128] tensors.  Returns false for strides the kernels cannot address: not multiples of
// 8 elements (16-byte accesses), not positive, or a key/value token stride whose 64-row tile
// offsets leave 31 bits.
constexpr int kStrideEntries = 7;
inline bool set_layout(TileTables& t, const int64_t* strides) {
  t.batch_rows = 0; t.q_batch_b = 0; t.kv_batch_b = 0;
  t.chunk_direct = nullptr;
  t.key_split_log2 = 0; t.part_stride = 0; t.xcd_block_log2 = 6; t.self_first = 0;
  t.self_skip = 0; t.q_shift = 0;
  if (!strides) {
    t.q_tok_b = (int64_t)t.H * kHeadDim * 2; t.q_head_b = kHeadDim * 2;
    t.kv_tok_b = (int64_t)t.Hkv * kHeadDim * 2; t.kv_head_b = kHeadDim * 2;
    return true;
  }
  for (int i = 0; i < 4; ++i)
    if (strides[i] <= 0 || (strides[i] & 7)) return false;
  if (strides[2] > (1 << 23) || strides[0] >= (1LL << 30)) return false;  // (byte strides of a token fit 32 bits)
  t.q_tok_b = strides[0] * 2; t.q_head_b = strides[1] * 2;
  t.kv_tok_b = strides[2] * 2; t.kv_head_b = strides[3] * 2;
  if (strides[4] != 0) {
    if (strides[4] < 0 || strides[4] > 0x7fffffffLL || strides[5] <= 0 || strides[6] <= 0 || (strides[5] & 7) || (strides[6] & 7))
      return false;
    t.batch_rows = (int)strides[4]; t.q_batch_b = strides[5] * 2; t.kv_batch_b = strides[6] * 2;
  }
  return true;
}

// One tile of up to TM query rows of one head, as seen by a lane.
struct Tile {
  int id;         // logical tile id
  int h;          // head
  int kv_tok0;    // token of key 0
  int nkeys;      // keys the tile attends (before masking)
  int row_count;  // valid rows
  int dest;       // this lane's row: destination slot row (token*H + h)*K1 + slot
  int tok;        // this lane's row: token
  int limit;      // this lane's row attends keys <= limit
  int wave_min_limit, wave_max_limit;  // over the wave's 32 rows
  int rot;        // history tiles may visit their key tiles in any order: start offset
  int base;       // history tile: index of row 0 in seg_dest; self tile: -(row 0 inside the chunk) - 1
  int direct;     // self tile of a chunk without history slots: dest is the output row token*H + h
};

// the tile counters of a kernel whose resident workgroups draw their tiles from per-XCD queues start at zero
// (a kernel, not a memset: safe to record into a graph)
// (`also`, if not null, is one more counter to clear)
static __global__ void zero_queues_kernel(int* queues, int* also) {
  queues[threadIdx.x] = 0;
  if (also && threadIdx.x == 0) *also = 0;
}

// Workgroup ids are dealt round-robin to the 8 XCDs; give each XCD runs of 1 << block_log2 (at most kXcdBlock)
// consecutive logical tiles so that tiles sharing a K/V chunk share an L2.  (A grid of few tiles takes shorter
// runs: whole runs of 64 would leave some XCDs with twice the tiles of others, or with none.)
__device__ __forceinline__ int logical_tile_id(int block_log2) {
  const int x = blockIdx.x & 7, y = blockIdx.x >> 3;
  return ((((y >> block_log2) << 3) + x) << block_log2) + (y & ((1 << block_log2) - 1));
}

// Tile decoding in steps, so that a kernel can start the key/value copies (which need only the
// wave-uniform part) before the per-row lookup has returned, and so that a kernel that walks many
// tiles can keep the lookups of later tiles in flight behind the work on the current one.
// Step 0, wave-uniform: the one entry of the big tables.  History tile: its segment (-1 for an unused
// id below hist_bound); self tile: its chunk; -2 past the last tile.
constexpr int kTileUnused = -1, kTilePastEnd = -2;
__device__ __forceinline__ int decode_tile_code(const TileTables& p, int logical) {
  if (logical < 0) return kTileUnused;
  if (logical < p.hist_bound) return table_load(p.tile_seg + logical);
  const int st = logical - p.hist_bound;
  if (st >= p.self_total) return kTilePastEnd;
  return table_load(p.self_tile_chunk + st / p.H);  // self_tile_prefix[c]*H <= st < self_tile_prefix[c+1]*H
}
// Step 1, wave-uniform: head, key range, number of rows, from the small per-segment / per-chunk tables.
// In two halves, so that a kernel can have the table entries on their way while it does something else:
// tile_head_entries starts the four lookups, decode_tile_head turns their results into the description.
// Returns false (and row_count = 0) for a code that is not a tile.
// (tm: rows per tile of the tables in p)
struct TileHeadEntries {
  int a, b, c, d;  // history tile: tile_off[seg], seg_off[seg], seg_off[seg+1], fchunk_tok[f];
                   // self tile: self_tile_prefix[c], self_tile_prefix[c+1], chunk_tok[c], chunk_tok[c+1]
  int e;           // self tile: chunk_direct[c] (0 without that table)
};
__device__ __forceinline__ TileHeadEntries tile_head_entries(const TileTables& p, int logical, int code) {
  TileHeadEntries e = {0, 0, 0, 0, 0};
  if (code < 0) return e;
  if (logical < p.hist_bound) {
    e.a = table_load(p.tile_off + code);
    e.b = table_load(p.seg_off + code);
    e.c = table_load(p.seg_off + code + 1);
    e.d = table_load(p.fchunk_tok + code / p.H);
  } else {
    e.a = table_load(p.self_tile_prefix + code);
    e.b = table_load(p.self_tile_prefix + code + 1);
    e.c = table_load(p.chunk_tok + code);
    e.d = table_load(p.chunk_tok + code + 1);
    if (p.chunk_direct) e.e = table_load(p.chunk_direct + code);
  }
  return e;
}
__device__ __forceinline__ bool decode_tile_head(const TileTables& p, int logical, int code, const TileHeadEntries& e,
                                                 Tile& t, int tm = TM) {
  const int H = p.H;
  t.id = logical;
  t.row_count = 0;
  t.base = -1;
  t.direct = 0;
  if (code < 0) return false;
  if (logical < p.hist_bound) {
    const int seg = code;
    const int tile = logical - e.a;
    const int f = seg / H;
    t.h = seg - f * H;
    t.base = e.b + tile * tm;
    t.row_count = min(tm, e.c - t.base);
    t.kv_tok0 = e.d;
    t.nkeys = p.B;
    t.rot = tile;
    return true;
  }
  const int st = logical - p.hist_bound;
  const int rem = st - e.a * H;
  const int nt = e.b - e.a;
  t.h = rem / nt;
  const int tin = nt - 1 - (rem - t.h * nt) + p.self_skip;  // longest tiles first
  const int c0 = e.c;
  const int len = e.d - c0;
  t.base = -1 - tin * tm;                   // self tile: -(first row of the tile inside its chunk) - 1
  t.row_count = min(tm, len - tin * tm);
  t.kv_tok0 = c0;
  t.nkeys = min(len, tin * tm + tm);
  t.rot = 0;
  t.direct = e.e;
  return true;
}
__device__ __forceinline__ bool decode_tile_head(const TileTables& p, int logical, int code, Tile& t, int tm = TM) {
  return decode_tile_head(p, logical, code, tile_head_entries(p, logical, code), t, tm);
}
__device__ __forceinline__ bool decode_tile_head(const TileTables& p, int logical, Tile& t, int tm = TM) {
  return decode_tile_head(p, logical, decode_tile_code(p, logical), t, tm);
}
// Step 2a, per row: the gather-list entry of row r (history tiles; self tiles need no lookup).
__device__ __forceinline__ int decode_tile_row_entry(const TileTables& p, int r, const Tile& t) {
  return (t.row_count > 0 && t.base >= 0) ? p.seg_dest[t.base + min(r, t.row_count - 1)] : 0;
}
// Step 2b, per row: everything else from that entry.  r = row of this lane inside the tile (wave*32 + lane%32).
__device__ __forceinline__ void decode_tile_rows(const TileTables& p, int wave, int r, int entry, Tile& t) {
  const int H = p.H;
  if (t.base >= 0) {
    t.dest = entry;
    t.tok = t.dest / (H * p.K1);
    t.limit = t.nkeys - 1;
    t.wave_min_limit = t.limit;
    t.wave_max_limit = t.limit;
  } else {
    const int r0 = -1 - t.base;
    t.tok = t.kv_tok0 + r0 + min(r, t.row_count - 1);
    t.dest = t.direct ? (t.tok - p.q_shift) * H + t.h : (t.tok * H + t.h) * p.K1;
    t.limit = r0 + min(r, t.row_count - 1);
    t.wave_min_limit = r0 + min(wave * 32, t.row_count - 1);
    t.wave_max_limit = r0 + min(wave * 32 + 31, t.row_count - 1);
  }
}
__device__ __forceinline__ void decode_tile_rows(const TileTables& p, int wave, int r, Tile& t) {
  decode_tile_rows(p, wave, r, decode_tile_row_entry(p, r, t), t);
}
__device__ __forceinline__ bool decode_tile(const TileTables& p, int logical, int wave, int r, Tile& t) {
  if (!decode_tile_head(p, logical, t)) return false;
  decode_tile_rows(p, wave, r, t);
  return true;
}

// max over the two halves of the wave (lane l and lane l^32), without LDS traffic
__device__ __forceinline__ float max_xhalf(float x) {
  const uint32_t u = __builtin_bit_cast(uint32_t, x);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return fmaxf(__builtin_bit_cast(float, (uint32_t)r[0]), __builtin_bit_cast(float, (uint32_t)r[1]));
}
__device__ __forceinline__ float sum_xhalf(float x) {
  const uint32_t u = __builtin_bit_cast(uint32_t, x);
  const auto r = __builtin_amdgcn_permlane32_swap(u, u, false, false);
  return __builtin_bit_cast(float, (uint32_t)r[0]) + __builtin_bit_cast(float, (uint32_t)r[1]);
}

// LDS layout of a [rows x 128] bf16 tile: row-major, 256 bytes per row, with the
// 16-byte column index XORed by a function of the row so that both access patterns
// are bank-conflict free: 16-byte row fragments read by 16 lanes holding 16 consecutive
// rows, and ds_read_b64_tr_b16 quads (4 consecutive rows x 32 bytes).
__device__ __forceinline__ int sw_col16(int row, int c16) { return c16 ^ ((row & 3) << 2) ^ ((row >> 2) & 3); }
__device__ __forceinline__ int tile_off16(int row, int c16) { return row * 256 + (sw_col16(row, c16) << 4); }

__device__ __forceinline__ void lds_read_tr(const char* p, bf16x4& out) {
  out = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((__attribute__((address_space(3))) bf16x4*)(p));
}
__device__ __forceinline__ void lds_read_tr(const char* p, f16x4& out) {
  typedef __attribute__((ext_vector_type(4))) short i16x4;
  out = __builtin_bit_cast(f16x4, __builtin_amdgcn_ds_read_tr16_b64_v4i16((__attribute__((address_space(3))) i16x4*)(p)));
}
template <class V4>
__device__ __forceinline__ V4 lds_read_tr(const char* p) {
  V4 r;
  lds_read_tr(p, r);
  return r;
}
// the same reads at an LDS byte address held as a number
template <class T>
__device__ __forceinline__ __attribute__((address_space(3))) T* lds_ptr(uint32_t addr) {
  return (__attribute__((address_space(3))) T*)(uintptr_t)addr;
}
__device__ __forceinline__ void lds_read_tr(uint32_t addr, bf16x4& out) {
  out = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(lds_ptr<bf16x4>(addr));
}
__device__ __forceinline__ void lds_read_tr(uint32_t addr, f16x4& out) {
  typedef __attribute__((ext_vector_type(4))) short i16x4;
  out = __builtin_bit_cast(f16x4, __builtin_amdgcn_ds_read_tr16_b64_v4i16(lds_ptr<i16x4>(addr)));
}
template <class V4>
__device__ __forceinline__ V4 lds_read_tr(uint32_t addr) {
  V4 r;
  lds_read_tr(addr, r);
  return r;
}

// asynchronous 16-byte copy global -> LDS: lane i of the wave fills lds_wave_base + 16*i.
// Issued as inline assembly so that completion is tracked by the explicit wait_vmem()
// before the tile barrier only (the copy must stay in flight across the compute phase).
// The statement overwrites M0 and says so to the compiler.
__device__ __forceinline__ void async_copy16(const void* gsrc, uint32_t lds_wave_base) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off"
               :
               : "v"(gsrc), "s"(lds_wave_base)
               : "memory", "m0");
}
// same with the global address split into a wave-uniform base and a per-lane byte offset
__device__ __forceinline__ void async_copy16_sv(const void* uniform_base, uint32_t lane_off, uint32_t lds_wave_base) {
  const uint64_t b = (uint64_t)uniform_base;
  const uint32_t lo = __builtin_amdgcn_readfirstlane((uint32_t)b);
  const uint32_t hi = __builtin_amdgcn_readfirstlane((uint32_t)(b >> 32));
  const uint64_t sb = ((uint64_t)hi << 32) | lo;
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1"
               :
               : "v"(lane_off), "s"(sb), "s"(lds_wave_base)
               : "memory", "m0");
}
// same for 4 bytes per lane: lane i fills lds_wave_base + 4*i
__device__ __forceinline__ void async_copy4(const void* gsrc, uint32_t lds_wave_base) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dword %0, off"
               :
               : "v"(gsrc), "s"(lds_wave_base)
               : "memory", "m0");
}
__device__ __forceinline__ uint32_t lds_addr(const char* p) {
  return (uint32_t)(uintptr_t)(__attribute__((address_space(3))) const char*)p;
}
// wait until this wave's outstanding global loads (including global -> LDS copies) have landed
__device__ __forceinline__ void wait_vmem() { __builtin_amdgcn_s_waitcnt(0x0F70); }

}  // namespace moba
