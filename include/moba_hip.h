/* C ABI of libmoba_hip.so: the MI355X (gfx950) kernels behind moba_attn_varlen.
 *
 * The reference (MoonshotAI/MoBA) has no native code: its hot path is torch ops plus
 * the private varlen entry points of the flash-attn wheel.  Each entry point below
 * names the reference lines whose arithmetic it replaces.  All pointers are device
 * pointers unless stated otherwise; tensors are contiguous except q, k, v (see `strides`);
 * `stream` is a hipStream_t.
 * The library allocates nothing, frees nothing, and never synchronises the device:
 * every launch is enqueued on `stream`.  Return value: 0, or a negative code that
 * moba_strerror() explains.  A HIP error already pending on the calling thread is neither reported
 * nor cleared; an error raised by an entry point's own launches is reported (-3) and cleared.  (With an error
 * pending, a launch failure of the entry point's own that carries the same code cannot be told from it and is
 * not reported: a caller that relies on the return value clears pending errors, hipGetLastError(), first.)
 * State the library keeps, all of it per device and filled on first use: the number of compute units,
 * which kernels have been allowed their dynamic LDS size, and the address of the array of
 * moba_chunk_mean_static.  First calls may come from several threads at once (the writes are idempotent,
 * the address is guarded by a mutex); nothing else is shared between calls.  One environment variable is read,
 * once: MOBA_RESIDENT_CUS=<n> (a diagnostic) makes the kernels whose workgroups stay resident occupy only n
 * compute units' worth of workgroups; results do not depend on it.
 * Inputs are expected to be finite: the attention kernels are compiled without NaN handling, and with an
 * infinity or a NaN in q, k, v or dout the outputs are unspecified (no fault, no hang).  Scores of any finite
 * size are handled (the softmax subtracts a row reference before it exponentiates; see `redo`).
 * Index limits, checked (code -4): S * H * (K + 1) < 2^31 (slot rows are 32-bit: 1M tokens x 64 heads x top-k 12
 * are 8.05e8 of them; a caller beyond the limit, or short of memory for that many partial results, makes one call per
 * group of heads -- heads are independent), K <= 64, chunks per sequence <= 13653, tile counts < 2^31.  head_dim 128 (D below; narrower heads are padded with zeros by the
 * caller, see softmax_scale); q, k, v and everything derived from them are
 * bf16 (dtype = MOBA_DTYPE_BF16) or fp16 (dtype = MOBA_DTYPE_F16, the dtype of the reference's
 * example, examples/llama.py:26); below, "elem" stands for that type.
 *
 * Shapes use: S packed tokens, H query heads, Hkv key/value heads (H is a multiple of Hkv;
 * query head h reads key/value head h / (H/Hkv); the reference operator has H == Hkv and
 * its wrapper repeats the key/value heads first, moba/wrapper.py:59-61), D head_dim, B chunk size, N chunks,
 * F filtered chunks (chunks that are not the last of their sequence), K selected
 * history chunks per (token, head), M = number of selected (token, head, chunk)
 * triples, P = number of (filtered chunk, later chunk of the same sequence) pairs.
 *
 * `strides` (a host pointer to seven int64, read during the call) describes q, k and v where an entry
 * point takes it: {q token stride, q head stride, k/v token stride, k/v head stride, rows per batch
 * entry, q batch stride, k/v batch stride} in elements; the D elements of one (token, head) are
 * contiguous, k and v share their strides, every stride is a positive multiple of 8 and the k/v token
 * stride is at most 2^23.  With rows per batch entry R > 0, packed token t lies in batch entry t / R at
 * position t % R (every sequence must then lie inside one batch entry): this is how a
 * [batch, heads, seqlen, D] tensor of the transformers layout is read without the transposing copy of
 * moba/wrapper.py:7-15; R = 0 (and batch strides 0): one affine range of tokens.  NULL means packed
 * [S,H,D] / [S,Hkv,D].  This is what lets a slice of a fused qkv projection or a
 * [heads, tokens, D] cache be read in place, as flash-attn reads them for the reference
 * (moba/moba_efficient.py:89-128 passes such views on unchanged).  Outputs are always packed.
 */
#ifndef MOBA_HIP_H
#define MOBA_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum { MOBA_DTYPE_BF16 = 0, MOBA_DTYPE_F16 = 1 };

#define MOBA_ABI_VERSION 115 /* the signatures below; moba_version() returns the number the library was built with */
int moba_version(void);
const char* moba_strerror(int code);

/* Host-side planner: counts, buffer sizes and the int32 index tables, all functions of the sequence lengths
 * alone.  Replaces calc_chunks, moba/moba_efficient.py:14-64, and the bookkeeping of :298-323 (number of filtered
 * chunks, effective top-k, the full-attention fallback).  Pure host code: host pointers, no device call.
 *   cu_seqlens_host [nseq+1] int32: starts at 0, strictly increasing
 * moba_plan fills `plan` (counts, table offsets and table_ints); moba_plan_fill does the same and writes the tables
 * into tables_host [plan->table_ints] int32, which the caller copies to the device once per batch layout: table X
 * then lives at device_base + plan->off_X (off_X = -1: the table does not exist in the full-attention fallback,
 * pass NULL).
 * Dense prefixes (dense = 1; no counterpart in the reference): a token in chunk c <= K of its sequence selects
 * every earlier chunk, so what it attends is the plain causal prefix of its sequence.  The plan then makes the chunks
 * 0..K of every sequence one *attention chunk* (dense_local = K) whose rows the kernels serve through their causal
 * self path alone: one partial result instead of c + 1, no picks in sel (moba_gate_topk writes -1 for them), no
 * list entries (pairs_per_head counts the other tokens' only).  The attended sets, and so the results up to
 * rounding, are those of dense = 0, where every chunk is its own attention chunk (dense_local = 0, NA = N).
 * It pays for problems of many tiles (ask moba_fwd_is_queued with the dense plan's counts); on a small problem the
 * long causal tiles of a prefix would run alone at the end.
 * Tables: cu_seqlens, chunk_tok [N+1], achunk_tok [NA+1] (first token of every attention chunk: the chunk_tok
 * argument of moba_fwd* and moba_bwd), fwd_self_tile_prefix [NA+1] / fwd_self_tile_chunk (the self_tile_* arguments of
 * moba_fwd*), self_tile_prefix [NA+1] / self_tile_chunk (those of moba_bwd), kv_tile_prefix [N+1] / kv_tile_chunk
 * and chunk_self_end [N] (moba_bwd), achunk_direct [NA] (the chunk_direct argument of moba_fwd*), mrg_start [nseq] and
 * mrg_prefix [nseq+1] (moba_fwd_merge), seq_fbase [nseq+1], fchunk_tok [F], chunk_fb [N], chunk_local [N], pair_off [F+1],
 * chunk_fid [N].
 * moba_plan_sizes gives, for H query and Hkv key/value heads, the size of every scratch buffer of the calls below. */
typedef struct moba_plan_t {
  int64_t S;
  int32_t nseq, chunk, topk;
  int32_t N, F, K, P, cmax;
  int32_t fallback;                        /* 1: full causal attention (K = 0, one "chunk" per sequence) */
  int32_t fwd_tile_rows, bwd_tile_rows;
  int32_t dense_local;                     /* chunks 0..dense_local of a sequence are one attention chunk */
  int32_t NA;                              /* attention chunks: the N argument of moba_fwd* and moba_bwd */
  int64_t pairs_per_head;                  /* M = pairs_per_head * H */
  int64_t fwd_self_tiles, bwd_self_tiles;  /* the self_tiles arguments of moba_fwd* and of moba_bwd */
  int64_t kv_tiles;                        /* the kv_tiles argument of moba_bwd */
  int64_t merge_tokens;                    /* the merge_tokens argument of moba_fwd_merge */
  double flops_per_head_per_dim;           /* forward flops = this * H * D */
  int64_t off_cu_seqlens, off_chunk_tok, off_achunk_tok, off_fwd_self_tile_prefix, off_fwd_self_tile_chunk,
      off_self_tile_prefix, off_self_tile_chunk, off_kv_tile_prefix, off_kv_tile_chunk, off_chunk_self_end,
      off_achunk_direct, off_mrg_start, off_mrg_prefix, off_seq_fbase, off_fchunk_tok, off_chunk_fb, off_chunk_local, off_pair_off, off_chunk_fid;
  int64_t table_ints;
} moba_plan_t;
typedef struct moba_sizes_t {
  int64_t kbar_elems;                      /* [F, Hkv, D] elem */
  int64_t chunk_mean_workspace_bytes;
  int64_t sel_ints;                        /* [S, H, K] */
  int64_t cnt_ints;                        /* [P*H + 1] */
  int64_t seg_off_ints;                    /* [F*H + 1]; tile_off has the same size */
  int64_t seg_dest_ints;                   /* [M] */
  int64_t fwd_hist_bound, bwd_hist_bound;  /* sizes of the two tile_seg tables = the hist_bound arguments */
  int64_t part_rows;                       /* S*H*(K+1): part_o, part_dq [part_rows, D] elem; part_lse [part_rows] fp32
                                              (times key_split for part_o, part_lse, times dq_key_split for part_dq) */
  int64_t redo_ints;
  int64_t lse_floats;                      /* [S, H] */
  int64_t delta_floats;                    /* [2, S, H] */
} moba_sizes_t;
int moba_plan(const int32_t* cu_seqlens_host, int nseq, int chunk, int topk, int dense, moba_plan_t* plan);
int moba_plan_fill(const int32_t* cu_seqlens_host, int nseq, int chunk, int topk, int dense, moba_plan_t* plan,
                   int32_t* tables_host);
int moba_plan_sizes(const moba_plan_t* plan, int H, int Hkv, int D, moba_sizes_t* sizes);

/* Key chunk-mean.  Replaces moba/moba_efficient.py:326-340 (index_select of the
 * filtered chunks, .mean(dim=1) on bf16, .float()).
 *   k          [S,H,D] elem (H here is the number of key/value heads); strides[2], strides[3] apply
 *   fchunk_tok [F] int32, first token of each filtered chunk
 *   kbar       [F,H,D] elem out (the mean rounded once to the element type)
 *   workspace  moba_chunk_mean_workspace_bytes() bytes, 8-byte aligned
 *   clear      optional: clear_ints int32 of the caller's that the call zeroes on the way -- the cnt array that
 *              moba_gate_topk then adds its counts into, one launch less than clearing it separately; NULL, 0
 *              for none.  (Not done when F = 0: there are no lists to count then.) */
size_t moba_chunk_mean_workspace_bytes(int H, int D, int F, int B);
int moba_chunk_mean(const void* k, const int32_t* fchunk_tok, void* kbar, void* workspace, int64_t S, int H, int D,
                    int F, int B, const int64_t* strides, int dtype, int32_t* clear, int64_t clear_ints,
                    void* stream);

/* moba_chunk_mean for callers that cannot allocate or bring a workspace (code under HIP graph capture, tight
 * serving loops, harnesses that forbid hipMalloc).  No counterpart in the reference.  Same arguments and
 * bit for bit the same kbar as moba_chunk_mean (the sums are exact in fp64 whatever the token split), but
 * the partial sums live in a fixed array inside the library, moba_chunk_mean_static_capacity() bytes (32 MiB)
 * per GPU, held until the process ends.  The call allocates and frees nothing.  Limit: F * H * D * 8 bytes
 * must fit the array (MOBA_ERR_LIMIT otherwise; F * H <= 32768 at D = 128).  All calls on one GPU share the
 * array: calls that overlap in time on one GPU (two streams) race.  The first call on a GPU looks the
 * array's address up (hipGetSymbolAddress); make that call outside any stream capture. */
size_t moba_chunk_mean_static_capacity(void);
int moba_chunk_mean_static(const void* k, const int32_t* fchunk_tok, void* kbar, int64_t S, int H, int D, int F, int B,
                           const int64_t* strides, int dtype, void* stream);

/* Gate scores + causal top-k.  Replaces moba/moba_efficient.py:341-371 (fp32 einsum,
 * -inf mask, torch.topk, dropping -inf picks).
 *   cu_seqlens [nseq+1] int32; seq_fbase [nseq+1] int32, first filtered id of each sequence
 *   sel        [S,H,K] int32 out: filtered-chunk ids, descending score, -1 padded
 *   scores_out optional [S,H,F] fp32, pre-filled with -inf by the caller; receives the
 *              score of every valid candidate (debug / test output), may be NULL
 *   cnt        optional [P*H+1] int32, zero on entry (moba_chunk_mean's `clear`): receives, as a by-product, the
 *              counts that moba_build_lists starts from (how many tokens of each query chunk and head picked
 *              each chunk; pass counted = 1 there); needs pair_off [F+1], the table of moba_build_lists.
 *              NULL: no counts.
 *   dense_local the plan's: the tokens of the chunks 0..dense_local of every sequence get no picks (-1) and no
 *              counts; 0 for the reference's selection
 * K <= 64.  strides[0], strides[1] apply to q; kbar is packed [F,Hkv,D]. */
int moba_gate_topk(const void* q, const void* kbar, const int32_t* cu_seqlens, const int32_t* seq_fbase, int32_t* sel,
                   float* scores_out, const int32_t* pair_off, int32_t* cnt, int64_t S, int H, int Hkv, int D,
                   int nseq, int F, int B, int K, int dense_local, const int64_t* strides, int dtype, void* stream);

/* The selection step of moba/moba_efficient.py:365-371 alone, on caller-supplied
 * scores [S,H,F] fp32 (-inf = not a candidate).  Same routine as moba_gate_topk. */
int moba_topk_from_scores(const float* scores, int32_t* sel, int64_t S, int H, int F, int K, void* stream);

/* Varlen gather lists.  Replaces moba/moba_efficient.py:373-423 (nonzero, per-segment
 * counts, gathered q and kv copies): index lists only, in the same (chunk, head, token)
 * order.
 *   chunk_tok [N+1], chunk_fb [N] (first filtered id of the chunk's sequence),
 *   chunk_local [N] (index of the chunk inside its sequence), pair_off [F+1]
 *   (prefix sum of the number of later chunks in the same sequence)   -- int32 tables
 *   cnt      [P*H+1] int32 scratch; with counted = 1 it holds on entry the counts moba_gate_topk left there
 *            (the call then skips its own counting pass over sel), with counted = 0 its contents do not matter
 *   seg_off  [F*H+1] out, list start of segment (f,h);  tile_off [F*H+1] out, prefix
 *            sum of ceil(rows/tile_rows);  seg_dest [M] out, entries
 *            (token*H + h)*(K+1) + 1 + slot
 *   tile_seg [hist_bound] out: segment f*H + h of every history tile id, -1 past the last tile
 * cmax = most chunks in a sequence minus one; tile_rows = rows per tile of the kernel that will read tile_off and
 * tile_seg (moba_fwd_tile_rows() or moba_bwd_tile_rows()); hist_bound: an upper bound on the number of tiles,
 * e.g. M / tile_rows + F * H.
 * tile_rows_b, tile_off_b [F*H+1], tile_seg_b [hist_bound_b]: optional second pair of tile tables for another tile
 * height (what moba_tile_tables would make from seg_off: a caller that will run the backward asks for its tables
 * here and saves that launch on small problems); tile_off_b NULL for none.
 * dense_local: the plan's -- the tokens of the chunks 0..dense_local of every sequence have no list entries (their
 * picks in sel, if any, are ignored, and their counts are zero); 0 for the reference's lists. */
int moba_build_lists(const int32_t* sel, const int32_t* chunk_tok, const int32_t* chunk_fb, const int32_t* chunk_local,
                     const int32_t* pair_off, int32_t* cnt, int32_t* seg_off, int32_t* tile_off, int32_t* seg_dest,
                     int32_t* tile_seg, int64_t S, int H, int K, int N, int F, int P, int cmax, int tile_rows,
                     int64_t hist_bound, int counted, int tile_rows_b, int32_t* tile_off_b, int32_t* tile_seg_b,
                     int64_t hist_bound_b, int dense_local, void* stream);

/* The tile tables of moba_build_lists alone, for another tile height: the forward and the backward kernels cut
 * the same gather lists into tiles of moba_fwd_tile_rows() and moba_bwd_tile_rows() rows.  No counterpart in the
 * reference (flash-attn tiles its varlen batches internally).
 *   seg_off [F*H+1] from moba_build_lists; tile_off [F*H+1] out; tile_seg [hist_bound] out */
int moba_tile_tables(const int32_t* seg_off, int32_t* tile_off, int32_t* tile_seg, int H, int F, int tile_rows,
                     int64_t hist_bound, void* stream);

/* Attention.  Replaces MixedAttention.forward, moba/moba_efficient.py:69-183 (two
 * flash-attn varlen forwards and the LSE merge), and with K = 0 and one chunk per
 * sequence the full-causal case of moba/moba_efficient.py:318-321.
 *   part_o [key_split*S*H*(K+1), D] elem and part_lse [key_split*S*H*(K+1)] fp32: per-slot partial results
 *   key_split: 1, or for small problems the power of two (up to 8) that moba_fwd_key_split() names: the kernel
 *              then cuts the keys of every history tile into that many parts, each a tile of its own, so that a
 *              problem of a few hundred tiles still spreads evenly over the compute units; the merge takes the
 *              parts as further slots (part g of a slot row lies S*H*(K+1) rows behind part g-1).  Refused
 *              (MOBA_ERR_ARG) for problems large enough for the resident-workgroup kernel or when B is not a
 *              multiple of 64*key_split.  The same value goes to moba_fwd_partials and moba_fwd_merge.
 *   chunk_tok [N+1], N: the attention chunks (the plan's achunk_tok and NA; the chunks themselves without dense
 *              prefixes): the rows of one attend its keys causally, in tiles of moba_fwd_tile_rows() rows
 *   self_tile_prefix [N+1] int32: prefix sum of ceil(attention chunk length / moba_fwd_tile_rows())
 *   self_tile_chunk [self_tile_prefix[N]] int32: the attention chunk of each of those tiles
 *   tile_off, tile_seg: from moba_build_lists or moba_tile_tables with tile_rows = moba_fwd_tile_rows()
 *              (may be NULL when K = 0)
 *   out [S,H,D] elem, lse [S,H] fp32 (natural log)
 *   chunk_direct [N] int32 or NULL: 1 for an attention chunk whose rows have no history slots (the first one of
 *              every sequence: the plan's achunk_direct).  moba_fwd_partials writes the result of such a chunk's
 *              rows straight into out and lse (there is nothing to merge it with) instead of into slot 0, and
 *              moba_fwd_merge is told to leave those rows alone: mrg_start [nranges] / mrg_prefix [nranges+1] name the
 *              token ranges it walks (range b: tokens mrg_start[b] + i, i < mrg_prefix[b+1] - mrg_prefix[b]) and
 *              merge_tokens = mrg_prefix[nranges] their number (0: no launch at all, e.g. with K = 0).  NULL, NULL,
 *              NULL, 0 and merge_tokens = S: every row goes through its slot and the merge.
 *   hist_bound: upper bound on the number of history tiles, e.g. M / moba_fwd_tile_rows() + F*H
 *   self_tiles: self_tile_prefix[N]
 *   queues [8] int32 scratch: the tile counters of the forward kernel, whose workgroups (one per CU) stay
 *              resident and draw tiles from one queue per XCD; the call zeroes them with a kernel of its own.
 *              Calls that overlap in time need their own eight counters each.
 *   redo   [1 + hist_bound + self_tiles * H] int32 scratch, or NULL.  With it, problems large enough for the
 *              resident-workgroup kernel take each tile's softmax relative to one fixed reference per row (the row
 *              maximum of the tile's first 32 keys) instead of a running maximum; a tile in which a row leaves the
 *              range that is safe -- scores that rise more than 96 powers of two above that reference (bf16) or 16
 *              (fp16: a probability beyond the type's range), or accumulators that leave fp32 (products with |v| of
 *              2^31 and more) -- is entered in this list and computed again by the kernel that tracks the maximum
 *              (redo[0] = number of such tiles after the call, normally 0).  The result is within rounding of the
 *              other path's either way.  NULL and small problems: running maximum only.
 *   softmax_scale: the factor on q k^T; 0 (or less) stands for D^-0.5, the reference's only choice
 *              (moba/moba_efficient.py:86).  A caller whose heads are narrower than D pads them with zeros
 *              and passes its own head_dim^-0.5.
 *   self_tile_skip, q_tok_shift (moba_fwd_partials only; 0, 0 otherwise): queries that are the tail of their
 *              sequence -- new tokens against a key/value cache, the decode branch of moba/wrapper.py:76-82 with
 *              more than one query token (flash_attn_func with a bottom-right aligned causal mask).  K = 0,
 *              chunk_direct set: the first self_tile_skip row tiles of every chunk do not exist (self_tile_prefix
 *              counts the others), and q, out and lse hold the rows from token q_tok_shift on
 *              (q_tok_shift <= self_tile_skip * moba_fwd_tile_rows(); the rows between the two are computed from
 *              whatever q holds there and land in out's rows of the same index: padding of the caller's). */
int moba_fwd_tile_rows(void);
int moba_bwd_tile_rows(void);
int moba_fwd_partials(const void* q, const void* k, const void* v, void* part_o, float* part_lse,
                      const int32_t* seg_off, const int32_t* tile_off, const int32_t* seg_dest,
                      const int32_t* fchunk_tok, const int32_t* chunk_tok, const int32_t* self_tile_prefix,
                      const int32_t* tile_seg, const int32_t* self_tile_chunk, const int32_t* chunk_direct, void* out,
                      float* lse, int64_t S, int H, int Hkv, int D, int K, int F, int N, int B, int64_t hist_bound,
                      int64_t self_tiles, int key_split, const int64_t* strides, int32_t* queues, int32_t* redo,
                      float softmax_scale, int dtype, int self_tile_skip, int64_t q_tok_shift, void* stream);
int moba_fwd_merge(const void* part_o, const float* part_lse, const int32_t* sel, void* out, float* lse, int64_t S,
                   int H, int D, int K, int key_split, const int32_t* mrg_start, const int32_t* mrg_prefix, int nranges,
                   int64_t merge_tokens, int dtype, void* stream);
int moba_fwd_key_split(int64_t S, int H, int K, int B, int64_t hist_bound, int64_t self_tiles);
/* 1 if moba_fwd_partials would run a problem of hist_bound + self_tiles * H tiles with resident workgroups drawing
 * from the tile queues, 0 if with one workgroup per tile (no counterpart in the reference). */
int moba_fwd_is_queued(int64_t hist_bound, int64_t self_tiles, int H);
int moba_fwd(const void* q, const void* k, const void* v, void* part_o, float* part_lse, const int32_t* sel,
             const int32_t* seg_off, const int32_t* tile_off, const int32_t* seg_dest, const int32_t* fchunk_tok,
             const int32_t* chunk_tok, const int32_t* self_tile_prefix, const int32_t* tile_seg,
             const int32_t* self_tile_chunk, const int32_t* chunk_direct, const int32_t* mrg_start,
             const int32_t* mrg_prefix, int nranges, int64_t merge_tokens, void* out, float* lse, int64_t S, int H,
             int Hkv, int D, int K, int F, int N, int B, int64_t hist_bound, int64_t self_tiles, int key_split,
             const int64_t* strides, int32_t* queues, int32_t* redo, float softmax_scale, int dtype, void* stream);

/* Backward.  Replaces MixedAttention.backward, moba/moba_efficient.py:185-267, and the
 * autograd scatter of its gathered gradients.  Deterministic (no floating-point atomics).
 *   dout, q, out, dq [S,H,D] elem; k, v, dk, dv [S,Hkv,D] elem; lse [S,H] fp32 from the forward
 *   (`strides` applies to q, k, v; dout, out, dq, dk, dv are packed)
 *   tile_off, tile_seg, chunk_tok, self_tile_prefix, self_tile_chunk, hist_bound, self_tiles, N: as in
 *   moba_fwd_partials (attention chunks), but for tiles of moba_bwd_tile_rows() rows (moba_tile_tables makes the
 *   first two from seg_off)
 *   chunk_fid [chunks] int32: filtered id of each chunk, -1 for the last chunk of a sequence
 *   kv_chunk_tok [chunks+1] (the plan's chunk_tok), kv_tile_prefix [chunks+1], kv_tile_chunk [kv_tiles],
 *   chunk_self_end [chunks], kv_tiles: the key tiles of the dK/dV kernel, moba_bwd_tile_rows() keys of one chunk
 *   each; the rows that attend a chunk's keys causally end at token chunk_self_end (the end of the chunk, or of
 *   the dense prefix it belongs to), the others come from the chunk's gather list
 *   chunk_direct, mrg_start, mrg_prefix, nranges, merge_tokens: as in moba_fwd (the dQ kernel writes the dQ of the
 *   rows without history slots itself, the sum over the slots walks the other tokens), or NULL, NULL, NULL, 0, S
 *   delta [2,S,H] fp32 scratch (rowsum(dO*O), then the LSE in the log2 domain); part_dq [dq_key_split*S*H*(K+1), D]
 *   elem scratch (the per-slot dQ, rounded as the per-chunk dQ that flash-attn returns to the reference is)
 *   dq_key_split: 1, or for small problems the power of two (up to 8) that moba_bwd_dq_key_split() names: the dQ
 *              kernel then cuts the keys of every history tile into that many parts, each a tile with slot rows of
 *              its own (as key_split does in the forward), and takes its self tiles first.  B must be a multiple
 *              of 64 * dq_key_split (MOBA_ERR_ARG otherwise).
 *   dq, dk, dv: out; dk and dv of a key/value head sum over its query heads
 *   queues [16] int32 scratch: tile counters of the dQ and dK/dV kernels (as in moba_fwd_partials)
 *   dkv_scratch: moba_bwd_dkv_scratch_bytes(S, Hkv, kv_tiles) bytes, 16-byte aligned, or null.  With few key tiles
 *              (fewer than two per compute unit, S >= 4096) the dK/dV kernel cuts each into up to 4 parts that run
 *              side by side and leave fp32 sums there, added up in a fixed order (deterministic all the same);
 *              without the scratch, or when the query returns 0, every tile is one piece.
 *   softmax_scale: as in the forward call */
size_t moba_bwd_dkv_scratch_bytes(int64_t S, int Hkv, int64_t kv_tiles);
int moba_bwd_dq_key_split(int64_t S, int H, int K, int B, int64_t hist_bound, int64_t self_tiles);
int moba_bwd(const void* dout, const void* q, const void* k, const void* v, const void* out, const float* lse,
             const int32_t* sel, const int32_t* seg_off, const int32_t* tile_off, const int32_t* seg_dest,
             const int32_t* fchunk_tok, const int32_t* chunk_tok, const int32_t* self_tile_prefix,
             const int32_t* tile_seg, const int32_t* self_tile_chunk, const int32_t* chunk_fid,
             const int32_t* kv_chunk_tok, const int32_t* kv_tile_prefix, const int32_t* kv_tile_chunk,
             const int32_t* chunk_self_end, const int32_t* chunk_direct, const int32_t* mrg_start,
             const int32_t* mrg_prefix, int nranges, int64_t merge_tokens, float* delta, void* part_dq, void* dq,
             void* dk, void* dv, int64_t S, int H,
             int Hkv, int D, int K, int F, int N, int B, int64_t hist_bound, int64_t self_tiles, int64_t kv_tiles,
             int dq_key_split, const int64_t* strides, int32_t* queues, void* dkv_scratch, int64_t dkv_scratch_bytes,
             float softmax_scale, int dtype, void* stream);

/* Decode: one query token per sequence against the key/value cache.  Replaces the
 * flash_attn_func call of the adapter's decode branch, moba/wrapper.py:76-82 (full attention
 * over the cache, grouped-query heads).
 *   q [B,H,D]: element strides q_stride_b, q_stride_h, D contiguous
 *   k, v [B,Hkv,Skv,D]: element strides kv_stride_b, kv_stride_h; key rows contiguous and D apart
 *   out [B,H,D] elem, contiguous
 *   part_o [B*H*splits, D] fp32 and part_lse [B*H*splits] fp32 scratch, splits = moba_decode_splits()
 * H/Hkv in {1,2,4,8}; strides multiples of 8 elements; scale = softmax scale. */
int moba_decode_splits(int B, int Hkv, int Skv);
int moba_decode(const void* q, const void* k, const void* v, void* out, float* part_o, float* part_lse, int B, int H,
                int Hkv, int Skv, int D, int64_t q_stride_b, int64_t q_stride_h, int64_t kv_stride_b,
                int64_t kv_stride_h, float scale, int dtype, void* stream);

/* Measurement aid, no counterpart in the reference: what the matrix pipes sustain when they do nothing else.
 * Launches `workgroups` workgroups (0: one per compute unit) of eight waves, two per SIMD as in the forward kernel;
 * every wave issues iters * 16 v_mfma_f32_32x32x16_bf16 on sixteen operand registers it loads once from
 * `operands` (16 KiB of bf16 on the device: constant or random data, the caller's choice) -- no LDS, no memory
 * traffic, no vector work.  Flops = workgroups * 8 * iters * 16 * 32768; the caller times the launch on
 * `stream`.  sink: one float on the device (never written in practice). */
int moba_mfma_probe(const void* operands, float* sink, int iters, int workgroups, void* stream);

#ifdef __cplusplus
}
#endif
#endif
