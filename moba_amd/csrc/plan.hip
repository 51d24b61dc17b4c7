// Host-side planner of the C ABI: everything the kernels need that depends only on the sequence
// lengths -- counts, buffer sizes and the small int32 index tables -- so that a host which is not Python
// has nothing to port.  Counterpart of calc_chunks (moba/moba_efficient.py:14-64) and of the bookkeeping
// around it (:298-323).  Pure host code: no device call, no allocation.
#include <algorithm>
#include <cstring>
#include "attn_common.h"

using namespace moba;

// The layout of this struct is part of the C ABI (include/moba_hip.h declares the same fields in the same order).
struct moba_plan_t {
  int64_t S;                // packed tokens
  int32_t nseq, chunk, topk;
  int32_t N;                // chunks (fallback: one per sequence)
  int32_t F;                // filtered chunks (0 in the fallback)
  int32_t K;                // selected history chunks per (token, head): min(topk - 1, F, most chunks per sequence - 1)
  int32_t P;                // (filtered chunk, later chunk of the same sequence) pairs
  int32_t cmax;             // most chunks in a sequence minus one
  int32_t fallback;         // 1: topk - 1 <= 0 or no filtered chunk -- full causal attention, K = 0
  int32_t fwd_tile_rows, bwd_tile_rows;
  int32_t dense_local;      // chunks 0..dense_local of every sequence form one attention chunk (0: every chunk its own)
  int32_t NA;               // attention chunks
  int64_t pairs_per_head;   // list entries per head: M = pairs_per_head * H
  int64_t fwd_self_tiles, bwd_self_tiles;  // row tiles of the attention chunks, per head
  int64_t kv_tiles;         // key tiles (bwd_tile_rows keys) of the chunks, per key/value head
  int64_t merge_tokens;     // tokens behind the first attention chunk of their sequence: the rows the merge walks
  double flops_per_head_per_dim;           // forward flops = this * H * head_dim
  // offsets (in int32 elements) of the tables inside the array moba_plan_fill writes, -1 = absent
  int64_t off_cu_seqlens, off_chunk_tok, off_achunk_tok, off_fwd_self_tile_prefix, off_fwd_self_tile_chunk,
      off_self_tile_prefix, off_self_tile_chunk, off_kv_tile_prefix, off_kv_tile_chunk, off_chunk_self_end,
      off_achunk_direct, off_mrg_start, off_mrg_prefix, off_seq_fbase, off_fchunk_tok, off_chunk_fb, off_chunk_local, off_pair_off, off_chunk_fid;
  int64_t table_ints;       // length of that array
};

static int plan_core(const int32_t* cu, int nseq, int chunk, int topk, int dense, moba_plan_t* pl, int32_t* tab) {
  if (!cu || !pl || nseq <= 0 || chunk <= 0 || topk <= 0) return MOBA_ERR_ARG;
  if (cu[0] != 0) return MOBA_ERR_ARG;
  for (int b = 0; b < nseq; ++b)
    if (cu[b + 1] <= cu[b]) return MOBA_ERR_ARG;  // strictly increasing: zero-length sequences are unsupported
  moba_plan_t p;
  std::memset(&p, 0, sizeof(p));
  p.S = cu[nseq]; p.nseq = nseq; p.chunk = chunk; p.topk = topk;
  p.fwd_tile_rows = kFwdTileRows; p.bwd_tile_rows = TM;
  int64_t nchunks = 0, F = 0;
  int cmax = 0;
  for (int b = 0; b < nseq; ++b) {
    const int64_t n = ((int64_t)cu[b + 1] - cu[b] + chunk - 1) / chunk;
    nchunks += n; F += n - 1;
    cmax = std::max<int64_t>(cmax, n - 1);
  }
  const int64_t k_eff = std::min<int64_t>(topk - 1, F);
  p.fallback = k_eff <= 0;
  if (p.fallback) { nchunks = nseq; F = 0; cmax = 0; }
  if (nchunks >= 0x7fffffffLL) return MOBA_ERR_LIMIT;
  p.N = (int32_t)nchunks; p.F = (int32_t)F; p.cmax = cmax;
  p.K = p.fallback ? 0 : (int32_t)std::min<int64_t>(k_eff, cmax);
  const int d = dense ? p.K : 0;
  p.dense_local = d;

  // first pass over the chunks: tile counts, pair counts, flops
  int64_t ftiles = 0, btiles = 0, ktiles = 0, pairs = 0, pairs_all = 0, pairs_self = 0, P = 0, NA = 0;
  auto add_achunk = [&](int64_t alen) {
    ftiles += (alen + kFwdTileRows - 1) / kFwdTileRows;
    btiles += (alen + TM - 1) / TM;
    ++NA;
  };
  for (int b = 0; b < nseq; ++b) {
    const int64_t len = (int64_t)cu[b + 1] - cu[b];
    const int64_t n = p.fallback ? 1 : (len + chunk - 1) / chunk;
    int64_t alen = 0;  // length of the attention chunk being put together
    for (int64_t c = 0; c < n; ++c) {
      const int64_t clen = p.fallback ? len : std::min<int64_t>(chunk, len - c * chunk);
      if (c == d + 1) p.merge_tokens += len - alen;  // (the tokens behind the sequence's first attention chunk)
      if (c > d) { add_achunk(alen); alen = 0; }
      alen += clen;
      ktiles += (clen + TM - 1) / TM;
      pairs_self += clen * (clen + 1) / 2;
      pairs_all += clen * std::min<int64_t>(p.K, c);
      if (c > d) pairs += clen * std::min<int64_t>(p.K, c);
      if (!p.fallback && c < n - 1) P += n - 1 - c;
    }
    add_achunk(alen);
  }
  if (P >= 0x7fffffffLL || ftiles >= 0x7fffffffLL || btiles >= 0x7fffffffLL || ktiles >= 0x7fffffffLL) return MOBA_ERR_LIMIT;
  p.fwd_self_tiles = ftiles; p.bwd_self_tiles = btiles; p.kv_tiles = ktiles; p.pairs_per_head = pairs; p.P = (int32_t)P;
  p.NA = (int32_t)NA;
  p.flops_per_head_per_dim = 4.0 * ((double)pairs_self + (double)pairs_all * chunk);

  int64_t off = 0;
  auto take = [&](int64_t n) { const int64_t o = off; off += n; return o; };
  p.off_chunk_tok = take(p.N + 1);
  p.off_achunk_tok = take(NA + 1);
  p.off_fwd_self_tile_prefix = take(NA + 1);
  p.off_fwd_self_tile_chunk = take(ftiles);
  p.off_self_tile_prefix = take(NA + 1);
  p.off_self_tile_chunk = take(btiles);
  p.off_kv_tile_prefix = take(p.N + 1);
  p.off_kv_tile_chunk = take(ktiles);
  p.off_chunk_self_end = take(p.N);
  p.off_achunk_direct = take(NA);
  p.off_mrg_start = take(nseq);
  p.off_mrg_prefix = take(nseq + 1);
  if (p.fallback) {
    p.off_seq_fbase = p.off_fchunk_tok = p.off_chunk_fb = p.off_chunk_local = p.off_pair_off = p.off_chunk_fid = -1;
  } else {
    p.off_seq_fbase = take(nseq + 1);
    p.off_fchunk_tok = take(p.F);
    p.off_chunk_fb = take(p.N);
    p.off_chunk_local = take(p.N);
    p.off_pair_off = take(p.F + 1);
    p.off_chunk_fid = take(p.N);
  }
  p.off_cu_seqlens = take(nseq + 1);
  p.table_ints = off;
  *pl = p;
  if (!tab) return MOBA_OK;

  // second pass: the tables
  std::memcpy(tab + p.off_cu_seqlens, cu, sizeof(int32_t) * (nseq + 1));
  int32_t* chunk_tok = tab + p.off_chunk_tok;
  int32_t* achunk_tok = tab + p.off_achunk_tok;
  int32_t* fpre = tab + p.off_fwd_self_tile_prefix;
  int32_t* fch = tab + p.off_fwd_self_tile_chunk;
  int32_t* bpre = tab + p.off_self_tile_prefix;
  int32_t* bch = tab + p.off_self_tile_chunk;
  int32_t* kpre = tab + p.off_kv_tile_prefix;
  int32_t* kch = tab + p.off_kv_tile_chunk;
  int32_t* self_end = tab + p.off_chunk_self_end;
  int32_t c_all = 0, f_all = 0, pair_all = 0, a_all = 0;
  int64_t ft = 0, bt = 0, kt = 0;
  int64_t merged = 0;
  auto close_achunk = [&](int32_t tok0, int64_t alen, int32_t first_chunk, int32_t end_chunk, int b, bool first) {
    achunk_tok[a_all] = tok0;
    tab[p.off_achunk_direct + a_all] = first ? 1 : 0;
    if (first) {
      tab[p.off_mrg_start + b] = (int32_t)(tok0 + alen);
      tab[p.off_mrg_prefix + b] = (int32_t)merged;
      merged += cu[b + 1] - (tok0 + alen);
    }
    fpre[a_all] = (int32_t)ft; bpre[a_all] = (int32_t)bt;
    for (int64_t i = 0; i < (alen + kFwdTileRows - 1) / kFwdTileRows; ++i) fch[ft++] = a_all;
    for (int64_t i = 0; i < (alen + TM - 1) / TM; ++i) bch[bt++] = a_all;
    for (int32_t cc = first_chunk; cc < end_chunk; ++cc) self_end[cc] = (int32_t)(tok0 + alen);
    ++a_all;
  };
  for (int b = 0; b < nseq; ++b) {
    const int64_t len = (int64_t)cu[b + 1] - cu[b];
    const int64_t n = p.fallback ? 1 : (len + chunk - 1) / chunk;
    if (!p.fallback) tab[p.off_seq_fbase + b] = f_all;
    const int32_t fb = f_all;
    int64_t alen = 0;
    int32_t a_tok0 = cu[b], a_first = c_all;
    for (int64_t c = 0; c < n; ++c, ++c_all) {
      const int64_t clen = p.fallback ? len : std::min<int64_t>(chunk, len - c * chunk);
      chunk_tok[c_all] = (int32_t)(cu[b] + c * chunk);
      if (c > d) {
        close_achunk(a_tok0, alen, a_first, c_all, b, c == d + 1);
        a_tok0 = chunk_tok[c_all]; a_first = c_all; alen = 0;
      }
      alen += clen;
      kpre[c_all] = (int32_t)kt;
      for (int64_t i = 0; i < (clen + TM - 1) / TM; ++i) kch[kt++] = c_all;
      if (p.fallback) continue;
      tab[p.off_chunk_fb + c_all] = fb;
      tab[p.off_chunk_local + c_all] = (int32_t)c;
      if (c < n - 1) {
        tab[p.off_chunk_fid + c_all] = f_all;
        tab[p.off_fchunk_tok + f_all] = chunk_tok[c_all];
        tab[p.off_pair_off + f_all] = pair_all;
        pair_all += (int32_t)(n - 1 - c);
        ++f_all;
      } else {
        tab[p.off_chunk_fid + c_all] = -1;
      }
    }
    close_achunk(a_tok0, alen, a_first, c_all, b, n <= (int64_t)d + 1);
  }
  tab[p.off_mrg_prefix + nseq] = (int32_t)merged;
  chunk_tok[c_all] = cu[nseq];
  achunk_tok[a_all] = cu[nseq];
  fpre[a_all] = (int32_t)ft; bpre[a_all] = (int32_t)bt;
  kpre[c_all] = (int32_t)kt;
  if (!p.fallback) {
    tab[p.off_seq_fbase + nseq] = f_all;
    tab[p.off_pair_off + f_all] = pair_all;
  }
  return MOBA_OK;
}

extern "C" int moba_plan(const int32_t* cu_seqlens_host, int nseq, int chunk, int topk, int dense, moba_plan_t* plan) {
  return plan_core(cu_seqlens_host, nseq, chunk, topk, dense, plan, nullptr);
}

extern "C" int moba_plan_fill(const int32_t* cu_seqlens_host, int nseq, int chunk, int topk, int dense,
                              moba_plan_t* plan, int32_t* tables_host) {
  if (!tables_host) return MOBA_ERR_ARG;
  return plan_core(cu_seqlens_host, nseq, chunk, topk, dense, plan, tables_host);
}

// Sizes, for H query heads, of every device buffer a forward (and backward) call takes besides q, k, v and the
// outputs.  Bytes for the element-typed ones (elem_bytes = 2), counts of int32 / fp32 / fp64 otherwise as named.
struct moba_sizes_t {
  int64_t kbar_elems;              // [F, Hkv, D]
  int64_t chunk_mean_workspace_bytes;
  int64_t sel_ints;                // [S, H, K]
  int64_t cnt_ints;                // [P*H + 1]
  int64_t seg_off_ints;            // [F*H + 1]  (tile_off has the same size)
  int64_t seg_dest_ints;           // [M] (at least 1)
  int64_t fwd_hist_bound, bwd_hist_bound;   // tile_seg sizes and the hist_bound arguments
  int64_t part_rows;               // S*H*(K+1): part_o [part_rows, D] elem, part_lse [part_rows] fp32, part_dq like part_o
  int64_t redo_ints;               // 1 + fwd_hist_bound + fwd_self_tiles*H
  int64_t lse_floats;              // [S, H]
  int64_t delta_floats;            // [2, S, H]
};

extern "C" size_t moba_chunk_mean_workspace_bytes(int H, int D, int F, int B);

extern "C" int moba_plan_sizes(const moba_plan_t* pl, int H, int Hkv, int D, moba_sizes_t* out) {
  if (!pl || !out || H <= 0 || Hkv <= 0 || H % Hkv != 0 || D <= 0) return MOBA_ERR_ARG;
  moba_sizes_t s;
  std::memset(&s, 0, sizeof(s));
  const int64_t M = pl->pairs_per_head * H;
  s.kbar_elems = (int64_t)pl->F * Hkv * D;
  s.chunk_mean_workspace_bytes = pl->F > 0 ? (int64_t)moba_chunk_mean_workspace_bytes(Hkv, D, pl->F, pl->chunk) : 0;
  s.sel_ints = pl->S * H * pl->K;
  s.cnt_ints = (int64_t)pl->P * H + 1;
  s.seg_off_ints = (int64_t)pl->F * H + 1;
  s.seg_dest_ints = std::max<int64_t>(M, 1);
  s.fwd_hist_bound = M / pl->fwd_tile_rows + (int64_t)pl->F * H;
  s.bwd_hist_bound = M / pl->bwd_tile_rows + (int64_t)pl->F * H;
  s.part_rows = pl->S * H * (pl->K + 1);
  s.redo_ints = 1 + s.fwd_hist_bound + pl->fwd_self_tiles * H;
  s.lse_floats = pl->S * H;
  s.delta_floats = 2 * pl->S * H;
  if (s.part_rows >= 0x7fffffffLL) return MOBA_ERR_LIMIT;
  *out = s;
  return MOBA_OK;
}
