// Row maps of the backward kernels: which "columns" a block of "rows" meets.
//
// dQ: rows are the queries of a set and columns its keys - the forward index map as it is
// (QueryRows).  dK / dV: rows are keys and columns the queries that see them.  For the patterns
// whose sets number queries and keys alike, the query range of a key follows from the forward
// map's monotone bounds by bisection (KeyRowsOf).  Block Scatter with a stripe offset and the
// per-token window have their own inverse maps.  Keys that are sinks are seen by every later
// query of every set; they are left out of those maps' results (`store`) and get a pass of their
// own (KeyRowsSinks), split over chunks of queries whose partial sums a small kernel adds up.
//
// Interface (host and device):
//   static num_sets(ge), max_rows(ge)      grid size: sets per (batch, kv head), rows of the largest
//   RowMap(ge, set, r0)                    r0: first row of the row block (rows r0 .. r0+255 at most)
//   n_rows(), n_cols()
//   row_pos(t), col_pos(c)                 token positions
//   lo(t), hi(t)                           row t meets the columns lo..hi (and those below kpre())
//   block_lo(r0, r1), block_hi(r0, r1)     union of the ranges of rows r0..r1
//   store(pos)                             whether the result row of token pos is written here
//   kBlockPredicate / sees(t, c)           maps whose rows do not meet one range of columns say per
//                                          row and 32-column block (first column c) whether the row
//                                          meets the block - all of it or nothing
//   kAccumulate                            the results are added to rows another pass has written
#pragma once
#include "intra_maps.h"

namespace intra {

template <class MAP>
struct QueryRows {
  MAP m;
  static IM_HD int num_sets(const IntraGeom& ge) { return MAP::num_sets(ge); }
  static IM_HD int max_rows(const IntraGeom& ge) { return MAP::max_nq(ge); }
  IM_HD QueryRows(const IntraGeom& ge, int set, int r0) : m(ge, set, r0) {}
  IM_HD int n_rows() const { return m.nq(); }
  IM_HD int n_cols() const { return m.nk(); }
  IM_HD int kpre() const { return m.kpre(); }
  IM_HD int row_pos(int t) const { return m.qpos(t); }
  IM_HD int col_pos(int c) const { return m.kpos(c); }
  IM_HD int lo(int t) const { return m.klo(t); }
  IM_HD int hi(int t) const { return im_min(m.khi(t), m.nk() - 1); }
  IM_HD int block_lo(int r0, int) const { return m.kpre() > 0 ? 0 : m.klo(r0); }
  IM_HD int block_hi(int, int r1) const { return hi(r1); }
  IM_HD bool store(int) const { return true; }
  static constexpr bool kBlockPredicate = false, kAccumulate = false;
  IM_HD bool sees(int, int) const { return true; }
};

// Keys of a set whose queries and keys carry the same numbering (LLM Scatter, Gather 1, window,
// block Scatter without offset): key r is seen by the queries from the first one whose upper key
// bound reaches r to the last one whose lower key bound does not exceed r; both are monotone in r.
template <class MAP>
struct KeyRowsOf {
  MAP m;
  static IM_HD int num_sets(const IntraGeom& ge) { return MAP::num_sets(ge); }
  static IM_HD int max_rows(const IntraGeom& ge) { return MAP::max_nq(ge); }
  IM_HD KeyRowsOf(const IntraGeom& ge, int set, int) : m(ge, set, 0) {}
  IM_HD int n_rows() const { return m.nk(); }
  IM_HD int n_cols() const { return m.nq(); }
  IM_HD int kpre() const { return 0; }
  IM_HD int row_pos(int t) const { return m.kpos(t); }
  IM_HD int col_pos(int c) const { return m.qpos(c); }
  IM_HD int lo(int r) const {  // first tq with min(khi(tq), nk-1) >= r
    int a = 0, b = m.nq();
    const int kmax = m.nk() - 1;
    while (a < b) {
      const int mid = (a + b) >> 1;
      if (im_min(m.khi(mid), kmax) >= r) b = mid;
      else a = mid + 1;
    }
    return a;
  }
  IM_HD int hi(int r) const {  // last tq with klo(tq) <= r
    int a = -1, b = m.nq() - 1;
    while (a < b) {
      const int mid = (a + b + 1) >> 1;
      if (m.klo(mid) <= r) a = mid;
      else b = mid - 1;
    }
    return a;
  }
  IM_HD int block_lo(int r0, int) const { return lo(r0); }
  IM_HD int block_hi(int, int r1) const { return hi(r1); }
  IM_HD bool store(int) const { return true; }
  static constexpr bool kBlockPredicate = false, kAccumulate = false;
  IM_HD bool sees(int, int) const { return true; }
};

// Keys of group gk of block Scatter (blocks kb = gk mod G), any stripe offset.  Without offset the
// queries that see them are the later tokens of the same group.  With offset `off` a key of block
// kb is seen by the later queries of its own block and by all queries of the blocks kb + G - off,
// kb + 2G - off, ... (the query blocks qb > kb with (qb + off) mod G = gk); the columns of a row
// block are numbered [own block][those blocks], which needs the row block inside one key block
// (block size a multiple of 256).  Sinks (positions < n_sink) are not stored here.
struct KeyRowsBlockScatter {
  int G, blk, gk, off, n, S, skip, a, kb, own_len, qb0, ncols;
  FastDiv dBlk;
  static IM_HD int num_sets(const IntraGeom& ge) { return ge.G; }
  static IM_HD int max_rows(const IntraGeom& ge) { return MapLlmBlockScatter::max_nq(ge); }
  IM_HD KeyRowsBlockScatter(const IntraGeom& ge, int set, int r0) {
    G = ge.G;
    blk = ge.blk;
    off = ge.off;
    S = ge.S;
    dBlk = ge.dBlk;
    gk = set;
    skip = im_min(ge.ns, ge.S);
    n = MapLlmBlockScatter::group_size(ge, gk);
    a = (int)fd_div(r0, dBlk);
    kb = a * G + gk;
    own_len = im_max(0, im_min(blk, S - kb * blk));
    qb0 = kb + G - off;
    if (off == 0) {
      ncols = n;
    } else {
      const int nbt = (int)fd_div(S + blk - 1, dBlk);  // blocks in the sequence, the last one maybe short
      int later = 0;
      if (qb0 < nbt) {
        const int cnt = (int)fd_div(nbt - 1 - qb0, ge.dG) + 1;  // blocks qb0, qb0 + G, ... below nbt
        const int last = qb0 + (cnt - 1) * G;
        later = (cnt - 1) * blk + im_min(blk, S - last * blk);
      }
      ncols = own_len + later;
    }
  }
  IM_HD int n_rows() const { return n; }
  IM_HD int n_cols() const { return ncols; }
  IM_HD int kpre() const { return 0; }
  IM_HD int row_pos(int t) const {
    const int b = (int)fd_div(t, dBlk);
    return (b * G + gk) * blk + (t - b * blk);
  }
  IM_HD int col_pos(int c) const {
    if (off == 0) return row_pos(c);
    if (c < own_len) return kb * blk + c;
    const int c2 = c - own_len;
    const int m = (int)fd_div(c2, dBlk);
    return (qb0 + m * G) * blk + (c2 - m * blk);
  }
  IM_HD int lo(int t) const { return off == 0 ? t : t - a * blk; }
  IM_HD int hi(int) const { return ncols - 1; }
  IM_HD int block_lo(int r0, int) const { return lo(r0); }
  IM_HD int block_hi(int, int) const { return ncols - 1; }
  IM_HD bool store(int pos) const { return pos >= skip; }
  static constexpr bool kBlockPredicate = false, kAccumulate = false;
  IM_HD bool sees(int, int) const { return true; }
};

// Keys of the per-token window with sinks: key j is seen by the queries j .. j + window - 1.
// Sinks (j < n_sink; seen by every later query) are not stored here.
struct KeyRowsWindowSink {
  int S, window, skip;
  static IM_HD int num_sets(const IntraGeom&) { return 1; }
  static IM_HD int max_rows(const IntraGeom& ge) { return ge.S; }
  IM_HD KeyRowsWindowSink(const IntraGeom& ge, int, int) {
    S = ge.S;
    window = ge.window;
    skip = im_min(ge.ns, ge.S);
  }
  IM_HD int n_rows() const { return S; }
  IM_HD int n_cols() const { return S; }
  IM_HD int kpre() const { return 0; }
  IM_HD int row_pos(int t) const { return t; }
  IM_HD int col_pos(int c) const { return c; }
  IM_HD int lo(int t) const { return t; }
  IM_HD int hi(int t) const { return (int)im_min64((int64_t)t + window - 1, S - 1); }
  IM_HD int block_lo(int r0, int) const { return r0; }
  IM_HD int block_hi(int, int r1) const { return hi(r1); }
  IM_HD bool store(int pos) const { return pos >= skip; }
  static constexpr bool kBlockPredicate = false, kAccumulate = false;
  IM_HD bool sees(int, int) const { return true; }
};

// The first ge.ns keys (LLM sinks; the text keys of the image patterns) against the queries of the
// whole sequence: every later query (CAUSAL) or every query.  set = chunk of ge.sink_chunk queries
// (chosen by the host so that the pass fills the GPU).  The results are partial sums over the chunk.
template <bool CAUSAL>
struct KeyRowsLeading {
  int S, ns, c0, c1;
  static IM_HD int num_sets(const IntraGeom& ge) { return (ge.S + ge.sink_chunk - 1) / ge.sink_chunk; }
  static IM_HD int max_rows(const IntraGeom& ge) { return im_min(ge.ns, ge.S); }
  IM_HD KeyRowsLeading(const IntraGeom& ge, int set, int) {
    S = ge.S;
    ns = im_min(ge.ns, ge.S);
    c0 = set * ge.sink_chunk;
    c1 = im_min(c0 + ge.sink_chunk, S);
  }
  IM_HD int n_rows() const { return ns; }
  IM_HD int n_cols() const { return S; }
  IM_HD int kpre() const { return 0; }
  IM_HD int row_pos(int t) const { return t; }
  IM_HD int col_pos(int c) const { return c; }
  IM_HD int lo(int t) const { return CAUSAL ? im_max(t, c0) : c0; }
  IM_HD int hi(int) const { return c1 - 1; }
  IM_HD int block_lo(int r0, int) const { return CAUSAL ? im_max(r0, c0) : c0; }
  IM_HD int block_hi(int, int) const { return c1 - 1; }
  IM_HD bool store(int) const { return true; }
  static constexpr bool kBlockPredicate = false, kAccumulate = false;
  IM_HD bool sees(int, int) const { return true; }
};
using KeyRowsSinks = KeyRowsLeading<true>;
using KeyRowsText = KeyRowsLeading<false>;

// Grid keys of group g of the image patterns (grid token (r, c) in group (r%2)*4 + c%4), against
// the queries of Scatter set g: its text chunk, then (unless TEXT_COLS_ONLY) its grid tokens; every
// pair is visible.  Scatter: dK / dV of the grid keys.  Gather 0: with TEXT_COLS_ONLY, what the text
// queries - which keep their Scatter rows - add to the grid keys' results of the window pass.
template <bool TEXT_COLS_ONLY>
struct KeyRowsImgGroup {
  MapImgScatter sc;
  static IM_HD int num_sets(const IntraGeom&) { return 8; }
  static IM_HD int max_rows(const IntraGeom& ge) { return ge.width * ge.width / 8; }
  IM_HD KeyRowsImgGroup(const IntraGeom& ge, int set, int) : sc(ge, set, 0, 0) {}
  IM_HD int n_rows() const { return sc.nimg; }
  IM_HD int n_cols() const { return TEXT_COLS_ONLY ? sc.chunk : sc.chunk + sc.nimg; }
  IM_HD int kpre() const { return 0; }
  IM_HD int row_pos(int t) const { return sc.imgpos(t); }
  IM_HD int col_pos(int c) const { return sc.qpos(c); }
  IM_HD int lo(int) const { return 0; }
  IM_HD int hi(int) const { return n_cols() - 1; }
  IM_HD int block_lo(int, int) const { return 0; }
  IM_HD int block_hi(int, int) const { return n_cols() - 1; }
  IM_HD bool store(int) const { return true; }
  static constexpr bool kBlockPredicate = false, kAccumulate = TEXT_COLS_ONLY;
  IM_HD bool sees(int, int) const { return true; }
};

// Grid keys of image Gather 0 against the grid queries.  Query patch (R, C) sees the grid rows
// win(R) .. win(R)+15 and columns win(C) .. win(C)+15, so key (r, c) is seen by whole 8x8 query
// patches: those with win(R) <= r < win(R)+16 and win(C) <= c < win(C)+16 - at most 3 x 3 of them
// around its own patch, 2 x 2 for a key away from the borders.  A set is a run of up to 4 key
// patches of one patch row (rows: patch after patch; inside a patch its upper 4 grid rows, then
// its lower 4, so that a wavefront owns 4 x 8 keys with few query patches between them); its
// columns are the query patches R-1 .. R+1 x C0-1 .. C0+4 (cut at the borders), 64 queries each,
// so a block of 32 columns lies inside one query patch and a row meets it entirely or not at all.
struct KeyRowsImgWindow {
  int W, T, np, Rk, Ck0, pk, Rlo, Clo, nR, nC;
  static constexpr int RUN = 4;
  static IM_HD int runs_per_row(const IntraGeom& ge) { return (ge.width / 8 + RUN - 1) / RUN; }
  static IM_HD int num_sets(const IntraGeom& ge) { return (ge.width / 8) * runs_per_row(ge); }
  static IM_HD int max_rows(const IntraGeom& ge) { return 64 * im_min(RUN, ge.width / 8); }
  IM_HD KeyRowsImgWindow(const IntraGeom& ge, int set, int) {
    W = ge.width;
    T = ge.text_len;
    np = W / 8;
    const int rpr = runs_per_row(ge);
    Rk = set / rpr;
    Ck0 = (set - Rk * rpr) * RUN;
    pk = im_min(RUN, np - Ck0);
    Rlo = im_max(Rk - 1, 0);
    Clo = im_max(Ck0 - 1, 0);
    nR = im_min(Rk + 1, np - 1) - Rlo + 1;
    nC = im_min(Ck0 + pk, np - 1) - Clo + 1;
  }
  IM_HD int n_rows() const { return 64 * pk; }
  IM_HD int n_cols() const { return 64 * nR * nC; }
  IM_HD int kpre() const { return 0; }
  IM_HD int key_r(int t) const { return 8 * Rk + ((t >> 3) & 7); }
  IM_HD int key_c(int t) const { return 8 * (Ck0 + (t >> 6)) + (t & 7); }
  IM_HD int row_pos(int t) const { return T + key_r(t) * W + key_c(t); }
  IM_HD int col_pos(int c) const {
    const int pi = c >> 6, u = c & 63;
    const int ri = pi / nC;
    return T + (8 * (Rlo + ri) + (u >> 3)) * W + 8 * (Clo + pi - ri * nC) + (u & 7);
  }
  IM_HD int lo(int) const { return 0; }
  IM_HD int hi(int) const { return n_cols() - 1; }
  IM_HD int block_lo(int, int) const { return 0; }
  IM_HD int block_hi(int, int) const { return n_cols() - 1; }
  IM_HD bool store(int) const { return true; }
  static constexpr bool kBlockPredicate = true, kAccumulate = false;
  IM_HD bool sees(int t, int c) const {
    const int pi = c >> 6, ri = pi / nC;
    const int wr = MapImgPatch::win_start(Rlo + ri, np), wc = MapImgPatch::win_start(Clo + pi - ri * nC, np);
    const int r = key_r(t), cc = key_c(t);
    return r >= wr && r < wr + 16 && cc >= wc && cc < wc + 16;
  }
};

}  // namespace intra
