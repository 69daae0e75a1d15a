// Computational Query Set (CQS) index maps and key bounds, shared by the gfx950 kernels and by
// the host-side model that the CPU tests walk.
//
// A "set" is a group of query tokens that share one packed key list.  Inside a set, queries are
// numbered tq = 0..nq-1 and keys tk = 0..nk-1 ("in-set indices"); qpos()/kpos() turn an in-set
// index into a token position of the (B, S, H, 128) tensors.  With hi = min(khi(tq), nk-1), query
// tq attends exactly the keys tk <= hi that are either below kpre() (a prefix every query of the
// set looks at, 0 for most maps) or at least klo(tq).  klo and khi are non-decreasing in tq for
// every pattern, which is what lets a wavefront classify a whole 32x32 score block as skipped /
// unmasked / partially masked from the bounds of its first and last query alone.
// A map is built for one row block of a set (constructor argument t0 = its first in-set query):
// the key numbering of some patterns depends on where the row block sits.
//
// Semantics follow the dense-mask specification of the reference:
//   LLM scatter   intra_attn/reference.py:14-17    index map csrc/flash_attn/src/gmem_tile.h:511,656
//   LLM gather1   intra_attn/reference.py:20-24    gmem_tile.h:847-864
//   LLM window    intra_attn/reference.py:27-32    csrc/flash_attn/src/flash_fwd_kernel.h:7008
//   image scatter intra_attn/reference.py:36-53    gmem_tile.h:286-340,388-389
//   image gather0 intra_attn/reference.py:56-74    gmem_tile.h:1220-1294,1334-1373
//   LLM block scatter (blocks, stripe offset, own block, sinks)  experiments/llm/llama_intra.py:93-110
//   LLM per-token window with sinks                             experiments/llm/llama_intra.py:57-72
// The maps here are re-derived from those predicates; nothing is shared with the reference code.
#pragma once
#include <stdint.h>

#if defined(__HIPCC__)
#define IM_HD __host__ __device__ __forceinline__
#else
#define IM_HD inline
#endif

// Pattern kinds used inside the library (the public pattern ids are per-entry-point).
enum IntraKind : int {
  KIND_LLM_SCATTER = 0,
  KIND_LLM_GATHER1 = 1,
  KIND_LLM_WINDOW = 2,
  KIND_IMG_SCATTER = 3,
  KIND_IMG_GATHER0 = 4,
  KIND_LLM_BLOCK_SCATTER = 5,
  KIND_LLM_WINDOW_SINK = 6,
};

// Division of a non-negative int below 2^31 by a divisor fixed per launch, as multiply-high and
// shift; the constants are worked out once on the host.
struct FastDiv {
  uint32_t d, mul, add, shift;
};
IM_HD uint32_t fd_div(uint32_t n, const FastDiv& f) {
  return ((uint32_t)(((uint64_t)n * f.mul) >> 32) + (f.add ? n : 0u)) >> f.shift;
}
IM_HD uint32_t fd_mod(uint32_t n, const FastDiv& f) { return n - fd_div(n, f) * f.d; }
inline FastDiv make_fastdiv(int d) {
  FastDiv f;
  f.d = (uint32_t)d;
  if (d <= 1) {  // n / 1 = (0 + n) >> 0
    f.d = 1;
    f.mul = 0;
    f.add = 1;
    f.shift = 0;
    return f;
  }
  int l = 0;
  while ((1ll << l) < d) ++l;  // 2^(l-1) < d <= 2^l
  // m = ceil(2^(31+l) / d) < 2^32 and floor(n * m / 2^(31+l)) = floor(n / d) for all n < 2^31
  f.mul = (uint32_t)((((uint64_t)1 << (31 + l)) + d - 1) / d);
  f.add = 0;
  f.shift = (uint32_t)(l - 1);
  return f;
}

struct IntraGeom {
  int S;         // tokens per sequence
  int G;         // LLM scatter / gather1 group count
  int window;    // LLM window width in keys (>= 64)
  int width;     // image latent grid side (tokens)
  int text_len;  // image: text tokens in front of the grid
  int text_only; // image scatter: only the text queries of each group (the text rows of gather0)
  int pg;        // image gather0: 8x8 patches per set (a run of pg patches in one patch row)
  int tm;        // image gather0, forward: text chunks (scatter groups) per set of text rows: 1 or 2
  int blk;       // LLM block scatter: tokens per block
  int off;       // LLM block scatter: stripe offset, 0 <= off < G
  int ns;        // LLM block scatter / window with sinks: leading tokens every query sees
  int sink_chunk;  // backward: queries per workgroup of the sink pass (a multiple of 64)
  // derived by geom_finish()
  FastDiv dG;        // / G
  FastDiv dWq;       // / (width / 4)
  FastDiv dPerRow;   // / ((width / 8) / pg)
  FastDiv dBlk;      // / blk
  int g1_full;       // gather1: (S / G^2) * G
  int g1_rem;        // gather1: S % G^2
};

inline void geom_finish(IntraGeom& ge) {
  ge.dG = make_fastdiv(ge.G);
  ge.dWq = make_fastdiv(ge.width / 4);
  ge.dPerRow = make_fastdiv((ge.width / 8) / (ge.pg > 0 ? ge.pg : 1));
  ge.dBlk = make_fastdiv(ge.blk);
  const long long gg = (long long)ge.G * ge.G;
  ge.g1_full = (int)((ge.S / gg) * ge.G);
  ge.g1_rem = (int)(ge.S % gg);
}

IM_HD int im_min(int a, int b) { return a < b ? a : b; }
IM_HD int im_max(int a, int b) { return a > b ? a : b; }
IM_HD int64_t im_min64(int64_t a, int64_t b) { return a < b ? a : b; }

// ---------------------------------------------------------------- LLM scatter: token i in group i % G
struct MapLlmScatter {
  static constexpr bool kHasPrefix = false;
  IM_HD int kpre() const { return 0; }
  int G, g, n;
  static IM_HD int num_sets(const IntraGeom& ge) { return ge.G; }
  static IM_HD int max_nq(const IntraGeom& ge) { return (ge.S + ge.G - 1) / ge.G; }
  IM_HD MapLlmScatter(const IntraGeom& ge, int set, int /*t0*/) {
    G = ge.G;
    g = set;
    n = ge.S > set ? (int)fd_div(ge.S - set + ge.G - 1, ge.dG) : 0;
  }
  IM_HD int nq() const { return n; }
  IM_HD int nk() const { return n; }
  IM_HD int qpos(int t) const { return t * G + g; }
  IM_HD int kpos(int t) const { return t * G + g; }
  IM_HD int klo(int) const { return 0; }
  IM_HD int khi(int tq) const { return tq; }
};

// ------------------------------------- LLM gather1: segments of G tokens, segment s in group s % G
// Token p = (G*G)*a + G*g + r (r < G) is in-set index G*a + r of group g; positions grow with the
// in-set index, so causality in positions equals causality in in-set indices.
struct MapLlmGather1 {
  static constexpr bool kHasPrefix = false;
  IM_HD int kpre() const { return 0; }
  int G, g, n;
  FastDiv dG;
  static IM_HD int num_sets(const IntraGeom& ge) { return ge.G; }
  static IM_HD int max_nq(const IntraGeom& ge) { return ge.g1_full + im_min(ge.G, ge.g1_rem); }
  IM_HD MapLlmGather1(const IntraGeom& ge, int set, int /*t0*/) {
    G = ge.G;
    g = set;
    dG = ge.dG;
    // g1_rem - G * g: tokens of this group in the last, partial G*G block
    n = ge.g1_full + im_max(0, im_min(G, ge.g1_rem - G * g));
  }
  IM_HD int nq() const { return n; }
  IM_HD int nk() const { return n; }
  IM_HD int qpos(int t) const {
    const int a = (int)fd_div(t, dG);
    return (a * G + g) * G + (t - a * G);
  }
  IM_HD int kpos(int t) const { return qpos(t); }
  IM_HD int klo(int) const { return 0; }
  IM_HD int khi(int tq) const { return tq; }
};

// -------------------------- LLM window: 64-query blocks see themselves plus window-64 earlier tokens
struct MapLlmWindow {
  static constexpr bool kHasPrefix = false;
  IM_HD int kpre() const { return 0; }
  int S, lookback;
  static IM_HD int num_sets(const IntraGeom&) { return 1; }
  static IM_HD int max_nq(const IntraGeom& ge) { return ge.S; }
  IM_HD MapLlmWindow(const IntraGeom& ge, int, int /*t0*/) {
    S = ge.S;
    lookback = ge.window - 64;
  }
  IM_HD int nq() const { return S; }
  IM_HD int nk() const { return S; }
  IM_HD int qpos(int t) const { return t; }
  IM_HD int kpos(int t) const { return t; }
  IM_HD int klo(int tq) const { return im_max((tq & ~63) - lookback, 0); }
  IM_HD int khi(int tq) const { return tq; }
};

// ------------- image scatter: 8 groups, grid token (r, c) in group (r%2)*4 + c%4, text chunk j rides
// with group j; every query sees all text keys plus the grid keys of its own group.
struct MapImgScatter {
  static constexpr bool kHasPrefix = false;
  IM_HD int kpre() const { return 0; }
  int W, T, chunk, j, a, b, wq, nimg, text_only;
  FastDiv dWq;
  static IM_HD int num_sets(const IntraGeom&) { return 8; }
  static IM_HD int max_nq(const IntraGeom& ge) {
    return ge.text_only ? ge.text_len / 8 : ge.text_len / 8 + ge.width * ge.width / 8;
  }
  IM_HD MapImgScatter(const IntraGeom& ge, int set, int /*t0*/, int only_text = -1) {
    W = ge.width;
    T = ge.text_len;
    chunk = T / 8;
    j = set;
    a = set >> 2;
    b = set & 3;
    wq = W / 4;
    nimg = W * W / 8;
    text_only = only_text < 0 ? ge.text_only : only_text;
    dWq = ge.dWq;
  }
  IM_HD int imgpos(int u) const {
    const int r = (int)fd_div(u, dWq);
    return T + (a + 2 * r) * W + b + 4 * (u - r * wq);
  }
  IM_HD int nq() const { return text_only ? chunk : chunk + nimg; }
  IM_HD int nk() const { return T + nimg; }
  IM_HD int qpos(int t) const { return t < chunk ? chunk * j + t : imgpos(t - chunk); }
  IM_HD int kpos(int t) const { return t < T ? t : imgpos(t - T); }
  IM_HD int klo(int) const { return 0; }
  IM_HD int khi(int) const { return T + nimg - 1; }
};

// Where the 64 keys of a tile sit when their positions are affine in the loader's coordinates: key
// 4 * g + r of the tile (row r of the 4-row group g a load instruction moves) is at position
// base + g * group_step + r * row_step.  A map that can tell (tile_rows) saves the loader the
// per-key index arithmetic for such tiles; the others answer no (map_tile_rows below), and so does
// any map for a tile that straddles two parts of its key list or its end.
struct TileRows {
  int base, group_step, row_step;
};


// ---- image gather0, grid queries: every 8x8 patch of grid queries sees all text plus a 16x16 grid
// window around it (shifted inwards at the borders).  A set is a run of pg patches of one patch
// row, so that the text keys (a prefix every query sees) and most of the window keys are shared.
// The window keys of the set are the union of the patches' windows, cut into blocks of 4 grid
// columns x 16 grid rows = 64 keys; window starts are multiples of 4, so a patch sees exactly 4
// consecutive blocks.  The text queries of gather0 keep their scatter rows (MapImgScatter in
// text_only mode); MapImgGather0 below puts both kinds of sets into one launch.
struct MapImgPatch {
  static constexpr bool kHasPrefix = true;
  int W, T, pg, np, R, C0, r0, cfirst, nblk;
  static IM_HD int win_start(int idx, int np) {
    if (idx == np - 1) return idx * 8 - 8;
    if (idx == 0) return 0;
    return idx * 8 - 4;
  }
  static IM_HD int num_sets(const IntraGeom& ge) { return (ge.width / 8) * ((ge.width / 8) / ge.pg); }
  static IM_HD int max_nq(const IntraGeom& ge) { return 64 * ge.pg; }
  IM_HD MapImgPatch(const IntraGeom& ge, int set, int /*t0*/) {
    W = ge.width;
    T = ge.text_len;
    pg = ge.pg;
    np = W / 8;
    R = (int)fd_div(set, ge.dPerRow);
    C0 = (set - R * (int)ge.dPerRow.d) * pg;
    r0 = win_start(R, np);
    cfirst = win_start(C0, np);
    nblk = (win_start(C0 + pg - 1, np) + 16 - cfirst) / 4;
  }
  IM_HD int nq() const { return 64 * pg; }
  IM_HD int nk() const { return T + 64 * nblk; }
  IM_HD int kpre() const { return T; }
  IM_HD int qpos(int t) const {
    const int w = t & 63;
    return T + (8 * R + (w >> 3)) * W + 8 * (C0 + (t >> 6)) + (w & 7);
  }
  IM_HD int kpos(int t) const {
    if (t < T) return t;
    const int u = t - T;
    return T + (r0 + ((u >> 2) & 15)) * W + cfirst + 4 * (u >> 6) + (u & 3);
  }
  IM_HD int klo(int tq) const { return T + 16 * (win_start(C0 + (tq >> 6), np) - cfirst); }
  IM_HD int khi(int tq) const { return klo(tq) + 255; }
  // A 64-key tile inside the text keys is 64 consecutive positions; one inside the window is a strip
  // of 4 columns by 16 rows.
  IM_HD bool tile_rows(int t_first, TileRows& a) const {
    if (t_first + 64 <= T) {
      a = TileRows{t_first, 4, 1};
      return true;
    }
    const int u = t_first - T;
    if (u < 0 || (u & 63) != 0 || t_first + 64 > nk()) return false;
    a = TileRows{T + r0 * W + cfirst + 4 * (u >> 6), W, 1};
    return true;
  }
};

// ---- image gather0, all rows: sets 0..7 are the text-only scatter sets (the longest work items,
// so they come first), sets 8.. the patch runs.
struct MapImgGather0 {
  static constexpr bool kHasPrefix = true;
  bool is_text;
  MapImgScatter sc;
  MapImgPatch pa;
  static IM_HD int num_sets(const IntraGeom& ge) { return 8 + MapImgPatch::num_sets(ge); }
  static IM_HD int max_nq(const IntraGeom& ge) { return im_max(ge.text_len / 8, MapImgPatch::max_nq(ge)); }
  IM_HD MapImgGather0(const IntraGeom& ge, int set, int t0)
      : is_text(set < 8), sc(ge, set < 8 ? set : 0, t0, 1), pa(ge, set < 8 ? 0 : set - 8, t0) {}
  IM_HD int nq() const { return is_text ? sc.nq() : pa.nq(); }
  IM_HD int nk() const { return is_text ? sc.nk() : pa.nk(); }
  IM_HD int kpre() const { return is_text ? 0 : pa.kpre(); }
  IM_HD int qpos(int t) const { return is_text ? sc.qpos(t) : pa.qpos(t); }
  IM_HD int kpos(int t) const { return is_text ? sc.kpos(t) : pa.kpos(t); }
  IM_HD int klo(int tq) const { return is_text ? 0 : pa.klo(tq); }
  IM_HD int khi(int tq) const { return is_text ? sc.khi(tq) : pa.khi(tq); }
};

// ---- The forward launch of image gather0 deals the text queries like this.  A scatter group has
// only text_len / 8 text queries (64 at 512 text tokens), a quarter of a row block, and they see
// the text keys and the group's grid keys; so the text chunks of tm = 1 or 2 groups share one row
// block (8 / tm sets of text rows per head).  With two groups A, B the key list is
// [grid keys of A][text keys][grid keys of B]: the queries of A see the first two parts, those of
// B the last two, each a contiguous range, and the text key tiles are loaded once for both.  A
// row block that holds one group's chunk only has the list [text keys][grid keys] of a scatter
// set.  (Image scatter keeps its text queries in front of the grid queries of their group,
// MapImgScatter: its key bounds are compile-time constants that way, which its main loop needs.)
struct MapImgTextRows {
  static constexpr bool kHasPrefix = false;
  IM_HD int kpre() const { return 0; }
  // (few fields: two of these maps are live in the kernel's main loop, in scalar registers)
  int W, T, nimg, nq_, lead, cA, cB, q0;
  FastDiv dWq;
  static IM_HD int num_sets(const IntraGeom& ge) { return 8 / ge.tm; }
  static IM_HD int max_nq(const IntraGeom& ge) { return ge.tm * (ge.text_len / 8); }
  IM_HD MapImgTextRows(const IntraGeom& ge, int set, int t0) {
    W = ge.width;
    T = ge.text_len;
    nimg = W * W / 8;
    dWq = ge.dWq;
    const int chunk = T / 8;
    const int first = ge.tm * set;
    const int g0 = ge.tm == 2 && t0 >= chunk ? 1 : 0;  // chunk of the row block's first query
    const int gA = first + g0;
    nq_ = ge.tm * chunk;
    q0 = first * chunk;
    lead = ge.tm - g0 == 2 ? nimg : 0;     // two groups: the grid keys of the first in front of the text keys
    cA = T + (gA >> 2) * W + (gA & 3);     // position of grid token 0 of group gA
    cB = cA + (lead ? 1 : 0);              // ... of the group whose grid keys follow the text keys
  }
  // Grid token u of scatter group g sits at row g / 4 + 2 * (u / (W/4)), column g % 4 + 4 * (u % (W/4)):
  // position T + (g / 4) * W + g % 4 + 4 * u + (u / (W/4)) * W.  Groups gA and gA + 1 of a two-group
  // list differ by one column.
  IM_HD int grid(int c0, int u) const { return c0 + 4 * u + (int)fd_div(u, dWq) * W; }
  IM_HD int nq() const { return nq_; }
  IM_HD int nk() const { return T + lead + nimg; }
  IM_HD int qpos(int t) const { return q0 + t; }
  IM_HD int kpos(int t) const {  // (runs per fetched key row: two compares, no mask arithmetic)
    const unsigned tt = (unsigned)(t - lead);  // index behind the leading part (huge inside it): text, then grid
    const bool front = t < lead;
    const int p = grid(front ? cA : cB, front ? t : (int)tt - T);
    return tt < (unsigned)T ? (int)tt : p;
  }
  // with two groups the queries of the second chunk start behind the first group's grid keys
  IM_HD int klo(int tq) const { return 8 * tq >= T ? lead : 0; }
  IM_HD int khi(int tq) const { return klo(tq) + T + nimg - 1; }
};

// image gather0, forward launch: the text rows, then the patch runs
struct MapImgGather0F {
  static constexpr bool kHasPrefix = true;
  bool is_text;
  MapImgTextRows tx;
  MapImgPatch pa;
  static IM_HD int num_sets(const IntraGeom& ge) { return MapImgTextRows::num_sets(ge) + MapImgPatch::num_sets(ge); }
  static IM_HD int max_nq(const IntraGeom& ge) { return im_max(MapImgTextRows::max_nq(ge), MapImgPatch::max_nq(ge)); }
  IM_HD MapImgGather0F(const IntraGeom& ge, int set, int t0)
      : is_text(set < 8 / ge.tm), tx(ge, is_text ? set : 0, t0), pa(ge, is_text ? 0 : set - 8 / ge.tm, t0) {}
  IM_HD int nq() const { return is_text ? tx.nq() : pa.nq(); }
  IM_HD int nk() const { return is_text ? tx.nk() : pa.nk(); }
  IM_HD int kpre() const { return is_text ? 0 : pa.kpre(); }
  IM_HD int qpos(int t) const { return is_text ? tx.qpos(t) : pa.qpos(t); }
  IM_HD int kpos(int t) const { return is_text ? tx.kpos(t) : pa.kpos(t); }
  IM_HD int klo(int tq) const { return is_text ? tx.klo(tq) : pa.klo(tq); }
  IM_HD int khi(int tq) const { return is_text ? tx.khi(tq) : pa.khi(tq); }
  IM_HD bool tile_rows(int t_first, TileRows& a) const { return !is_text && pa.tile_rows(t_first, a); }
};

// tile_rows of a map that has one, else false
template <class MAP>
IM_HD auto map_tile_rows_(const MAP& map, int t_first, TileRows& a, int) -> decltype(map.tile_rows(t_first, a)) {
  return map.tile_rows(t_first, a);
}
template <class MAP>
IM_HD bool map_tile_rows_(const MAP&, int, TileRows&, long) { return false; }
template <class MAP>
IM_HD bool map_tile_rows(const MAP& map, int t_first, TileRows& a) { return map_tile_rows_(map, t_first, a, 0); }

// ------- LLM block scatter: blocks of blk tokens, block b in group b % G.  A query of block qb sees,
// causally, the blocks of group (qb + off) % G, the first ns tokens ("sinks", ns <= blk) and, when
// off != 0, its own block.  The key list of a row block is numbered
//   [sinks, unless the next part starts with them] [blocks of the target group] [own block, off != 0]
// where the own block follows the last target block in front of it, so that every query sees the
// contiguous range 0..khi.  With off != 0 the numbering depends on the query block, hence row
// blocks must not straddle query blocks (the host picks the row-block size accordingly).
struct MapLlmBlockScatter {
  static constexpr bool kHasPrefix = false;
  IM_HD int kpre() const { return 0; }
  int G, blk, g, gt, off, n, E, own_base, own_len, qb;
  FastDiv dBlk;
  static IM_HD int group_size(const IntraGeom& ge, int g) {  // tokens in blocks b = g (mod G)
    const int nb = (int)fd_div(ge.S, ge.dBlk);               // full blocks
    const int tail = ge.S - nb * ge.blk;
    const int full = nb > g ? (int)fd_div(nb - 1 - g, ge.dG) + 1 : 0;
    return full * ge.blk + ((tail > 0 && (int)fd_mod(nb, ge.dG) == g) ? tail : 0);
  }
  static IM_HD int num_sets(const IntraGeom& ge) { return ge.G; }
  static IM_HD int max_nq(const IntraGeom& ge) {
    int m = 0;
    for (int g = 0; g < ge.G; ++g) m = im_max(m, group_size(ge, g));
    return m;
  }
  IM_HD MapLlmBlockScatter(const IntraGeom& ge, int set, int t0) {
    G = ge.G;
    blk = ge.blk;
    off = ge.off;
    dBlk = ge.dBlk;
    g = set;
    gt = g + off >= G ? g + off - G : g + off;  // target group
    n = group_size(ge, g);
    const int a = (int)fd_div(t0, dBlk);         // query block of the row block, within the group
    qb = a * G + g;
    const int ns = im_min(ge.ns, ge.S);
    own_len = im_max(0, im_min(blk, ge.S - qb * blk));  // tokens the own block really has
    if (off == 0) {
      E = g == 0 ? 0 : ns;
      own_base = 0x7fffffff;                     // no own-block part
    } else {
      E = (gt == 0 || qb == 0) ? 0 : ns;         // block 0 is in front already / is the own block
      own_base = E + (a + (gt < g ? 1 : 0)) * blk;
    }
  }
  IM_HD int nq() const { return n; }
  IM_HD int nk() const { return off == 0 ? E + n : own_base + own_len; }
  IM_HD int qpos(int t) const {
    const int a = (int)fd_div(t, dBlk);
    return (a * G + g) * blk + (t - a * blk);
  }
  IM_HD int kpos(int t) const {
    if (t < E) return t;
    if (t >= own_base) return qb * blk + (t - own_base);
    const int c = t - E;
    const int m = (int)fd_div(c, dBlk);
    return (m * G + gt) * blk + (c - m * blk);
  }
  IM_HD int klo(int) const { return 0; }
  IM_HD int khi(int tq) const {
    if (off == 0) return E + tq;
    return own_base + (tq - (int)fd_div(tq, dBlk) * blk);
  }
};

// ------- LLM per-token sliding window with sinks: query i sees the keys j <= i with i - j < window
// or j < ns.  One set; the key list of a row block is numbered [sinks][positions wlo, wlo+1, ...]
// with wlo = the first position outside the sinks that its first query sees, so that tiles start
// at the window and not at position 0.
struct MapLlmWindowSink {
  static constexpr bool kHasPrefix = true;
  int S, window, ns, wlo;
  static IM_HD int num_sets(const IntraGeom&) { return 1; }
  static IM_HD int max_nq(const IntraGeom& ge) { return ge.S; }
  IM_HD MapLlmWindowSink(const IntraGeom& ge, int, int t0) {
    S = ge.S;
    window = ge.window;
    ns = im_min(ge.ns, ge.S);
    wlo = im_max(t0 - window + 1, ns);
  }
  IM_HD int nq() const { return S; }
  IM_HD int nk() const { return ns + (S - wlo); }
  IM_HD int kpre() const { return ns; }
  IM_HD int qpos(int t) const { return t; }
  IM_HD int kpos(int t) const { return t < ns ? t : wlo + (t - ns); }
  IM_HD int klo(int tq) const { return ns + im_max(tq - window + 1, wlo) - wlo; }
  IM_HD int khi(int tq) const { return tq < ns ? tq : ns + (tq - wlo); }
};

// --------------------------------------------------------------------------- block classification
// A wavefront owns the queries wq0..wq_last of a set.
struct WaveBounds {
  int w_lo, w_hi;  // union of the [klo, hi] ranges of the wavefront's queries
  int f_lo, f_hi;  // intersection of them
};

template <class MAP>
IM_HD WaveBounds wave_bounds(const MAP& map, int wq0, int wq_last) {
  int kmax = map.nk() - 1;
  WaveBounds wb;
  wb.w_lo = map.klo(wq0);
  wb.w_hi = im_min(map.khi(wq_last), kmax);
  wb.f_lo = map.klo(wq_last);
  wb.f_hi = im_min(map.khi(wq0), kmax);
  return wb;
}

// Does the wavefront look at the 32 keys sb_lo..sb_lo+31 at all, and can it skip the mask?
IM_HD bool block_wanted(const WaveBounds& wb, int kpre, int sb_lo) {
  return sb_lo <= wb.w_hi && (sb_lo < kpre || sb_lo + 31 >= wb.w_lo);
}
IM_HD bool block_unmasked(const WaveBounds& wb, int kpre, int sb_lo) {
  return sb_lo + 31 <= wb.f_hi && (sb_lo + 31 < kpre || (sb_lo >= kpre && sb_lo >= wb.f_lo));
}
IM_HD bool key_visible(int key, int kpre, int lo, int hi) { return key <= hi && (key < kpre || key >= lo); }

// Host walk of the kernel's decomposition for one index map: sets -> row blocks of nw * 32 / hp
// in-set queries -> wavefronts -> key tiles of `tile_keys` keys -> 32-key blocks, with the same block
// tests and per-element bound test as the device code.  Adds 1 (saturating) to
// count[q_pos * S + k_pos] for every score the kernel computes and keeps; `count` holds S * S bytes.
// Host only: what the library's intra_model_mask* entry points run, and what a sanitizer build of
// this header checks for out-of-range positions and integer overflow.
template <class MAP>
inline void im_model_walk(const IntraGeom& ge, int hp, int nw, int tile_keys, uint8_t* count) {
  const int pos = nw * 32 / hp;
  const int S = ge.S;
  const int n_sets = MAP::num_sets(ge);
  const int n_mblocks = (MAP::max_nq(ge) + pos - 1) / pos;
  for (int set = 0; set < n_sets; ++set) {
    for (int mblk = 0; mblk < n_mblocks; ++mblk) {
      const int t0 = mblk * pos;
      const MAP map(ge, set, t0);
      const int nq = map.nq(), nk = map.nk(), kpre = map.kpre();
      if (t0 >= nq) continue;
      const int t1 = im_min(t0 + pos, nq) - 1;
      const int kt_lo = MAP::kHasPrefix ? 0 : map.klo(t0);
      const int kt_hi = im_min(map.khi(t1), nk - 1);
      const int ntiles = (kt_hi - kt_lo + tile_keys) / tile_keys;
      for (int pw = 0; pw < pos / 32; ++pw) {  // the wavefronts of one head
        const int wq0 = t0 + pw * 32;
        if (wq0 > t1) continue;
        const int wq_last = im_min(wq0 + 31, t1);
        const WaveBounds wb = wave_bounds(map, wq0, wq_last);
        for (int blk = 0; blk < (tile_keys / 32) * ntiles; ++blk) {
          const int sb_lo = kt_lo + 32 * blk;
          if (!block_wanted(wb, kpre, sb_lo)) continue;
          const bool unmasked = block_unmasked(wb, kpre, sb_lo);
          for (int l = 0; l < 32; ++l) {
            if (wq0 + l > t1) continue;  // rows the kernel computes but never stores
            const int tq = wq0 + l;
            const int lo = map.klo(tq), hi = im_min(map.khi(tq), nk - 1);
            for (int e = 0; e < 32; ++e) {
              const int key = sb_lo + e;
              if (!unmasked && !key_visible(key, kpre, lo, hi)) continue;
              // an unmasked block keeps every element: clamp the loaded row like the loader does
              const int tk = im_min(key, nk - 1);
              const int64_t qp = map.qpos(tq), kp = map.kpos(tk);
              uint8_t& c8 = count[qp * S + kp];
              if (c8 < 255) ++c8;
            }
          }
        }
      }
    }
  }
}
