// C ABI of libintra_hip.so: validation, launch planning and dispatch.  See include/intra_hip.h.
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdarg.h>
#include <stdio.h>
#include <stdlib.h>
#include <string.h>

#include <algorithm>
#include <atomic>
#include <type_traits>

#include "../../include/intra_hip.h"
#include "intra_kernel_narrow.hip.h"
#include "intra_bwd_kernel.hip.h"
#include "intra_diag.hip.h"

namespace {

thread_local char g_err[512] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

struct Request {
  int kind;
  int B, S, H, Hkv;
  IntraGeom geom;
};

// Translate the public (domain, pattern, args) triple and check everything that does not need
// pointers.  Mirrors the checks of intra_attn/interface.py:41-42,60-63 and
// csrc/flash_attn/flash_api.cpp:576-612 where they still apply.
int make_request(int domain, int pattern, int B, int S, int H, int Hkv, int arg0, int arg1,
                 Request* r, int block = 0, int offset = 0, int n_sink = 0, bool extended = false) {
  if (B < 1 || S < 1 || H < 1 || Hkv < 1)
    return fail(INTRA_ERR_INVALID, "B, S, H, Hkv must be positive (got %d, %d, %d, %d)", B, S, H, Hkv);
  if (H % Hkv != 0)
    return fail(INTRA_ERR_INVALID, "query heads (%d) must be a multiple of kv heads (%d)", H, Hkv);
  r->B = B;
  r->S = S;
  r->H = H;
  r->Hkv = Hkv;
  r->geom = IntraGeom{S, 1, 64, 16, 8, 0, 1, 1, 64, 0, 0};  // derived fields: geom_finish() in shape_for()
  r->geom.sink_chunk = 1024;  // backward: set by leading_chunk() once the number of leading keys is known
  if (domain == 0) {
    if (!extended && (pattern == INTRA_LLM_BLOCK_SCATTER || pattern == INTRA_LLM_WINDOW_SINK))
      return fail(INTRA_ERR_INVALID, "unknown LLM pattern id %d (0 scatter, 1 gather1, 4 window)", pattern);
    if (pattern == INTRA_LLM_SCATTER || pattern == INTRA_LLM_GATHER1) {
      if (arg0 < 1) return fail(INTRA_ERR_INVALID, "group_num must be >= 1 (got %d)", arg0);
      if (arg0 > 32768) return fail(INTRA_ERR_INVALID, "group_num too large (%d)", arg0);
      r->geom.G = arg0;
      r->kind = pattern == INTRA_LLM_SCATTER ? KIND_LLM_SCATTER : KIND_LLM_GATHER1;
    } else if (pattern == INTRA_LLM_WINDOW) {
      if (arg1 < 64)
        return fail(INTRA_ERR_INVALID,
                    "window must be >= 64: every 64-query block sees itself (got %d)", arg1);
      r->geom.window = arg1;
      r->kind = KIND_LLM_WINDOW;
    } else if (pattern == INTRA_LLM_BLOCK_SCATTER) {
      if (arg0 < 1 || arg0 > 32768) return fail(INTRA_ERR_INVALID, "group_num must be in [1, 32768] (got %d)", arg0);
      if (block < 64 || block % 64 != 0)
        return fail(INTRA_ERR_INVALID, "block must be a positive multiple of 64 (got %d)", block);
      if (offset < 0 || offset >= arg0)
        return fail(INTRA_ERR_INVALID, "offset must be in [0, group_num) (got %d)", offset);
      if (n_sink < 0 || n_sink > block)
        return fail(INTRA_ERR_INVALID, "n_sink must be in [0, block] (got %d)", n_sink);
      r->geom.G = arg0;
      r->geom.blk = block;
      r->geom.off = offset;
      r->geom.ns = n_sink;
      r->kind = KIND_LLM_BLOCK_SCATTER;
    } else if (pattern == INTRA_LLM_WINDOW_SINK) {
      if (arg1 < 1) return fail(INTRA_ERR_INVALID, "window must be >= 1 (got %d)", arg1);
      if (n_sink < 0) return fail(INTRA_ERR_INVALID, "n_sink must be >= 0 (got %d)", n_sink);
      r->geom.window = arg1;
      r->geom.ns = n_sink;
      r->kind = KIND_LLM_WINDOW_SINK;
    } else {
      return fail(INTRA_ERR_INVALID,
                  "unknown LLM pattern id %d (0 scatter, 1 gather1, 4 window, 8 block scatter, 9 window with sinks)",
                  pattern);
    }
  } else if (domain == 1) {
    if (pattern != INTRA_IMAGE_SCATTER && pattern != INTRA_IMAGE_GATHER0)
      return fail(INTRA_ERR_INVALID, "unknown image pattern id %d (0 scatter, 4 gather0)", pattern);
    if (arg0 < 16 || arg0 % 8 != 0 || arg0 > 4096)
      return fail(INTRA_ERR_INVALID, "width must be a multiple of 8 in [16, 4096] (got %d)", arg0);
    if (arg1 < 8 || arg1 % 8 != 0)
      return fail(INTRA_ERR_INVALID, "text_len must be a positive multiple of 8 (got %d)", arg1);
    if ((int64_t)S != (int64_t)arg1 + (int64_t)arg0 * arg0)
      return fail(INTRA_ERR_INVALID, "expected %d text + %dx%d image tokens, got %d", arg1, arg0, arg0, S);
    r->geom.width = arg0;
    r->geom.text_len = arg1;
    r->kind = pattern == INTRA_IMAGE_SCATTER ? KIND_IMG_SCATTER : KIND_IMG_GATHER0;
  } else {
    return fail(INTRA_ERR_INVALID, "unknown domain %d (0 LLM, 1 image)", domain);
  }
  return INTRA_OK;
}

// The kernel launch of a request: an index map, its geometry and the workgroup shape (HP query heads
// of one kv head share a workgroup of NW wavefronts, so a row block has NW * 32 / HP in-set queries).
enum MapId : int {
  MAP_LLM_SCATTER, MAP_LLM_GATHER1, MAP_LLM_WINDOW, MAP_IMG_SCATTER, MAP_LLM_BLOCK_SCATTER,
  MAP_LLM_WINDOW_SINK, MAP_IMG_GATHER0
};
struct Shape {
  int map;
  IntraGeom geom;
  int hp, nw;
};

int default_hp(int ratio) { return ratio % 4 == 0 ? 4 : (ratio % 2 == 0 ? 2 : 1); }

// Every pattern is one launch of 8-wavefront workgroups.  Image gather0 runs its grid queries as
// sets of `pg` neighbouring 8x8 patches (as many as fit into a row block) and its text queries -
// which see what the scatter pattern shows them - as sets of the same launch, the text chunks of
// one or two scatter groups each (MapImgTextRows, pick_text_merge).
// Text chunks per set of text rows of image gather0 (IntraGeom::tm).  Two chunks in one row block
// share the text key tiles, but the item then walks through the grid keys of both groups with a
// quarter of the wavefronts busy, and the static dealing of work items wants items of about one
// size: 2 if the estimated cost stays within 15 % of a patch item's, else 1.  A key tile with w of
// 8 wavefronts busy is taken to cost 5/9 + w/18 of a full one (2/3 at w = 2, measured).
int pick_text_merge(const IntraGeom& ge, int pos, int pg, int nw) {
  const int chunk = ge.text_len / 8, nimg = ge.width * ge.width / 8;
  if (chunk % 32 != 0 || 2 * chunk > pos) return 1;  // (more chunks than a row block holds share nothing)
  auto busy = [nw](int w) { return 5.0 / 9 + std::min(w, nw) * (8 / nw) / 18.0; };
  const double patch_item = (ge.text_len + 16 * (16 + 8 * (pg - 1))) / 64.0;
  const double cost = ge.text_len / 64.0 * busy(2 * chunk / 32) + 2 * (nimg / 64.0) * busy(chunk / 32);
  return cost <= 1.15 * patch_item ? 2 : 1;
}

bool shape_for(const Request& r, int hp, Shape* ph, int nw = 8) {  // false: no kernel shape fits
  ph->geom = r.geom;
  ph->hp = hp;
  ph->nw = nw;
  switch (r.kind) {
    case KIND_LLM_SCATTER: ph->map = MAP_LLM_SCATTER; break;
    case KIND_LLM_GATHER1: ph->map = MAP_LLM_GATHER1; break;
    case KIND_LLM_WINDOW: ph->map = MAP_LLM_WINDOW; break;
    case KIND_IMG_SCATTER: ph->map = MAP_IMG_SCATTER; break;
    case KIND_LLM_WINDOW_SINK: ph->map = MAP_LLM_WINDOW_SINK; break;
    case KIND_LLM_BLOCK_SCATTER:
      // with a stripe offset a row block (256 / hp queries) has to stay inside one query block
      ph->map = MAP_LLM_BLOCK_SCATTER;
      if (r.geom.off != 0 && r.geom.blk % (nw * 32 / hp) != 0) return false;
      break;
    default: {
      const int np = r.geom.width / 8;
      if (nw * 32 / hp < 64) return false;  // a row block holds whole patches
      int pg = (nw * 32 / hp) / 64;
      while (np % pg != 0) --pg;
      ph->map = MAP_IMG_GATHER0;
      ph->geom.pg = pg;
      ph->geom.tm = pick_text_merge(r.geom, nw * 32 / hp, pg, nw);
    }
  }
  geom_finish(ph->geom);
  return true;
}

struct LaunchDims {
  int pos, n_sets, n_mblocks, hgroups, n_pairs, work_items;
};

template <class MAP>
LaunchDims dims_of(const Request& r, const Shape& ph) {
  LaunchDims d;
  d.pos = ph.nw * 32 / ph.hp;
  d.n_sets = MAP::num_sets(ph.geom);
  d.n_mblocks = (MAP::max_nq(ph.geom) + d.pos - 1) / d.pos;
  d.hgroups = (r.H / r.Hkv) / ph.hp;
  const int64_t n_pairs = (int64_t)r.B * r.Hkv * d.n_sets;
  const int64_t items = 8 * ((n_pairs + 7) / 8) * d.hgroups * d.n_mblocks;
  d.n_pairs = n_pairs > 0x7fffffff ? -1 : (int)n_pairs;
  d.work_items = items > 0x7fffffff ? -1 : (int)items;
  return d;
}

template <class MAP>
int64_t pairs_of(const IntraGeom& ge) {
  int64_t pairs = 0;
  const int n_sets = MAP::num_sets(ge);
  for (int set = 0; set < n_sets; ++set) {
    const int nq = MAP(ge, set, 0).nq();
    for (int tq = 0; tq < nq; ++tq) {
      const MAP map(ge, set, tq & ~63);  // a row block of 64 queries starting at a multiple of 64
      const int hi = im_min(map.khi(tq), map.nk() - 1), kpre = map.kpre();
      const int lo = im_max(map.klo(tq), kpre);
      pairs += im_min(kpre, hi + 1) + (hi >= lo ? hi - lo + 1 : 0);
    }
  }
  return pairs;
}

template <template <class> class F, class... A>
auto by_map(int map, A&&... a) {
  switch (map) {
    case MAP_LLM_SCATTER: return F<MapLlmScatter>::go(a...);
    case MAP_LLM_GATHER1: return F<MapLlmGather1>::go(a...);
    case MAP_LLM_WINDOW: return F<MapLlmWindow>::go(a...);
    case MAP_IMG_SCATTER: return F<MapImgScatter>::go(a...);
    case MAP_LLM_BLOCK_SCATTER: return F<MapLlmBlockScatter>::go(a...);
    case MAP_LLM_WINDOW_SINK: return F<MapLlmWindowSink>::go(a...);
    default: return F<MapImgGather0F>::go(a...);
  }
}
template <class MAP> struct DimsOf { static LaunchDims go(const Request& r, const Shape& ph) { return dims_of<MAP>(r, ph); } };
template <class MAP> struct PairsOf { static int64_t go(const IntraGeom& ge) { return pairs_of<MAP>(ge); } };

// CUs of the current device (cached per device; -1 if it cannot be asked)
int cu_count() {
  static std::atomic<int> cus[64];  // 0 = not asked yet (same answer from every thread)
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return -1;
  int n = cus[dev].load(std::memory_order_relaxed);
  if (n == 0) {
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) return -1;
    cus[dev].store(n, std::memory_order_relaxed);
  }
  return n;
}

// Wavefronts per workgroup of a forward launch.  Half-size workgroups, two per CU, pay for every key
// tile twice as often per query (measured: 7 % on the long rows of LLM Scatter), and gain where the
// work items are short or few:
//  * image gather0 (short items, and the wavefronts of one use different key tiles: the two
//    workgroups of a CU fill each other's waits): 0.0775 -> 0.0694 ms at 1024^2, 0.266 -> 0.235 at 2048^2;
//  * launches with so few row blocks that the CU with the most work gets at least a fifth less of it
//    when the blocks are half as large (8 kv heads at S <= 1024: 22 -> 18 us; image scatter at
//    1024^2, whose 576 row blocks of 256 queries are 2.25 per CU).
// The environment variable INTRA_WAVES (4 or 8) overrides the choice for measurements, where the
// shape exists.
int pick_waves(const Request& r, int hp) {
  Shape narrow, wide;
  if (!shape_for(r, hp, &narrow, intra::NARROW_WAVES)) return 8;
  if (!shape_for(r, hp, &wide, 8)) return intra::NARROW_WAVES;  // (block scatter with an offset: smaller row blocks fit smaller blocks)
  if (const char* e = getenv("INTRA_WAVES")) {
    const int n = atoi(e);
    if (n == 8 || n == intra::NARROW_WAVES) return n;
  }
  if (r.kind == KIND_IMG_GATHER0) return intra::NARROW_WAVES;
  int cus = cu_count();
  if (cus <= 0) cus = 256;  // (planning without a device)
  const int64_t items8 = by_map<DimsOf>(wide.map, r, wide).work_items, items4 = by_map<DimsOf>(narrow.map, r, narrow).work_items;
  if (items8 <= 0 || items4 <= 0) return 8;
  const int64_t share8 = 2 * ((items8 + cus - 1) / cus), share4 = (items4 + cus - 1) / cus;  // in half-size items
  return 5 * share4 <= 4 * share8 ? intra::NARROW_WAVES : 8;
}

int plan_for(const Request& r, int hp, IntraPlan* plan) {
  Shape ph;
  if (!shape_for(r, hp, &ph, pick_waves(r, hp)))
    return fail(INTRA_ERR_UNSUPPORTED, "block size does not fit the row blocks of this head layout");
  const LaunchDims d = by_map<DimsOf>(ph.map, r, ph);
  plan->kind = r.kind;
  plan->heads_per_block = ph.hp;
  plan->waves = ph.nw;
  plan->pos_per_block = d.pos;
  plan->n_sets = d.n_sets;
  plan->n_mblocks = d.n_mblocks;
  plan->launches = 1;
  plan->lds_bytes = ph.nw == intra::NARROW_WAVES ? intra::NARROW_LDS_BYTES : intra::LDS_BYTES;
  plan->work_items = d.work_items;
  plan->grid = plan->work_items;  // upper bound; a launch uses min(its work items, 8 * (CUs / 8))
  plan->pairs_per_head = by_map<PairsOf>(ph.map, ph.geom);
  return INTRA_OK;
}

template <class MAP> struct ModelWalk {
  static int go(const IntraGeom& ge, int hp, int nw, uint8_t* count) { im_model_walk<MAP>(ge, hp, nw, intra::BN, count); return 0; }
};

// Host enumeration of the dealing: every workgroup of a grid asks locate_item for its items, round
// after round, like the kernels do.
template <class MAP, int POS>
void deal_walk(const intra::KParams& p, int grid, int n_mblocks, uint8_t* visits) {
  const int cols = grid / 8;
  for (int wg = 0; wg < grid; ++wg) {
    intra::Where w;
    for (int round = 0; intra::locate_item<MAP, POS, false>(p, wg & 7, cols, wg >> 3, nullptr, round, w); round = w.round + 1) {
      const int64_t pair = ((int64_t)w.set * p.B + w.batch) * p.Hkv + w.kvh;
      uint8_t& c = visits[(pair * n_mblocks + w.mblk) * p.hgroups + w.hg];
      if (c < 255) ++c;
    }
  }
}
template <class MAP> struct DealWalk {
  static int go(const intra::KParams& p, int pos, int grid, int n_mblocks, uint8_t* visits) {
    switch (pos) {
      case 32: deal_walk<MAP, 32>(p, grid, n_mblocks, visits); break;
      case 64: deal_walk<MAP, 64>(p, grid, n_mblocks, visits); break;
      case 128: deal_walk<MAP, 128>(p, grid, n_mblocks, visits); break;
      default: deal_walk<MAP, 256>(p, grid, n_mblocks, visits); break;
    }
    return 0;
  }
};

// Persistent workgroups, as many as the CUs hold at once (LDS allows one of 8 wavefronts or two of
// 4 per CU), in multiples of the 8 XCDs.
int launch_grid(int work_items, int nw) {
  const int n = cu_count();
  if (n <= 0) return -1;
  int g = (n / 8) * 8;
  if (g < 8) g = 8;
  g *= 8 / nw;
  return work_items < g ? work_items : g;
}

template <class MAP, int HP, int NW, int SM>
int launch(const intra::KParams& p, int grid, hipStream_t stream) {
  hipLaunchKernelGGL((intra::intra_fwd_kernel<MAP, HP, NW, SM>), dim3(grid), dim3(NW * 64), 0, stream, p);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(INTRA_ERR_HIP, "kernel launch failed: %s", hipGetErrorString(e));
  return INTRA_OK;
}

template <class MAP, int HP>
int launch_sm(const intra::KParams& p, int sm, int grid, hipStream_t stream) {
  switch (sm) {
    case intra::SM_SCALED: return launch<MAP, HP, 8, intra::SM_SCALED>(p, grid, stream);
    case intra::SM_FOLDED: return launch<MAP, HP, 8, intra::SM_FOLDED>(p, grid, stream);
    default: return launch<MAP, HP, 8, intra::SM_EXACT>(p, grid, stream);
  }
}

template <class MAP, int HP, int SM>
int launch_narrow(const intra::KParams& p, int grid, hipStream_t stream) {
  hipLaunchKernelGGL((intra::intra_fwd_kernel_narrow<MAP, HP, SM>), dim3(grid), dim3(intra::NARROW_WAVES * 64), 0, stream, p);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(INTRA_ERR_HIP, "kernel launch failed: %s", hipGetErrorString(e));
  return INTRA_OK;
}

template <class MAP, int HP>
int launch_narrow_sm(const intra::KParams& p, int sm, int grid, hipStream_t stream) {
  switch (sm) {
    case intra::SM_SCALED: return launch_narrow<MAP, HP, intra::SM_SCALED>(p, grid, stream);
    case intra::SM_FOLDED: return launch_narrow<MAP, HP, intra::SM_FOLDED>(p, grid, stream);
    default: return launch_narrow<MAP, HP, intra::SM_EXACT>(p, grid, stream);
  }
}

template <class MAP>
struct LaunchMap {
  static int go(const intra::KParams& p, int hp, int nw, int sm, int grid, hipStream_t stream) {
    if (nw == 8) {
      switch (hp) {
        case 4: return launch_sm<MAP, 4>(p, sm, grid, stream);
        case 2: return launch_sm<MAP, 2>(p, sm, grid, stream);
        case 1: return launch_sm<MAP, 1>(p, sm, grid, stream);
      }
    } else if (nw == intra::NARROW_WAVES) {
      switch (hp) {
        case 4: return launch_narrow_sm<MAP, 4>(p, sm, grid, stream);
        case 2: return launch_narrow_sm<MAP, 2>(p, sm, grid, stream);
        case 1: return launch_narrow_sm<MAP, 1>(p, sm, grid, stream);
      }
    }
    return fail(INTRA_ERR_UNSUPPORTED, "no kernel for heads_per_block=%d, waves=%d", hp, nw);
  }
};

// Device buffer of the phase timers of an INTRA_DIAG_TIMERS build (intra_diag_set_buffer)
std::atomic<long long*> g_diag{nullptr};
std::atomic<int64_t> g_diag_values{0};

// What a call that names no softmax arithmetic gets (INTRA_SOFTMAX_* values; 0 = by softmax_scale,
// see pick_softmax).  Starts from the environment variable INTRA_SOFTMAX (auto / exact / folded /
// scaled; "fast" is the older name of folded).
std::atomic<int>& softmax_mode() {
  static std::atomic<int> mode{[] {
    const char* e = getenv("INTRA_SOFTMAX");
    if (e && !strcmp(e, "exact")) return (int)INTRA_SOFTMAX_EXACT;
    if (e && (!strcmp(e, "folded") || !strcmp(e, "fast"))) return (int)INTRA_SOFTMAX_FOLDED;
    if (e && !strcmp(e, "scaled")) return (int)INTRA_SOFTMAX_SCALED;
    return (int)INTRA_SOFTMAX_AUTO;
  }()};
  return mode;
}

// The kernel's softmax arithmetic for a call: what its flags name, else the process default.  Auto
// takes SCALED - fp32 scores times scale like the reference, no running maximum, out-of-band
// queries recomputed - while |softmax_scale| <= INTRA_SCALED_SOFTMAX_MAX_SCALE; beyond that the
// scores of ordinary inputs spread over so many powers of two that most work items would be
// computed twice, and EXACT runs from the start.  FOLDED is never picked by auto: its error grows
// with the magnitude of q and k (every product q_d * k_d moves by up to 2^-9 of itself when
// Q * scale * log2(e) is rounded to bf16).
int pick_softmax(float scale, unsigned flags) {
  int mode = (int)(flags & INTRA_SOFTMAX_MASK);
  if (mode == INTRA_SOFTMAX_AUTO) mode = softmax_mode().load(std::memory_order_relaxed);
  switch (mode) {
    case INTRA_SOFTMAX_EXACT: return intra::SM_EXACT;
    case INTRA_SOFTMAX_FOLDED: return intra::SM_FOLDED;
    case INTRA_SOFTMAX_SCALED: return intra::SM_SCALED;
    default: return fabsf(scale) <= INTRA_SCALED_SOFTMAX_MAX_SCALE ? intra::SM_SCALED : intra::SM_EXACT;
  }
}

// Order of an XCD's work items (see KParams::Section).  One section - every pair, all row blocks -
// except where a launch mixes kinds of items:
//  * image scatter: a set has text_len / 8 + width^2 / 8 queries, so its last row block is partial
//    (64 of 256 rows at 24 heads); where it is at most half full, those row blocks of all pairs
//    form a second section behind the full ones;
//  * image gather0: the text rows (the first sets; pairs are numbered set-major, so they are the
//    first pair slots) and the patch runs can have different numbers of row blocks; each kind gets
//    its section, so that no number goes to an empty item, text rows first.
void set_sections(intra::KParams& p, const Request& r, const Shape& ph, const LaunchDims& d) {
  const int pslots = (d.n_pairs + 7) / 8;
  auto section = [&](int p_lo, int p_n, int mb_lo, int mb_hi) {
    intra::KParams::Section s;
    s.p_lo = p_lo;
    s.mb_hi = mb_hi;
    s.slots = p_n * (mb_hi - mb_lo) * d.hgroups;
    s.d_ipp = make_fastdiv(std::max(1, (mb_hi - mb_lo) * d.hgroups));
    return s;
  };
  p.sec[0] = section(0, pslots, 0, d.n_mblocks);
  p.sec[1] = section(0, 0, 0, 1);
  if (ph.map == MAP_IMG_SCATTER) {
    const int nq = r.geom.text_len / 8 + r.geom.width * r.geom.width / 8;
    if (d.n_mblocks >= 2 && nq % d.pos != 0 && 2 * (nq % d.pos) <= d.pos) {
      p.sec[0] = section(0, pslots, 0, d.n_mblocks - 1);
      p.sec[1] = section(0, pslots, d.n_mblocks - 1, d.n_mblocks);
    }
  } else if (ph.map == MAP_IMG_GATHER0) {
    // pair slots that hold text rows only (a slot mixing both kinds goes with the patch runs and
    // then keeps the larger number of row blocks)
    const int text_pairs = (8 / ph.geom.tm) * r.B * r.Hkv;
    const int text_slots = text_pairs / 8;
    const int text_mb = std::min(d.n_mblocks, (ph.geom.tm * (r.geom.text_len / 8) + d.pos - 1) / d.pos);
    const int patch_mb = text_pairs % 8 != 0 ? d.n_mblocks : std::min(d.n_mblocks, (64 * ph.geom.pg + d.pos - 1) / d.pos);
    p.sec[0] = section(0, text_slots, 0, text_mb);
    p.sec[1] = section(text_slots, pslots - text_slots, 0, patch_mb);
  }
  p.n_slots = p.sec[0].slots + p.sec[1].slots;
}

// what locate_item needs of a launch: geometry, item counts, sections, divisors
void set_dealing(intra::KParams& p, const Request& r, const Shape& ph, const LaunchDims& dims) {
  p.B = r.B; p.H = r.H; p.Hkv = r.Hkv; p.ratio = r.H / r.Hkv;
  p.geom = ph.geom;
  p.n_sets = dims.n_sets;
  p.n_mblocks = dims.n_mblocks;
  p.hgroups = dims.hgroups;
  p.n_pairs = dims.n_pairs;
  set_sections(p, r, ph, dims);
  p.d_nbh = make_fastdiv(r.B * r.Hkv);
  p.d_hkv = make_fastdiv(r.Hkv);
  p.d_hgroups = make_fastdiv(p.hgroups);
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

// `written`: the tensor is an output, so its elements may not alias (a zero stride over a dimension
// larger than 1); inputs are only read, so expanded views (e.g. the gradient of a mean over tokens,
// or one kv head broadcast over several) are fine.
int check_strides(const char* name, const int64_t* st, int B, int S, int heads, bool written = false) {
  if (!st) return fail(INTRA_ERR_INVALID, "%s strides pointer is null", name);
  for (int i = 0; i < 3; ++i) {
    if (st[i] < 0) return fail(INTRA_ERR_INVALID, "%s stride %d is negative", name, i);
    if (st[i] % 8 != 0)
      return fail(INTRA_ERR_INVALID, "%s stride %d (%lld elements) breaks 16-byte alignment", name, i,
                  (long long)st[i]);
  }
  if (written && ((S > 1 && st[1] == 0) || (heads > 1 && st[2] == 0) || (B > 1 && st[0] == 0)))
    return fail(INTRA_ERR_INVALID, "%s has a zero stride over a dimension larger than 1", name);
  return INTRA_OK;
}

int run(int domain, const void* q, const void* k, const void* v, void* o, int B, int S, int H,
        int Hkv, const int64_t* qs, const int64_t* ks, const int64_t* vs, const int64_t* os,
        int pattern, int arg0, int arg1, float scale, void* stream, float* lse = nullptr,
        const int64_t* ls = nullptr, bool want_lse = false, int block = 0, int offset = 0, int n_sink = 0,
        bool extended = false, unsigned flags = 0) {
  g_err[0] = 0;
  if (flags & ~(unsigned)INTRA_SOFTMAX_MASK) return fail(INTRA_ERR_INVALID, "unknown bits in flags (0x%x)", flags);
  Request r;
  int rc = make_request(domain, pattern, B, S, H, Hkv, arg0, arg1, &r, block, offset, n_sink, extended);
  if (rc) return rc;
  if (!q || !k || !v || !o) return fail(INTRA_ERR_INVALID, "q, k, v and o must be non-null device pointers");
  if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(o))
    return fail(INTRA_ERR_INVALID, "q, k, v and o must be 16-byte aligned");
  if ((rc = check_strides("q", qs, B, S, H))) return rc;
  if ((rc = check_strides("k", ks, B, S, Hkv))) return rc;
  if ((rc = check_strides("v", vs, B, S, Hkv))) return rc;
  if ((rc = check_strides("o", os, B, S, H, true))) return rc;
  if (!isfinite(scale)) return fail(INTRA_ERR_INVALID, "softmax_scale must be finite");
  if (want_lse) {
    if (!lse) return fail(INTRA_ERR_INVALID, "lse must be a non-null device pointer");
    if (reinterpret_cast<uintptr_t>(lse) & 3) return fail(INTRA_ERR_INVALID, "lse must be 4-byte aligned");
    if (!ls) return fail(INTRA_ERR_INVALID, "lse strides pointer is null");
    for (int i = 0; i < 3; ++i)
      if (ls[i] < 0) return fail(INTRA_ERR_INVALID, "lse stride %d is negative", i);
    if ((B > 1 && ls[0] == 0) || (H > 1 && ls[1] == 0) || (S > 1 && ls[2] == 0))
      return fail(INTRA_ERR_INVALID, "lse has a zero stride over a dimension larger than 1");
  }

  if (qs[1] >= ((int64_t)1 << 31) || ks[1] >= ((int64_t)1 << 31) || vs[1] >= ((int64_t)1 << 31))
    return fail(INTRA_ERR_UNSUPPORTED, "q / k / v token stride must stay below 2^31 elements");

  intra::KParams p;
  p.q = static_cast<const uint16_t*>(q);
  p.k = static_cast<const uint16_t*>(k);
  p.v = static_cast<const uint16_t*>(v);
  p.o = static_cast<uint16_t*>(o);
  p.q_bs = qs[0]; p.q_rs = qs[1]; p.q_hs = qs[2];
  p.k_bs = ks[0]; p.k_rs = ks[1]; p.k_hs = ks[2];
  p.v_bs = vs[0]; p.v_rs = vs[1]; p.v_hs = vs[2];
  p.o_bs = os[0]; p.o_rs = os[1]; p.o_hs = os[2];
  p.lse = want_lse ? lse : nullptr;
  p.lse_bs = want_lse ? ls[0] : 0; p.lse_hs = want_lse ? ls[1] : 0; p.lse_ts = want_lse ? ls[2] : 0;
  p.B = B; p.H = H; p.Hkv = Hkv; p.ratio = H / Hkv;
  p.scale_log2 = fabsf(scale) * 1.4426950408889634f;
  if (p.scale_log2 < 1e-30f) p.scale_log2 = 1e-30f;  // scale 0: uniform weights without 0 * inf on masked scores
  p.negate_q = scale < 0.f;
  p.q_fold = scale * 1.4426950408889634f;
  p.k_rs_bytes = (uint32_t)(ks[1] * 2);
  p.v_rs_bytes = (uint32_t)(vs[1] * 2);
  p.q_rs_bytes = (uint32_t)(qs[1] * 2);

  Shape ph;
  if (!shape_for(r, default_hp(H / Hkv), &ph, pick_waves(r, default_hp(H / Hkv))))
    return fail(INTRA_ERR_UNSUPPORTED, "block scatter with an offset needs block %% 128 == 0 unless H / Hkv is even");
  const LaunchDims dims = by_map<DimsOf>(ph.map, r, ph);
  if (dims.work_items <= 0 || dims.n_pairs <= 0)
    return fail(INTRA_ERR_UNSUPPORTED, "problem needs more than 2^31 work items");
  const int grid = launch_grid(dims.work_items, ph.nw);
  if (grid <= 0)
    return fail(INTRA_ERR_HIP, "cannot query the current device: %s", hipGetErrorString(hipGetLastError()));
  set_dealing(p, r, ph, dims);
  p.diag = (int64_t)grid * intra::DIAG_SLOTS <= g_diag_values.load() ? g_diag.load() : nullptr;
  return by_map<LaunchMap>(ph.map, p, ph.hp, ph.nw, pick_softmax(scale, flags), grid, static_cast<hipStream_t>(stream));
}


// ------------------------------------------------------------------------------------ backward
template <class RMAP, int MODE, int HP, bool PARTIAL = false>
int launch_bwd(const intra::BParams& p, int64_t grid, hipStream_t stream) {
  if (grid <= 0 || grid > 0x7fffffff) return fail(INTRA_ERR_UNSUPPORTED, "backward needs more than 2^31 workgroups");
  hipLaunchKernelGGL((intra::intra_bwd_kernel<RMAP, MODE, HP, PARTIAL>), dim3((unsigned)grid), dim3(intra::bwd_waves(MODE) * 64), 0, stream, p);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(INTRA_ERR_HIP, "kernel launch failed: %s", hipGetErrorString(e));
  return INTRA_OK;
}

// Grid of one backward launch: per XCD, bundles of pairs x items of a pair (see the kernel).
int64_t bwd_grid(intra::BParams& p, int64_t pairs) {
  p.items_per_pair = p.n_rblocks * p.hgroups;
  const int64_t pairs_per_xcd = (pairs + 7) / 8;
  const int64_t want = (32 + p.items_per_pair - 1) / p.items_per_pair;  // pairs that fill an XCD's 32 CUs
  p.bundle = (int)std::max<int64_t>(1, std::min<int64_t>(want, pairs_per_xcd));
  const int64_t bundles = (pairs_per_xcd + p.bundle - 1) / p.bundle;
  return 8 * bundles * p.bundle * p.items_per_pair;
}

// dQ of a forward map: row blocks of 256 / hp queries of hp heads; also writes D = rowsum(dO o O)
template <class MAP>
int run_bwd_dq(intra::BParams p, int hp, hipStream_t stream) {
  using R = intra::QueryRows<MAP>;
  const int64_t pairs = (int64_t)R::num_sets(p.geom) * p.B * p.Hkv;
  p.hgroups = p.ratio / hp;
  p.n_rblocks = (R::max_rows(p.geom) + 256 / hp - 1) / (256 / hp);
  const int64_t grid = bwd_grid(p, pairs);
  switch (hp) {
    case 4: return launch_bwd<R, intra::BWD_DQ, 4>(p, grid, stream);
    case 2: return launch_bwd<R, intra::BWD_DQ, 2>(p, grid, stream);
    default: return launch_bwd<R, intra::BWD_DQ, 1>(p, grid, stream);
  }
}

// One launch over a key-row map: row blocks of one kv head's keys (32 per wavefront of the mode's
// workgroups), all query heads of its group streamed past
template <class R, bool PARTIAL, int MODE>
int run_bwd_keys_mode(intra::BParams p, hipStream_t stream) {
  constexpr int rows = intra::bwd_waves(MODE) * 32;
  const int64_t pairs = (int64_t)R::num_sets(p.geom) * p.B * p.Hkv;
  p.hgroups = 1;
  p.n_rblocks = (R::max_rows(p.geom) + rows - 1) / rows;
  return launch_bwd<R, MODE, 1, PARTIAL>(p, bwd_grid(p, pairs), stream);
}
// dK and dV over a key-row map, in one pass
template <class R>
int run_bwd_keys(const intra::BParams& p, hipStream_t stream) {
  return run_bwd_keys_mode<R, false, intra::BWD_DKV>(p, stream);
}

// Queries per workgroup of the pass over the `ns` leading keys (LLM sinks, image text keys): about
// one workgroup per CU (`cus`: the device's count; the workspace size and the launch have to use the
// same one), at least 128 queries each, a multiple of 64.
constexpr int MODEL_CUS = 256;  // host-only walks of the decomposition: any value gives a valid split
// The workspace is sized for a device of WS_CUS CUs (no device has to be current to ask for the size);
// a launch splits for min(its device's CUs, WS_CUS), which never needs more chunks than that.
constexpr int WS_CUS = 320;
int leading_chunk(int S, int B, int Hkv, int ns, int cus) {
  const int64_t row_wgs = (int64_t)B * Hkv * ((ns + 255) / 256);
  int64_t chunks = std::max<int64_t>(1, cus / row_wgs);  // at most one workgroup per CU: no second, thin round
  chunks = std::min<int64_t>(chunks, std::max(1, S / 128));
  return (int)(64 * ((S + 64 * chunks - 1) / (64 * chunks)));
}

// The rows of dk and dv of the leading keys: partial sums per chunk of queries, then their sum
// (twice: dk and dv share the partial buffer; everything is ordered by the stream).
template <class R>
int run_bwd_leading(const intra::BParams& p, hipStream_t stream) {
  const int ns = R::max_rows(p.geom), chunks = R::num_sets(p.geom);
  const int64_t threads = (int64_t)p.B * p.Hkv * ns * 32;
  const unsigned blocks = (unsigned)((threads + 255) / 256);
  for (int mode = 0; mode < 2; ++mode) {
    int rc = mode == 0 ? run_bwd_keys_mode<R, true, intra::BWD_DK>(p, stream)
                       : run_bwd_keys_mode<R, true, intra::BWD_DV>(p, stream);
    if (rc) return rc;
    if (mode == 0)
      hipLaunchKernelGGL(intra::intra_bwd_sink_reduce, dim3(blocks), dim3(256), 0, stream, p.part, chunks, p.B, p.Hkv,
                         ns, p.dk, p.dk_bs, p.dk_rs, p.dk_hs);
    else
      hipLaunchKernelGGL(intra::intra_bwd_sink_reduce, dim3(blocks), dim3(256), 0, stream, p.part, chunks, p.B, p.Hkv,
                         ns, p.dv, p.dv_bs, p.dv_rs, p.dv_hs);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) return fail(INTRA_ERR_HIP, "kernel launch failed: %s", hipGetErrorString(e));
  }
  return INTRA_OK;
}

// keys every query sees, handled by run_bwd_leading
int leading_keys(const Request& r) {
  if (r.kind == KIND_LLM_BLOCK_SCATTER || r.kind == KIND_LLM_WINDOW_SINK) return std::min(r.geom.ns, r.S);
  if (r.kind == KIND_IMG_SCATTER || r.kind == KIND_IMG_GATHER0) return r.geom.text_len;
  return 0;
}

// floats of workspace: -D = -rowsum(dO o O) and lse * log2(e) per (batch, head, token), then the partial
// sums of the leading keys
int64_t bwd_dsum_floats(int B, int S, int H) { return ((int64_t)B * H * S + 3) & ~(int64_t)3; }
int64_t bwd_workspace_floats(const Request& r, int cus) {
  int64_t n = 2 * bwd_dsum_floats(r.B, r.S, r.H);
  const int ns = leading_keys(r);
  if (ns > 0) {
    const int chunk = leading_chunk(r.S, r.B, r.Hkv, ns, cus);
    n += (int64_t)((r.S + chunk - 1) / chunk) * r.B * r.Hkv * ns * 128;
  }
  return n;
}

// Does the backward pass cover this request?
int bwd_supported(const Request& r) {
  if (r.kind == KIND_LLM_BLOCK_SCATTER && r.geom.off != 0 && r.geom.blk % 256 != 0)
    return fail(INTRA_ERR_UNSUPPORTED, "backward: block scatter with a stripe offset needs block % 256 == 0");
  return INTRA_OK;
}

int run_bwd(int domain, const void* q, const void* k, const void* v, const void* o, const float* lse, const void* dout,
            void* dq, void* dk, void* dv, float* dsum, int B, int S, int H, int Hkv, const int64_t* qs,
            const int64_t* ks, const int64_t* vs, const int64_t* os, const int64_t* dos, const int64_t* dqs,
            const int64_t* dks, const int64_t* dvs, const int64_t* ls, int pattern, int group_num, int window,
            int block, int offset, int n_sink, float scale, void* stream) {
  g_err[0] = 0;
  Request r;
  int rc = make_request(domain, pattern, B, S, H, Hkv, group_num, window, &r, block, offset, n_sink, domain == 0);
  if (rc) return rc;
  if ((rc = bwd_supported(r))) return rc;
  const void* ins[] = {q, k, v, o, dout, dq, dk, dv};
  for (const void* ptr : ins) {
    if (!ptr) return fail(INTRA_ERR_INVALID, "q, k, v, o, dout, dq, dk and dv must be non-null device pointers");
    if (!aligned16(ptr)) return fail(INTRA_ERR_INVALID, "q, k, v, o, dout, dq, dk and dv must be 16-byte aligned");
  }
  if (!lse || (reinterpret_cast<uintptr_t>(lse) & 3)) return fail(INTRA_ERR_INVALID, "lse must be a non-null, 4-byte aligned device pointer");
  if (!dsum || !aligned16(dsum)) return fail(INTRA_ERR_INVALID, "the workspace must be a non-null, 16-byte aligned device pointer");
  if ((rc = check_strides("q", qs, B, S, H)) || (rc = check_strides("k", ks, B, S, Hkv)) ||
      (rc = check_strides("v", vs, B, S, Hkv)) || (rc = check_strides("o", os, B, S, H)) ||
      (rc = check_strides("dout", dos, B, S, H)) || (rc = check_strides("dq", dqs, B, S, H, true)) ||
      (rc = check_strides("dk", dks, B, S, Hkv, true)) || (rc = check_strides("dv", dvs, B, S, Hkv, true)))
    return rc;
  if (!ls) return fail(INTRA_ERR_INVALID, "lse strides pointer is null");
  for (int i = 0; i < 3; ++i)
    if (ls[i] < 0) return fail(INTRA_ERR_INVALID, "lse stride %d is negative", i);
  if (!isfinite(scale)) return fail(INTRA_ERR_INVALID, "softmax_scale must be finite");
  if (scale == 0.f) return fail(INTRA_ERR_UNSUPPORTED, "backward: softmax_scale must not be zero");
  const int64_t* all[] = {qs, ks, vs, dos};
  for (const int64_t* st : all)
    if (st[1] >= ((int64_t)1 << 31)) return fail(INTRA_ERR_UNSUPPORTED, "token strides must stay below 2^31 elements");

  intra::BParams p;
  p.q = static_cast<const uint16_t*>(q);
  p.k = static_cast<const uint16_t*>(k);
  p.v = static_cast<const uint16_t*>(v);
  p.o = static_cast<const uint16_t*>(o);
  p.dout = static_cast<const uint16_t*>(dout);
  p.lse = lse;
  p.dsum = dsum;
  p.l2 = dsum + bwd_dsum_floats(B, S, H);
  p.part = p.l2 + bwd_dsum_floats(B, S, H);
  p.dq = static_cast<uint16_t*>(dq);
  p.dk = static_cast<uint16_t*>(dk);
  p.dv = static_cast<uint16_t*>(dv);
  p.q_bs = qs[0]; p.q_rs = qs[1]; p.q_hs = qs[2];
  p.k_bs = ks[0]; p.k_rs = ks[1]; p.k_hs = ks[2];
  p.v_bs = vs[0]; p.v_rs = vs[1]; p.v_hs = vs[2];
  p.o_bs = os[0]; p.o_rs = os[1]; p.o_hs = os[2];
  p.do_bs = dos[0]; p.do_rs = dos[1]; p.do_hs = dos[2];
  p.dq_bs = dqs[0]; p.dq_rs = dqs[1]; p.dq_hs = dqs[2];
  p.dk_bs = dks[0]; p.dk_rs = dks[1]; p.dk_hs = dks[2];
  p.dv_bs = dvs[0]; p.dv_rs = dvs[1]; p.dv_hs = dvs[2];
  p.lse_bs = ls[0]; p.lse_hs = ls[1]; p.lse_ts = ls[2];
  p.ds_bs = (int64_t)H * S; p.ds_hs = S;
  p.B = B; p.H = H; p.Hkv = Hkv; p.ratio = H / Hkv;
  p.scale = scale;
  p.scale_log2 = scale * 1.4426950408889634f;
  Shape sh;
  if (!shape_for(r, default_hp(H / Hkv), &sh)) return fail(INTRA_ERR_UNSUPPORTED, "no kernel shape for this request");
  p.geom = sh.geom;
  const int ns = leading_keys(r);
  if (ns > 0) {
    p.geom.ns = ns;
    const int cus = cu_count();
    if (cus <= 0) return fail(INTRA_ERR_HIP, "cannot query the current device: %s", hipGetErrorString(hipGetLastError()));
    p.geom.sink_chunk = leading_chunk(S, B, Hkv, ns, std::min(cus, WS_CUS));
  }
  hipStream_t st = static_cast<hipStream_t>(stream);
  switch (sh.map) {
    case MAP_LLM_SCATTER:
      if ((rc = run_bwd_dq<MapLlmScatter>(p, sh.hp, st))) return rc;
      return run_bwd_keys<intra::KeyRowsOf<MapLlmScatter>>(p, st);
    case MAP_LLM_GATHER1:
      if ((rc = run_bwd_dq<MapLlmGather1>(p, sh.hp, st))) return rc;
      return run_bwd_keys<intra::KeyRowsOf<MapLlmGather1>>(p, st);
    case MAP_LLM_WINDOW:
      if ((rc = run_bwd_dq<MapLlmWindow>(p, sh.hp, st))) return rc;
      return run_bwd_keys<intra::KeyRowsOf<MapLlmWindow>>(p, st);
    case MAP_LLM_BLOCK_SCATTER:
      if ((rc = run_bwd_dq<MapLlmBlockScatter>(p, sh.hp, st))) return rc;
      if ((rc = run_bwd_keys<intra::KeyRowsBlockScatter>(p, st))) return rc;
      return ns > 0 ? run_bwd_leading<intra::KeyRowsSinks>(p, st) : INTRA_OK;
    case MAP_LLM_WINDOW_SINK:
      if ((rc = run_bwd_dq<MapLlmWindowSink>(p, sh.hp, st))) return rc;
      if ((rc = run_bwd_keys<intra::KeyRowsWindowSink>(p, st))) return rc;
      return ns > 0 ? run_bwd_leading<intra::KeyRowsSinks>(p, st) : INTRA_OK;
    case MAP_IMG_SCATTER:  // grid keys against their group's queries, text keys against all queries
      if ((rc = run_bwd_dq<MapImgScatter>(p, sh.hp, st))) return rc;
      if ((rc = run_bwd_keys<intra::KeyRowsImgGroup<false>>(p, st))) return rc;
      return run_bwd_leading<intra::KeyRowsText>(p, st);
    case MAP_IMG_GATHER0:  // grid keys against the grid queries around them, plus their group's text queries
      if ((rc = run_bwd_dq<MapImgGather0>(p, sh.hp, st))) return rc;
      if ((rc = run_bwd_keys<intra::KeyRowsImgWindow>(p, st))) return rc;
      if ((rc = run_bwd_keys<intra::KeyRowsImgGroup<true>>(p, st))) return rc;
      return run_bwd_leading<intra::KeyRowsText>(p, st);
    default: return fail(INTRA_ERR_UNSUPPORTED, "backward: no kernels for this pattern");
  }
}

// ------------------------------------------------------------------------------------ no-allocation backward
// Workspace of intra_llm_bwd_noalloc: one array per GPU inside the library's own device image, so the
// entry point never calls an allocator.  In host code the array's name only stands for the symbol; the
// address the kernels get comes from hipGetSymbolAddress, asked once per device with that device current.
static __device__ __align__(256) float scratch[INTRA_NOALLOC_SCRATCH_FLOATS];

float* noalloc_scratch() {
  static std::atomic<float*> ptrs[64];  // per device; nullptr = not asked yet
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) {
    fail(INTRA_ERR_HIP, "cannot query the current device: %s", hipGetErrorString(hipGetLastError()));
    return nullptr;
  }
  float* ptr = ptrs[dev].load(std::memory_order_acquire);
  if (ptr == nullptr) {
    const hipError_t e = hipGetSymbolAddress(reinterpret_cast<void**>(&ptr), HIP_SYMBOL(scratch));
    if (e != hipSuccess || ptr == nullptr) {
      fail(INTRA_ERR_HIP, "hipGetSymbolAddress of the built-in workspace failed: %s", hipGetErrorString(e));
      return nullptr;
    }
    ptrs[dev].store(ptr, std::memory_order_release);  // every thread gets the same answer for a device
  }
  return ptr;
}

// Host walk of the backward decomposition: count[q * S + k] += 1 for every (query, key) pair that
// the dK / dV launches (key-row maps with their `store` rule, then the sink pass) multiply.
template <class R>
void bwd_walk(const IntraGeom& ge, uint8_t* count, int rows) {  // rows: keys per row block of the launch
  const int S = ge.S;
  for (int set = 0; set < R::num_sets(ge); ++set)
    for (int r0 = 0; r0 < R::max_rows(ge); r0 += rows) {
      const R m(ge, set, r0);
      const int r1 = std::min(r0 + rows, m.n_rows()) - 1;
      for (int t = r0; t <= r1; ++t) {
        const int kp = m.row_pos(t);
        if (!m.store(kp)) continue;
        const int lo = std::max(m.lo(t), m.block_lo(r0, r1));
        const int hi = std::min(std::min(m.hi(t), m.n_cols() - 1), m.block_hi(r0, r1));
        for (int c = lo; c <= hi; ++c)
          if (!R::kBlockPredicate || m.sees(t, c & ~31)) ++count[(size_t)m.col_pos(c) * S + kp];
      }
    }
}

int model_mask_bwd(const Request& r, uint8_t* count) {
  if (int rc = bwd_supported(r)) return rc;
  Shape sh;
  if (!shape_for(r, 1, &sh)) return fail(INTRA_ERR_UNSUPPORTED, "no kernel shape for this request");
  switch (sh.map) {
    case MAP_LLM_SCATTER: bwd_walk<intra::KeyRowsOf<MapLlmScatter>>(sh.geom, count, intra::bwd_waves(intra::BWD_DKV) * 32); break;
    case MAP_LLM_GATHER1: bwd_walk<intra::KeyRowsOf<MapLlmGather1>>(sh.geom, count, intra::bwd_waves(intra::BWD_DKV) * 32); break;
    case MAP_LLM_WINDOW: bwd_walk<intra::KeyRowsOf<MapLlmWindow>>(sh.geom, count, intra::bwd_waves(intra::BWD_DKV) * 32); break;
    case MAP_LLM_BLOCK_SCATTER: bwd_walk<intra::KeyRowsBlockScatter>(sh.geom, count, intra::bwd_waves(intra::BWD_DKV) * 32); break;
    case MAP_LLM_WINDOW_SINK: bwd_walk<intra::KeyRowsWindowSink>(sh.geom, count, intra::bwd_waves(intra::BWD_DKV) * 32); break;
    default: return fail(INTRA_ERR_UNSUPPORTED, "backward: no kernels for this pattern");
  }
  if (leading_keys(r) > 0) {
    sh.geom.sink_chunk = leading_chunk(r.S, 1, 1, leading_keys(r), MODEL_CUS);
    bwd_walk<intra::KeyRowsSinks>(sh.geom, count, 256);
  }
  return INTRA_OK;
}

int model_mask(const Request& r, int heads_per_block, int waves, uint8_t* count) {
  const int hp = heads_per_block > 0 ? heads_per_block : 1;
  if ((hp != 1 && hp != 2 && hp != 4) || (waves > 0 && waves != 8 && waves != intra::NARROW_WAVES))
    return fail(INTRA_ERR_INVALID, "no kernel for heads_per_block=%d, waves=%d", hp, waves);
  Shape ph;
  if (!shape_for(r, hp, &ph, waves > 0 ? waves : 8))
    return fail(INTRA_ERR_UNSUPPORTED, "block size does not fit the row blocks of this head layout");
  by_map<ModelWalk>(ph.map, ph.geom, ph.hp, ph.nw, count);
  return INTRA_OK;
}

int model_mask_image_bwd(const Request& r, uint8_t* count) {
  Shape sh;
  if (!shape_for(r, 1, &sh)) return fail(INTRA_ERR_UNSUPPORTED, "no kernel shape for this request");
  IntraGeom ge = sh.geom;
  ge.ns = ge.text_len;  // the text keys are the leading keys every query sees
  ge.sink_chunk = leading_chunk(r.S, 1, 1, ge.ns, MODEL_CUS);
  if (r.kind == KIND_IMG_SCATTER) {
    bwd_walk<intra::KeyRowsImgGroup<false>>(ge, count, intra::bwd_waves(intra::BWD_DKV) * 32);
  } else {
    bwd_walk<intra::KeyRowsImgWindow>(ge, count, intra::bwd_waves(intra::BWD_DKV) * 32);
    bwd_walk<intra::KeyRowsImgGroup<true>>(ge, count, intra::bwd_waves(intra::BWD_DKV) * 32);
  }
  bwd_walk<intra::KeyRowsText>(ge, count, 256);
  return INTRA_OK;
}

}  // namespace

extern "C" {

int intra_llm_fwd(const void* q, const void* k, const void* v, void* o, int B, int S, int H,
                  int Hkv, const int64_t q_strides[3], const int64_t k_strides[3],
                  const int64_t v_strides[3], const int64_t o_strides[3], int pattern,
                  int group_num, int window, float softmax_scale, void* hip_stream) {
  return run(0, q, k, v, o, B, S, H, Hkv, q_strides, k_strides, v_strides, o_strides, pattern,
             group_num, window, softmax_scale, hip_stream);
}

int intra_image_fwd(const void* q, const void* k, const void* v, void* o, int B, int S, int H,
                    int Hkv, const int64_t q_strides[3], const int64_t k_strides[3],
                    const int64_t v_strides[3], const int64_t o_strides[3], int pattern,
                    int width, int text_len, float softmax_scale, void* hip_stream) {
  return run(1, q, k, v, o, B, S, H, Hkv, q_strides, k_strides, v_strides, o_strides, pattern,
             width, text_len, softmax_scale, hip_stream);
}

int intra_llm_fwd_lse(const void* q, const void* k, const void* v, void* o, int B, int S, int H,
                      int Hkv, const int64_t q_strides[3], const int64_t k_strides[3],
                      const int64_t v_strides[3], const int64_t o_strides[3], int pattern,
                      int group_num, int window, float softmax_scale, void* hip_stream, float* lse,
                      const int64_t lse_strides[3]) {
  return run(0, q, k, v, o, B, S, H, Hkv, q_strides, k_strides, v_strides, o_strides, pattern,
             group_num, window, softmax_scale, hip_stream, lse, lse_strides, true);
}

int intra_image_fwd_lse(const void* q, const void* k, const void* v, void* o, int B, int S, int H,
                        int Hkv, const int64_t q_strides[3], const int64_t k_strides[3],
                        const int64_t v_strides[3], const int64_t o_strides[3], int pattern,
                        int width, int text_len, float softmax_scale, void* hip_stream, float* lse,
                        const int64_t lse_strides[3]) {
  return run(1, q, k, v, o, B, S, H, Hkv, q_strides, k_strides, v_strides, o_strides, pattern,
             width, text_len, softmax_scale, hip_stream, lse, lse_strides, true);
}

int intra_llm_bwd(const void* q, const void* k, const void* v, const void* o, const float* lse, const void* dout,
                  void* dq, void* dk, void* dv, float* workspace, int B, int S, int H, int Hkv,
                  const int64_t q_strides[3], const int64_t k_strides[3], const int64_t v_strides[3],
                  const int64_t o_strides[3], const int64_t dout_strides[3], const int64_t dq_strides[3],
                  const int64_t dk_strides[3], const int64_t dv_strides[3], const int64_t lse_strides[3],
                  int pattern, int group_num, int window, int block, int offset, int n_sink,
                  float softmax_scale, void* hip_stream) {
  return run_bwd(0, q, k, v, o, lse, dout, dq, dk, dv, workspace, B, S, H, Hkv, q_strides, k_strides, v_strides,
                 o_strides, dout_strides, dq_strides, dk_strides, dv_strides, lse_strides, pattern, group_num,
                 window, block, offset, n_sink, softmax_scale, hip_stream);
}

int intra_llm_bwd_noalloc(const void* q, const void* k, const void* v, const void* o, const float* lse, const void* dout,
                          void* dq, void* dk, void* dv, int B, int S, int H, int Hkv, const int64_t q_strides[3],
                          const int64_t k_strides[3], const int64_t v_strides[3], const int64_t o_strides[3],
                          const int64_t dout_strides[3], const int64_t dq_strides[3], const int64_t dk_strides[3],
                          const int64_t dv_strides[3], const int64_t lse_strides[3], int pattern, int group_num,
                          int window, int block, int offset, int n_sink, float softmax_scale, void* hip_stream) {
  g_err[0] = 0;
  Request r;
  int rc = make_request(0, pattern, B, S, H, Hkv, group_num, window, &r, block, offset, n_sink, true);
  if (rc) return rc;
  if ((rc = bwd_supported(r))) return rc;
  const int64_t need = bwd_workspace_floats(r, WS_CUS);
  if (need > (int64_t)INTRA_NOALLOC_SCRATCH_FLOATS)
    return fail(INTRA_ERR_UNSUPPORTED,
                "intra_llm_bwd_noalloc: this call needs %lld floats of workspace, the built-in one holds %lld; "
                "use intra_llm_bwd with a workspace of the caller", (long long)need, (long long)INTRA_NOALLOC_SCRATCH_FLOATS);
  float* work = noalloc_scratch();
  if (work == nullptr) return INTRA_ERR_HIP;
  return run_bwd(0, q, k, v, o, lse, dout, dq, dk, dv, work, B, S, H, Hkv, q_strides, k_strides, v_strides, o_strides,
                 dout_strides, dq_strides, dk_strides, dv_strides, lse_strides, pattern, group_num, window, block, offset,
                 n_sink, softmax_scale, hip_stream);
}

int64_t intra_llm_bwd_workspace(int B, int S, int H, int Hkv, int pattern, int group_num, int window, int block,
                                int offset, int n_sink) {
  g_err[0] = 0;
  Request r;
  if (make_request(0, pattern, B, S, H, Hkv, group_num, window, &r, block, offset, n_sink, true)) return -1;
  if (bwd_supported(r)) return -1;
  return bwd_workspace_floats(r, WS_CUS);
}

int intra_image_bwd(const void* q, const void* k, const void* v, const void* o, const float* lse, const void* dout,
                    void* dq, void* dk, void* dv, float* workspace, int B, int S, int H, int Hkv,
                    const int64_t q_strides[3], const int64_t k_strides[3], const int64_t v_strides[3],
                    const int64_t o_strides[3], const int64_t dout_strides[3], const int64_t dq_strides[3],
                    const int64_t dk_strides[3], const int64_t dv_strides[3], const int64_t lse_strides[3],
                    int pattern, int width, int text_len, float softmax_scale, void* hip_stream) {
  return run_bwd(1, q, k, v, o, lse, dout, dq, dk, dv, workspace, B, S, H, Hkv, q_strides, k_strides, v_strides,
                 o_strides, dout_strides, dq_strides, dk_strides, dv_strides, lse_strides, pattern, width, text_len,
                 0, 0, 0, softmax_scale, hip_stream);
}

int64_t intra_image_bwd_workspace(int B, int S, int H, int Hkv, int pattern, int width, int text_len) {
  g_err[0] = 0;
  Request r;
  if (make_request(1, pattern, B, S, H, Hkv, width, text_len, &r)) return -1;
  return bwd_workspace_floats(r, WS_CUS);
}

int intra_model_mask_llm_bwd(int pattern, int S, int group_num, int window, int block, int offset, int n_sink,
                             uint8_t* count) {
  g_err[0] = 0;
  if (!count) return fail(INTRA_ERR_INVALID, "count is null");
  Request r;
  int rc = make_request(0, pattern, 1, S, 1, 1, group_num, window, &r, block, offset, n_sink, true);
  if (rc) return rc;
  return model_mask_bwd(r, count);
}

int intra_model_mask_image_bwd(int pattern, int S, int width, int text_len, uint8_t* count) {
  g_err[0] = 0;
  if (!count) return fail(INTRA_ERR_INVALID, "count is null");
  Request r;
  int rc = make_request(1, pattern, 1, S, 1, 1, width, text_len, &r);
  if (rc) return rc;
  return model_mask_image_bwd(r, count);
}

const char* intra_last_error(void) { return g_err; }

int intra_version(void) { return INTRA_VERSION; }

int intra_set_softmax_mode(int mode) {
  g_err[0] = 0;
  if (mode < 0 || mode > 3)
    return fail(INTRA_ERR_INVALID, "softmax mode must be 0 (auto), 1 (exact), 2 (folded) or 3 (scaled), got %d", mode);
  softmax_mode().store(mode, std::memory_order_relaxed);
  return INTRA_OK;
}

int intra_get_softmax_mode(void) { return softmax_mode().load(std::memory_order_relaxed); }

int intra_diag_set_buffer(long long* counters, int64_t n_values) {
  g_err[0] = 0;
#ifdef INTRA_DIAG_TIMERS
  if (counters != nullptr && (n_values < intra::DIAG_SLOTS || (reinterpret_cast<uintptr_t>(counters) & 7)))
    return fail(INTRA_ERR_INVALID, "the timer buffer must be 8-byte aligned and hold at least %d values", intra::DIAG_SLOTS);
  g_diag_values.store(0);
  g_diag.store(counters);
  g_diag_values.store(counters ? n_values : 0);
  return INTRA_OK;
#else
  (void)counters;
  (void)n_values;
  return fail(INTRA_ERR_UNSUPPORTED, "this library was built without -DINTRA_DIAG_TIMERS (python -m intra_amd.build --diag)");
#endif
}

int intra_diag_ablation(void) { return INTRA_ABLATE; }

int intra_diag_mfma_ceiling(const void* table, float* sink, long long* clocks, int workgroups, int iters,
                            int shape, void* hip_stream) {
  g_err[0] = 0;
  if (!table || !sink || !clocks) return fail(INTRA_ERR_INVALID, "table, sink and clocks must be non-null device pointers");
  if (!aligned16(table)) return fail(INTRA_ERR_INVALID, "table must be 16-byte aligned");
  if (workgroups < 1 || workgroups > 65536 || iters < 1)
    return fail(INTRA_ERR_INVALID, "workgroups must be in [1, 65536] and iters positive (got %d, %d)", workgroups, iters);
  if (shape != 16 && shape != 32) return fail(INTRA_ERR_INVALID, "shape must be 16 (16x16x32) or 32 (32x32x16), got %d", shape);
  if (shape == 16)
    hipLaunchKernelGGL(intra::mfma_ceiling_kernel<true>, dim3(workgroups), dim3(512), 0, static_cast<hipStream_t>(hip_stream),
                       static_cast<const uint4*>(table), sink, iters, clocks);
  else
    hipLaunchKernelGGL(intra::mfma_ceiling_kernel<false>, dim3(workgroups), dim3(512), 0, static_cast<hipStream_t>(hip_stream),
                       static_cast<const uint4*>(table), sink, iters, clocks);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(INTRA_ERR_HIP, "kernel launch failed: %s", hipGetErrorString(e));
  return INTRA_OK;
}

int intra_plan(int domain, int pattern, int B, int S, int H, int Hkv, int arg0, int arg1,
               IntraPlan* plan) {
  g_err[0] = 0;
  if (!plan) return fail(INTRA_ERR_INVALID, "plan pointer is null");
  Request r;
  int rc = make_request(domain, pattern, B, S, H, Hkv, arg0, arg1, &r);
  if (rc) return rc;
  return plan_for(r, default_hp(H / Hkv), plan);
}

int intra_model_mask(int domain, int pattern, int S, int arg0, int arg1, int heads_per_block,
                     int waves, uint8_t* count) {
  g_err[0] = 0;
  if (!count) return fail(INTRA_ERR_INVALID, "count pointer is null");
  Request r;
  int rc = make_request(domain, pattern, 1, S, 1, 1, arg0, arg1, &r);
  if (rc) return rc;
  return model_mask(r, heads_per_block, waves, count);
}

int intra_model_deal(int domain, int pattern, int B, int S, int H, int Hkv, int arg0, int arg1,
                     int waves, int grid, uint8_t* visits, int64_t n_visits) {
  g_err[0] = 0;
  if (!visits) return fail(INTRA_ERR_INVALID, "visits pointer is null");
  Request r;
  int rc = make_request(domain, pattern, B, S, H, Hkv, arg0, arg1, &r);
  if (rc) return rc;
  if (waves != 8 && waves != intra::NARROW_WAVES) return fail(INTRA_ERR_INVALID, "waves must be 8 or 4");
  Shape ph;
  if (!shape_for(r, default_hp(H / Hkv), &ph, waves))
    return fail(INTRA_ERR_UNSUPPORTED, "no kernel shape of %d wavefronts for this request", waves);
  const LaunchDims dims = by_map<DimsOf>(ph.map, r, ph);
  if (dims.work_items <= 0 || dims.n_pairs <= 0)
    return fail(INTRA_ERR_UNSUPPORTED, "problem needs more than 2^31 work items");
  if (grid < 8 || grid % 8 != 0 || grid > dims.work_items)
    return fail(INTRA_ERR_INVALID, "grid must be a multiple of 8 in 8 .. work_items (%d)", dims.work_items);
  if (n_visits < dims.work_items) return fail(INTRA_ERR_INVALID, "visits holds %lld values, %d needed", (long long)n_visits, dims.work_items);
  intra::KParams p{};
  set_dealing(p, r, ph, dims);
  return by_map<DealWalk>(ph.map, p, dims.pos, grid, dims.n_mblocks, visits);
}

int intra_llm_fwd_ex(const void* q, const void* k, const void* v, void* o, int B, int S, int H,
                     int Hkv, const int64_t q_strides[3], const int64_t k_strides[3],
                     const int64_t v_strides[3], const int64_t o_strides[3], int pattern,
                     int group_num, int window, int block, int offset, int n_sink,
                     float softmax_scale, void* hip_stream, float* lse, const int64_t lse_strides[3],
                     unsigned flags) {
  return run(0, q, k, v, o, B, S, H, Hkv, q_strides, k_strides, v_strides, o_strides, pattern,
             group_num, window, softmax_scale, hip_stream, lse, lse_strides, lse != nullptr, block, offset,
             n_sink, true, flags);
}

int intra_image_fwd_ex(const void* q, const void* k, const void* v, void* o, int B, int S, int H,
                       int Hkv, const int64_t q_strides[3], const int64_t k_strides[3],
                       const int64_t v_strides[3], const int64_t o_strides[3], int pattern,
                       int width, int text_len, float softmax_scale, void* hip_stream, float* lse,
                       const int64_t lse_strides[3], unsigned flags) {
  return run(1, q, k, v, o, B, S, H, Hkv, q_strides, k_strides, v_strides, o_strides, pattern,
             width, text_len, softmax_scale, hip_stream, lse, lse_strides, lse != nullptr, 0, 0, 0, false,
             flags);
}

int intra_plan_llm_ex(int pattern, int B, int S, int H, int Hkv, int group_num, int window,
                      int block, int offset, int n_sink, IntraPlan* plan) {
  g_err[0] = 0;
  if (!plan) return fail(INTRA_ERR_INVALID, "plan pointer is null");
  Request r;
  int rc = make_request(0, pattern, B, S, H, Hkv, group_num, window, &r, block, offset, n_sink, true);
  if (rc) return rc;
  return plan_for(r, default_hp(H / Hkv), plan);
}

int intra_model_mask_llm_ex(int pattern, int S, int group_num, int window, int block, int offset,
                            int n_sink, int heads_per_block, uint8_t* count) {
  g_err[0] = 0;
  if (!count) return fail(INTRA_ERR_INVALID, "count pointer is null");
  Request r;
  int rc = make_request(0, pattern, 1, S, 1, 1, group_num, window, &r, block, offset, n_sink, true);
  if (rc) return rc;
  return model_mask(r, heads_per_block, 8, count);
}

}  // extern "C"
