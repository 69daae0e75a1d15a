// Forward sparse-attention kernel for gfx950 (MI355X): one template for all five INTRA patterns.
//
// Replaces the reference's five CUDA kernels (csrc/flash_attn/src/flash_fwd_kernel.h:3970-6158
// with their loaders in gmem_tile.h) by one wave64/MFMA design, which also runs the block-level
// Scatter and window-with-sinks layers of experiments/llm/llama_intra.py:
//
//  * A workgroup of NW wavefronts owns a row block of one set: POS = NW*32/HP consecutive in-set
//    queries of HP query heads that share one KV head (GQA packing), so every gathered K/V tile
//    is used by all HP heads.  Each wavefront owns 32 queries of one head.
//  * Scores are computed transposed, S^T = K Q^T, with v_mfma_f32_16x16x32_bf16 (per flop it draws
//    about a tenth less power than the 32x32x16 shape, and this kernel runs against the board's
//    power limit): the A operand is a K tile row read from LDS (16 B per lane), the B operand is Q
//    held in registers for a whole work item.  A 32-key block times the wavefront's 32 queries is
//    2 x 2 tiles; in the accumulator layout a lane holds 4 keys per tile of ONE query per query
//    tile, so the rescale factors are plain per-lane scalars and a query's maximum or sum is a
//    reduction over four lanes (l, l ^ 16, l ^ 32, l ^ 48).
//  * O^T = V^T P^T: P^T is the softmax output still in registers (packed to bf16, no LDS round
//    trip): the lane's 8 weights of a query tile ARE its B operand, under a numbering of the 32-key
//    reduction that the V^T operand follows; V^T comes from ds_read_b64_tr_b16 transposing reads of
//    the row-major V tile.
//  * Software pipeline in steps of 32 keys: in step j a wavefront issues the 16 QK^T MFMAs of key
//    block j+1 and the 16 PV MFMAs of block j, with the softmax VALU work of block j spread over
//    both phases and every LDS operand read issued about a phase ahead.
//  * K/V rows are gathered from HBM straight into LDS (global_load_lds_dwordx4, 16 lanes per
//    256-byte row, no register staging), three tiles ahead; one barrier per 64-key tile, which
//    only waits for the requests of the previous iteration.  The tiles of all work items of a
//    workgroup form one stream through the ring, so the first tiles of a work item arrive while
//    the previous one still computes.  The Q rows of a work item travel in the same stream, as
//    two ring slots in front of its key tiles: they are requested three slots ahead like any
//    tile, arrive as whole 256-byte rows, and each wavefront picks its 32 rows out of LDS with
//    the K operand's read pattern.  The output rows of a finished item are stored right behind its
//    tile loop, in front of the barrier that opens the next item.  An LDS tile is 16 groups
//    of 4 rows with an XOR chunk swizzle inside the group and 32 bytes of padding between groups,
//    so the row-per-lane K reads and the 4-row transposing V reads are both free of bank conflicts.
//  * The softmax reference stays 0 (weights exp2(score*c), exact after normalisation because
//    numerator and denominator share it) unless a block maximum leaves the +-60 exponent band;
//    then the query is re-centred and O rescaled.  No per-block rescale in the common case.
//  * Blocks outside a wavefront's key range are skipped; only blocks cut by a bound are masked.
//  * The grid is persistent (about one workgroup per CU); work items are dealt per XCD so that
//    one (batch, kv head, set) stays in one XCD's L2, in an order that balances causal triangles.
//  * Three softmax modes.  SM_EXACT scales the fp32 scores after the MFMA and watches every
//    block's maximum (the reference's arithmetic, csrc/flash_attn/src/softmax.h:65-91).
//    SM_SCALED (what a plain call gets) scales the fp32 scores the same way, so its accuracy does
//    not depend on the size of q and k, but keeps no running maximum at all: weights are
//    exp2(score * c); a query whose weight sum left the safe exponent band marks its work item
//    in an LDS bitmap, and after the last item the workgroup runs the marked items again in
//    SM_EXACT mode.  SM_FOLDED (opt-in per call) saves the multiply per score as well: it folds
//    softmax_scale * log2(e) into the bf16 Q fragments once per work item and exponentiates the
//    raw MFMA results; the bf16 rounding of Q * c perturbs a score in proportion to the
//    magnitudes of q and k, so it is only as accurate as the other two for inputs of unit scale.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "intra_maps.h"

namespace intra {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef float floatx2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

struct KParams {
  const uint16_t* q;
  const uint16_t* k;
  const uint16_t* v;
  uint16_t* o;
  // element strides: batch, row (token), head
  int64_t q_bs, q_rs, q_hs;
  int64_t k_bs, k_rs, k_hs;
  int64_t v_bs, v_rs, v_hs;
  int64_t o_bs, o_rs, o_hs;
  float* lse;          // optional (B, H, S) log-sum-exp output, or null
  int64_t lse_bs, lse_hs, lse_ts;  // its element strides: batch, head, token
  int B, H, Hkv, ratio;
  IntraGeom geom;
  float scale_log2;    // |softmax_scale| * log2(e)
  int negate_q;        // softmax_scale < 0: flip the sign of Q instead
  float q_fold;        // SM_FOLDED: softmax_scale * log2(e), signed, multiplied into Q
  uint32_t k_rs_bytes, v_rs_bytes, q_rs_bytes;  // token strides of k, v, q in bytes (< 4 GiB, checked on the host)
  int n_sets;          // sets per (batch, kv head)
  int n_mblocks;       // row blocks of the largest set
  int hgroups;         // ratio / HP
  int n_pairs;         // B * Hkv * n_sets
  int n_slots;         // work items per XCD: sum of the sections' slots
  // The work items of an XCD are numbered section by section (costly kinds of items first, so
  // that the cheap ones fill the last, partial round of the workgroups; kinds of sets with
  // different numbers of row blocks apart, so that no number goes to an empty item): a section is
  // a range of the XCD's pairs times a range of row blocks, taken pair by pair, last row block first.
  struct Section {
    int p_lo;          // first pair slot (pair = 8 * pair slot + XCD)
    int mb_hi;         // one past its last row block
    int slots;         // pair slots * row blocks * hgroups
    FastDiv d_ipp;     // division by its items per pair: row blocks * hgroups
  } sec[2];
  FastDiv d_nbh, d_hkv, d_hgroups;  // divisions by B * Hkv, Hkv, hgroups
  long long* diag;     // INTRA_DIAG_TIMERS builds: DIAG_SLOTS counters per workgroup, or null
};

// Phase timers of diagnostic builds (-DINTRA_DIAG_TIMERS): wavefront 0 of every workgroup adds up,
// over its work items, the 100 MHz wall clock spent in each phase and the shader cycles of the tile
// loop, and stores DIAG_SLOTS values at the end: [0] item set-up, [1] first barrier, [2] first key
// block, [3] tile loop, [4] next-item look-up, normalisation and output stores, [5] work items,
// [6] tiles, [7] shader cycles of the tile loops; then shader cycles spent at the barriers, split into
// the wait for the wavefront's own requests and LDS reads and the wait for the other wavefronts:
// [8], [9] the barrier in front of the Q slots, [10], [11] the one in front of the first key block,
// [12], [13] the one that opens tile 0, [14], [15] all barriers between tiles.  Production builds
// compile none of it.
constexpr int DIAG_SLOTS = 16;
#ifdef INTRA_DIAG_TIMERS
#define INTRA_DIAG(...) __VA_ARGS__
#else
#define INTRA_DIAG(...)
#endif

// Ablations for measurement builds: -DINTRA_ABLATE=<n> removes one ingredient of the hand-scheduled
// step so that its share of the time can be read off the phase timers.  The results of such a build
// are wrong by construction (the instruction mix is what is measured), so it only compiles together
// with the timers, and intra_diag_ablation() reports the number.
//   1: the V^T operands are not read from LDS (a Q fragment stands in)
//   2: the K operands are not re-read in the PV slots (the first block's stay)
//   3: no barrier between tiles
//   4: no exponentials, packing or row sums (Q fragments stand in for the weights)
//   5: every exponential, packing and row-sum instruction issued twice
//   6: the loader requests the same 64 rows for every tile (no address arithmetic, and every request hits the L2)
#ifndef INTRA_ABLATE
#define INTRA_ABLATE 0
#endif
#if INTRA_ABLATE != 0 && !defined(INTRA_DIAG_TIMERS)
#error "INTRA_ABLATE belongs to measurement builds (-DINTRA_DIAG_TIMERS): its results are wrong on purpose"
#endif

// softmax arithmetic of a pass (template argument SM)
constexpr int SM_EXACT = 0, SM_FOLDED = 1, SM_SCALED = 2;

constexpr int BN = 64;             // keys per tile (one barrier per tile)
// LDS tile layout.  A tile is 16 groups of 4 rows; a group is 1024 contiguous bytes (what one
// 16-bytes-per-lane direct-to-LDS load instruction writes) followed by padding.  Inside a group,
// the 16-byte chunk c of row i (0..3) sits at chunk slot c ^ (4 * i).  The padding is chosen for
// the operand reads of the MFMA shape in use, which must touch 16 distinct 16-byte bank groups per
// LDS cycle.  A 16-bytes-per-lane read is served 16 lanes per cycle, in the lane sets
// {0-3, 12-15, 20-23, 24-27}, {4-7, 8-11, 16-19, 28-31} and the same + 32 (found by counting
// SQ_LDS_BANK_CONFLICT for both layouts below); an 8-bytes-per-lane transposing read 32 lanes per cycle.
//  * 32 bytes of padding suits 16x16x32 MFMAs (this kernel and the backward kernels): lane l reads
//    row l % 16 at chunk 4 * ks + l / 16, and its transposing reads take 4 rows x 32 bytes of two
//    neighbouring groups.
//  * (16 bytes of padding suits the operand pattern of 32x32x16 MFMAs: lane l reads row l % 32 at
//    chunk 2 * ks + l / 32, and its transposing reads take 4 rows x 64 bytes of one group.)
constexpr int FGROUP_STRIDE = 1024 + 32;
constexpr int FTILE = (BN / 4) * FGROUP_STRIDE;
constexpr int FBLOCK32 = 8 * FGROUP_STRIDE;  // 32 rows
constexpr int NKBUF = 4, NVBUF = 4;   // tiles i-1 (being overwritten) .. i+2 of K and of V
constexpr int VBASE = NKBUF * FTILE;  // K ring then V ring
constexpr int RING_BYTES = (NKBUF + NVBUF) * FTILE;
constexpr int REDO_WORDS = 64;        // bitmap of work-item rounds to run again in EXACT mode (round % 2048)
constexpr int LDS_BYTES = RING_BYTES + REDO_WORDS * 4;

// 64 lanes x 16 bytes from per-lane global addresses to 1024 consecutive LDS bytes at lds_addr
// (wave-uniform).  Issued as inline assembly so that the compiler does not put a full vmcnt(0)
// wait in front of every later LDS read; completion is tracked by hand with vmcnt (see the main
// loop), and the "memory" clobber keeps LDS accesses from moving across it at compile time.
__device__ __forceinline__ void dma_group(const void* gsrc, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dwordx4 %0, off" : : "v"(gsrc), "s"(lds_addr) : "memory");
}

// Workgroup barrier that leaves the `pending` most recent direct-to-LDS loads of this wavefront
// in flight: waits for all its LDS reads (so buffers it was reading may be overwritten) and for
// all but `pending` of its loads (so older tiles are complete), then s_barrier.
template <int PENDING>
__device__ __forceinline__ void tile_barrier() {
  asm volatile("" ::: "memory");
  __builtin_amdgcn_s_waitcnt((PENDING & 15) | ((PENDING >> 4) << 14) | (7 << 4) | (0 << 8));
  __builtin_amdgcn_s_barrier();
  asm volatile("" ::: "memory");
}

__device__ __forceinline__ float lane_xor32_max(float x) {
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float lane_xor32_sum(float x) {
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}
// the same over the four lanes l % 16, l % 16 + 16, + 32, + 48 (the lanes that share a query in the
// 16x16 accumulator layout of the forward kernel)
__device__ __forceinline__ float lane_quad_max(float x) {
  auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return lane_xor32_max(fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1])));
}
__device__ __forceinline__ float lane_quad_sum(float x) {
  auto r = __builtin_amdgcn_permlane16_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return lane_xor32_sum(__uint_as_float(r[0]) + __uint_as_float(r[1]));
}

#ifdef INTRA_DIAG_TIMERS
// the same, adding the shader cycles of its two waits to w[0] (own requests, LDS reads) and w[1] (barrier)
template <int PENDING>
__device__ __forceinline__ void tile_barrier_timed(long long* w) {
  asm volatile("" ::: "memory");
  const long long a = __builtin_readcyclecounter();
  __builtin_amdgcn_s_waitcnt((PENDING & 15) | ((PENDING >> 4) << 14) | (7 << 4) | (0 << 8));
  const long long b = __builtin_readcyclecounter();
  __builtin_amdgcn_s_barrier();
  const long long c = __builtin_readcyclecounter();
  w[0] += b - a;
  w[1] += c - b;
  asm volatile("" ::: "memory");
}
#define INTRA_TILE_BARRIER(PENDING, W) tile_barrier_timed<PENDING>(W)
#else
#define INTRA_TILE_BARRIER(PENDING, W) tile_barrier<PENDING>()
#endif

// A work item: round = the workgroup's round it was dealt in
struct Where {
  int round, set, batch, kvh, mblk, hg;
};
// Key range of a row block: tiles of BN keys counted from kt_lo.
struct Range {
  int kt_lo, ntiles;
};
template <class MAP, int POS>
IM_HD Range range_of_block(const MAP& map, int mblk) {
  const int t0 = mblk * POS;
  const int t1 = im_min(t0 + POS, map.nq()) - 1;
  const int kt_lo = MAP::kHasPrefix ? 0 : map.klo(t0);  // first key the row block looks at
  const int kt_hi = im_min(map.khi(t1), map.nk() - 1);
  return Range{kt_lo, (kt_hi - kt_lo + BN) / BN};
}

// Dealing of work items.  Workgroups are handed to the 8 XCDs round-robin by id, so workgroup
// id % 8 names the XCD.  All row blocks of one (batch, kv head, set) "pair" go to one XCD, one pair
// after the other, longest row block first, so that the pair's K/V stays in that XCD's L2 while its
// row blocks run.  Inside an XCD the slots are dealt to its workgroups in boustrophedon order
// (0..w-1, w-1..0, ...), which balances the triangular causal workloads.
// locate_item: the first non-empty work item of workgroup `wg_in_xcd` (of `wgs_per_xcd`) of XCD `xcd`
// at or after `round`; false when there is none.  `redo` (device, second pass only): bitmap of the
// rounds to visit.  Also runs on the host, where tests enumerate what every workgroup is dealt.
template <class MAP, int POS, bool REDO>
IM_HD bool locate_item(const KParams& p, int xcd, int wgs_per_xcd, int wg_in_xcd, const uint32_t* redo, int round, Where& w) {
  for (;; ++round) {
    const int slot = round * wgs_per_xcd + ((round & 1) ? wgs_per_xcd - 1 - wg_in_xcd : wg_in_xcd);
    if (slot >= p.n_slots) return false;
    if (REDO && !((redo[(round >> 5) & (REDO_WORDS - 1)] >> (round & 31)) & 1u)) continue;
    const bool second = slot >= p.sec[0].slots;
    const int sslot = second ? slot - p.sec[0].slots : slot;
    const KParams::Section& sc = p.sec[second ? 1 : 0];
    const int pq = (int)fd_div(sslot, sc.d_ipp);
    const int pair = (sc.p_lo + pq) * 8 + xcd;
    if (pair >= p.n_pairs) continue;
    const int rem = sslot - pq * (int)sc.d_ipp.d;
    const int rblk = (int)fd_div(rem, p.d_hgroups);
    w.round = round;
    w.set = (int)fd_div(pair, p.d_nbh);
    const int bh = pair - w.set * (int)p.d_nbh.d;
    w.batch = (int)fd_div(bh, p.d_hkv);
    w.kvh = bh - w.batch * p.Hkv;
    w.mblk = sc.mb_hi - 1 - rblk;
    w.hg = rem - rblk * p.hgroups;
    if (w.mblk * POS >= MAP(p.geom, w.set, w.mblk * POS).nq()) continue;
    return true;
  }
}

template <int V>
using ic = std::integral_constant<int, V>;

// One pass of a workgroup over its work items.  SM: softmax arithmetic, see the file comment.
// REDO: visit only the items whose round is marked in `redo` (the SM_EXACT second pass of a kernel
// whose first pass keeps no running maximum).
template <class MAP, int HP, int NW, int SM, bool REDO>
__device__ __forceinline__ void run_pass(const KParams& p, unsigned char* smem, uint32_t* redo) {
  constexpr int POS = NW * 32 / HP;          // in-set queries per row block
  constexpr bool FAST = SM != SM_EXACT;      // no running maximum: the weight sums are checked at the end
  static_assert(BN % NW == 0, "tile rows must split evenly over the wavefronts");
  static_assert(!(FAST && REDO), "the second pass is exact");

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l16 = lane & 15;  // row or column of a 16x16 MFMA tile
  const int g4 = lane >> 4;   // which quarter of the wavefront

  // ---------------------------------------------------------------- persistent loop over work items
  // The grid holds about one workgroup per CU and every workgroup walks through several work items
  // (row blocks), which saves the dispatch gap between consecutive workgroups on a CU; see
  // locate_item for the order.
  const int xcd = blockIdx.x & 7;
  const int wgs_per_xcd = gridDim.x >> 3;
  const int wg_in_xcd = blockIdx.x >> 3;
  auto locate = [&](int round, Where& w) {
    return locate_item<MAP, POS, REDO>(p, xcd, wgs_per_xcd, wg_in_xcd, redo, round, w);
  };
  auto range_of = [&](const MAP& map, int mblk) { return range_of_block<MAP, POS>(map, mblk); };

  // ---------------------------------------------------------------- loader: HBM rows -> LDS
  // One global_load_lds_dwordx4 moves a 4-row group: lane L fetches 16 bytes of row L/16 and the
  // hardware writes the 64 x 16 bytes to consecutive LDS addresses from M0, so lane L has to
  // fetch the chunk that belongs into slot L%16 of its row.  No VGPR staging and no LDS store
  // instructions; rows past the last key are clamped to it.
  //
  // The K/V tiles of all work items of this workgroup form one stream that runs through the LDS
  // ring without a break: the loader has its own cursor (`fd`), three tiles ahead of the
  // computation, and moves on to the next work item when it has requested the last tile of one.
  // So the first tiles of a work item arrive while the previous one is still computing.
  constexpr int GROUPS_PER_WAVE = (BN / 4) / NW;
  static_assert((BN / 4) % NW == 0, "tile groups must split evenly over the wavefronts");
  const int ld_row = lane >> 4;                                  // row of the group this lane fetches
  const uint32_t ld_col = (((lane & 15) ^ (4 * ld_row)) << 4);   // byte column it fetches
  const uint32_t k_rs_b = p.k_rs_bytes, v_rs_b = p.v_rs_bytes, q_rs_b = p.q_rs_bytes;
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)smem;
  // The stream of a work item: slots -2 and -1 carry its 256 Q rows (wavefront w reads rows
  // 32 * (w % 2) .. of the K part (w / 2 even) or V part (w / 2 odd) of slot w / 4), slots 0 .. ntiles-1
  // its key tiles.
  static_assert(NW == 8, "the Q slots are laid out for 8 wavefronts");
  struct Feed {
    MAP map;
    Range rg;
    int nk, tile;      // tile: -2, -1 (Q slots), then the key tile being requested next
    bool more;         // false once the last work item has been requested completely
    const char *kbase, *vbase, *qbase;
    int t0, t1;        // first and last in-set query of the row block
    Where w;           // the work item whose slots are being requested
    int prev_round;    // round of the work item before it
  };
  auto feed_for = [&](const Where& w, int prev_round) {
    const MAP map(p.geom, w.set, w.mblk * POS);
    return Feed{map, range_of(map, w.mblk), map.nk(), -2, true,
                reinterpret_cast<const char*>(p.k + w.batch * p.k_bs + w.kvh * p.k_hs),
                reinterpret_cast<const char*>(p.v + w.batch * p.v_bs + w.kvh * p.v_hs),
                reinterpret_cast<const char*>(p.q + w.batch * p.q_bs + (int64_t)(w.kvh * p.ratio + w.hg * HP) * p.q_hs),
                w.mblk * POS, im_min(w.mblk * POS + POS, map.nq()) - 1, w, prev_round};
  };
  Where cw;
  if (!locate(0, cw)) return;
  long long* dgw = nullptr;  // measurement builds: the barrier counters
  INTRA_DIAG(long long dg[DIAG_SLOTS] = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0}; dgw = dg + 8;)
  Feed fd = feed_for(cw, -1);
  // request the next slot of the stream into a ring slot (byte offset inside the K ring and the V ring)
  auto feed_tile = [&](int slot_off) {
    if (fd.tile < 0) {  // 128 Q rows: rows of four wavefronts, two per part
#pragma unroll
      for (int gi = 0; gi < GROUPS_PER_WAVE; ++gi) {
        const int grp = wave * GROUPS_PER_WAVE + gi;
        const int rho = 4 * grp + ld_row;  // row of the part
#pragma unroll
        for (int part = 0; part < 2; ++part) {
          const int wq = (fd.tile + 2) * 4 + part * 2 + (rho >> 5);  // the wavefront that will read this row
          const int t = im_min(fd.t0 + (wq / HP) * 32 + (rho & 31), fd.t1);
          const uint32_t pos = fd.map.qpos(t);
          dma_group(fd.qbase + ((int64_t)(wq % HP) * p.q_hs * 2 + (uint64_t)pos * q_rs_b + ld_col),
                    lds_base + part * VBASE + slot_off + grp * FGROUP_STRIDE);
        }
      }
    } else if (TileRows tr; INTRA_ABLATE != 6 && map_tile_rows(fd.map, fd.rg.kt_lo + fd.tile * BN, tr)) {
      // (wave-uniform) a tile whose key positions are affine: no per-key index arithmetic
      const uint32_t row = (uint32_t)(ld_row * tr.row_step);
#pragma unroll
      for (int gi = 0; gi < GROUPS_PER_WAVE; ++gi) {
        const int grp = wave * GROUPS_PER_WAVE + gi;
        const uint32_t pos = (uint32_t)(tr.base + grp * tr.group_step) + row;
        dma_group(fd.kbase + ((uint64_t)pos * k_rs_b + ld_col), lds_base + slot_off + grp * FGROUP_STRIDE);
        dma_group(fd.vbase + ((uint64_t)pos * v_rs_b + ld_col), lds_base + VBASE + slot_off + grp * FGROUP_STRIDE);
      }
    } else {
#pragma unroll
      for (int gi = 0; gi < GROUPS_PER_WAVE; ++gi) {
        const int grp = wave * GROUPS_PER_WAVE + gi;
        if (INTRA_ABLATE == 6) {
          const char* row = reinterpret_cast<const char*>(p.k) + ((uint32_t)(4 * grp + ld_row) * k_rs_b + ld_col);
          dma_group(row, lds_base + slot_off + grp * FGROUP_STRIDE);
          dma_group(row + 256, lds_base + VBASE + slot_off + grp * FGROUP_STRIDE);
          continue;
        }
        const int tk = im_min(fd.rg.kt_lo + fd.tile * BN + 4 * grp + ld_row, fd.nk - 1);
        const uint32_t pos = fd.map.kpos(tk);
        dma_group(fd.kbase + ((uint64_t)pos * k_rs_b + ld_col), lds_base + slot_off + grp * FGROUP_STRIDE);
        dma_group(fd.vbase + ((uint64_t)pos * v_rs_b + ld_col), lds_base + VBASE + slot_off + grp * FGROUP_STRIDE);
      }
    }
    ++fd.tile;
    if (fd.tile == fd.rg.ntiles && fd.more) {
      Where w;
      if (locate(fd.w.round + 1, w)) fd = feed_for(w, fd.w.round);
      else fd.more = false;  // nothing left: keep requesting the (clamped) last row, nobody reads it
    }
  };
  constexpr int PER_TILE = 2 * GROUPS_PER_WAVE;  // requests per wavefront per slot (K + V parts)

  // LDS operand addresses.  A 32-key block times the wavefront's 32 queries is 2 x 2 MFMA tiles of
  // 16 x 16 with 4 k-steps of 32 head dims; lane (l16, g4) supplies head dims 32 * ks + 8 * g4 .. + 7,
  // the 16-byte chunk 4 * ks + g4, of key row 16 * kt + l16.  With the chunk swizzle c ^ 4i of a
  // group that chunk sits at byte 64 * (ks ^ r) + 16 * g4 of its row slot, r = l16 % 4: four
  // lane-dependent bases (one per ks) and compile-time offsets for everything else, which the
  // ds_read offset field takes.  The bases carry the ring slot and are advanced once per tile:
  // kb[] follows the tile AFTER the one being multiplied (whose K rows the pipeline reads ahead),
  // vb[] the current one.
  const int lane_chunks = (l16 & 3) * 256 + 16 * g4;  // row slot inside the group + chunk g4, before the swizzle
  int kb[4], vb[4];
  {
    const int r = l16 & 3;
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) kb[ks] = FTILE + (l16 >> 2) * FGROUP_STRIDE + lane_chunks + 64 * (ks ^ r);
    // V^T operand (A of O^T = V^T P^T) through transposing reads.  Within each group of 16 lanes,
    // lane i supplies the address of 4 head dims (4*(i%4)..) of key row i/4 and receives head dim i
    // of those 4 key rows.  The MFMA's 32-key reduction is numbered so that lane quarter g4 holds
    // keys 4*g4 .. +3 and 16 + 4*g4 .. +3 of the block (what the score accumulators of that lane
    // hold, see below): two reads, of row groups g4 and 4 + g4.  vb[a]: head dims 32*a .. 32*a+31,
    // the 16-dim tile 2*a + b another 32 bytes further.
    const int ri = l16 >> 2;
#pragma unroll
    for (int a = 0; a < 4; ++a)
      vb[a] = VBASE + g4 * FGROUP_STRIDE + ri * 256 + 64 * (a ^ ri) + 16 * ((l16 & 3) >> 1) + 8 * (l16 & 1);
  }
  // Q^T fragments (B operand of S^T = K Q^T): qf[qt][ks] is chunk 4 * ks + g4 of query 16 * qt + l16
  bf16x8 qf[2][4];
  auto kread_q = [&](int addr) { return *reinterpret_cast<const bf16x8*>(smem + addr); };

  // Ring slots (byte offsets into the K ring; the V ring uses the same offsets behind VBASE) of
  // the stream tiles i, i+1, i+2, i+3 seen from the computation; they rotate once per tile and
  // carry on from one work item to the next.
  int k0 = 0, k1 = FTILE, k2 = 2 * FTILE, k3 = 3 * FTILE;
  feed_tile(k0);  // the two Q slots of the first work item and its first key tile
  feed_tile(k1);
  feed_tile(k2);
  auto rotate = [&] {  // one slot further in the stream
    const int dk = k2 - k1, dv = k1 - k0;  // one tile, or minus three where the ring wraps
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      kb[a] += dk;
      vb[a] += dv;
    }
    const int tk = k0;
    k0 = k1; k1 = k2; k2 = k3; k3 = tk;
  };
  // Barrier in front of a slot, leaving this wavefront's requests for the slot after the next in
  // flight (PER_TILE operations) and the `extra` stores of the previous work item's output (0, 8 or
  // 9; wave-uniform), wherever those sit among the PER_TILE + extra most recent operations.  The
  // operation counter retires in issue order, so everything older than that has landed.
  auto slot_barrier = [&](int extra, long long* w) {
    (void)w;
    if (extra == 0) INTRA_TILE_BARRIER(PER_TILE, w);
    else if (extra == 8) INTRA_TILE_BARRIER(PER_TILE + 8, w);
    else INTRA_TILE_BARRIER(PER_TILE + 9, w);
  };
  // Vector-memory stores this wavefront issued for the output of the previous work item (0, 8, or 9
  // with a log-sum-exp).  They go out right after the item's tile loop - the wavefronts leave that
  // loop at different times (the diagonal tile gives some of them one block more), so the early ones
  // get their stores through the memory pipeline while the late ones still compute - and may stay in
  // flight across the first two barriers of the next item.
  int stored = 0;

  for (;;) {
  INTRA_DIAG(const long long t_a = wall_clock64();)
  const int set = cw.set, batch = cw.batch, kvh = cw.kvh, mblk = cw.mblk, hg = cw.hg;
  const int t0 = mblk * POS;
  const MAP map(p.geom, set, t0);
  const int nq = map.nq();
  const int nk = map.nk();
  const int t1 = im_min(t0 + POS, nq) - 1;
  const int kpre = map.kpre();  // keys every query of the set sees (0 if none)
  const Range rg = range_of(map, mblk);
  const int kt_lo = rg.kt_lo, ntiles = rg.ntiles;

  // ---------------------------------------------------------------- this wavefront's queries
  // A lane works for two queries: 16 * qt + l16 of the wavefront's 32, qt = 0, 1.  Rows past the
  // end of the row block are clamped to its last row, for Q and for O alike: such lanes compute
  // that row once more and store the same bytes to the same place, so every active wavefront
  // issues all of its stores.
  const int hw = wave % HP;
  const int wq0 = t0 + (wave / HP) * 32;
  const bool wave_active = wq0 <= t1;
  const int wq_last = im_min(wq0 + 31, t1);
  bool row_valid[2];
  int lo_l[2], hi_l[2];
  int64_t qpos[2];
#pragma unroll
  for (int qt = 0; qt < 2; ++qt) {
    row_valid[qt] = wq0 + 16 * qt + l16 <= t1;
    const int tq = im_min(wq0 + 16 * qt + l16, t1);
    lo_l[qt] = map.klo(tq);
    hi_l[qt] = im_min(map.khi(tq), nk - 1);
    qpos[qt] = map.qpos(tq);
  }
  WaveBounds wb = wave_bounds(map, im_min(wq0, t1), wq_last);
  // 32-key blocks (counted from kt_lo) this wavefront has to look at: those of its own key range
  // and, for maps with a prefix, the prefix blocks in front of it.
  int bw_lo = __builtin_amdgcn_readfirstlane((wb.w_lo - kt_lo) / 32);
  int bw_hi = __builtin_amdgcn_readfirstlane((wb.w_hi - kt_lo) / 32);
  // last prefix block it looks at (a causal bound may end the prefix early)
  int bp_hi = MAP::kHasPrefix && kpre > 0 ? __builtin_amdgcn_readfirstlane(im_min(kpre - 1, wb.w_hi) / 32) : -1;
  if (!wave_active || wb.w_lo > wb.w_hi) {  // no own range: an empty run of steps
    bw_lo = 2;
    bw_hi = 0;
  }
  if (!wave_active) bp_hi = -1;
  wb.f_lo = __builtin_amdgcn_readfirstlane(wb.f_lo);
  wb.f_hi = __builtin_amdgcn_readfirstlane(wb.f_hi);
  wb.w_lo = __builtin_amdgcn_readfirstlane(wb.w_lo);
  wb.w_hi = __builtin_amdgcn_readfirstlane(wb.w_hi);

  const int hq = kvh * p.ratio + hg * HP + hw;

  // ---------------------------------------------------------------- slot -2: the Q rows arrive
  INTRA_DIAG(const long long t_b = wall_clock64();)
  const int in_flight = stored;
  slot_barrier(in_flight, dgw);  // both Q slots have landed; behind them: the first key tile's requests, then the stores
  INTRA_DIAG(const long long t_c = wall_clock64();)
  feed_tile(k3);
  {
    // this wavefront's 32 rows: slot wave / 4 (ring slot 0 or 1 of the stream as it stands), part
    // (wave / 2) % 2, rows 32 * (wave % 2) .. of the part; read with the K operand's pattern
    // address of row l16's chunk g4 before the k-step swizzle
    const int qa = ((wave >> 1) & 1) * VBASE + ((wave >> 2) ? k1 : k0) + (wave & 1) * FBLOCK32 +
                   (l16 >> 2) * FGROUP_STRIDE + lane_chunks;
    constexpr int qstep = 4 * FGROUP_STRIDE;  // from query tile 0 to 1
    const int r = l16 & 3;
    u32x4 raw[8];
#pragma unroll
    for (int qt = 0; qt < 2; ++qt)
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) raw[4 * qt + ks] = __builtin_bit_cast(u32x4, kread_q(qa + qt * qstep + 64 * (ks ^ r)));
    if (SM == SM_FOLDED) {  // Q <- bf16(Q * softmax_scale * log2 e): the MFMA then yields exponents directly
      const float cq = p.q_fold;
#pragma unroll
      for (int f = 0; f < 8; ++f)
#pragma unroll
        for (int d = 0; d < 4; ++d) {
          const uint32_t x = raw[f][d];
          floatx2 y = {__uint_as_float(x << 16) * cq, __uint_as_float(x & 0xffff0000u) * cq};
          raw[f][d] = __builtin_bit_cast(uint32_t, __builtin_convertvector(y, bf16x2));
        }
    } else if (p.negate_q) {  // softmax_scale < 0: flip the sign of Q (exact) and use |scale| below
#pragma unroll
      for (int f = 0; f < 8; ++f) raw[f] ^= 0x80008000u;
    }
#pragma unroll
    for (int f = 0; f < 8; ++f) qf[f >> 2][f & 3] = __builtin_bit_cast(bf16x8, raw[f]);
  }
  rotate();

  // ---------------------------------------------------------------- running softmax state
  // oacc[dt][qt]: O^T tile of head dims 16 * dt .. + 15 and query tile qt; the lane holds head dims
  // 16 * dt + 4 * g4 .. + 3 of query 16 * qt + l16.
  floatx4 oacc[8][2];
#pragma unroll
  for (int dt = 0; dt < 8; ++dt)
#pragma unroll
    for (int qt = 0; qt < 2; ++qt) oacc[dt][qt] = floatx4{0.f, 0.f, 0.f, 0.f};
  // Raw scores q.k of two consecutive 32-key blocks, [kt][qt]: the lane holds keys
  // 16 * kt + 4 * g4 .. + 3 of the block for query 16 * qt + l16.
  floatx4 s0[2][2], s1[2][2];
  // Exponent reference of each of the lane's queries.  Weights are exp2(score * c - mref) and
  // numerator and denominator always share mref, so any value gives the exact softmax as long as
  // nothing overflows or underflows.  fp32 and bf16 both span 2^+-126, so mref stays 0 (and costs
  // nothing) for every query whose scores stay within +-60 of it; it is re-centred on a block's
  // maximum when that maximum leaves this band upwards, or downwards before anything was
  // accumulated.  SM_SCALED and SM_FOLDED have no reference at all (weights exp2(score * c), or
  // exp2(score) with the scores already in exponent units).
  float mref[2] = {0.f, 0.f};
  float l_acc[2] = {0.f, 0.f};  // this lane's share of the two queries' weight sums
  const float c = p.scale_log2;  // |softmax_scale| * log2(e)

  // operand reads: base register + compile-time byte offset
  auto kread_at = [&](int base, int off) { return *reinterpret_cast<const bf16x8*>(smem + (base + off)); };
  auto vread_at = [&](int base, int off) {
    bf16x4 x0 = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((__attribute__((address_space(3))) bf16x4*)(smem + (base + off)));
    bf16x4 x1 = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
        (__attribute__((address_space(3))) bf16x4*)(smem + (base + off + 4 * FGROUP_STRIDE)));
    return __builtin_shufflevector(x0, x1, 0, 1, 2, 3, 4, 5, 6, 7);
  };
  auto mfma = [](bf16x8 a, bf16x8 b, floatx4 acc) { return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, acc, 0, 0, 0); };
  const floatx4 zero4 = {0.f, 0.f, 0.f, 0.f};

  // ----- unscheduled pieces, used at the edges of a wavefront's key range
  // K operands of a 32-key block, ka[2 * ks + kt] in the order the MFMAs take them: `delta` = its
  // tile's ring slot minus the slot kb[] points to
  auto load_ka = [&](bf16x8 (&ka)[8], int delta, int half) {
#pragma unroll
    for (int f = 0; f < 8; ++f) ka[f] = kread_at(kb[f >> 1] + delta, (f & 1) * 4 * FGROUP_STRIDE + half);
  };
  auto mask_block = [&](floatx4 (&s)[2][2], int kb32) {
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int qt = 0; qt < 2; ++qt)
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          const int key = kb32 + 16 * kt + 4 * g4 + e;
          if (!key_visible(key, kpre, lo_l[qt], hi_l[qt])) s[kt][qt][e] = -INFINITY;
        }
  };
  // this lane's part of a block's maximum for query tile qt, and the whole of it
  auto lane_max = [&](const floatx4 (&s)[2][2], int qt) {
    const float a = fmaxf(fmaxf(s[0][qt][0], s[0][qt][1]), fmaxf(s[0][qt][2], s[0][qt][3]));
    const float b = fmaxf(fmaxf(s[1][qt][0], s[1][qt][1]), fmaxf(s[1][qt][2], s[1][qt][3]));
    return fmaxf(a, b);
  };
  auto block_max = [&](const floatx4 (&s)[2][2], float (&mx)[2]) {
    mx[0] = lane_quad_max(lane_max(s, 0));
    mx[1] = lane_quad_max(lane_max(s, 1));
  };
  // EXACT mode: what can happen to a freshly computed block of raw scores q.k before it is
  // exponentiated as exp2(score * c - mref); all of it is rare.  `mx` are the block maxima of the
  // raw scores of the lane's two queries.  Four lanes hold a query (disjoint keys and head dims),
  // so every decision here is taken per query: maximum and running sum are taken over the four.
  auto settle = [&](floatx4 (&nxt)[2][2], float (&mx)[2], bool masked, int kb32) {
    if (masked) {  // block cut by a bound: mask in place, then redo the maximum
      mask_block(nxt, kb32);
      block_max(nxt, mx);
    }
    const float mxs[2] = {__builtin_fmaf(mx[0], c, -mref[0]), __builtin_fmaf(mx[1], c, -mref[1])};  // in exponent units
    if (__builtin_amdgcn_ballot_w64(fmaxf(__builtin_fabsf(mxs[0]), __builtin_fabsf(mxs[1])) > 60.f) == 0) return;  // the usual case
#pragma unroll
    for (int qt = 0; qt < 2; ++qt) {
      const float l_run = lane_quad_sum(l_acc[qt]);  // of the query, not of this lane's keys
      const bool need = mxs[qt] > 60.f || (l_run == 0.f && mxs[qt] < -60.f && mxs[qt] > -INFINITY);
      if (__builtin_amdgcn_ballot_w64(need) != 0) {
        const float delta = need ? mxs[qt] : 0.f;
        const float alpha = l_run == 0.f ? 1.f : __builtin_amdgcn_exp2f(-delta);
        mref[qt] += delta;
        l_acc[qt] *= alpha;
#pragma unroll
        for (int dt = 0; dt < 8; ++dt) oacc[dt][qt] *= alpha;
      }
    }
  };
  // a freshly computed block of scores, before its weights are formed
  auto finish_scores = [&](floatx4 (&nxt)[2][2], float (&mx)[2], bool masked, int kb32) {
    if (FAST) {
      if (masked) mask_block(nxt, kb32);
    } else {
      settle(nxt, mx, masked, kb32);
    }
  };

  // ----- hand-scheduled step: QK^T of the next key block (16 MFMAs) and PV of the current one
  // (16 MFMAs) with the softmax VALU work spread between them.  One "slot" is one MFMA.  LDS
  // operands are fetched about a phase ahead: the V^T operands of this step's PV during its QK^T
  // slots, the K operands of the NEXT step's QK^T during the second half of this step's PV slots
  // (ka lives across steps and across the tile barrier: the K tile it reads was made visible by an
  // earlier barrier and is not overwritten before the next one).  The score accumulators are the
  // B operand of PV as they stand: the lane's 8 weights of query tile qt, packed to bf16, are
  // keys 4*g4 .. +3 and 16 + 4*g4 .. +3 of the block, the numbering the V^T reads follow.  PV
  // runs query tile 0 first, so the weights of query tile 1 are only needed 8 slots later: the
  // exponentials of the 8 bf16 pairs are spread over slots 0..20 of the 32, the packing and the row sums
  // follow two slots behind, and in EXACT mode the maximum of the next block is taken in the last
  // PV slots once its MFMA chain has drained.  sched_barrier keeps the compiler from regrouping
  // the slots.
  bf16x8 ka[8];
  // HALF: which half of its tile the V reads (block j) and the K reads (block j + 2, one tile
  // further) address: the same for both.
  auto steady = [&](const floatx4 (&s)[2][2], floatx4 (&n)[2][2], auto half_c, bool mask_next, int kb32_next) {
    constexpr int HALF = decltype(half_c)::value;
    bf16x8 va[8], pb[2];
    float px[8][2];
    // pair u = 4 * qt + 2 * kt + h: weights of keys 16 * kt + 4 * g4 + 2 * h, + 1 for query tile qt
    auto stage_e = [&](int u) {
      const int qt = u >> 2, kt = (u >> 1) & 1, h = u & 1;
      if (SM == SM_FOLDED) {
        px[u][0] = __builtin_amdgcn_exp2f(s[kt][qt][2 * h]);
        px[u][1] = __builtin_amdgcn_exp2f(s[kt][qt][2 * h + 1]);
      } else if (SM == SM_SCALED) {
        px[u][0] = __builtin_amdgcn_exp2f(s[kt][qt][2 * h] * c);
        px[u][1] = __builtin_amdgcn_exp2f(s[kt][qt][2 * h + 1] * c);
      } else {
        px[u][0] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[kt][qt][2 * h], c, -mref[qt]));
        px[u][1] = __builtin_amdgcn_exp2f(__builtin_fmaf(s[kt][qt][2 * h + 1], c, -mref[qt]));
      }
    };
    uint32_t hx[8];
    auto stage_c = [&](int u) {
      floatx2 f = {px[u][0], px[u][1]};
      bf16x2 h2 = __builtin_convertvector(f, bf16x2);
      hx[u] = __builtin_bit_cast(uint32_t, h2);
      pb[u >> 2][2 * (u & 3)] = h2[0];
      pb[u >> 2][2 * (u & 3) + 1] = h2[1];
    };
    // The row sum takes what PV multiplies: the two rounded weights of the pair, by one dot-product
    // instruction with (1, 1).  (Widening them back to fp32 with a shift and a mask and adding
    // twice - four plain instructions - measured 7 % slower: in this loop every instruction issued
    // beside the MFMAs costs its cycles.)
    auto stage_s = [&](int u) {
      const bf16x2 ones2 = {(__bf16)1.0f, (__bf16)1.0f};
      l_acc[u >> 2] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, hx[u]), ones2, l_acc[u >> 2], false);
    };
    // slot (0..31, PV slots from 16) in which the exponentials of pair u are issued
    auto valu_slot = [&](int k) {
      if (INTRA_ABLATE == 4) return;
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int es = u < 4 ? 4 * u : 2 * u + 6;
        if (es == k) stage_e(u);
        if (es + 2 == k) stage_c(u);
        if (es + 2 == k) stage_s(u);
        if (INTRA_ABLATE == 5) {  // the same instructions once more (the sums count twice, the rest is rewritten)
          if (es == k) {
            asm volatile("" : "+v"(px[u][0]), "+v"(px[u][1]));
            stage_e(u);
          }
          if (es + 2 == k) {
            asm volatile("" : "+v"(px[u][0]), "+v"(px[u][1]));
            stage_c(u);
          }
          if (es + 2 == k) stage_s(u);
        }
      }
    };
    if (INTRA_ABLATE == 4) pb[0] = qf[0][0], pb[1] = qf[1][0];
#pragma unroll
    for (int k = 0; k < 16; ++k) {  // QK^T: k-step ks, key tile kt, query tile qt
      const int ks = k >> 2, kt = (k >> 1) & 1, qt = k & 1;
      if ((k & 1) == 0) va[k >> 1] = INTRA_ABLATE == 1 ? qf[0][(k >> 1) & 3] : vread_at(vb[k >> 2], 32 * ((k >> 1) & 1) + HALF * FBLOCK32);
      n[kt][qt] = mfma(ka[2 * ks + kt], qf[qt][ks], ks == 0 ? zero4 : n[kt][qt]);
      valu_slot(k);
      __builtin_amdgcn_sched_barrier(0);
    }
    float m[2] = {0.f, 0.f};
#pragma unroll
    for (int k = 0; k < 16; ++k) {  // PV: query tile qt, head-dim tile dt
      const int qt = k >> 3, dt = k & 7;
      if (k >= 8 && INTRA_ABLATE != 2) ka[k - 8] = kread_at(kb[(k - 8) >> 1], (k & 1) * 4 * FGROUP_STRIDE + HALF * FBLOCK32);
      oacc[dt][qt] = mfma(va[dt], pb[qt], oacc[dt][qt]);
      valu_slot(16 + k);
      if (!FAST) {
        if (k == 12) m[0] = lane_max(n, 0);
        if (k == 14) m[1] = lane_max(n, 1);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
    if (!FAST) {
      m[0] = lane_quad_max(m[0]);
      m[1] = lane_quad_max(m[1]);
    }
    finish_scores(n, m, mask_next, kb32_next);
  };

  // Step j: softmax + PV of key block j (scores in `cur`, V rows in the current tile) and QK^T of
  // key block j+1 into `nxt` (its K rows are in ka already; those of block j+2 are read meanwhile).
  // A wavefront runs the steps jq..jp for a run of blocks jq+1..jp it looks at: in step jq only the
  // QK^T half matters, so its scores are preset to -inf (weights 0); in step jp the QK^T half
  // computes a block the wavefront does not look at, which the per-element mask turns into -inf.
  // That keeps one code path through the accumulators.  Maps with a prefix have two such runs
  // (prefix blocks, own range); they are merged when they touch.
  int jq1 = bw_lo - 1, jp1 = bw_hi, jq2 = 1, jp2 = 0;
  if (MAP::kHasPrefix && bp_hi >= 0) {
    if (bw_lo - 1 <= bp_hi) {  // the ranges touch: one run from the first prefix block on
      jq1 = -1;
      jp1 = im_max(bw_hi, bp_hi);
    } else {
      jq1 = -1;
      jp1 = bp_hi;
      jq2 = bw_lo - 1;
      jp2 = bw_hi;
    }
  }
  auto needs_mask = [&](int j) { return !block_unmasked(wb, kpre, kt_lo + 32 * j); };
  // half_c: which half of its tile block j is (0 / 1).  Block j + 1 is the other half of the same
  // tile (half 0) or the first half of the next tile (half 1).
  auto step = [&](int j, floatx4 (&cur)[2][2], floatx4 (&nxt)[2][2], auto half_c, auto with_loader, int free_slot) {
    constexpr int HALF = decltype(half_c)::value;
    if (decltype(with_loader)::value) feed_tile(free_slot);
    const bool in1 = j >= jq1 && j <= jp1, in2 = j >= jq2 && j <= jp2;
    if (!in1 && !in2) return;
    if (j == jq1 || (in2 && j == jq2)) {
#pragma unroll
      for (int t = 0; t < 4; ++t) cur[t >> 1][t & 1] = floatx4{-INFINITY, -INFINITY, -INFINITY, -INFINITY};
      if (HALF == 0) load_ka(ka, k0 - k1, FBLOCK32);  // second half of the current tile
      else load_ka(ka, 0, 0);                         // first half of the next tile
    }
    steady(cur, nxt, half_c, needs_mask(j + 1), kt_lo + 32 * (j + 1));
  };

  // ---------------------------------------------------------------- main loop
  // Stream tile t lives in ring slot t % 4 (of the K ring and of the V ring).  At the top of
  // iteration i the LDS holds tiles i and i+1; tile i+2 was requested during iteration i-1 and
  // may still be in flight.  Iteration i requests tile i+3 into the slot of tile i-1, which no
  // wavefront reads after the barrier that opened iteration i.  The barrier that opens iteration
  // i+1 only waits for the older requests, so every row has a whole iteration to arrive.
  // The two Q slots in front of a work item's tiles are iterations of the same kind without
  // tile work: the first reads Q out of LDS, the second computes the scores of key block 0.
  // ---------------------------------------------------------------- slot -1: the first key tile has landed
  slot_barrier(in_flight, dgw + 2);
  feed_tile(k3);
  if (jq1 < 0 && jp1 >= 0) {  // scores of key block 0, ahead of the pipeline (the tile sits in slot k1)
    load_ka(ka, 0, 0);
#pragma unroll
    for (int t = 0; t < 4; ++t) s0[t >> 1][t & 1] = zero4;
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      const int ks = k >> 2, kt = (k >> 1) & 1, qt = k & 1;
      s0[kt][qt] = mfma(ka[2 * ks + kt], qf[qt][ks], s0[kt][qt]);
    }
    float mx[2] = {0.f, 0.f};
    if (!FAST) block_max(s0, mx);
    finish_scores(s0, mx, needs_mask(0), kt_lo);
    load_ka(ka, 0, FBLOCK32);
  }
  rotate();
  INTRA_DIAG(const long long t_d = wall_clock64(); const long long c_d = __builtin_readcyclecounter();)
  INTRA_TILE_BARRIER(PER_TILE, dgw + 4);  // opens tile 0 (tile 1 was requested behind the stores: they are done too)
  for (int i = 0;;) {
    step(2 * i, s0, s1, ic<0>{}, ic<1>{}, k3);
    step(2 * i + 1, s1, s0, ic<1>{}, ic<0>{}, 0);
    rotate();
    if (++i == ntiles) break;
    if (INTRA_ABLATE != 3) INTRA_TILE_BARRIER(PER_TILE, dgw + 6);
  }

  INTRA_DIAG(const long long t_e = wall_clock64(); dg[7] += __builtin_readcyclecounter() - c_d;)
  // The loader is ahead by three slots, so it usually knows the next work item already.
  Where nw = fd.w;
  bool more = true;
  if (fd.w.round == cw.round) more = false;  // (the loader only stays on an item when it is the last)
  else if (fd.prev_round != cw.round) more = locate(cw.round + 1, nw);

  // ---------------------------------------------------------------- normalise and store
  {
  const float l_tot[2] = {lane_quad_sum(l_acc[0]), lane_quad_sum(l_acc[1])};
  if (FAST) {
    // Weights were formed without a reference: the result is good iff the weight sum stayed inside
    // 2^-100 .. 2^60 (no weight overflowed, and the largest ones are far from underflow).  The
    // integer comparison of the bit patterns also catches a negative or NaN sum.
    const uint32_t lb0 = __float_as_uint(l_tot[0]), lb1 = __float_as_uint(l_tot[1]);
    const bool bad = wave_active && ((row_valid[0] && !(lb0 >= 0x0d800000u && lb0 <= 0x5d800000u)) ||
                                     (row_valid[1] && !(lb1 >= 0x0d800000u && lb1 <= 0x5d800000u)));
    if (INTRA_ABLATE == 0 && __builtin_amdgcn_ballot_w64(bad) != 0 && lane == 0)  // (an ablated pass is not run again)
      __hip_atomic_fetch_or(&redo[(cw.round >> 5) & (REDO_WORDS - 1)], 1u << (cw.round & 31), __ATOMIC_RELAXED,
                            __HIP_MEMORY_SCOPE_WORKGROUP);
  }
  const float inv[2] = {l_tot[0] > 0.f ? 1.f / l_tot[0] : 0.f, l_tot[1] > 0.f ? 1.f / l_tot[1] : 0.f};
  stored = wave_active ? (p.lse != nullptr ? 9 : 8) : 0;
  if (wave_active) {
    // The four lanes of a query hold head dims 4 * g4 .. + 3 of every 16-dim tile.  For the tile pair
    // 2m, 2m+1 a lane quarter and its neighbour (g4 ^ 1) trade 8 bytes: the even one keeps its 4 dims
    // of tile 2m and receives the neighbour's (the next 4 dims), the odd one does the same for tile
    // 2m+1.  Each lane then owns one whole 16-byte chunk of the row, 4m + 2 * (g4 % 2) + g4 / 2, and
    // the four lanes of a query store 64 contiguous bytes per instruction.
    const int64_t ohead = batch * p.o_bs + hq * p.o_hs + (2 * (g4 & 1) + (g4 >> 1)) * 8;
#pragma unroll
    for (int qt = 0; qt < 2; ++qt) {
      uint16_t* orow = p.o + (ohead + qpos[qt] * p.o_rs);
#pragma unroll
      for (int m = 0; m < 4; ++m) {
        uint32_t w[2][2];
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int k = 0; k < 2; ++k) {
            floatx2 f = {oacc[2 * m + t][qt][2 * k] * inv[qt], oacc[2 * m + t][qt][2 * k + 1] * inv[qt]};
            w[t][k] = __builtin_bit_cast(uint32_t, __builtin_convertvector(f, bf16x2));
          }
        auto r0 = __builtin_amdgcn_permlane16_swap(w[0][0], w[1][0], false, false);
        auto r1 = __builtin_amdgcn_permlane16_swap(w[0][1], w[1][1], false, false);
        *reinterpret_cast<u32x4*>(orow + 32 * m) = u32x4{r0[0], r1[0], r0[1], r1[1]};
      }
    }
    // ln sum_j exp(scale * q.k_j) = (mref + log2 l) * ln 2; the lane quarters g4 = 0, 1 store the values of
    // query tiles 0, 1, the other two (and lanes of clamped rows) repeat them
    if (p.lse != nullptr) {
      const int qt = g4 & 1;
      p.lse[batch * p.lse_bs + hq * p.lse_hs + (qt ? qpos[1] : qpos[0]) * p.lse_ts] =
          ((qt ? mref[1] : mref[0]) + __builtin_amdgcn_logf(qt ? l_tot[1] : l_tot[0])) * 0.6931471805599453f;
    }
  }
  }
  INTRA_DIAG(dg[0] += t_b - t_a; dg[1] += t_c - t_b; dg[2] += t_d - t_c; dg[3] += t_e - t_d;
             dg[4] += wall_clock64() - t_e; dg[5] += 1; dg[6] += ntiles;)
  if (!more) break;
  cw = nw;
  }  // work items
  INTRA_DIAG(if (p.diag != nullptr && tid == 0) for (int i = 0; i < DIAG_SLOTS; ++i)
               p.diag[(size_t)blockIdx.x * DIAG_SLOTS + i] += dg[i];)
}

template <class MAP, int HP, int NW, int SM>
__global__ __launch_bounds__(NW * 64) void intra_fwd_kernel(const KParams p) {
  __shared__ __attribute__((aligned(1024))) unsigned char smem[LDS_BYTES];
  uint32_t* redo = reinterpret_cast<uint32_t*>(smem + RING_BYTES);
  constexpr bool FAST = SM != SM_EXACT;
  if (FAST) {
    if (threadIdx.x < REDO_WORDS) redo[threadIdx.x] = 0;  // visible after the first tile barrier
    run_pass<MAP, HP, NW, SM, false>(p, smem, redo);
    // Every wavefront has left the first pass: its marks are in, nobody reads the ring any more and
    // the loader's last (unused) requests have landed before new ones reuse their slots.
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    const uint32_t mine = redo[threadIdx.x & (REDO_WORDS - 1)];
    if (__builtin_amdgcn_ballot_w64(mine != 0) == 0) return;  // the usual case
  }
  run_pass<MAP, HP, NW, SM_EXACT, FAST>(p, smem, redo);
}

}  // namespace intra
