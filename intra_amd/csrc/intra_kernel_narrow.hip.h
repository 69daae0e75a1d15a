// Forward sparse-attention kernel for gfx950 in half-size workgroups: 4 wavefronts, two workgroups
// per CU, for patterns whose work items are short (a window of a few hundred keys, the patches of
// image gather0).
//
// The step of 32 keys, the operand layouts, the softmax arithmetics and the dealing of work items are
// those of intra_kernel.hip.h; what differs is everything around the step:
//
//  * A workgroup owns POS = 128 / HP in-set queries.  Two workgroups share a CU (and every SIMD has
//    one wavefront of each), and they are not in step: while one waits at an item boundary - for the
//    wavefronts on the causal diagonal, for its Q rows, for its first key block - the other one has
//    the SIMDs' issue slots to itself.  The wide kernel's eight wavefronts all wait together.
//  * The LDS ring of a workgroup is 2 K tiles + 2 V tiles (66 KiB).  K is requested one tile ahead of
//    V: iteration t multiplies the V rows of stream tile t and reads the K rows of tile t + 1, so at
//    its top, behind the barrier, a wavefront requests the K rows of tile t + 2 into the slot of
//    tile t (last read before that barrier) and the V rows of tile t + 1 into the slot of tile t - 1.
//    Every request has one iteration to arrive, and every barrier waits for all of them.  The V
//    request uses the row positions its K request computed one iteration earlier (4 registers).
//  * The Q rows of the next item come from HBM straight into the operand registers when the tile
//    loop has ended (they are dead then), by ordinary loads in front of the normalisation and the
//    output stores; the other workgroup covers their latency.
#pragma once
#include "intra_kernel.hip.h"

namespace intra {

constexpr int NARROW_WAVES = 4;
constexpr int NARROW_VBASE = 2 * FTILE;                  // 2 K slots, then 2 V slots
constexpr int NARROW_RING_BYTES = 4 * FTILE;
constexpr int NARROW_LDS_BYTES = NARROW_RING_BYTES + REDO_WORDS * 4;
static_assert(2 * NARROW_LDS_BYTES <= 160 * 1024, "two workgroups per CU");

// One pass of a workgroup over its work items.  SM: softmax arithmetic, see the file comment.
// REDO: visit only the items whose round is marked in `redo` (the SM_EXACT second pass of a kernel
// whose first pass keeps no running maximum).
template <class MAP, int HP, int SM, bool REDO>
__device__ __forceinline__ void run_pass_narrow(const KParams& p, unsigned char* smem, uint32_t* redo) {
  constexpr int NW = NARROW_WAVES;
  constexpr int VBASE = NARROW_VBASE;        // (shadows the wide kernel's)
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
  // Two workgroups per CU, each walking through its work items in the order of locate_item.
  const int xcd = blockIdx.x & 7;
  const int wgs_per_xcd = gridDim.x >> 3;
  const int wg_in_xcd = blockIdx.x >> 3;
  auto locate = [&](int round, Where& w) {
    return locate_item<MAP, POS, REDO>(p, xcd, wgs_per_xcd, wg_in_xcd, redo, round, w);
  };
  auto range_of = [&](const MAP& map, int mblk) { return range_of_block<MAP, POS>(map, mblk); };

  // ---------------------------------------------------------------- loader: HBM rows -> LDS
  // One global_load_lds_dwordx4 moves a 4-row group (see the wide kernel's loader): 16 groups per
  // tile, 4 per wavefront.  The K rows of all work items of this workgroup form one stream of tiles,
  // and so do the V rows, one tile behind: the loader's cursor (`fd`) names the K tile to request
  // next, two tiles ahead of the computation, and moves on to the next work item when it has
  // requested the last tile of one.  The V rows of a tile are requested one call later, from the
  // positions (`v_pos`, per lane) and the base address (`v_base`) its K request left behind.
  constexpr int GROUPS_PER_WAVE = (BN / 4) / NW;
  static_assert((BN / 4) % NW == 0, "tile groups must split evenly over the wavefronts");
  const int ld_row = lane >> 4;                                  // row of the group this lane fetches
  const uint32_t ld_col = (((lane & 15) ^ (4 * ld_row)) << 4);   // byte column it fetches
  const uint32_t k_rs_b = p.k_rs_bytes, v_rs_b = p.v_rs_bytes;
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)smem;
  struct Feed {
    MAP map;
    Range rg;
    int nk, tile;      // tile: the key tile whose K rows are requested next
    bool more;         // false once the last work item has been requested completely
    const char *kbase, *vbase;
    Where w;           // the work item whose tiles are being requested
    int prev_round;    // round of the work item before it
  };
  auto feed_for = [&](const Where& w, int prev_round) {
    const MAP map(p.geom, w.set, w.mblk * POS);
    return Feed{map, range_of(map, w.mblk), map.nk(), 0, true,
                reinterpret_cast<const char*>(p.k + w.batch * p.k_bs + w.kvh * p.k_hs),
                reinterpret_cast<const char*>(p.v + w.batch * p.v_bs + w.kvh * p.v_hs), w, prev_round};
  };
  Where cw;
  if (!locate(0, cw)) return;
  // measurement builds: the wide kernel's phase timers, where they have a counterpart here ([1] stays
  // 0: no barriers at the item boundary; [14], [15]: the barrier of every tile; [8] .. [11] are
  // written at the end)
  long long* dgw = nullptr;
  INTRA_DIAG(long long dg[DIAG_SLOTS] = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0}; dgw = dg + 8;)
  (void)dgw;
  Feed fd = feed_for(cw, -1);
  uint32_t v_pos[GROUPS_PER_WAVE];
  const char* v_base = fd.vbase;
  // request the V rows of the tile whose K rows were requested last (into the V slot at v_off) and
  // the K rows of the next tile of the stream (into the K slot at k_off)
  auto feed_tile = [&](int k_off, int v_off, auto with_v) {
    if (decltype(with_v)::value) {
#pragma unroll
      for (int gi = 0; gi < GROUPS_PER_WAVE; ++gi)
        dma_group(v_base + ((uint64_t)v_pos[gi] * v_rs_b + ld_col),
                  lds_base + VBASE + v_off + (wave * GROUPS_PER_WAVE + gi) * FGROUP_STRIDE);
    }
    TileRows tr;
    if (map_tile_rows(fd.map, fd.rg.kt_lo + fd.tile * BN, tr)) {  // (wave-uniform)
      const uint32_t row = (uint32_t)(ld_row * tr.row_step);
#pragma unroll
      for (int gi = 0; gi < GROUPS_PER_WAVE; ++gi) {
        const int grp = wave * GROUPS_PER_WAVE + gi;
        const uint32_t pos = (uint32_t)(tr.base + grp * tr.group_step) + row;
        dma_group(fd.kbase + ((uint64_t)pos * k_rs_b + ld_col), lds_base + k_off + grp * FGROUP_STRIDE);
        v_pos[gi] = pos;
      }
    } else {
#pragma unroll
      for (int gi = 0; gi < GROUPS_PER_WAVE; ++gi) {
        const int grp = wave * GROUPS_PER_WAVE + gi;
        const int tk = im_min(fd.rg.kt_lo + fd.tile * BN + 4 * grp + ld_row, fd.nk - 1);
        const uint32_t pos = fd.map.kpos(tk);
        dma_group(fd.kbase + ((uint64_t)pos * k_rs_b + ld_col), lds_base + k_off + grp * FGROUP_STRIDE);
        v_pos[gi] = pos;
      }
    }
    v_base = fd.vbase;
    ++fd.tile;
    if (fd.tile == fd.rg.ntiles && fd.more) {
      Where w;
      if (locate(fd.w.round + 1, w)) fd = feed_for(w, fd.w.round);
      else fd.more = false;  // nothing left: keep requesting the (clamped) last row, nobody reads it
    }
  };

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
  // Q^T fragments (B operand of S^T = K Q^T): qf[qt][ks] is chunk 4 * ks + g4 of query 16 * qt + l16.
  // They come from HBM straight into registers (16 rows x 64 bytes per instruction), requested for
  // the NEXT work item when the tile loop of the current one has ended, and first used at the top of
  // the next item.  These are ordinary loads (the compiler places their wait); nothing is requested
  // through the hand-counted direct-to-LDS path between their issue and their first use.
  u32x4 qf[2][4];
  auto request_q = [&](const Where& w) {
    const int t0 = w.mblk * POS;
    const MAP map(p.geom, w.set, t0);
    const int t1 = im_min(t0 + POS, map.nq()) - 1;
    const uint16_t* base = p.q + (w.batch * p.q_bs + (int64_t)(w.kvh * p.ratio + w.hg * HP + wave % HP) * p.q_hs + g4 * 8);
#pragma unroll
    for (int qt = 0; qt < 2; ++qt) {
      const int tq = im_min(t0 + (wave / HP) * 32 + 16 * qt + l16, t1);  // rows past the end: the last row once more
      const uint16_t* row = base + (int64_t)map.qpos(tq) * p.q_rs;
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) qf[qt][ks] = *reinterpret_cast<const u32x4*>(row + 32 * ks);
    }
    asm volatile("" ::: "memory");  // the requests stay where they are written
  };

  // Ring slots (byte offsets into the K ring; the V ring uses the same offsets behind VBASE): k0
  // holds stream tile t while iteration t runs, k1 tile t + 1 (and, in the V ring, tile t - 1 until
  // the request at the top of the iteration); they swap once per tile and carry on from one work
  // item to the next.
  int k0 = 0, k1 = FTILE;
  feed_tile(k0, 0, ic<0>{});   // K rows of the first tile of the stream
  feed_tile(k1, k0, ic<1>{});  // its V rows and the K rows of the second
  request_q(cw);
  tile_barrier<0>();           // all of it has landed (once per pass; later items find their first tile in place)
  auto rotate = [&] {  // one tile further in the stream
    const int d = k0 - k1;
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      kb[a] += d;
      vb[a] -= d;
    }
    const int tk = k0;
    k0 = k1; k1 = tk;
  };

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

  // ---------------------------------------------------------------- the Q rows have been requested
  if (SM == SM_FOLDED) {  // Q <- bf16(Q * softmax_scale * log2 e): the MFMA then yields exponents directly
    const float cq = p.q_fold;
#pragma unroll
    for (int f = 0; f < 8; ++f)
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        const uint32_t x = qf[f >> 2][f & 3][d];
        floatx2 y = {__uint_as_float(x << 16) * cq, __uint_as_float(x & 0xffff0000u) * cq};
        qf[f >> 2][f & 3][d] = __builtin_bit_cast(uint32_t, __builtin_convertvector(y, bf16x2));
      }
  } else if (p.negate_q) {  // softmax_scale < 0: flip the sign of Q (exact) and use |scale| below
#pragma unroll
    for (int f = 0; f < 8; ++f) qf[f >> 2][f & 3] ^= 0x80008000u;
  }

  INTRA_DIAG(const long long t_c = wall_clock64();)
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
#pragma unroll
      for (int u = 0; u < 8; ++u) {
        const int es = u < 4 ? 4 * u : 2 * u + 6;
        if (es == k) stage_e(u);
        if (es + 2 == k) stage_c(u);
        if (es + 2 == k) stage_s(u);
      }
    };
#pragma unroll
    for (int k = 0; k < 16; ++k) {  // QK^T: k-step ks, key tile kt, query tile qt
      const int ks = k >> 2, kt = (k >> 1) & 1, qt = k & 1;
      if ((k & 1) == 0) va[k >> 1] = vread_at(vb[k >> 2], 32 * ((k >> 1) & 1) + HALF * FBLOCK32);
      n[kt][qt] = mfma(ka[2 * ks + kt], __builtin_bit_cast(bf16x8, qf[qt][ks]), ks == 0 ? zero4 : n[kt][qt]);
      valu_slot(k);
      __builtin_amdgcn_sched_barrier(0);
    }
    float m[2] = {0.f, 0.f};
#pragma unroll
    for (int k = 0; k < 16; ++k) {  // PV: query tile qt, head-dim tile dt
      const int qt = k >> 3, dt = k & 7;
      if (k >= 8) ka[k - 8] = kread_at(kb[(k - 8) >> 1], (k & 1) * 4 * FGROUP_STRIDE + HALF * FBLOCK32);
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
  //
  // A run only starts in the second half of a tile (an odd step) or with the block ahead of the
  // pipeline: a start in the first half would read K rows of the current tile, whose slot the loader
  // has just given to the tile after the next.  Such a run starts one step earlier instead; the block
  // that adds lies outside the wavefront's range, so the mask removes all of it.
  auto odd_start = [](int jq) { return jq >= 0 && (jq & 1) == 0 ? jq - 1 : jq; };
  int jq1 = odd_start(bw_lo - 1), jp1 = bw_hi, jq2 = 1, jp2 = 0;
  if (MAP::kHasPrefix && bp_hi >= 0) {
    if (jq1 <= bp_hi) {  // the ranges touch: one run from the first prefix block on
      jq1 = -1;
      jp1 = im_max(bw_hi, bp_hi);
    } else {
      jq2 = jq1;
      jp2 = bw_hi;
      jq1 = -1;
      jp1 = bp_hi;
    }
  }
  auto needs_mask = [&](int j) { return !block_unmasked(wb, kpre, kt_lo + 32 * j); };
  // half_c: which half of its tile block j is (0 / 1).  Block j + 1 is the other half of the same
  // tile (half 0) or the first half of the next tile (half 1).
  auto step = [&](int j, floatx4 (&cur)[2][2], floatx4 (&nxt)[2][2], auto half_c) {
    constexpr int HALF = decltype(half_c)::value;
    const bool in1 = j >= jq1 && j <= jp1, in2 = j >= jq2 && j <= jp2;
    if (!in1 && !in2) return;
    if (HALF == 1 && (j == jq1 || (in2 && j == jq2))) {
#pragma unroll
      for (int t = 0; t < 4; ++t) cur[t >> 1][t & 1] = floatx4{-INFINITY, -INFINITY, -INFINITY, -INFINITY};
      load_ka(ka, 0, 0);  // first half of the next tile
    }
    steady(cur, nxt, half_c, needs_mask(j + 1), kt_lo + 32 * (j + 1));
  };

  // ---------------------------------------------------------------- main loop
  // Stream tile t lives in ring slot t % 2 of the K ring and of the V ring.  Behind the barrier that
  // opens iteration t every wavefront's requests up to K rows of tile t + 1 and V rows of tile t have
  // landed, and nobody reads the K rows of tile t or the V rows of tile t - 1 any more: those two
  // slots take the requests for the K rows of tile t + 2 and the V rows of tile t + 1.  The first
  // block of a work item is computed ahead of the pipeline from K rows that landed before the
  // barrier of the previous item's last tile.
  if (jq1 < 0 && jp1 >= 0) {  // scores of key block 0 (its tile sits in slot k0)
    load_ka(ka, k0 - k1, 0);
#pragma unroll
    for (int t = 0; t < 4; ++t) s0[t >> 1][t & 1] = zero4;
#pragma unroll
    for (int k = 0; k < 16; ++k) {
      const int ks = k >> 2, kt = (k >> 1) & 1, qt = k & 1;
      s0[kt][qt] = mfma(ka[2 * ks + kt], __builtin_bit_cast(bf16x8, qf[qt][ks]), s0[kt][qt]);
    }
    float mx[2] = {0.f, 0.f};
    if (!FAST) block_max(s0, mx);
    finish_scores(s0, mx, needs_mask(0), kt_lo);
    load_ka(ka, k0 - k1, FBLOCK32);
  }
  INTRA_DIAG(const long long t_d = wall_clock64(); const long long c_d = __builtin_readcyclecounter();)
  for (int i = 0;;) {
    INTRA_TILE_BARRIER(0, dgw + 6);
    feed_tile(k0, k1, ic<1>{});
    step(2 * i, s0, s1, ic<0>{});
    step(2 * i + 1, s1, s0, ic<1>{});
    rotate();
    if (++i == ntiles) break;
  }

  INTRA_DIAG(const long long t_e = wall_clock64(); dg[7] += __builtin_readcyclecounter() - c_d;)
  // The loader is ahead by two tiles, so it usually knows the next work item already.
  Where nw = fd.w;
  bool more = true;
  if (fd.w.round == cw.round) more = false;  // (the loader only stays on an item when it is the last)
  else if (fd.prev_round != cw.round) more = locate(cw.round + 1, nw);
  if (more) request_q(nw);

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
    if (__builtin_amdgcn_ballot_w64(bad) != 0 && lane == 0)
      __hip_atomic_fetch_or(&redo[(cw.round >> 5) & (REDO_WORDS - 1)], 1u << (cw.round & 31), __ATOMIC_RELAXED,
                            __HIP_MEMORY_SCOPE_WORKGROUP);
  }
  const float inv[2] = {l_tot[0] > 0.f ? 1.f / l_tot[0] : 0.f, l_tot[1] > 0.f ? 1.f / l_tot[1] : 0.f};
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
  INTRA_DIAG(dg[0] += t_c - t_a; dg[2] += t_d - t_c; dg[3] += t_e - t_d; dg[4] += wall_clock64() - t_e;
             dg[5] += 1; dg[6] += ntiles;)
  if (!more) break;
  cw = nw;
  }  // work items
  INTRA_DIAG(if (p.diag != nullptr && tid == 0) for (int i = 0; i < DIAG_SLOTS; ++i)
               p.diag[(size_t)blockIdx.x * DIAG_SLOTS + i] += dg[i];)
  // [8 + w]: where the hardware put wavefront w (HW_ID register: wave slot, SIMD, CU, shader engine;
  // XCC_ID in the upper half), from which a reader sees which workgroups share a CU
  INTRA_DIAG(if (p.diag != nullptr && lane == 0) {
    uint32_t hw, xcc;
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_HW_ID)" : "=s"(hw));
    asm volatile("s_getreg_b32 %0, hwreg(HW_REG_XCC_ID)" : "=s"(xcc));
    p.diag[(size_t)blockIdx.x * DIAG_SLOTS + 8 + wave] = (long long)hw | ((long long)xcc << 32);
  })
}

template <class MAP, int HP, int SM>
__global__ __launch_bounds__(NARROW_WAVES * 64, 2) void intra_fwd_kernel_narrow(const KParams p) {
  __shared__ __attribute__((aligned(1024))) unsigned char smem[NARROW_LDS_BYTES];
  uint32_t* redo = reinterpret_cast<uint32_t*>(smem + NARROW_RING_BYTES);
  constexpr bool FAST = SM != SM_EXACT;
  if (FAST) {
    if (threadIdx.x < REDO_WORDS) redo[threadIdx.x] = 0;  // visible after the first barrier
    run_pass_narrow<MAP, HP, SM, false>(p, smem, redo);
    // Every wavefront has left the first pass: its marks are in, nobody reads the ring any more and
    // the loader's last (unused) requests have landed before new ones reuse their slots.
    __builtin_amdgcn_s_waitcnt(0);
    __syncthreads();
    const uint32_t mine = redo[threadIdx.x & (REDO_WORDS - 1)];
    if (__builtin_amdgcn_ballot_w64(mine != 0) == 0) return;  // the usual case
  }
  run_pass_narrow<MAP, HP, SM_EXACT, FAST>(p, smem, redo);
}

}  // namespace intra
