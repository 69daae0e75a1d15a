// Backward kernels of the sparse attention for gfx950 (MI355X): dQ, dK and dV for the causal LLM
// patterns (Scatter, Gather 1, 64-aligned window, block Scatter with stripe offsets and sinks,
// per-token window with sinks) and the image patterns (Scatter, Gather 0).  Which rows meet which
// columns comes from the row maps of intra_bwd_maps.h.
//
// The reference has no backward kernels (its README names them as missing; training there runs
// through masked SDPA / FlexAttention, experiments/llm/llama_intra.py:26).  The math is the usual
//   P = exp(scale * S - lse),  dV = P^T dO,  dP = dO V^T,  dS = P o (dP - D),  D_i = dO_i . O_i,
//   dQ = scale * dS K,  dK = scale * dS^T Q.
//
// One template serves the three results.  A workgroup owns 256 / HP "rows" (queries for dQ, keys
// for dK and dV; 32 per wavefront, held as MFMA B operands in registers like Q in the forward
// kernel) and streams the "columns" that see them through LDS in tiles of 64 (K and V rows for
// dQ, Q and dO rows of every query head of the group for dK / dV) through three slots.  Per 32
// columns a wavefront forms the scores S^T = C1 R1^T and dP^T = C2 R2^T, turns them into the
// weights (P or dS), packed to bf16 straight from the accumulators, and adds X^T W^T to its
// accumulators, X being the K, Q or dO tile read with transposing LDS reads - the data flow of
// the forward kernel without the online softmax.
#pragma once
#include "intra_bwd_maps.h"
#include "intra_kernel.hip.h"

namespace intra {

// BWD_DKV forms dK and dV in one pass (the scores of a block are computed once for both): the two
// accumulators, the K and V fragments of the key rows, the scores, dP, both sets of weights and the
// operand ring need more than the 256 registers of a wavefront at two wavefronts per SIMD, so this
// mode runs workgroups of 4 wavefronts, one per SIMD, with up to 512 registers each.
// f(ic<B>{}), f(ic<B + 1>{}), ..., f(ic<E - 1>{})
template <int B, int E, class F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (B < E) {
    f(ic<B>{});
    static_for<B + 1, E>(f);
  }
}

enum BwdMode : int { BWD_DQ = 0, BWD_DK = 1, BWD_DV = 2, BWD_DKV = 3 };
constexpr int bwd_waves(int mode) { return mode == BWD_DKV ? 4 : 8; }

struct BParams {
  const uint16_t *q, *k, *v, *o, *dout;  // bf16 (B, S, heads, 128)
  const float* lse;                      // (B, H, S): ln sum exp(scale * q.k) from the forward pass
  float* dsum;                           // (B, H, S) workspace: -D = -rowsum(dO o O), written by dQ, read by dK
  float* l2;                             // (B, H, S) workspace: lse * log2(e), written by dQ, read by dK / dV
  uint16_t *dq, *dk, *dv;
  float* part;  // partial sums of the sink pass: (chunk, batch, kv head, sink, 128) fp32
  // element strides: batch, row (token), head
  int64_t q_bs, q_rs, q_hs, k_bs, k_rs, k_hs, v_bs, v_rs, v_hs, o_bs, o_rs, o_hs, do_bs, do_rs, do_hs;
  int64_t dq_bs, dq_rs, dq_hs, dk_bs, dk_rs, dk_hs, dv_bs, dv_rs, dv_hs;
  int64_t lse_bs, lse_hs, lse_ts, ds_bs, ds_hs;  // dsum is contiguous over tokens
  int B, H, Hkv, ratio;
  IntraGeom geom;
  float scale;       // softmax scale
  float scale_log2;  // scale * log2(e)
  int n_rblocks;     // row blocks per set
  int hgroups;       // ratio / HP (dQ only)
  int items_per_pair;  // n_rblocks * hgroups
  int bundle;        // pairs of one XCD that are worked on together
};

constexpr int BWD_SLOT = 2 * FTILE + 512;  // two tiles and 2 x 64 column scalars
constexpr int BWD_LDS_BYTES = 3 * BWD_SLOT;
constexpr int bwd_ring_slots(int mode) { return mode == BWD_DKV ? 4 : 3; }

// 64 lanes x 4 bytes from per-lane global addresses to 256 consecutive LDS bytes at lds_addr (the
// active lanes' parts of them), like dma_group
__device__ __forceinline__ void dma_dwords(const void* gsrc, uint32_t lds_addr) {
  asm volatile("s_mov_b32 m0, %1\n\tglobal_load_lds_dword %0, off" : : "v"(gsrc), "s"(lds_addr) : "memory");
}

// RMAP: row map (intra_bwd_maps.h).  PARTIAL: the results are partial sums over the set's columns,
// written as fp32 to p.part instead of bf16 to dk / dv (sink pass).
//
// MFMA layout (v_mfma_f32_16x16x32_bf16, as in the forward kernel): a block of 32 columns times the
// wavefront's 32 rows is 2 x 2 tiles [ct][rt] with 4 k-steps; lane (l16 = lane % 16, g4 = lane / 16)
// holds columns 16*ct + 4*g4 .. +3 of row 16*rt + l16.  The packed weights of a row tile are the B
// operand of the accumulation, whose 32-column reduction is numbered slot s of lane quarter g4 =
// column 16*(s/4) + 4*g4 + s%4; the transposing reads of the X tile follow that numbering.
template <class RMAP, int MODE, int HP, bool PARTIAL = false>
__global__ __launch_bounds__(bwd_waves(MODE) * 64) void intra_bwd_kernel(const BParams p) {
  constexpr int NW = bwd_waves(MODE);
  constexpr bool HAS_DP = MODE != BWD_DV;                    // forms dP and dS
  constexpr bool HAS_V = MODE == BWD_DV || MODE == BWD_DKV;  // accumulates dV (weights P)
  static_assert(!(MODE == BWD_DKV && PARTIAL), "the partial sums of the sink pass come from the separate modes");
  constexpr bool ROWS_ARE_QUERIES = MODE == BWD_DQ;
  constexpr int POS = ROWS_ARE_QUERIES ? NW * 32 / HP : NW * 32;  // rows per row block (of one head)

  // BWD_DKV: a step of its single wavefront per SIMD is about as long as a tile takes to arrive, so
  // its ring is one slot deeper and a tile has two steps to land; the column scalars travel the same
  // way (every wavefront requests those of 16 columns) instead of through registers.
  constexpr bool DEEP = MODE == BWD_DKV;
  constexpr bool TWO_STAGES = MODE == BWD_DKV || MODE == BWD_DQ;  // P and dS = P * dP formed apart
  __shared__ __attribute__((aligned(1024))) unsigned char smem[bwd_ring_slots(MODE) * BWD_SLOT];
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)smem;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l16 = lane & 15;
  const int g4 = lane >> 4;

  // ---------------------------------------------------------------- work item
  // Workgroups start in blockIdx order, round-robin over the 8 XCDs, and a CU takes the next one
  // when it has finished one.  Per XCD the (set, batch, kv head) pairs are taken in bundles of
  // `bundle` pairs - as few as fill its 32 CUs - so that the workgroups running together stream the
  // same few megabytes of columns through the XCD's L2; within a bundle the row blocks with the
  // most columns come first (the last query blocks for dQ, the first key blocks for dK / dV).
  const int xcd = blockIdx.x & 7, slot = blockIdx.x >> 3;
  const int per_bundle = p.bundle * p.items_per_pair;
  const int bun = slot / per_bundle, rem = slot - bun * per_bundle;
  const int heavy = rem / p.bundle;
  const int nbh = p.B * p.Hkv;
  const int pair = (bun * p.bundle + (rem - heavy * p.bundle)) * 8 + xcd;
  if (pair >= RMAP::num_sets(p.geom) * nbh) return;
  int hg = 0, rblk = heavy;
  if (ROWS_ARE_QUERIES) {
    hg = heavy % p.hgroups;
    rblk = p.n_rblocks - 1 - heavy / p.hgroups;
  }
  const int set = pair / nbh;
  const int bh = pair % nbh;
  const int batch = bh / p.Hkv;
  const int kvh = bh % p.Hkv;

  const int r0 = rblk * POS;
  const RMAP map(p.geom, set, r0);
  const int kpre = map.kpre();
  const int n_rows = map.n_rows(), n_cols = map.n_cols();
  if (r0 >= n_rows) return;
  const int r1 = im_min(r0 + POS, n_rows) - 1;

  // Row r meets the columns lo(r)..hi(r) (plus those below kpre for maps that have such a prefix).
  const int cb = map.block_lo(r0, r1);  // first column of the row block
  const int ce = map.block_hi(r0, r1);  // last one
  const int ntiles = ce >= cb ? (ce - cb + BN) / BN : 0;

  // ---------------------------------------------------------------- this wavefront's rows
  // a lane works for two rows: 16 * rt + l16 of the wavefront's 32 (rows past the end repeat the last)
  const int hw = ROWS_ARE_QUERIES ? wave % HP : 0;
  const int wr0 = r0 + (ROWS_ARE_QUERIES ? wave / HP : wave) * 32;
  const bool wave_active = wr0 <= r1;
  bool row_valid[2];
  int row[2], lo_l[2], hi_l[2];
  int64_t rpos[2];
#pragma unroll
  for (int rt = 0; rt < 2; ++rt) {
    row_valid[rt] = wr0 + 16 * rt + l16 <= r1;
    row[rt] = im_min(wr0 + 16 * rt + l16, r1);
    lo_l[rt] = map.lo(row[rt]);
    hi_l[rt] = map.hi(row[rt]);
    rpos[rt] = map.row_pos(row[rt]);
  }
  // union and intersection of the ranges of the wavefront's rows
  WaveBounds wb;
  {
    int a = im_min(lo_l[0], lo_l[1]), b = im_max(hi_l[0], hi_l[1]), c = im_max(lo_l[0], lo_l[1]), d = im_min(hi_l[0], hi_l[1]);
#pragma unroll
    for (int m = 1; m < 16; m <<= 1) {
      a = im_min(a, __shfl_xor(a, m));
      b = im_max(b, __shfl_xor(b, m));
      c = im_max(c, __shfl_xor(c, m));
      d = im_min(d, __shfl_xor(d, m));
    }
    wb.w_lo = __builtin_amdgcn_readfirstlane(a);
    wb.w_hi = __builtin_amdgcn_readfirstlane(b);
    wb.f_lo = __builtin_amdgcn_readfirstlane(c);
    wb.f_hi = __builtin_amdgcn_readfirstlane(d);
  }
  // The blocks of 32 columns (counted from cb) that this wavefront's rows meet: one range; with a
  // prefix it starts at the first block (blocks between prefix and own range are few and masked).
  const bool any = wave_active && wb.w_hi >= cb && (kpre > 0 || wb.w_hi >= wb.w_lo);  // (early rows may meet prefix columns only)
  const int jb_lo = !any ? 1 : kpre > 0 ? 0 : (im_max(wb.w_lo, cb) - cb) >> 5;
  const int jb_hi = !any ? 0 : (wb.w_hi - cb) >> 5;
  const int hq = kvh * p.ratio + hg * HP + hw;  // query head of a query row

  // ---------------------------------------------------------------- row operands (MFMA B fragments)
  // [rt][ks]: lane holds row 16 * rt + l16, head dims 32 * ks + 8 * g4 .. +7
  bf16x8 r1f[2][4], r2f[2][4];
  float L2_row[2] = {0.f, 0.f}, D_row[2] = {0.f, 0.f};
  auto load_rows = [&] {
#pragma unroll
  for (int rt = 0; rt < 2; ++rt) {
    const uint16_t *a1, *a2;
    if (ROWS_ARE_QUERIES) {
      a1 = p.q + (batch * p.q_bs + rpos[rt] * p.q_rs + hq * p.q_hs + g4 * 8);
      a2 = p.dout + (batch * p.do_bs + rpos[rt] * p.do_rs + hq * p.do_hs + g4 * 8);
    } else {
      a1 = p.k + (batch * p.k_bs + rpos[rt] * p.k_rs + kvh * p.k_hs + g4 * 8);
      a2 = p.v + (batch * p.v_bs + rpos[rt] * p.v_rs + kvh * p.v_hs + g4 * 8);
    }
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
      r1f[rt][ks] = *reinterpret_cast<const bf16x8*>(a1 + ks * 32);
      if (HAS_DP) r2f[rt][ks] = *reinterpret_cast<const bf16x8*>(a2 + ks * 32);
    }
    if (ROWS_ARE_QUERIES) {
      // D = dO . O of the row: this lane's 32 head dims, then the rest from the other three lanes of the row
      const uint16_t* ao = p.o + (batch * p.o_bs + rpos[rt] * p.o_rs + hq * p.o_hs + g4 * 8);
      float part = 0.f;
#pragma unroll
      for (int ks = 0; ks < 4; ++ks) {
        const bf16x8 of = *reinterpret_cast<const bf16x8*>(ao + ks * 32);
#pragma unroll
        for (int d = 0; d < 8; ++d) part += (float)r2f[rt][ks][d] * (float)of[d];
      }
      D_row[rt] = lane_quad_sum(part);
      L2_row[rt] = p.lse[batch * p.lse_bs + hq * p.lse_hs + rpos[rt] * p.lse_ts] * 1.4426950408889634f;
      if (row_valid[rt] && g4 == 0) {  // what the dK / dV launches need per query, in the form they use it
        p.dsum[batch * p.ds_bs + hq * p.ds_hs + rpos[rt]] = -D_row[rt];
        p.l2[batch * p.ds_bs + hq * p.ds_hs + rpos[rt]] = L2_row[rt];
      }
    }
  }
  };
  if (!DEEP) load_rows();  // (the deep ring requests its first tiles before them, see below)

  // ---------------------------------------------------------------- LDS addressing (as in the forward kernel)
  const int ld_row = lane >> 4;
  const uint32_t ld_col = (((lane & 15) ^ (4 * ld_row)) << 4);
  int kaddr[4];
  {
    const int r = l16 & 3;
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) kaddr[ks] = (l16 >> 2) * FGROUP_STRIDE + r * 256 + 64 * (ks ^ r) + 16 * g4;
  }
  int vaddr[4];
  {
    const int ri = l16 >> 2;
#pragma unroll
    for (int a = 0; a < 4; ++a)
      vaddr[a] = g4 * FGROUP_STRIDE + ri * 256 + 64 * (a ^ ri) + 16 * ((l16 & 3) >> 1) + 8 * (l16 & 1);
  }
  // LDS operands are read from per-lane bases that carry the ring slot (b0: the step's slot, b1: the
  // next one's), advanced once per step, so that everything else is a compile-time offset.
  // kread_b: row-per-lane operand 2 * ks + ct of a 32-row block (rows 16 * ct + l16, head dims of
  // k-step ks); vread_b: transposed operand (head dims 16 * dt .. + 15 of the block's 32 rows).
  // sb0, sb1: the same for the column scalars of the deep ring.
  int kb0[4], kb1[4], vb0[4], sb0 = 0, sb1 = 0;
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    kb0[i] = kaddr[i];
    kb1[i] = BWD_SLOT + kaddr[i];
    vb0[i] = vaddr[i];
  }
  sb0 = 2 * FTILE + 16 * g4;
  sb1 = BWD_SLOT + 2 * FTILE + 16 * g4;
  auto kread_b = [&](const int (&kb)[4], int off, int f) {
    return *reinterpret_cast<const bf16x8*>(smem + (kb[f >> 1] + (off + (f & 1) * 4 * FGROUP_STRIDE)));
  };
  auto vread_b = [&](int off, int dt) {
    const int o2 = vb0[dt >> 1] + (off + 32 * (dt & 1));
    bf16x4 v0 = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((__attribute__((address_space(3))) bf16x4*)(smem + o2));
    bf16x4 v1 = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
        (__attribute__((address_space(3))) bf16x4*)(smem + (o2 + 4 * FGROUP_STRIDE)));
    return __builtin_shufflevector(v0, v1, 0, 1, 2, 3, 4, 5, 6, 7);
  };
  auto mfma = [](bf16x8 a, bf16x8 b, floatx4 c) { return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0); };
  const floatx4 zero4 = {0.f, 0.f, 0.f, 0.f};

  floatx4 acc[8][2];  // [head-dim tile][row tile]: head dims 16 * dt + 4 * g4 .. + 3 of row 16 * rt + l16
  floatx4 acc_v[MODE == BWD_DKV ? 8 : 1][2];  // BWD_DKV: dV (acc is dK)
#pragma unroll
  for (int dt = 0; dt < 8; ++dt)
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) {
      acc[dt][rt] = zero4;
      if (MODE == BWD_DKV) acc_v[dt][rt] = zero4;
    }
  const float c2 = p.scale_log2;
  const float s_hidden = c2 >= 0.f ? -INFINITY : INFINITY;  // score that gives exp2(s * c2 - lse) = 0

  // ---------------------------------------------------------------- column steps
  // dQ meets one stream of columns (the K / V rows of the kv head), tile after tile from the first.
  // dK / dV meet one per query head of the group (its Q / dO rows); they take the tiles from the
  // last one down and, per tile, head after head: all key blocks of a (set, batch, kv head) start
  // at the last tile together and stay in step, so that a tile fetched for one of them is in the
  // L2 for the others.  A step is one (tile, head).
  const int n_streams = ROWS_ARE_QUERIES ? 1 : p.ratio;
  const int n_steps = ntiles * n_streams;
  struct Cursor {
    int tile, head;
  };
  auto advance = [&](Cursor& c) {
    if (ROWS_ARE_QUERIES) {
      ++c.tile;
    } else if (++c.head == n_streams) {
      c.head = 0;
      --c.tile;
    }
  };
  const char *c1base, *c2base;
  uint32_t c1rs, c2rs;
  int64_t c1hs = 0, c2hs = 0;  // byte stride between the heads of the group (dK / dV)
  if (ROWS_ARE_QUERIES) {
    c1base = reinterpret_cast<const char*>(p.k + batch * p.k_bs + kvh * p.k_hs);
    c2base = reinterpret_cast<const char*>(p.v + batch * p.v_bs + kvh * p.v_hs);
    c1rs = (uint32_t)(p.k_rs * 2);
    c2rs = (uint32_t)(p.v_rs * 2);
  } else {
    c1base = reinterpret_cast<const char*>(p.q + batch * p.q_bs + kvh * p.ratio * p.q_hs);
    c2base = reinterpret_cast<const char*>(p.dout + batch * p.do_bs + kvh * p.ratio * p.do_hs);
    c1rs = (uint32_t)(p.q_rs * 2);
    c2rs = (uint32_t)(p.do_rs * 2);
    c1hs = p.q_hs * 2;
    c2hs = p.do_hs * 2;
  }
  auto col_pos = [&](int c) { return map.col_pos(c); };
  // dK / dV take a tile once per query head of the group, head after head: the rows' positions are
  // worked out for the first head and kept for the others
  uint32_t pos_kept[16 / NW] = {};
  int64_t spos_kept = 0;
  auto load_group = [&](const Cursor& cu, int slot_off, int gi) {  // this wavefront's group gi of both tiles
    const int grp = wave * (16 / NW) + gi;
    if (ROWS_ARE_QUERIES || cu.head == 0) pos_kept[gi] = col_pos(im_min(cb + cu.tile * BN + 4 * grp + ld_row, n_cols - 1));
    const uint32_t pos = pos_kept[gi];
    dma_group(c1base + (cu.head * c1hs + (uint64_t)pos * c1rs + ld_col), lds_base + slot_off + grp * FGROUP_STRIDE);
    dma_group(c2base + (cu.head * c2hs + (uint64_t)pos * c2rs + ld_col),
              lds_base + slot_off + FTILE + grp * FGROUP_STRIDE);
  };
  auto load_tile = [&](const Cursor& cu, int slot_off) {
#pragma unroll
    for (int gi = 0; gi < 16 / NW; ++gi) load_group(cu, slot_off, gi);
  };
  // requests per wavefront for one step of the deep ring: its groups of both tiles and two for the scalars
  constexpr int DEEP_REQUESTS = 2 * (16 / NW) + 2;
  auto load_scalars = [&](const Cursor& cu, int slot_off) {  // (deep ring) lse * log2(e) and -D of the step's 64 columns
    static_assert(!DEEP || NW == 4, "16 columns per wavefront");
    if (cu.head == 0) spos_kept = col_pos(im_min(cb + cu.tile * BN + lane, n_cols - 1));
    if ((lane >> 4) == wave) {
      const int64_t pos = spos_kept;
      const int hcol = kvh * p.ratio + cu.head;
      dma_dwords(p.l2 + (batch * p.ds_bs + hcol * p.ds_hs + pos), lds_base + slot_off + 2 * FTILE);
      dma_dwords(p.dsum + (batch * p.ds_bs + hcol * p.ds_hs + pos), lds_base + slot_off + 2 * FTILE + 256);
    }
  };
  // column scalars of a step (dK / dV): wavefront 0 fetches lse * log2(e) and -D of its 64 columns
  float sc_l = 0.f, sc_d = 0.f;
  auto fetch_scalars = [&](const Cursor& cu) {
    if (!ROWS_ARE_QUERIES && !DEEP && wave == 0) {
      const int c = im_min(cb + cu.tile * BN + lane, n_cols - 1);
      const int64_t pos = col_pos(c);
      const int hcol = kvh * p.ratio + cu.head;
      sc_l = p.l2[batch * p.ds_bs + hcol * p.ds_hs + pos];
      if (HAS_DP) sc_d = p.dsum[batch * p.ds_bs + hcol * p.ds_hs + pos];
    }
  };
  auto put_scalars = [&](int slot_off) {
    if (!ROWS_ARE_QUERIES && !DEEP && wave == 0) {
      float* sc = reinterpret_cast<float*>(smem + slot_off + 2 * FTILE);
      sc[lane] = sc_l;
      sc[64 + lane] = sc_d;
    }
  };
  // Three tile slots: while step t works on its tile, the tile of step t+1 has landed (the scores
  // of its first block are formed at the end of step t) and the tile of step t+2 is in flight.
  Cursor cur{ROWS_ARE_QUERIES ? 0 : ntiles - 1, 0};  // step being computed
  Cursor ld = cur;                                   // step being requested
  // (Deep ring: one slot more, the tile of step t+3 is requested during step t, and the barrier of a
  // step leaves the most recent request in flight where one was made during the step before.)
  for (int t = 0; t < (DEEP ? 3 : 2) && t < n_steps; ++t) {
    load_tile(ld, t * BWD_SLOT);
    if (DEEP) load_scalars(ld, t * BWD_SLOT);
    fetch_scalars(ld);
    put_scalars(t * BWD_SLOT);
    advance(ld);
  }
  // The deep ring's barriers leave requests in flight.  The row operands are ordinary loads the
  // compiler waits for at their first use, inside the main loop, with a count that knows nothing of
  // the requests issued by hand - it would wait for those as well, every time round.  So they are
  // requested here, behind the first tiles (whose latency they share), and land here, once.
  if (DEEP) {
    load_rows();
    __builtin_amdgcn_s_waitcnt((0 & 15) | (7 << 4) | (15 << 8) | (0 << 14));  // vmcnt(0)
  }
  int slot0 = 0, slot1 = BWD_SLOT, slot2 = 2 * BWD_SLOT, slot3 = 3 * BWD_SLOT;
  bool fresh = DEEP && n_steps >= 3;  // the most recent request is for the step after the next
  floatx4 s_cur[2][2];  // [ct][rt]
#pragma unroll
  for (int t = 0; t < 4; ++t) s_cur[t >> 1][t & 1] = zero4;
  bool have = false;  // s_cur and fr hold what a previous block prepared for the one that comes next
  // One slot is one MFMA; an LDS operand serves two consecutive slots (the two row tiles).
  constexpr int NFRAG = MODE == BWD_DV ? 16 : MODE == BWD_DKV ? 32 : 24;  // LDS operands per block
  constexpr int LA = MODE == BWD_DK ? 4 : MODE == BWD_DQ ? 6 : 8;  // operands between the request of one and its use
  static_assert(NFRAG % LA == 0, "a block must leave the ring where the next block expects it");
  // slot of the first weight stage and slots from one stage to the next; BWD_DKV: of the dS stages
  // (its P stages run in slots 5 .. 15, in front of the dV accumulation)
  constexpr int WS = MODE == BWD_DV ? 4 : MODE == BWD_DKV ? 22 : 16;
  constexpr int WSTEP = MODE == BWD_DV ? 1 : MODE == BWD_DKV ? 3 : 2;
  bf16x8 fr[LA];
#pragma unroll
  for (int i = 0; i < LA; ++i) fr[i] = bf16x8{};
  floatx4 l4_keep[2] = {zero4, zero4}, d4_keep[2] = {zero4, zero4};
  // dQ: -D of the lane's two rows, as the accumulators of dP start from it
  const floatx4 nd_row[2] = {floatx4{-D_row[0], -D_row[0], -D_row[0], -D_row[0]}, floatx4{-D_row[1], -D_row[1], -D_row[1], -D_row[1]}};
  for (int t = 0; t < n_steps; ++t) {
    // the tiles of steps t and t+1 have landed for everybody; nobody reads that of t-1
    if (DEEP && fresh) tile_barrier<DEEP_REQUESTS>();
    else tile_barrier<0>();
    if (DEEP) {
      fresh = t + 3 < n_steps;
      if (fresh) {
        load_tile(ld, slot3);
        load_scalars(ld, slot3);
        advance(ld);
      }
    } else if (t + 2 < n_steps) {
      load_tile(ld, slot2);
      fetch_scalars(ld);
      advance(ld);
    }
#pragma unroll
    for (int blk = 0; blk < 2; ++blk) {
      const int jb = 2 * cur.tile + blk;
      if (jb < jb_lo || jb > jb_hi) {
        have = false;
        continue;
      }
      const int sb_lo = cb + 32 * jb;  // first column of the block
      // maps with a block predicate: a row meets the whole block or nothing of it
      bool lane_sees[2] = {true, true};
      bool masked;
      if (RMAP::kBlockPredicate) {
        lane_sees[0] = map.sees(row[0], sb_lo);
        lane_sees[1] = map.sees(row[1], sb_lo);
        if (__builtin_amdgcn_ballot_w64(lane_sees[0] || lane_sees[1]) == 0) {
          have = false;
          continue;
        }
        masked = __builtin_amdgcn_ballot_w64(lane_sees[0] && lane_sees[1]) != ~0ull;
      } else {
        masked = !block_unmasked(wb, kpre, sb_lo);
      }
      // Hand-scheduled.  dQ / dK: slots 0-15 dP of this block, 16-31 the scores of the next block,
      // 32-47 the accumulation; dV: 0-15 scores of the next block, 16-31 the accumulation.  LDS
      // operand f (slots 2f, 2f+1) is requested LA operands earlier into a ring of LA fragments,
      // across block and step boundaries (both following blocks have landed); the weights of
      // element pair u are formed in slot WS + WSTEP * u, after dP has drained and before the
      // accumulation needs them.  sched_barrier keeps the compiler from regrouping the slots.
      auto fetch = [&](int f) {
        const int here = blk * FBLOCK32;  // the block inside the step's slot
        // rows of the block that follows in this order, at tile `which` of its slot
        auto next_rows = [&](int which, int ff) {
          return blk == 0 ? kread_b(kb0, FBLOCK32 + which * FTILE, ff) : kread_b(kb1, which * FTILE, ff);
        };
        if (MODE == BWD_DKV) {
          if (f < 8) return kread_b(kb0, here + FTILE, f);   // dO rows: dP
          if (f < 16) return vread_b(here + FTILE, f - 8);   // dO^T: dV accumulation
          if (f < 24) return next_rows(0, f - 16);           // Q rows of the next block: its scores
          if (f < 32) return vread_b(here, f - 24);          // Q^T: dK accumulation
          return next_rows(1, f - 32);
        }
        if (MODE == BWD_DV) {
          if (f < 8) return next_rows(0, f);
          if (f < 16) return vread_b(here + FTILE, f - 8);
          return blk == 0 ? kread_b(kb1, 0, f - 16) : kread_b(kb1, FBLOCK32, f - 16);  // the block after the next
        }
        if (f < 8) return kread_b(kb0, here + FTILE, f);
        if (f < 16) return next_rows(0, f - 8);
        if (f < 24) return vread_b(here, f - 16);
        return next_rows(1, f - 24);
      };
      const float* sc = DEEP ? reinterpret_cast<const float*>(smem + (sb0 + 128 * blk))
                             : reinterpret_cast<const float*>(smem + slot0 + 2 * FTILE) + 32 * blk + 4 * g4;
      // scalars of the block that follows in this order
      const float* scn = blk == 0 ? sc + 32 : reinterpret_cast<const float*>(smem + sb1);
      if (!have) {  // first block of a run: nothing was prepared by a previous block
        if (MODE == BWD_DKV) {
          l4_keep[0] = *reinterpret_cast<const floatx4*>(sc);
          l4_keep[1] = *reinterpret_cast<const floatx4*>(sc + 16);
          d4_keep[0] = *reinterpret_cast<const floatx4*>(sc + 64);
          d4_keep[1] = *reinterpret_cast<const floatx4*>(sc + 64 + 16);
        }
#pragma unroll
        for (int t4 = 0; t4 < 4; ++t4) s_cur[t4 >> 1][t4 & 1] = zero4;
#pragma unroll
        for (int f = 0; f < 8; ++f) {
          const bf16x8 a = kread_b(kb0, blk * FBLOCK32, f);
#pragma unroll
          for (int rt = 0; rt < 2; ++rt) s_cur[f & 1][rt] = mfma(a, r1f[rt][f >> 1], s_cur[f & 1][rt]);
        }
#pragma unroll
        for (int i = 0; i < LA; ++i) fr[i] = fetch(i);
      }
      if (masked) {  // scores of invisible pairs become -inf (for a positive scale): weight 0
#pragma unroll
        for (int ct = 0; ct < 2; ++ct)
#pragma unroll
          for (int rt = 0; rt < 2; ++rt)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const bool vis = RMAP::kBlockPredicate ? lane_sees[rt]
                                                     : key_visible(sb_lo + 16 * ct + 4 * g4 + e, kpre, lo_l[rt], hi_l[rt]);
              if (!vis) s_cur[ct][rt][e] = s_hidden;
            }
      }
      floatx4 dp[2][2], s_next[2][2];
      bf16x8 wp[2];
      bf16x8 wp_p[MODE == BWD_DKV ? 2 : 1];   // BWD_DKV: the weights P (wp holds dS)
      floatx4 pf[TWO_STAGES ? 2 : 1][2];       // P before rounding, for dS
      floatx4 l4_[2], d4_[2];  // column scalars of the lane's columns, per column tile
      // (BWD_DKV keeps them across blocks: a block reads those of the next one in its last slots)
      floatx4 (&l4)[2] = MODE == BWD_DKV ? l4_keep : l4_;
      floatx4 (&d4)[2] = MODE == BWD_DKV ? d4_keep : d4_;
      // weights of pair u = 4 * rt + 2 * ct + h (columns 16 * ct + 4 * g4 + 2 * h, + 1 of row tile rt): P, or dS = P * (dP - D)
      auto stage = [&](int u) {
        const int rt = u >> 2, ct = (u >> 1) & 1, h = u & 1;
        float w[2];
#pragma unroll
        for (int v = 0; v < 2; ++v) {
          const int e = 2 * h + v;
          const float l = ROWS_ARE_QUERIES ? L2_row[rt] : l4[ct][e];
          float x = __builtin_amdgcn_exp2f(__builtin_fmaf(s_cur[ct][rt][e], c2, -l));
          if (MODE == BWD_DK) x *= dp[ct][rt][e] + d4[ct][e];
          w[v] = x;
        }
        if (MODE == BWD_DQ) {  // (the P stage: dS follows when dP is there)
          pf[ct][rt][2 * h] = w[0];
          pf[ct][rt][2 * h + 1] = w[1];
          return;
        }
        floatx2 f2 = {w[0], w[1]};
        bf16x2 h2 = __builtin_convertvector(f2, bf16x2);
        if (MODE == BWD_DKV) {  // (this is the P stage: keep the unrounded values for dS)
          pf[ct][rt][2 * h] = w[0];
          pf[ct][rt][2 * h + 1] = w[1];
          wp_p[rt][4 * ct + 2 * h] = h2[0];
          wp_p[rt][4 * ct + 2 * h + 1] = h2[1];
        } else {
          wp[rt][4 * ct + 2 * h] = h2[0];
          wp[rt][4 * ct + 2 * h + 1] = h2[1];
        }
      };
      // dQ and BWD_DKV: dS = P * (dP - D) of pair u; the accumulators of dP start from -D
      auto stage_ds = [&](int u) {
        const int rt = u >> 2, ct = (u >> 1) & 1, h = u & 1;
        floatx2 f2 = {pf[ct][rt][2 * h] * dp[ct][rt][2 * h], pf[ct][rt][2 * h + 1] * dp[ct][rt][2 * h + 1]};  // (dP started from -D)
        bf16x2 h2 = __builtin_convertvector(f2, bf16x2);
        wp[rt][4 * ct + 2 * h] = h2[0];
        wp[rt][4 * ct + 2 * h + 1] = h2[1];
      };
      constexpr int NSLOT = 2 * NFRAG;
      // (compile-time slot numbers: a loop of this size is beyond what the compiler unrolls in full)
      static_for<0, NSLOT>([&](auto slot_c) {
        constexpr int i = decltype(slot_c)::value;
        constexpr int f = i >> 1, rt = i & 1;
        const bf16x8 a = fr[f % LA];
        if (MODE == BWD_DKV) {
          if (f < 8) dp[f & 1][rt] = mfma(a, r2f[rt][f >> 1], f < 2 ? d4[f & 1] : dp[f & 1][rt]);  // from -D of the tile's columns
          else if (f < 16) acc_v[f - 8][rt] = mfma(a, wp_p[rt], acc_v[f - 8][rt]);
          else if (f < 24) s_next[f & 1][rt] = mfma(a, r1f[rt][(f - 16) >> 1], f < 18 ? zero4 : s_next[f & 1][rt]);
          else acc[f - 24][rt] = mfma(a, wp[rt], acc[f - 24][rt]);
        } else if (MODE == BWD_DV) {
          if (f < 8) s_next[f & 1][rt] = mfma(a, r1f[rt][f >> 1], f < 2 ? zero4 : s_next[f & 1][rt]);
          else acc[f - 8][rt] = mfma(a, wp[rt], acc[f - 8][rt]);
        } else {
          if (f < 8) dp[f & 1][rt] = mfma(a, r2f[rt][f >> 1], f < 2 ? (ROWS_ARE_QUERIES ? nd_row[rt] : zero4) : dp[f & 1][rt]);  // dQ: from -D of the row
          else if (f < 16) s_next[f & 1][rt] = mfma(a, r1f[rt][(f - 8) >> 1], f < 10 ? zero4 : s_next[f & 1][rt]);
          else acc[f - 16][rt] = mfma(a, wp[rt], acc[f - 16][rt]);
        }
        if (rt == 1) fr[f % LA] = fetch(f + LA);
        if (MODE == BWD_DKV) {  // P in front of the dV accumulation, dS behind dP
          // the next block's scalars, when this block has used its own for the last time
          if (i == 50) l4[0] = *reinterpret_cast<const floatx4*>(scn);
          if (i == 52) l4[1] = *reinterpret_cast<const floatx4*>(scn + 16);
          if (i == 54) d4[0] = *reinterpret_cast<const floatx4*>(scn + 64);
          if (i == 56) d4[1] = *reinterpret_cast<const floatx4*>(scn + 64 + 16);
          if (i >= 5 && i < 16 && (i - 5) % 3 != 2) stage((i - 5) - (i - 5) / 3);  // slots 5, 6, 8, 9, 11, 12, 14, 15
          if (i >= WS && (i - WS) % WSTEP == 0 && (i - WS) / WSTEP < 8) stage_ds((i - WS) / WSTEP);
        } else {
        if (!ROWS_ARE_QUERIES) {  // column scalars, four slots ahead of the first weight stage
          if (i == WS - 4) l4[0] = *reinterpret_cast<const floatx4*>(sc);
          if (i == WS - 3) l4[1] = *reinterpret_cast<const floatx4*>(sc + 16);
          if (MODE == BWD_DK && i == WS - 2) d4[0] = *reinterpret_cast<const floatx4*>(sc + 64);
          if (MODE == BWD_DK && i == WS - 1) d4[1] = *reinterpret_cast<const floatx4*>(sc + 64 + 16);
        }
        // dQ: P while dP is formed (the scores are then free for those of the next block), dS behind it
        if (MODE == BWD_DQ && i < 16 && i % 2 == 0) stage(i / 2);
        if (i >= WS && (i - WS) % WSTEP == 0 && (i - WS) / WSTEP < 8) {
          if (MODE == BWD_DQ) stage_ds((i - WS) / WSTEP);
          else stage((i - WS) / WSTEP);
        }
        }
        __builtin_amdgcn_sched_barrier(0);
      });
#pragma unroll
      for (int t4 = 0; t4 < 4; ++t4) s_cur[t4 >> 1][t4 & 1] = s_next[t4 >> 1][t4 & 1];
      have = true;
    }
    if (t + 2 < n_steps) put_scalars(slot2);
    advance(cur);
    const int ts = slot0;
    slot0 = slot1;
    slot1 = slot2;
    {
      const int d0 = slot0 - ts, d1 = slot1 - slot0;  // (slot0 and slot1 are the new ones already; ts the old slot0)
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        kb0[i] += d0;
        vb0[i] += d0;
        kb1[i] += d1;
        // (opaque to the compiler, which would otherwise keep the lane parts and add the slot at every read)
        asm volatile("" : "+v"(kb0[i]), "+v"(vb0[i]), "+v"(kb1[i]));
      }
      if (DEEP) {
        sb0 += d0;
        sb1 += d1;
        asm volatile("" : "+v"(sb0), "+v"(sb1));
      }
    }
    if (DEEP) {
      slot2 = slot3;
      slot3 = ts;
    } else {
      slot2 = ts;
    }
  }

  // ---------------------------------------------------------------- scale, round, store
  if (!wave_active) return;
  const float f = MODE == BWD_DV ? 1.f : p.scale;
  if (PARTIAL) {
    // fp32 partial sums: part[((set * B + batch) * Hkv + kvh) * n_rows + row][128]
#pragma unroll
    for (int rt = 0; rt < 2; ++rt)
      if (row_valid[rt]) {
        float* prow = p.part + ((((int64_t)set * p.B + batch) * p.Hkv + kvh) * n_rows + row[rt]) * 128 + 4 * g4;
#pragma unroll
        for (int dt = 0; dt < 8; ++dt) *reinterpret_cast<floatx4*>(prow + 16 * dt) = acc[dt][rt] * f;
      }
    return;
  }
  // The four lanes of a row hold head dims 4 * g4 .. + 3 of every 16-dim tile; a lane quarter and
  // its neighbour trade 8 bytes per tile pair so that each lane owns the whole 16-byte chunk
  // 4 * m + 2 * (g4 % 2) + g4 / 2 of its row.
  auto store_rows = [&](const floatx4 (&a)[8][2], int what, float factor) {
#pragma unroll
    for (int rt = 0; rt < 2; ++rt) {
      const bool keep = row_valid[rt] && map.store((int)rpos[rt]);
      uint16_t* orow;
      const int cofs = (2 * (g4 & 1) + (g4 >> 1)) * 8;
      if (what == BWD_DQ) orow = p.dq + (batch * p.dq_bs + rpos[rt] * p.dq_rs + hq * p.dq_hs + cofs);
      else if (what == BWD_DK) orow = p.dk + (batch * p.dk_bs + rpos[rt] * p.dk_rs + kvh * p.dk_hs + cofs);
      else orow = p.dv + (batch * p.dv_bs + rpos[rt] * p.dv_rs + kvh * p.dv_hs + cofs);
#pragma unroll
      for (int m = 0; m < 4; ++m) {
        uint32_t w[2][2];
#pragma unroll
        for (int t = 0; t < 2; ++t)
#pragma unroll
          for (int k2 = 0; k2 < 2; ++k2) {
            floatx2 v2 = {a[2 * m + t][rt][2 * k2] * factor, a[2 * m + t][rt][2 * k2 + 1] * factor};
            w[t][k2] = __builtin_bit_cast(uint32_t, __builtin_convertvector(v2, bf16x2));
          }
        auto q0 = __builtin_amdgcn_permlane16_swap(w[0][0], w[1][0], false, false);
        auto q1 = __builtin_amdgcn_permlane16_swap(w[0][1], w[1][1], false, false);
        if (keep) {
          u32x4 pk = {q0[0], q1[0], q0[1], q1[1]};
          if (RMAP::kAccumulate) {  // add to what an earlier pass has written (both rounded to bf16)
            const u32x4 old = *reinterpret_cast<const u32x4*>(orow + 32 * m);
#pragma unroll
            for (int i = 0; i < 4; ++i) {
              floatx2 s2 = {__uint_as_float(pk[i] << 16) + __uint_as_float(old[i] << 16),
                            __uint_as_float(pk[i] & 0xffff0000u) + __uint_as_float(old[i] & 0xffff0000u)};
              pk[i] = __builtin_bit_cast(uint32_t, __builtin_convertvector(s2, bf16x2));
            }
          }
          *reinterpret_cast<u32x4*>(orow + 32 * m) = pk;
        }
      }
    }
  };
  if constexpr (MODE == BWD_DKV) {
    store_rows(acc, BWD_DK, p.scale);
    store_rows(acc_v, BWD_DV, 1.f);
  } else {
    store_rows(acc, MODE, f);
  }
}

// Adds up the partial sums of the sink pass over the chunks and writes the sink rows of dk or dv:
// one thread per (batch, kv head, sink, 4 head dims).
__global__ void intra_bwd_sink_reduce(const float* part, int n_chunks, int B, int Hkv, int ns, uint16_t* out,
                                      int64_t o_bs, int64_t o_rs, int64_t o_hs) {
  const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
  const int64_t total = (int64_t)B * Hkv * ns * 32;
  if (i >= total) return;
  const int d4 = (int)(i & 31);
  const int64_t row = i >> 5;  // (batch * Hkv + kvh) * ns + sink
  floatx4 s = {0.f, 0.f, 0.f, 0.f};
  for (int c = 0; c < n_chunks; ++c) s += *reinterpret_cast<const floatx4*>(part + ((int64_t)c * B * Hkv * ns + row) * 128 + 4 * d4);
  const int sink = (int)(row % ns);
  const int64_t bh = row / ns;
  const int kvh = (int)(bh % Hkv), batch = (int)(bh / Hkv);
  floatx2 a = {s[0], s[1]}, b = {s[2], s[3]};
  uint32_t lo = __builtin_bit_cast(uint32_t, __builtin_convertvector(a, bf16x2));
  uint32_t hi = __builtin_bit_cast(uint32_t, __builtin_convertvector(b, bf16x2));
  uint16_t* o = out + (batch * o_bs + sink * o_rs + kvh * o_hs + 4 * d4);
  *reinterpret_cast<uint2*>(o) = make_uint2(lo, hi);
}

}  // namespace intra
