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

typedef float floatx4 __attribute__((ext_vector_type(4)));

enum BwdMode : int { BWD_DQ = 0, BWD_DK = 1, BWD_DV = 2 };

struct BParams {
  const uint16_t *q, *k, *v, *o, *dout;  // bf16 (B, S, heads, 128)
  const float* lse;                      // (B, H, S): ln sum exp(scale * q.k) from the forward pass
  float* dsum;                           // (B, H, S) workspace: D = rowsum(dO o O), written by dQ, read by dK
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

constexpr int BWD_SLOT = 2 * TILE_BYTES + 512;  // two tiles and 2 x 64 column scalars
constexpr int BWD_LDS_BYTES = 3 * BWD_SLOT;

// RMAP: row map (intra_bwd_maps.h).  PARTIAL: the results are partial sums over the set's columns,
// written as fp32 to p.part instead of bf16 to dk / dv (sink pass).
template <class RMAP, int MODE, int HP, bool PARTIAL = false>
__global__ __launch_bounds__(512) void intra_bwd_kernel(const BParams p) {
  constexpr int NW = 8;
  constexpr bool ROWS_ARE_QUERIES = MODE == BWD_DQ;
  constexpr int POS = ROWS_ARE_QUERIES ? NW * 32 / HP : NW * 32;  // rows per row block (of one head)

  __shared__ __attribute__((aligned(1024))) unsigned char smem[BWD_LDS_BYTES];
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) unsigned char*)smem;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int h32 = lane >> 5;
  const int l32 = lane & 31;

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
  const int hw = ROWS_ARE_QUERIES ? wave % HP : 0;
  const int wr0 = r0 + (ROWS_ARE_QUERIES ? wave / HP : wave) * 32;
  const bool wave_active = wr0 <= r1;
  const bool row_valid = wr0 + l32 <= r1;
  const int row = im_min(wr0 + l32, r1);
  const int lo_l = map.lo(row), hi_l = map.hi(row);
  // union and intersection of the ranges of the wavefront's rows (rows past the end repeat the last)
  WaveBounds wb;
  {
    int a = lo_l, b = hi_l, c = lo_l, d = hi_l;
#pragma unroll
    for (int m = 1; m < 32; m <<= 1) {
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
  const int64_t rpos = map.row_pos(row);
  const int hq = kvh * p.ratio + hg * HP + hw;  // query head of a query row

  // ---------------------------------------------------------------- row operands (MFMA B fragments)
  // lane holds row l32, head dims 16*ks + 8*h32 .. +7 for ks = 0..7
  bf16x8 r1f[8], r2f[8];
  float L2_row = 0.f, D_row = 0.f;
  {
    const uint16_t *a1, *a2;
    if (ROWS_ARE_QUERIES) {
      a1 = p.q + (batch * p.q_bs + rpos * p.q_rs + hq * p.q_hs + h32 * 8);
      a2 = p.dout + (batch * p.do_bs + rpos * p.do_rs + hq * p.do_hs + h32 * 8);
    } else {
      a1 = p.k + (batch * p.k_bs + rpos * p.k_rs + kvh * p.k_hs + h32 * 8);
      a2 = p.v + (batch * p.v_bs + rpos * p.v_rs + kvh * p.v_hs + h32 * 8);
    }
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      r1f[ks] = *reinterpret_cast<const bf16x8*>(a1 + ks * 16);
      if (MODE != BWD_DV) r2f[ks] = *reinterpret_cast<const bf16x8*>(a2 + ks * 16);
    }
    if (ROWS_ARE_QUERIES) {
      // D = dO . O of the row: this lane's 64 head dims, then the other half from lane ^ 32
      const uint16_t* ao = p.o + (batch * p.o_bs + rpos * p.o_rs + hq * p.o_hs + h32 * 8);
      float part = 0.f;
#pragma unroll
      for (int ks = 0; ks < 8; ++ks) {
        const bf16x8 of = *reinterpret_cast<const bf16x8*>(ao + ks * 16);
#pragma unroll
        for (int d = 0; d < 8; ++d) part += (float)r2f[ks][d] * (float)of[d];
      }
      D_row = lane_xor32_sum(part);
      L2_row = p.lse[batch * p.lse_bs + hq * p.lse_hs + rpos * p.lse_ts] * 1.4426950408889634f;
      if (row_valid && h32 == 0) p.dsum[batch * p.ds_bs + hq * p.ds_hs + rpos] = D_row;
    }
  }

  // ---------------------------------------------------------------- LDS addressing (as in the forward kernel)
  const int ld_row = lane >> 4;
  const uint32_t ld_col = (((lane & 15) ^ (4 * ld_row)) << 4);
  int kaddr[8];
#pragma unroll
  for (int ks = 0; ks < 8; ++ks)
    kaddr[ks] = (l32 >> 2) * GROUP_STRIDE + (l32 & 3) * 256 + (((2 * ks + h32) ^ (4 * (l32 & 3))) << 4);
  int vaddr[4];
  {
    const int i16 = lane & 15, g2 = (lane >> 4) & 1, ri = i16 >> 2;
#pragma unroll
    for (int db = 0; db < 4; ++db)
      vaddr[db] = h32 * GROUP_STRIDE + ri * 256 + (((4 * db + 2 * g2 + ((i16 & 3) >> 1)) ^ (4 * ri)) << 4) + 8 * (i16 & 1);
  }
  auto kread = [&](int off, int ks) { return *reinterpret_cast<const bf16x8*>(smem + off + kaddr[ks]); };
  auto vread = [&](int off, int j) {
    const int o2 = off + vaddr[j & 3] + (j >> 2) * 4 * GROUP_STRIDE;
    bf16x4 v0 = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((__attribute__((address_space(3))) bf16x4*)(smem + o2));
    bf16x4 v1 = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
        (__attribute__((address_space(3))) bf16x4*)(smem + o2 + 2 * GROUP_STRIDE));
    return __builtin_shufflevector(v0, v1, 0, 1, 2, 3, 4, 5, 6, 7);
  };

  floatx16 acc[4];
#pragma unroll
  for (int db = 0; db < 4; ++db)
#pragma unroll
    for (int e = 0; e < 16; ++e) acc[db][e] = 0.f;
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
  auto load_tile = [&](const Cursor& cu, int slot_off) {
#pragma unroll
    for (int gi = 0; gi < 2; ++gi) {
      const int grp = wave * 2 + gi;
      const int c = im_min(cb + cu.tile * BN + 4 * grp + ld_row, n_cols - 1);
      const uint32_t pos = col_pos(c);
      dma_group(c1base + (cu.head * c1hs + (uint64_t)pos * c1rs + ld_col), lds_base + slot_off + grp * GROUP_STRIDE);
      dma_group(c2base + (cu.head * c2hs + (uint64_t)pos * c2rs + ld_col),
                lds_base + slot_off + TILE_BYTES + grp * GROUP_STRIDE);
    }
  };
  // column scalars of a step (dK / dV): wavefront 0 fetches lse * log2(e) and D of its 64 columns
  float sc_l = 0.f, sc_d = 0.f;
  auto fetch_scalars = [&](const Cursor& cu) {
    if (!ROWS_ARE_QUERIES && wave == 0) {
      const int c = im_min(cb + cu.tile * BN + lane, n_cols - 1);
      const int64_t pos = col_pos(c);
      const int hcol = kvh * p.ratio + cu.head;
      sc_l = p.lse[batch * p.lse_bs + hcol * p.lse_hs + pos * p.lse_ts] * 1.4426950408889634f;
      if (MODE == BWD_DK) sc_d = p.dsum[batch * p.ds_bs + hcol * p.ds_hs + pos];
    }
  };
  auto put_scalars = [&](int slot_off) {
    if (!ROWS_ARE_QUERIES && wave == 0) {
      float* sc = reinterpret_cast<float*>(smem + slot_off + 2 * TILE_BYTES);
      sc[lane] = sc_l;
      sc[64 + lane] = sc_d;
    }
  };
  auto zero16 = [] {
    floatx16 z;
#pragma unroll
    for (int e = 0; e < 16; ++e) z[e] = 0.f;
    return z;
  };
  auto scores = [&](int off) {
    floatx16 s = zero16();
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) s = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kread(off, ks), r1f[ks], s, 0, 0, 0);
    return s;
  };

  // Three tile slots: while step t works on its tile, the tile of step t+1 has landed (the scores
  // of its first block are formed at the end of step t) and the tile of step t+2 is in flight.
  Cursor cur{ROWS_ARE_QUERIES ? 0 : ntiles - 1, 0};  // step being computed
  Cursor ld = cur;                                   // step being requested
  for (int t = 0; t < 2 && t < n_steps; ++t) {
    load_tile(ld, t * BWD_SLOT);
    fetch_scalars(ld);
    put_scalars(t * BWD_SLOT);
    advance(ld);
  }
  int slot0 = 0, slot1 = BWD_SLOT, slot2 = 2 * BWD_SLOT;
  floatx16 s_cur;
#pragma unroll
  for (int e = 0; e < 16; ++e) s_cur[e] = 0.f;
  bool have = false;  // s_cur and fr hold what a previous block prepared for the one that comes next
  constexpr int NSLOT = MODE == BWD_DV ? 16 : 24;  // MFMAs per block
  constexpr int LA = MODE == BWD_DK ? 4 : MODE == BWD_DV ? 8 : 6;  // slots between the request of an LDS operand and its use
  static_assert(NSLOT % LA == 0, "a block must leave the ring where the next block expects it");
  constexpr int W0 = MODE == BWD_DV ? 2 : 10;      // slot of the first weight stage
  bf16x8 fr[LA];
#pragma unroll
  for (int i = 0; i < LA; ++i) fr[i] = bf16x8{};
  for (int t = 0; t < n_steps; ++t) {
    tile_barrier<0>();  // the tiles of steps t and t+1 have landed for everybody; nobody reads that of t-1
    if (t + 2 < n_steps) {
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
      bool lane_sees = true;
      uint64_t seeing = ~0ull;
      if (RMAP::kBlockPredicate) {
        lane_sees = map.sees(row, sb_lo);
        seeing = __builtin_amdgcn_ballot_w64(lane_sees);
        if (seeing == 0) {
          have = false;
          continue;
        }
      }
      const bool masked = RMAP::kBlockPredicate ? seeing != ~0ull : !block_unmasked(wb, kpre, sb_lo);
      // this block, the one that follows in this order, and the one after that
      const int c1off = slot0 + blk * BLOCK32, c2off = c1off + TILE_BYTES;
      const int c1n = blk == 0 ? c1off + BLOCK32 : slot1, c2n = c1n + TILE_BYTES;
      const int c1nn = blk == 0 ? slot1 : slot1 + BLOCK32;
      // Hand-scheduled: one slot is one MFMA.  dQ / dK: slots 0-7 dP of this block, 8-15 the
      // scores of the next block, 16-23 the accumulation; dV: 0-7 scores of the next block, 8-15
      // the accumulation.  The LDS operand of slot i is requested in slot i - LA into a ring of
      // LA fragments, across block and step boundaries (both following blocks have landed); the
      // weights of element pair u are formed in slot W0 + u, after dP has drained and before the
      // accumulation needs them.  sched_barrier keeps the compiler from regrouping the slots.
      auto fetch = [&](int i) {
        if (MODE == BWD_DV) {
          if (i < 8) return kread(c1n, i);
          if (i < 16) return vread(c2off, i - 8);
          return kread(c1nn, i - 16);
        }
        if (i < 8) return kread(c2off, i);
        if (i < 16) return kread(c1n, i - 8);
        if (i < 24) return vread(c1off, i - 16);
        return kread(c2n, i - 24);
      };
      if (!have) {  // first block of a run: nothing was prepared by a previous block
        s_cur = scores(c1off);
#pragma unroll
        for (int i = 0; i < LA; ++i) fr[i] = fetch(i);
      }
      const float* sc = reinterpret_cast<const float*>(smem + slot0 + 2 * TILE_BYTES) + 32 * blk + 4 * h32;
      if (masked) {  // scores of invisible pairs become -inf (for a positive scale): weight 0
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const bool vis = RMAP::kBlockPredicate ? lane_sees
                                                 : key_visible(sb_lo + 8 * (e >> 2) + 4 * h32 + (e & 3), kpre, lo_l, hi_l);
          if (!vis) s_cur[e] = s_hidden;
        }
      }
      floatx16 dp, s_next;
      bf16x8 wp[2];
      floatx4 l4[4], d4[4];
      auto stage = [&](int u) {  // weights of elements 2u, 2u+1: P, or dS = P * (dP - D)
        float w[2];
#pragma unroll
        for (int v = 0; v < 2; ++v) {
          const int e = 2 * u + v;
          const float l = ROWS_ARE_QUERIES ? L2_row : l4[e >> 2][e & 3];
          float x = __builtin_amdgcn_exp2f(__builtin_fmaf(s_cur[e], c2, -l));
          if (MODE != BWD_DV) x *= dp[e] - (ROWS_ARE_QUERIES ? D_row : d4[e >> 2][e & 3]);
          w[v] = x;
        }
        floatx2 f = {w[0], w[1]};
        bf16x2 h = __builtin_convertvector(f, bf16x2);
        wp[u >> 2][2 * (u & 3)] = h[0];
        wp[u >> 2][2 * (u & 3) + 1] = h[1];
      };
#pragma unroll
      for (int i = 0; i < NSLOT; ++i) {
        const bf16x8 a = fr[i % LA];
        if (MODE == BWD_DV) {
          if (i < 8) s_next = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, r1f[i], i == 0 ? zero16() : s_next, 0, 0, 0);
          else acc[(i - 8) & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, wp[(i - 8) >> 2], acc[(i - 8) & 3], 0, 0, 0);
        } else {
          if (i < 8) dp = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, r2f[i], i == 0 ? zero16() : dp, 0, 0, 0);
          else if (i < 16) s_next = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, r1f[i - 8], i == 8 ? zero16() : s_next, 0, 0, 0);
          else acc[(i - 16) & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, wp[(i - 16) >> 2], acc[(i - 16) & 3], 0, 0, 0);
        }
        fr[i % LA] = fetch(i + LA);
        if (!ROWS_ARE_QUERIES && i >= W0 - 2 && i < W0 + 6 && ((i - (W0 - 2)) & 1) == 0) {
          const int t4 = (i - (W0 - 2)) >> 1;  // column scalars of elements 4*t4 .. 4*t4+3, two slots ahead
          l4[t4] = *reinterpret_cast<const floatx4*>(sc + 8 * t4);
          if (MODE == BWD_DK) d4[t4] = *reinterpret_cast<const floatx4*>(sc + 64 + 8 * t4);
        }
        if (i >= W0 && i < W0 + 8) stage(i - W0);
        __builtin_amdgcn_sched_barrier(0);
      }
      s_cur = s_next;
      have = true;
    }
    if (t + 2 < n_steps) put_scalars(slot2);
    advance(cur);
    const int ts = slot0;
    slot0 = slot1;
    slot1 = slot2;
    slot2 = ts;
  }

  // ---------------------------------------------------------------- scale, round, store
  if (!wave_active) return;
  const float f = MODE == BWD_DV ? 1.f : p.scale;
  if (PARTIAL) {
    // fp32 partial sums: part[((set * B + batch) * Hkv + kvh) * n_rows + row][128]; lane holds, per
    // 32 head dims db, the dims 8*(e>>2) + 4*h32 + (e&3) of its row
    if (row_valid) {
      float* prow = p.part + ((((int64_t)set * p.B + batch) * p.Hkv + kvh) * n_rows + row) * 128 + 4 * h32;
#pragma unroll
      for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int g4 = 0; g4 < 4; ++g4) {
          floatx4 o4 = {acc[db][4 * g4] * f, acc[db][4 * g4 + 1] * f, acc[db][4 * g4 + 2] * f, acc[db][4 * g4 + 3] * f};
          *reinterpret_cast<floatx4*>(prow + 32 * db + 8 * g4) = o4;
        }
    }
    return;
  }
  const bool keep = row_valid && map.store((int)rpos);
  uint16_t* orow;
  if (MODE == BWD_DQ) orow = p.dq + (batch * p.dq_bs + rpos * p.dq_rs + hq * p.dq_hs + 8 * h32);
  else if (MODE == BWD_DK) orow = p.dk + (batch * p.dk_bs + rpos * p.dk_rs + kvh * p.dk_hs + 8 * h32);
  else orow = p.dv + (batch * p.dv_bs + rpos * p.dv_rs + kvh * p.dv_hs + 8 * h32);
#pragma unroll
  for (int db = 0; db < 4; ++db)
#pragma unroll
    for (int g2 = 0; g2 < 2; ++g2) {
      uint32_t w[4];
#pragma unroll
      for (int half = 0; half < 2; ++half)
#pragma unroll
        for (int k2 = 0; k2 < 2; ++k2) {
          const int e = 8 * g2 + 4 * half + 2 * k2;
          floatx2 v2 = {acc[db][e] * f, acc[db][e + 1] * f};
          w[2 * half + k2] = __builtin_bit_cast(uint32_t, __builtin_convertvector(v2, bf16x2));
        }
      auto q0 = __builtin_amdgcn_permlane32_swap(w[0], w[2], false, false);
      auto q1 = __builtin_amdgcn_permlane32_swap(w[1], w[3], false, false);
      if (keep) {
        u32x4 pk = {q0[0], q1[0], q0[1], q1[1]};
        if (RMAP::kAccumulate) {  // add to what an earlier pass has written (both rounded to bf16)
          const u32x4 old = *reinterpret_cast<const u32x4*>(orow + 32 * db + 16 * g2);
#pragma unroll
          for (int i = 0; i < 4; ++i) {
            floatx2 s2 = {__uint_as_float(pk[i] << 16) + __uint_as_float(old[i] << 16),
                          __uint_as_float(pk[i] & 0xffff0000u) + __uint_as_float(old[i] & 0xffff0000u)};
            pk[i] = __builtin_bit_cast(uint32_t, __builtin_convertvector(s2, bf16x2));
          }
        }
        *reinterpret_cast<u32x4*>(orow + 32 * db + 16 * g2) = pk;
      }
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
