// Forward sparse-attention kernel for gfx950 (MI355X): one template for all five INTRA patterns.
//
// Replaces the reference's five CUDA kernels (csrc/flash_attn/src/flash_fwd_kernel.h:3970-6158
// with their loaders in gmem_tile.h) by one wave64/MFMA design:
//
//  * A workgroup of NW wavefronts owns a row block of one set: POS = NW*32/HP consecutive in-set
//    queries of HP query heads that share one KV head (GQA packing), so every gathered K/V tile
//    is used by all HP heads.  Each wavefront owns 32 queries of one head.
//  * Scores are computed transposed, S^T = K Q^T, with v_mfma_f32_32x32x16_bf16: the A operand
//    is a K tile row read from LDS (16 B per lane), the B operand is Q held in registers for the
//    whole kernel.  In the accumulator layout a lane then holds 16 keys of ONE query per 32x32
//    block, so the online softmax needs a single cross-lane exchange (lane ^ 32) per tile and the
//    rescale factors are plain per-lane scalars.
//  * O^T = V^T P^T: P^T is the softmax output still in registers (packed to bf16, no LDS round
//    trip); V^T comes from ds_read_b64_tr_b16 transposing reads of the row-major V tile.
//  * Software pipeline in steps of 32 keys: in step j a wavefront issues the 8 QK^T MFMAs of key
//    block j+1 next to the softmax VALU work of block j, then the 8 PV MFMAs of block j, with
//    all LDS operand reads issued two MFMAs ahead.  K therefore runs up to one tile ahead of V
//    in LDS: three K buffers, two V buffers, one barrier per 64-key tile.
//  * K/V rows are gathered from HBM with 16-byte loads, 16 lanes per 256-byte row, staged in
//    registers during the iteration and written to the free LDS buffers at its end.  LDS rows
//    are padded (K: 272 B, V: 320 B) so that the row-per-lane K reads and the 4-row transposing
//    V reads both spread over all 64 banks with plain base + immediate addressing.
//  * The running maximum is only raised (and O rescaled) when a tile's maximum exceeds it by
//    more than 2^8 in the exponent; softmax weights are exact after the final normalisation
//    because numerator and denominator share the reference maximum.
//  * Tiles outside a wavefront's key range are skipped; only tiles cut by a bound are masked.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include <type_traits>

#include "intra_maps.h"

namespace intra {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

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
  int B, H, Hkv, ratio;
  IntraGeom geom;
  float scale_log2;    // |softmax_scale| * log2(e), > 0
  float rescale_gap;   // raw-score gap that forces a new reference maximum: 8 / scale_log2
  int negate_q;        // softmax_scale < 0: flip the sign of Q instead
  int small_offsets;   // K/V row offsets fit 32 bits and the factors 24 bits
  uint32_t k_rs_bytes, v_rs_bytes;
  int n_sets;          // sets per (batch, kv head)
  int n_mblocks;       // row blocks of the largest set
  int hgroups;         // ratio / HP
  int n_pairs;         // B * Hkv * n_sets
  int items_per_pair;  // hgroups * n_mblocks
};

constexpr int BN = 64;            // keys per tile (one barrier per tile)
constexpr int KSTRIDE = 272;      // bytes per K row in LDS: 16 consecutive rows hit 16 distinct 16-byte slots
constexpr int VSTRIDE = 320;      // bytes per V row in LDS: 4 consecutive rows cover 4 distinct 64-byte spans
constexpr int KTILE = BN * KSTRIDE;
constexpr int VTILE = BN * VSTRIDE;
constexpr int VBASE = 3 * KTILE;  // K[3] then V[2]
constexpr int LDS_BYTES = 3 * KTILE + 2 * VTILE;

__device__ __forceinline__ float lane_xor32_max(float x) {
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float lane_xor32_sum(float x) {
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

template <int V>
using ic = std::integral_constant<int, V>;

template <class MAP, int HP, int NW>
__global__ __launch_bounds__(NW * 64) void intra_fwd_kernel(const KParams p) {
  constexpr int NT = NW * 64;
  constexpr int POS = NW * 32 / HP;          // in-set queries per row block
  constexpr int LD_PASSES = (BN * 16) / NT;  // 16-byte chunks per thread per tile (K or V)
  static_assert((BN * 16) % NT == 0, "tile must split evenly over the threads");

  __shared__ __attribute__((aligned(1024))) unsigned char smem[LDS_BYTES];

  // ---------------------------------------------------------------- which work item is this?
  // Workgroups are handed to the 8 XCDs round-robin by id.  All row blocks of one (batch, kv head,
  // set) "pair" go to one XCD, one pair after the other, longest row block first, so that the
  // pair's K/V stays in that XCD's L2 while its row blocks run.
  const int wg = blockIdx.x;
  const int xcd = wg & 7;
  const int slot = wg >> 3;
  const int pair = (slot / p.items_per_pair) * 8 + xcd;
  if (pair >= p.n_pairs) return;
  const int rem = slot % p.items_per_pair;
  const int mblk = p.n_mblocks - 1 - rem / p.hgroups;
  const int hg = rem % p.hgroups;
  const int nbh = p.B * p.Hkv;
  const int set = pair / nbh;
  const int bh = pair % nbh;
  const int batch = bh / p.Hkv;
  const int kvh = bh % p.Hkv;

  const MAP map(p.geom, set);
  const int nq = map.nq();
  const int nk = map.nk();
  const int t0 = mblk * POS;
  if (t0 >= nq) return;
  const int t1 = im_min(t0 + POS, nq) - 1;
  const int kt_lo = map.klo(t0);
  const int kt_hi = im_min(map.khi(t1), nk - 1);
  const int ntiles = (kt_hi - kt_lo + BN) / BN;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int h32 = lane >> 5;  // which half of the wavefront
  const int l32 = lane & 31;

  // ---------------------------------------------------------------- this wavefront's queries
  const int hw = wave % HP;
  const int wq0 = t0 + (wave / HP) * 32;
  const bool wave_active = wq0 <= t1;
  const int wq_last = im_min(wq0 + 31, t1);
  const bool row_valid = wq0 + l32 <= t1;
  const int tq = im_min(wq0 + l32, t1);
  const int lo_l = map.klo(tq);
  const int hi_l = im_min(map.khi(tq), nk - 1);
  WaveBounds wb = wave_bounds(map, im_min(wq0, t1), wq_last);
  // 32-key blocks (counted from kt_lo) this wavefront has to look at; blocks inside
  // [f_lo, f_hi] need no mask
  int bw_lo = __builtin_amdgcn_readfirstlane((wb.w_lo - kt_lo) / 32);
  int bw_hi = __builtin_amdgcn_readfirstlane((wb.w_hi - kt_lo) / 32);
  if (!wave_active) {
    bw_lo = 1;
    bw_hi = 0;
  }
  const int f_lo = __builtin_amdgcn_readfirstlane(wb.f_lo);
  const int f_hi = __builtin_amdgcn_readfirstlane(wb.f_hi);

  const int hq = kvh * p.ratio + hg * HP + hw;
  const int64_t qpos = map.qpos(tq);

  // Q^T fragments: lane holds query l32, head dims 16*ks + 8*h32 .. +7 for ks = 0..7
  bf16x8 qf[8];
  {
    const uint16_t* qrow = p.q + batch * p.q_bs + qpos * p.q_rs + hq * p.q_hs + h32 * 8;
#pragma unroll
    for (int ks = 0; ks < 8; ++ks) {
      u32x4 raw = *reinterpret_cast<const u32x4*>(qrow + ks * 16);
      if (p.negate_q) raw ^= 0x80008000u;
      qf[ks] = __builtin_bit_cast(bf16x8, raw);
    }
  }

  // ---------------------------------------------------------------- loader addressing
  // thread handles 16-byte chunk (tid % 16) of tile rows tid/16 + (NT/16)*pass
  const int ld_chunk = tid & 15;
  const int ld_row0 = tid >> 4;
  // Row gather addresses: uniform base pointer + per-lane 32-bit byte offset whenever every row of
  // the (batch, kv head) slice lies within 4 GiB of its base (checked on the host), which keeps
  // the address arithmetic to a couple of 24-bit multiplies per tile.
  const char* kbase = reinterpret_cast<const char*>(p.k + batch * p.k_bs + kvh * p.k_hs);
  const char* vbase = reinterpret_cast<const char*>(p.v + batch * p.v_bs + kvh * p.v_hs);
  u32x4 kst[LD_PASSES], vst[LD_PASSES];
  const int ld_koff = ld_row0 * KSTRIDE + ld_chunk * 16;
  const int ld_voff = VBASE + ld_row0 * VSTRIDE + ld_chunk * 16;
  const uint32_t k_rs_b = p.k_rs_bytes, v_rs_b = p.v_rs_bytes;
  const uint32_t ld_col = ld_chunk * 16;

  auto load_k = [&](int tile) {
    const int kb = kt_lo + tile * BN;
#pragma unroll
    for (int ps = 0; ps < LD_PASSES; ++ps) {
      int tk = im_min(kb + ld_row0 + ps * (NT / 16), nk - 1);
      uint32_t pos = map.kpos(tk);
      if (p.small_offsets)
        kst[ps] = *reinterpret_cast<const u32x4*>(kbase + (__umul24(pos, k_rs_b) + ld_col));
      else
        kst[ps] = *reinterpret_cast<const u32x4*>(kbase + ((int64_t)pos * p.k_rs * 2 + ld_col));
    }
  };
  auto load_v = [&](int tile) {
    const int kb = kt_lo + tile * BN;
#pragma unroll
    for (int ps = 0; ps < LD_PASSES; ++ps) {
      int tk = im_min(kb + ld_row0 + ps * (NT / 16), nk - 1);
      uint32_t pos = map.kpos(tk);
      if (p.small_offsets)
        vst[ps] = *reinterpret_cast<const u32x4*>(vbase + (__umul24(pos, v_rs_b) + ld_col));
      else
        vst[ps] = *reinterpret_cast<const u32x4*>(vbase + ((int64_t)pos * p.v_rs * 2 + ld_col));
    }
  };
  auto store_k = [&](int kbuf_off) {
#pragma unroll
    for (int ps = 0; ps < LD_PASSES; ++ps)
      *reinterpret_cast<u32x4*>(smem + kbuf_off + ld_koff + ps * (NT / 16) * KSTRIDE) = kst[ps];
  };
  auto store_v = [&](int vbuf_off) {
#pragma unroll
    for (int ps = 0; ps < LD_PASSES; ++ps)
      *reinterpret_cast<u32x4*>(smem + vbuf_off + ld_voff + ps * (NT / 16) * VSTRIDE) = vst[ps];
  };

  // K operand (A of S^T = K Q^T): lane reads 16 bytes of key row l32 at head dims 16*ks + 8*h32
  const int klane = l32 * KSTRIDE + h32 * 16;
  // V^T operand (A of O^T = V^T P^T) through transposing reads.  Within each group of 16 lanes,
  // lane i supplies the address of 4 head dims (4*(i%4)..) of key row i/4 and receives head dim i
  // of those 4 key rows.  Lane groups 0/1 take head dims 0-15/16-31 of a 32-dim block, the upper
  // 32 lanes the key rows 4..7 of each group of 8.
  const int vlane = VBASE + (4 * h32 + ((lane & 15) >> 2)) * VSTRIDE + 32 * ((lane >> 4) & 1) + 8 * (lane & 3);

  // ---------------------------------------------------------------- running softmax state
  floatx16 oacc[4];
#pragma unroll
  for (int db = 0; db < 4; ++db)
#pragma unroll
    for (int e = 0; e < 16; ++e) oacc[db][e] = 0.f;
  floatx16 s0, s1;  // scores of two consecutive 32-key blocks
  float m_run = -INFINITY;  // reference maximum of the exponentials (raw score units)
  float mc = 0.f;           // m_run * c, 0 while m_run is still -inf
  float l_run = 0.f;
  const float c = p.scale_log2;
  const bf16x2 ones2 = {(__bf16)1.0f, (__bf16)1.0f};
  const float gap = p.rescale_gap;

  // operand reads; koff / voff are byte offsets of (buffer, 32-key block) in LDS
  auto kread = [&](int koff, int ks) {
    return *reinterpret_cast<const bf16x8*>(smem + koff + klane + ks * 32);
  };
  auto vread = [&](int voff, int j) {  // j = 4 * t + db: keys 16t..16t+15 of the block, head dims 32db..
    const int off = (j >> 2) * 16 * VSTRIDE + (j & 3) * 64;
    bf16x4 v0 = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
        (__attribute__((address_space(3))) bf16x4*)(smem + voff + vlane + off));
    bf16x4 v1 = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
        (__attribute__((address_space(3))) bf16x4*)(smem + voff + vlane + off + 8 * VSTRIDE));
    return __builtin_shufflevector(v0, v1, 0, 1, 2, 3, 4, 5, 6, 7);
  };
  auto zero16 = [] {
    floatx16 z;
#pragma unroll
    for (int e = 0; e < 16; ++e) z[e] = 0.f;
    return z;
  };

  // ----- unscheduled pieces, used at the edges of a wavefront's key range
  auto qk_block = [&](floatx16& acc, int koff) {
    acc = zero16();
#pragma unroll
    for (int ks = 0; ks < 8; ++ks)
      acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(kread(koff, ks), qf[ks], acc, 0, 0, 0);
  };
  auto mask_block = [&](floatx16& s, int kb32) {
#pragma unroll
    for (int e = 0; e < 16; ++e) {
      int key = kb32 + 8 * (e >> 2) + 4 * h32 + (e & 3);
      if (key < lo_l || key > hi_l) s[e] = -INFINITY;
    }
  };
  // The running maximum only moves when some query's block maximum exceeds it by more than
  // `gap`; until then the exponentials just grow up to 2^8, which fp32/bf16 hold easily.
  auto raise_max = [&](float mx) {
    if (__builtin_amdgcn_ballot_w64(mx > m_run + gap) != 0) {
      const float m_new = fmaxf(m_run, mx);
      const float m_use = m_new == -INFINITY ? 0.f : m_new;
      const float alpha = __builtin_amdgcn_exp2f((m_run - m_use) * c);
      m_run = m_new;
      mc = m_use * c;
      l_run *= alpha;
#pragma unroll
      for (int db = 0; db < 4; ++db)
#pragma unroll
        for (int e = 0; e < 16; ++e) oacc[db][e] *= alpha;
    }
  };
  // ----- loader work of one tile iteration: put the rows fetched during the previous iteration
  // (K(i+2), V(i+1), waiting in registers) into the LDS buffers of K(i-1) and V(i-1), then start
  // fetching K(i+3) and V(i+2).  Rows past the end are clamped to the last key, so the tail
  // iterations just re-read one cached row instead of branching.
  auto loader = [&](int i, int kdst, int vdst) {
    store_k(kdst);
    store_v(vdst);
    load_k(i + 3);
    load_v(i + 2);
  };

  // ----- hand-scheduled step: QK^T of the next key block (8 MFMAs) and PV of the current one
  // (8 MFMAs) with the softmax VALU work of the current block spread between them.  One "slot"
  // is one MFMA.  LDS operands are fetched a whole phase (8 slots) ahead: the V^T operands of
  // this step's PV during its QK^T slots, the K operands of the NEXT step's QK^T during this
  // step's PV slots (ka lives across steps and across the tile barrier: the K tile it reads was
  // made visible by an earlier barrier and is not overwritten before the next one), so each
  // phase opens with a single wait.  The exponentials are cut into 8 units of one bf16 pair and
  // run through a 3-stage pipeline (scale, exp2, pack + row sum) one slot apart, so that no VALU
  // instruction waits for the one issued just before it; P^T half 0 is complete at slot 7, half
  // 1 at slot 11.  The first step of a tile also carries the tile's loader work in slots 12..15,
  // where the VALU is otherwise idle.  sched_barrier keeps the compiler from regrouping.
  bf16x8 ka[8];
  auto steady = [&](const floatx16& s, floatx16& n, int koff_next, int voff, auto with_loader, int i,
                    int kdst, int vdst) {
    bf16x8 va[8], pb[2];
    float mx0, mx1;
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): ka[] has landed
#pragma unroll
    for (int g = 0; g < 2; ++g) {
      va[g] = vread(voff, g);
      n = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka[g], qf[g], g == 0 ? zero16() : n, 0, 0, 0);
      const int e0 = 8 * g;
      float m = fmaxf(fmaxf(s[e0], s[e0 + 1]), s[e0 + 2]);
      m = fmaxf(fmaxf(m, s[e0 + 3]), s[e0 + 4]);
      m = fmaxf(fmaxf(m, s[e0 + 5]), s[e0 + 6]);
      m = fmaxf(m, s[e0 + 7]);
      if (g == 0) mx0 = m;
      else mx1 = m;
      __builtin_amdgcn_sched_barrier(0);
    }
    raise_max(lane_xor32_max(fmaxf(mx0, mx1)));
    float rs = 0.f;
    float fx[8][2], px[8][2];
    auto stage_f = [&](int u) {
      fx[u][0] = __builtin_fmaf(s[2 * u], c, -mc);
      fx[u][1] = __builtin_fmaf(s[2 * u + 1], c, -mc);
    };
    auto stage_e = [&](int u) {
      px[u][0] = __builtin_amdgcn_exp2f(fx[u][0]);
      px[u][1] = __builtin_amdgcn_exp2f(fx[u][1]);
    };
    auto stage_c = [&](int u) {
      floatx2 f = {px[u][0], px[u][1]};
      bf16x2 h = __builtin_convertvector(f, bf16x2);
      rs = __builtin_amdgcn_fdot2_f32_bf16(h, ones2, rs, false);  // sums what PV will multiply
      pb[u >> 2][2 * (u & 3)] = h[0];
      pb[u >> 2][2 * (u & 3) + 1] = h[1];
    };
    auto valu_slot = [&](int k) {  // slot k: scale unit k-2, exp2 unit k-3, pack unit k-4
      if (k - 2 >= 0 && k - 2 < 8) stage_f(k - 2);
      if (k - 3 >= 0 && k - 3 < 8) stage_e(k - 3);
      if (k - 4 >= 0 && k - 4 < 8) stage_c(k - 4);
    };
#pragma unroll
    for (int g = 2; g < 8; ++g) {
      va[g] = vread(voff, g);
      n = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ka[g], qf[g], n, 0, 0, 0);
      valu_slot(g);
      __builtin_amdgcn_sched_barrier(0);
    }
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): va[] has landed
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      ka[j] = kread(koff_next, j);
      oacc[j & 3] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va[j], pb[j >> 2], oacc[j & 3], 0, 0, 0);
      valu_slot(8 + j);

      __builtin_amdgcn_sched_barrier(0);
    }
    l_run += rs;
  };

  // Step j: softmax + PV of key block j (scores in `cur`, V rows at voff) and QK^T of key block
  // j+1 into `nxt` (its K rows at koff; those of block j+2 at koff_next).  A wavefront runs the
  // steps jq..jp with jq = bw_lo - 1: in step jq only the QK^T half matters, so its scores are
  // preset to -inf (weights 0, the maximum stays -inf); in step jp the QK^T half computes a block
  // nobody reads.  That keeps one code path through the accumulators.
  const int jq = bw_lo - 1, jp = bw_hi;
  auto step = [&](int j, floatx16& cur, floatx16& nxt, int koff, int koff_next, int voff, auto with_loader,
                  int i, int kdst, int vdst) {
    if (decltype(with_loader)::value) loader(i, kdst, vdst);
    if (j < jq || j > jp) return;
    const int kb32 = kt_lo + 32 * j;
    if (j == jq) {
#pragma unroll
      for (int e = 0; e < 16; ++e) cur[e] = -INFINITY;
#pragma unroll
      for (int g = 0; g < 8; ++g) ka[g] = kread(koff, g);
    } else if (kb32 < f_lo || kb32 + 31 > f_hi) {
      mask_block(cur, kb32);
    }
    steady(cur, nxt, koff_next, voff, with_loader, i, kdst, vdst);
  };

  // ---------------------------------------------------------------- main loop
  // At the top of iteration i the LDS holds K(i), K(i+1) and V(i), and the staging registers hold
  // (or are receiving) K(i+2) and V(i+1).  During the iteration those go into the buffers of
  // K(i-1) and V(i-1), which no wavefront reads after the barrier that opened iteration i, and
  // the fetch of K(i+3) and V(i+2) starts: every global load has a whole iteration to arrive.
  load_k(0);
  load_v(0);
  store_k(0);
  store_v(0);
  load_k(1);
  store_k(KTILE);
  load_k(2);
  load_v(1);
  __syncthreads();
  if (jq < 0 && jp >= 0) {
    qk_block(s0, 0);
#pragma unroll
    for (int g = 0; g < 8; ++g) ka[g] = kread(32 * KSTRIDE, g);
  }
  int kcur = 0, knext = KTILE, knext2 = 2 * KTILE;
  for (int i = 0; i < ntiles; ++i) {
    __syncthreads();
    const int vcur = (i & 1) * VTILE;
    step(2 * i, s0, s1, kcur + 32 * KSTRIDE, knext, vcur, ic<1>{}, i, knext2, VTILE - vcur);
    step(2 * i + 1, s1, s0, knext, knext + 32 * KSTRIDE, vcur + 32 * VSTRIDE, ic<0>{}, i, 0, 0);
    const int t = kcur;
    kcur = knext;
    knext = knext2;
    knext2 = t;
  }

  // ---------------------------------------------------------------- normalise and scatter-store
  if (!wave_active) return;
  const float l_tot = lane_xor32_sum(l_run);
  const float inv = l_tot > 0.f ? 1.f / l_tot : 0.f;
  if (row_valid) {
    uint16_t* orow = p.o + batch * p.o_bs + qpos * p.o_rs + hq * p.o_hs + 4 * h32;
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        floatx2 f0 = {oacc[db][4 * g] * inv, oacc[db][4 * g + 1] * inv};
        floatx2 f1 = {oacc[db][4 * g + 2] * inv, oacc[db][4 * g + 3] * inv};
        bf16x2 b0 = __builtin_convertvector(f0, bf16x2);
        bf16x2 b1 = __builtin_convertvector(f1, bf16x2);
        u32x2 pk = {__builtin_bit_cast(uint32_t, b0), __builtin_bit_cast(uint32_t, b1)};
        *reinterpret_cast<u32x2*>(orow + 32 * db + 8 * g) = pk;
      }
  }
}

}  // namespace intra
