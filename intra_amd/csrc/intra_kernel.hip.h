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
//  * K/V rows are gathered from HBM with 16-byte loads, 16 lanes per 256-byte row, staged in
//    registers during the MFMA work of the current tile and written to the other LDS buffer
//    (one barrier per tile).  LDS rows are XOR-swizzled in 16-byte chunks so that both the
//    row-per-lane K reads and the 4-row transposing V reads spread over all banks.
//  * Blocks of 32 keys that no query of the wavefront may see are skipped; only blocks cut by a
//    bound get the per-element mask.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

#include "intra_maps.h"

namespace intra {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4 __attribute__((ext_vector_type(4)));
typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
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
  float scale_log2;  // |softmax_scale| * log2(e), > 0
  int negate_q;      // softmax_scale < 0: flip the sign of Q instead
  int n_sets;        // sets per (batch, kv head)
  int n_mblocks;     // row blocks of the largest set
  int hgroups;       // ratio / HP
  int n_pairs;       // B * Hkv * n_sets
  int items_per_pair;  // hgroups * n_mblocks
};

constexpr int BN = 64;                 // keys per tile
constexpr int TILE_BYTES = BN * 256;   // one K or V tile in LDS
constexpr int BUF_BYTES = 2 * TILE_BYTES;

// 16-byte chunk c of tile row r lives at chunk slot c ^ swz(r).  swz is a bijection of r % 16
// whose two high bits differ for four consecutive rows.
__device__ __forceinline__ int swz(int r) { return ((r & 3) << 2) | ((r >> 2) & 3); }

__device__ __forceinline__ float lane_xor32_max(float x) {
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return fmaxf(__uint_as_float(r[0]), __uint_as_float(r[1]));
}
__device__ __forceinline__ float lane_xor32_sum(float x) {
  auto r = __builtin_amdgcn_permlane32_swap(__float_as_uint(x), __float_as_uint(x), false, false);
  return __uint_as_float(r[0]) + __uint_as_float(r[1]);
}

typedef __attribute__((address_space(3))) unsigned char lds_byte;

template <class MAP, int HP, int NW>
__global__ __launch_bounds__(NW * 64) void intra_fwd_kernel(const KParams p) {
  constexpr int NT = NW * 64;
  constexpr int POS = NW * 32 / HP;      // in-set queries per row block
  constexpr int LD_PASSES = (BN * 16) / NT;  // 16-byte chunks per thread per tile (K or V)
  static_assert((BN * 16) % NT == 0, "tile must split evenly over the threads");

  __shared__ __attribute__((aligned(1024))) unsigned char smem[2 * BUF_BYTES];

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
  wb.w_lo = __builtin_amdgcn_readfirstlane(wb.w_lo);
  wb.w_hi = __builtin_amdgcn_readfirstlane(wb.w_hi);
  wb.f_lo = __builtin_amdgcn_readfirstlane(wb.f_lo);
  wb.f_hi = __builtin_amdgcn_readfirstlane(wb.f_hi);

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
  const uint16_t* kbase = p.k + batch * p.k_bs + kvh * p.k_hs + ld_chunk * 8;
  const uint16_t* vbase = p.v + batch * p.v_bs + kvh * p.v_hs + ld_chunk * 8;
  u32x4 kst[LD_PASSES], vst[LD_PASSES];

  auto issue_loads = [&](int tile) {
    const int kb = kt_lo + tile * BN;
#pragma unroll
    for (int ps = 0; ps < LD_PASSES; ++ps) {
      int tk = im_min(kb + ld_row0 + ps * (NT / 16), nk - 1);
      int64_t pos = map.kpos(tk);
      kst[ps] = *reinterpret_cast<const u32x4*>(kbase + pos * p.k_rs);
      vst[ps] = *reinterpret_cast<const u32x4*>(vbase + pos * p.v_rs);
    }
  };
  auto store_lds = [&](int buf) {
#pragma unroll
    for (int ps = 0; ps < LD_PASSES; ++ps) {
      int r = ld_row0 + ps * (NT / 16);
      int off = r * 256 + ((ld_chunk ^ swz(r)) << 4);
      *reinterpret_cast<u32x4*>(smem + buf * BUF_BYTES + off) = kst[ps];
      *reinterpret_cast<u32x4*>(smem + buf * BUF_BYTES + TILE_BYTES + off) = vst[ps];
    }
  };

  // K operand (A of S^T = K Q^T): lane reads row l32 (+32 per block), chunk 2*ks + h32
  int kaddr[8];
#pragma unroll
  for (int ks = 0; ks < 8; ++ks) kaddr[ks] = l32 * 256 + (((2 * ks + h32) ^ swz(l32)) << 4);
  // V^T operand (A of O^T = V^T P^T) through transposing reads.  Within each group of 16 lanes,
  // lane i supplies the address of 4 head dims (4*(i%4)..) of key row i/4 and receives head dim i
  // of those 4 key rows.  vaddr[db][u]: d block db (32 dims), key sub-row group u (rows 8u+4*h32..).
  int vaddr[4][2];
  {
    const int i16 = lane & 15;
    const int g2 = (lane >> 4) & 1;
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int u = 0; u < 2; ++u) {
        int r = 8 * u + 4 * h32 + (i16 >> 2);
        int chunk = 4 * db + 2 * g2 + ((i16 & 3) >> 1);
        vaddr[db][u] = TILE_BYTES + r * 256 + ((chunk ^ swz(r)) << 4) + 8 * (i16 & 1);
      }
  }

  // ---------------------------------------------------------------- running softmax state
  floatx16 oacc[4];
#pragma unroll
  for (int db = 0; db < 4; ++db)
#pragma unroll
    for (int e = 0; e < 16; ++e) oacc[db][e] = 0.f;
  float m_run = -INFINITY;
  float l_run = 0.f;
  const float c = p.scale_log2;

  auto compute_tile = [&](int tile, int buf) {
    const int kb = kt_lo + tile * BN;
    int cls[2];
#pragma unroll
    for (int b = 0; b < 2; ++b) cls[b] = wave_active ? classify_block(wb, kb + 32 * b) : BLK_SKIP;
    if (cls[0] == BLK_SKIP && cls[1] == BLK_SKIP) return;
    const unsigned char* sb = smem + buf * BUF_BYTES;

    floatx16 s[2];
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      if (cls[b] != BLK_SKIP) {
#pragma unroll
        for (int e = 0; e < 16; ++e) s[b][e] = 0.f;
#pragma unroll
        for (int ks = 0; ks < 8; ++ks) {
          bf16x8 a = *reinterpret_cast<const bf16x8*>(sb + kaddr[ks] + b * 32 * 256);
          s[b] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, qf[ks], s[b], 0, 0, 0);
        }
        if (cls[b] == BLK_PARTIAL) {
#pragma unroll
          for (int e = 0; e < 16; ++e) {
            int key = kb + 32 * b + 8 * (e >> 2) + 4 * h32 + (e & 3);
            if (key < lo_l || key > hi_l) s[b][e] = -INFINITY;
          }
        }
      } else {
#pragma unroll
        for (int e = 0; e < 16; ++e) s[b][e] = -INFINITY;
      }
    }

    // online softmax; each lane owns one query
    float mx = s[0][0];
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int e = 0; e < 16; ++e) mx = fmaxf(mx, s[b][e]);
    mx = lane_xor32_max(mx);
    const float m_new = fmaxf(m_run, mx);
    const float m_use = m_new == -INFINITY ? 0.f : m_new;
    const float alpha = __builtin_amdgcn_exp2f((m_run - m_use) * c);
    m_run = m_new;
    const float mc = m_use * c;
    float rs = 0.f;
    bf16x8 pb[2][2];
#pragma unroll
    for (int b = 0; b < 2; ++b)
#pragma unroll
      for (int t = 0; t < 2; ++t)
#pragma unroll
        for (int e2 = 0; e2 < 4; ++e2) {
          float p0 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[b][8 * t + 2 * e2], c, -mc));
          float p1 = __builtin_amdgcn_exp2f(__builtin_fmaf(s[b][8 * t + 2 * e2 + 1], c, -mc));
          rs += p0 + p1;
          floatx2 f = {p0, p1};
          bf16x2 h = __builtin_convertvector(f, bf16x2);
          pb[b][t][2 * e2] = h[0];
          pb[b][t][2 * e2 + 1] = h[1];
        }
    l_run = l_run * alpha + rs;
#pragma unroll
    for (int db = 0; db < 4; ++db)
#pragma unroll
      for (int e = 0; e < 16; ++e) oacc[db][e] *= alpha;

    // O^T += V^T P^T
#pragma unroll
    for (int b = 0; b < 2; ++b) {
      if (cls[b] == BLK_SKIP) continue;
#pragma unroll
      for (int t = 0; t < 2; ++t) {
#pragma unroll
        for (int db = 0; db < 4; ++db) {
          const int roff = (32 * b + 16 * t) * 256;
          bf16x4 v0 = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
              (__attribute__((address_space(3))) bf16x4*)(sb + vaddr[db][0] + roff));
          bf16x4 v1 = __builtin_amdgcn_ds_read_tr16_b64_v4bf16(
              (__attribute__((address_space(3))) bf16x4*)(sb + vaddr[db][1] + roff));
          bf16x8 a = __builtin_shufflevector(v0, v1, 0, 1, 2, 3, 4, 5, 6, 7);
          oacc[db] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, pb[b][t], oacc[db], 0, 0, 0);
        }
      }
    }
  };

  // ---------------------------------------------------------------- main loop
  issue_loads(0);
  store_lds(0);
  for (int tile = 0; tile < ntiles; ++tile) {
    __syncthreads();
    const bool more = tile + 1 < ntiles;
    if (more) issue_loads(tile + 1);
    compute_tile(tile, tile & 1);
    if (more) store_lds((tile + 1) & 1);
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
