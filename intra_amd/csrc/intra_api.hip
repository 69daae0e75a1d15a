// C ABI of libintra_hip.so: validation, launch planning and dispatch.  See include/intra_hip.h.
#include <hip/hip_runtime.h>
#include <math.h>
#include <stdarg.h>
#include <stdio.h>
#include <string.h>

#include "../../include/intra_hip.h"
#include "intra_kernel.hip.h"

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
                 Request* r) {
  if (B < 1 || S < 1 || H < 1 || Hkv < 1)
    return fail(INTRA_ERR_INVALID, "B, S, H, Hkv must be positive (got %d, %d, %d, %d)", B, S, H, Hkv);
  if (H % Hkv != 0)
    return fail(INTRA_ERR_INVALID, "query heads (%d) must be a multiple of kv heads (%d)", H, Hkv);
  r->B = B;
  r->S = S;
  r->H = H;
  r->Hkv = Hkv;
  r->geom = IntraGeom{S, 1, 64, 16, 8};
  if (domain == 0) {
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
    } else {
      return fail(INTRA_ERR_INVALID, "unknown LLM pattern id %d (0 scatter, 1 gather1, 4 window)", pattern);
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

// Workgroup shape: HP query heads of one kv head share a workgroup.  Gather0 sets are single
// 64-query blocks, so its workgroups shrink with HP; the other patterns always run 8 wavefronts.
void pick_shape(int kind, int ratio, int* hp, int* nw) {
  int h = ratio % 4 == 0 ? 4 : (ratio % 2 == 0 ? 2 : 1);
  *hp = h;
  *nw = kind == KIND_IMG_GATHER0 ? 2 * h : 8;
}

bool shape_ok(int kind, int hp, int nw) {
  if (hp != 1 && hp != 2 && hp != 4) return false;
  if (kind == KIND_IMG_GATHER0) return nw == 2 * hp;
  return nw == 8;
}

template <class MAP>
void fill_plan(const Request& r, int hp, int nw, IntraPlan* plan) {
  const int pos = nw * 32 / hp;
  plan->kind = r.kind;
  plan->heads_per_block = hp;
  plan->waves = nw;
  plan->pos_per_block = pos;
  plan->n_sets = MAP::num_sets(r.geom);
  plan->n_mblocks = (MAP::max_nq(r.geom) + pos - 1) / pos;
  const int hgroups = (r.H / r.Hkv) / hp;
  const int64_t n_pairs = (int64_t)r.B * r.Hkv * plan->n_sets;
  const int64_t items = 8 * ((n_pairs + 7) / 8) * hgroups * plan->n_mblocks;
  plan->work_items = items > 0x7fffffff ? -1 : (int)items;
  plan->grid = plan->work_items;  // upper bound; a launch uses min(work_items, 8 * (CUs / 8))
  plan->lds_bytes = intra::LDS_BYTES;
  int64_t pairs = 0;
  for (int set = 0; set < plan->n_sets; ++set) {
    MAP map(r.geom, set);
    const int nq = map.nq(), nk = map.nk();
    for (int tq = 0; tq < nq; ++tq) {
      int hi = im_min(map.khi(tq), nk - 1);
      int lo = map.klo(tq);
      if (hi >= lo) pairs += hi - lo + 1;
    }
  }
  plan->pairs_per_head = pairs;
}

void plan_for(const Request& r, int hp, int nw, IntraPlan* plan) {
  switch (r.kind) {
    case KIND_LLM_SCATTER: fill_plan<MapLlmScatter>(r, hp, nw, plan); break;
    case KIND_LLM_GATHER1: fill_plan<MapLlmGather1>(r, hp, nw, plan); break;
    case KIND_LLM_WINDOW: fill_plan<MapLlmWindow>(r, hp, nw, plan); break;
    case KIND_IMG_SCATTER: fill_plan<MapImgScatter>(r, hp, nw, plan); break;
    default: fill_plan<MapImgGather0>(r, hp, nw, plan); break;
  }
}

// Host walk of the kernel's decomposition: sets -> row blocks -> wavefronts -> key tiles ->
// 32-key blocks, with the same classification and per-element bound test as the device code.
template <class MAP>
void model_walk(const IntraGeom& ge, int hp, int nw, uint8_t* count) {
  const int pos = nw * 32 / hp;
  const int S = ge.S;
  const int n_sets = MAP::num_sets(ge);
  const int n_mblocks = (MAP::max_nq(ge) + pos - 1) / pos;
  for (int set = 0; set < n_sets; ++set) {
    MAP map(ge, set);
    const int nq = map.nq(), nk = map.nk();
    for (int mblk = 0; mblk < n_mblocks; ++mblk) {
      const int t0 = mblk * pos;
      if (t0 >= nq) continue;
      const int t1 = im_min(t0 + pos, nq) - 1;
      const int kt_lo = map.klo(t0);
      const int kt_hi = im_min(map.khi(t1), nk - 1);
      const int ntiles = (kt_hi - kt_lo + intra::BN) / intra::BN;
      for (int pw = 0; pw < pos / 32; ++pw) {  // the wavefronts of one head
        const int wq0 = t0 + pw * 32;
        if (wq0 > t1) continue;
        const int wq_last = im_min(wq0 + 31, t1);
        const WaveBounds wb = wave_bounds(map, wq0, wq_last);
        for (int tile = 0; tile < ntiles; ++tile) {
          for (int b = 0; b < 2; ++b) {
            const int sb_lo = kt_lo + tile * intra::BN + 32 * b;
            const int cls = classify_block(wb, sb_lo);
            if (cls == BLK_SKIP) continue;
            for (int l = 0; l < 32; ++l) {
              if (wq0 + l > t1) continue;  // rows the kernel computes but never stores
              const int tq = wq0 + l;
              const int lo = map.klo(tq), hi = im_min(map.khi(tq), nk - 1);
              for (int e = 0; e < 32; ++e) {
                const int key = sb_lo + e;
                if (cls == BLK_PARTIAL && (key < lo || key > hi)) continue;
                // a FULL block keeps every element: clamp the loaded row like the loader does
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
}

// One persistent workgroup per CU (LDS allows no more), in multiples of the 8 XCDs.
int launch_grid(int work_items) {
  static int cus[64] = {0};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return -1;
  if (cus[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0) return -1;
    cus[dev] = n;
  }
  int g = (cus[dev] / 8) * 8;
  if (g < 8) g = 8;
  return work_items < g ? work_items : g;
}

template <class MAP, int HP, int NW>
int launch(const intra::KParams& p, int grid, hipStream_t stream) {
  hipLaunchKernelGGL((intra::intra_fwd_kernel<MAP, HP, NW>), dim3(grid), dim3(NW * 64), 0, stream, p);
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(INTRA_ERR_HIP, "kernel launch failed: %s", hipGetErrorString(e));
  return INTRA_OK;
}

template <class MAP>
int launch_hp8(const intra::KParams& p, int hp, int grid, hipStream_t stream) {
  switch (hp) {
    case 4: return launch<MAP, 4, 8>(p, grid, stream);
    case 2: return launch<MAP, 2, 8>(p, grid, stream);
    default: return launch<MAP, 1, 8>(p, grid, stream);
  }
}

bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15) == 0; }

int check_strides(const char* name, const int64_t* st, int B, int S, int heads) {
  if (!st) return fail(INTRA_ERR_INVALID, "%s strides pointer is null", name);
  for (int i = 0; i < 3; ++i) {
    if (st[i] < 0) return fail(INTRA_ERR_INVALID, "%s stride %d is negative", name, i);
    if (st[i] % 8 != 0)
      return fail(INTRA_ERR_INVALID, "%s stride %d (%lld elements) breaks 16-byte alignment", name, i,
                  (long long)st[i]);
  }
  if ((S > 1 && st[1] == 0) || (heads > 1 && st[2] == 0) || (B > 1 && st[0] == 0 && name[0] == 'o'))
    return fail(INTRA_ERR_INVALID, "%s has a zero stride over a dimension larger than 1", name);
  return INTRA_OK;
}

int run(int domain, const void* q, const void* k, const void* v, void* o, int B, int S, int H,
        int Hkv, const int64_t* qs, const int64_t* ks, const int64_t* vs, const int64_t* os,
        int pattern, int arg0, int arg1, float scale, void* stream) {
  g_err[0] = 0;
  Request r;
  int rc = make_request(domain, pattern, B, S, H, Hkv, arg0, arg1, &r);
  if (rc) return rc;
  if (!q || !k || !v || !o) return fail(INTRA_ERR_INVALID, "q, k, v and o must be non-null device pointers");
  if (!aligned16(q) || !aligned16(k) || !aligned16(v) || !aligned16(o))
    return fail(INTRA_ERR_INVALID, "q, k, v and o must be 16-byte aligned");
  if ((rc = check_strides("q", qs, B, S, H))) return rc;
  if ((rc = check_strides("k", ks, B, S, Hkv))) return rc;
  if ((rc = check_strides("v", vs, B, S, Hkv))) return rc;
  if ((rc = check_strides("o", os, B, S, H))) return rc;
  if (!isfinite(scale)) return fail(INTRA_ERR_INVALID, "softmax_scale must be finite");

  int hp, nw;
  pick_shape(r.kind, H / Hkv, &hp, &nw);
  IntraPlan plan;
  plan_for(r, hp, nw, &plan);
  if (plan.work_items <= 0) return fail(INTRA_ERR_UNSUPPORTED, "problem needs more than 2^31 work items");
  const int grid = launch_grid(plan.work_items);
  if (grid <= 0) return fail(INTRA_ERR_HIP, "cannot query the current device: %s", hipGetErrorString(hipGetLastError()));

  intra::KParams p;
  p.q = static_cast<const uint16_t*>(q);
  p.k = static_cast<const uint16_t*>(k);
  p.v = static_cast<const uint16_t*>(v);
  p.o = static_cast<uint16_t*>(o);
  p.q_bs = qs[0]; p.q_rs = qs[1]; p.q_hs = qs[2];
  p.k_bs = ks[0]; p.k_rs = ks[1]; p.k_hs = ks[2];
  p.v_bs = vs[0]; p.v_rs = vs[1]; p.v_hs = vs[2];
  p.o_bs = os[0]; p.o_rs = os[1]; p.o_hs = os[2];
  p.B = B; p.H = H; p.Hkv = Hkv; p.ratio = H / Hkv;
  p.geom = r.geom;
  p.scale_log2 = fabsf(scale) * 1.4426950408889634f;
  if (p.scale_log2 < 1e-30f) p.scale_log2 = 1e-30f;  // scale 0: uniform weights without 0 * inf on masked scores
  p.negate_q = scale < 0.f;
  if (ks[1] >= ((int64_t)1 << 31) || vs[1] >= ((int64_t)1 << 31))
    return fail(INTRA_ERR_UNSUPPORTED, "k / v token stride must stay below 2^31 elements");
  p.k_rs_bytes = (uint32_t)(ks[1] * 2);
  p.v_rs_bytes = (uint32_t)(vs[1] * 2);
  p.n_sets = plan.n_sets;
  p.n_mblocks = plan.n_mblocks;
  p.hgroups = p.ratio / hp;
  p.n_pairs = B * Hkv * plan.n_sets;
  p.items_per_pair = p.hgroups * plan.n_mblocks;
  p.n_slots = plan.work_items / 8;

  hipStream_t st = static_cast<hipStream_t>(stream);
  switch (r.kind) {
    case KIND_LLM_SCATTER: return launch_hp8<MapLlmScatter>(p, hp, grid, st);
    case KIND_LLM_GATHER1: return launch_hp8<MapLlmGather1>(p, hp, grid, st);
    case KIND_LLM_WINDOW: return launch_hp8<MapLlmWindow>(p, hp, grid, st);
    case KIND_IMG_SCATTER: return launch_hp8<MapImgScatter>(p, hp, grid, st);
    default:
      switch (hp) {
        case 4: return launch<MapImgGather0, 4, 8>(p, grid, st);
        case 2: return launch<MapImgGather0, 2, 4>(p, grid, st);
        default: return launch<MapImgGather0, 1, 2>(p, grid, st);
      }
  }
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

const char* intra_last_error(void) { return g_err; }

int intra_version(void) { return 100; }

int intra_plan(int domain, int pattern, int B, int S, int H, int Hkv, int arg0, int arg1,
               IntraPlan* plan) {
  g_err[0] = 0;
  if (!plan) return fail(INTRA_ERR_INVALID, "plan pointer is null");
  Request r;
  int rc = make_request(domain, pattern, B, S, H, Hkv, arg0, arg1, &r);
  if (rc) return rc;
  int hp, nw;
  pick_shape(r.kind, H / Hkv, &hp, &nw);
  plan_for(r, hp, nw, plan);
  return INTRA_OK;
}

int intra_model_mask(int domain, int pattern, int S, int arg0, int arg1, int heads_per_block,
                     int waves, uint8_t* count) {
  g_err[0] = 0;
  if (!count) return fail(INTRA_ERR_INVALID, "count pointer is null");
  Request r;
  int rc = make_request(domain, pattern, 1, S, 1, 1, arg0, arg1, &r);
  if (rc) return rc;
  int hp, nw;
  pick_shape(r.kind, 1, &hp, &nw);
  if (heads_per_block > 0) hp = heads_per_block;
  if (waves > 0) nw = waves;
  if (!shape_ok(r.kind, hp, nw))
    return fail(INTRA_ERR_INVALID, "no kernel for heads_per_block=%d, waves=%d", hp, nw);
  switch (r.kind) {
    case KIND_LLM_SCATTER: model_walk<MapLlmScatter>(r.geom, hp, nw, count); break;
    case KIND_LLM_GATHER1: model_walk<MapLlmGather1>(r.geom, hp, nw, count); break;
    case KIND_LLM_WINDOW: model_walk<MapLlmWindow>(r.geom, hp, nw, count); break;
    case KIND_IMG_SCATTER: model_walk<MapImgScatter>(r.geom, hp, nw, count); break;
    default: model_walk<MapImgGather0>(r.geom, hp, nw, count); break;
  }
  return INTRA_OK;
}

}  // extern "C"
