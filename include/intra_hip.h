/* C ABI of libintra_hip.so: MI355X (gfx950) forward sparse-attention kernels of INTRA.
 *
 * This header is the drop-in boundary.  It replaces the pybind11 module `intra_attn_cuda` of the
 * reference (csrc/flash_attn/flash_api.cpp:1766-1770, functions `fwd_llm` and `fwd`).  All tensor
 * arguments are raw device pointers to bf16 data laid out (batch, token, head, 128) with the
 * last dimension contiguous; strides are passed in ELEMENTS as {batch, token, head}.  Every
 * pointer and every stride must keep 16-byte alignment (pointer % 16 == 0, stride % 8 == 0).
 * The library allocates nothing; the caller owns `o`.  Launches are asynchronous on `hip_stream`
 * (a hipStream_t, NULL = default stream).  State the library keeps between calls: the process
 * default of the softmax arithmetic (intra_set_softmax_mode; a call can name its own in the flags
 * of the *_ex entry points), the 16 MiB per-GPU array behind intra_llm_bwd_noalloc, the timer buffer
 * of measurement builds (intra_diag_set_buffer), and per-device caches of the CU count.
 * Environment variables read by the library, both for experiments only: INTRA_SOFTMAX (the
 * starting value of that default) and INTRA_WAVES (8 or 4: the workgroup size of the forward
 * launches, where the named shape exists; otherwise the library picks - workgroups of 4 wavefronts,
 * two per CU, for image gather0 and for launches with few row blocks, 8 wavefronts for the rest).
 *
 * Every function returns INTRA_OK or an error code; intra_last_error() then describes the failure
 * (thread-local string).  Argument validation happens before any HIP call, so it can be exercised
 * on a machine without a GPU.
 */
#ifndef INTRA_HIP_H
#define INTRA_HIP_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

enum {
  INTRA_OK = 0,
  INTRA_ERR_INVALID = 1,     /* bad argument (null pointer, shape, stride, pattern id ...) */
  INTRA_ERR_UNSUPPORTED = 2, /* valid request this build has no kernel for */
  INTRA_ERR_HIP = 3          /* HIP runtime / launch failure */
};

/* Pattern ids, identical to the reference's `mask` argument
 * (intra_attn/interface.py:12-13: LLM_PATTERNS, IMAGE_PATTERNS). */
enum { INTRA_LLM_SCATTER = 0, INTRA_LLM_GATHER1 = 1, INTRA_LLM_WINDOW = 4 };
/* Patterns of the reference's model-level experiments that its kernels do not cover (see
 * intra_llm_fwd_ex); ids chosen here. */
enum { INTRA_LLM_BLOCK_SCATTER = 8, INTRA_LLM_WINDOW_SINK = 9 };
enum { INTRA_IMAGE_SCATTER = 0, INTRA_IMAGE_GATHER0 = 4 };

/* Causal language-model attention.  Replaces `fwd_llm` / mha_fwd_llm
 * (csrc/flash_attn/flash_api.cpp:556-763) as called by intra_llm_attn
 * (intra_attn/interface.py:30-45).
 *   q, o: (B, S, H, 128); k, v: (B, S, Hkv, 128); H % Hkv == 0; query head h reads kv head
 *   h / (H / Hkv).
 *   pattern INTRA_LLM_SCATTER: group_num >= 1, any S.
 *   pattern INTRA_LLM_GATHER1: group_num >= 1, any S (the reference is limited to 8 / S % 64 == 0).
 *   pattern INTRA_LLM_WINDOW : window >= 64, any S; group_num ignored.
 *   softmax_scale: any finite float. */
int intra_llm_fwd(const void* q, const void* k, const void* v, void* o, int B, int S, int H,
                  int Hkv, const int64_t q_strides[3], const int64_t k_strides[3],
                  const int64_t v_strides[3], const int64_t o_strides[3], int pattern,
                  int group_num, int window, float softmax_scale, void* hip_stream);

/* Bidirectional attention over `text_len` text tokens followed by a width x width token grid.
 * Replaces `fwd` / mha_fwd (csrc/flash_attn/flash_api.cpp:355-552) as called by intra_image_attn
 * (intra_attn/interface.py:48-66).  S must equal text_len + width*width; width % 8 == 0,
 * width >= 16, text_len % 8 == 0, text_len >= 8 (the reference fixes text_len = 512 and
 * width in {64, 128}). */
int intra_image_fwd(const void* q, const void* k, const void* v, void* o, int B, int S, int H,
                    int Hkv, const int64_t q_strides[3], const int64_t k_strides[3],
                    const int64_t v_strides[3], const int64_t o_strides[3], int pattern,
                    int width, int text_len, float softmax_scale, void* hip_stream);

/* The same two operations with the softmax log-sum-exp as a second output: for query token t of
 * head h, lse[b*lse_strides[0] + h*lse_strides[1] + t*lse_strides[2]] = ln sum_j exp(softmax_scale
 * * q_t . k_j) over the keys j the pattern shows to t (fp32; strides in elements: batch, head,
 * token).  This is the `softmax_lse` tensor that mha_fwd / mha_fwd_llm allocate and fill
 * (csrc/flash_attn/flash_api.cpp:470,670) and that the reference's Python layer discards
 * (intra_attn/interface.py:44,65); here it is indexed by token position, not by in-group row.
 * It is what a backward pass or a merge of partial results over key shards needs.  Accuracy: the
 * sum runs over the bf16-rounded weights that multiply V, so lse is within ln(1 + 2^-8) = 3.9e-3
 * of the exact value. */
int intra_llm_fwd_lse(const void* q, const void* k, const void* v, void* o, int B, int S, int H,
                      int Hkv, const int64_t q_strides[3], const int64_t k_strides[3],
                      const int64_t v_strides[3], const int64_t o_strides[3], int pattern,
                      int group_num, int window, float softmax_scale, void* hip_stream, float* lse,
                      const int64_t lse_strides[3]);
int intra_image_fwd_lse(const void* q, const void* k, const void* v, void* o, int B, int S, int H,
                        int Hkv, const int64_t q_strides[3], const int64_t k_strides[3],
                        const int64_t v_strides[3], const int64_t o_strides[3], int pattern,
                        int width, int text_len, float softmax_scale, void* hip_stream, float* lse,
                        const int64_t lse_strides[3]);

/* intra_llm_fwd with the two further causal patterns that the reference's LLaMA / Qwen integration
 * runs through FlexAttention or gathered SDPA because its kernels lack them
 * (experiments/llm/llama_intra.py:57-72, 93-110), and an optional log-sum-exp output (lse may be
 * NULL).  Patterns 0, 1, 4 behave as in intra_llm_fwd and ignore block, offset, n_sink.
 *   INTRA_LLM_BLOCK_SCATTER: tokens form blocks of `block` (a multiple of 64); query i in block qb
 *     sees key j <= i in block kb iff kb % group_num == (qb + offset) % group_num, or j < n_sink,
 *     or (offset != 0 and kb == qb).  0 <= offset < group_num, 0 <= n_sink <= block.  With
 *     offset != 0, block must be a multiple of 128 when H / Hkv is odd (any multiple of 64 otherwise).
 *   INTRA_LLM_WINDOW_SINK: query i sees key j <= i iff i - j < window or j < n_sink
 *     (window >= 1, n_sink >= 0; group_num ignored).
 *   flags: INTRA_SOFTMAX_* (below) for this call; other bits must be 0. */
int intra_llm_fwd_ex(const void* q, const void* k, const void* v, void* o, int B, int S, int H,
                     int Hkv, const int64_t q_strides[3], const int64_t k_strides[3],
                     const int64_t v_strides[3], const int64_t o_strides[3], int pattern,
                     int group_num, int window, int block, int offset, int n_sink,
                     float softmax_scale, void* hip_stream, float* lse, const int64_t lse_strides[3],
                     unsigned flags);
/* intra_image_fwd with an optional log-sum-exp output (lse may be NULL) and per-call flags. */
int intra_image_fwd_ex(const void* q, const void* k, const void* v, void* o, int B, int S, int H,
                       int Hkv, const int64_t q_strides[3], const int64_t k_strides[3],
                       const int64_t v_strides[3], const int64_t o_strides[3], int pattern,
                       int width, int text_len, float softmax_scale, void* hip_stream, float* lse,
                       const int64_t lse_strides[3], unsigned flags);

/* Description of the last failure on the calling thread ("" if none).  Replaces the
 * TORCH_CHECK messages of flash_api.cpp. */
const char* intra_last_error(void);

/* Library version, major*10000 + minor*100 + patch (0.3.0). */
#define INTRA_VERSION 300
int intra_version(void);

/* Softmax arithmetic of the forward entry points.  The reference scales the fp32 scores after the
 * first product and subtracts a running maximum (csrc/flash_attn/src/softmax.h:65-91).
 *   INTRA_SOFTMAX_EXACT:  that arithmetic (the running reference only moves when a block maximum
 *       leaves +-60 powers of two, which changes no result).
 *   INTRA_SOFTMAX_SCALED: the same fp32 scaling, weights exp2(score * scale * log2 e) with no
 *       running maximum; queries whose weight sum leaves 2^-100 .. 2^60 are recomputed in EXACT
 *       arithmetic inside the same launch, so results stay finite and correct for any input.  Equal
 *       to EXACT up to the rounding of the weights; accuracy does not depend on the size of q, k.
 *   INTRA_SOFTMAX_FOLDED: multiplies softmax_scale * log2(e) into the bf16 query rows instead (one
 *       multiply per score less; about 2 % faster), then as SCALED.  Rounding the scaled query to
 *       bf16 perturbs a score by about 1.1e-3 * scale * sqrt(sum_d q_d^2 k_d^2) rms, i.e. in
 *       proportion to the magnitudes of q and k: as accurate as the other two for unit-variance
 *       inputs, outside the 1.6e-2 output bound once q and k are about twice as large.  Opt-in.
 *   INTRA_SOFTMAX_AUTO (0): the process default, which starts as "SCALED iff |softmax_scale| <=
 *       INTRA_SCALED_SOFTMAX_MAX_SCALE (four times 128^-1/2), else EXACT".
 * A call names its arithmetic in the `flags` of intra_llm_fwd_ex / intra_image_fwd_ex; the entry
 * points without flags use the process default.  intra_set_softmax_mode changes that default for
 * the whole process (it starts from the environment variable INTRA_SOFTMAX: auto / exact / folded
 * / scaled); it is meant for experiments - callers that need a fixed arithmetic pass it per call.
 * No counterpart in the reference. */
enum {
  INTRA_SOFTMAX_AUTO = 0, INTRA_SOFTMAX_EXACT = 1, INTRA_SOFTMAX_FOLDED = 2, INTRA_SOFTMAX_SCALED = 3,
  INTRA_SOFTMAX_MASK = 3
};
#define INTRA_SCALED_SOFTMAX_MAX_SCALE 0.35355339f
int intra_set_softmax_mode(int mode);
int intra_get_softmax_mode(void);

/* Backward pass of intra_llm_fwd / intra_llm_fwd_ex: gradients of the inputs given the gradient
 * `dout` of the output.  The reference ships no backward kernels (README.md lists them as missing;
 * its training experiments differentiate masked SDPA / FlexAttention instead,
 * experiments/llm/llama_intra.py:26); this entry point has no counterpart there and is what an
 * autograd wrapper of intra_llm_attn needs.
 *   o, lse:    output and log-sum-exp of the forward call with the same arguments
 *   dout:      gradient of o, bf16, shaped like q
 *   dq/dk/dv:  results, bf16, shaped like q / k / v (every element is written)
 *   workspace: intra_llm_bwd_workspace(...) floats of device memory owned by the caller, 16-byte
 *              aligned (rowsum(dout * o), and the partial sums of the sink keys); contents on
 *              entry do not matter
 * Patterns: all five of intra_llm_fwd_ex; INTRA_LLM_BLOCK_SCATTER with offset != 0 needs
 * block % 256 == 0, softmax_scale must not be 0; otherwise INTRA_ERR_UNSUPPORTED.  Launches on
 * hip_stream: dq, dk, dv, and with sinks four more for the sink rows of dk and dv; nothing is
 * allocated.  Accuracy: weights are rounded to bf16 before the second product, as in the forward
 * pass, accumulation is fp32. */
int intra_llm_bwd(const void* q, const void* k, const void* v, const void* o, const float* lse,
                  const void* dout, void* dq, void* dk, void* dv, float* workspace, int B, int S,
                  int H, int Hkv, const int64_t q_strides[3], const int64_t k_strides[3],
                  const int64_t v_strides[3], const int64_t o_strides[3],
                  const int64_t dout_strides[3], const int64_t dq_strides[3],
                  const int64_t dk_strides[3], const int64_t dv_strides[3],
                  const int64_t lse_strides[3], int pattern, int group_num, int window, int block,
                  int offset, int n_sink, float softmax_scale, void* hip_stream);
/* Floats of workspace that intra_llm_bwd needs for such a call (twice B*H*S rounded up to 4, plus with
 * sinks chunks * B * Hkv * min(n_sink, S) * 128, the queries being cut into chunks so that the
 * sink pass has about one workgroup per CU; the size is the same on every device - it allows for
 * 320 CUs, and a launch never splits finer than that); -1 if the request is invalid or unsupported
 * (intra_last_error() says why).  No counterpart in the reference. */
int64_t intra_llm_bwd_workspace(int B, int S, int H, int Hkv, int pattern, int group_num,
                                int window, int block, int offset, int n_sink);

/* intra_llm_bwd for callers that cannot allocate device memory and have no workspace to hand
 * over: code under HIP graph capture, tight serving or training loops, harnesses that forbid
 * hipMalloc.  No counterpart in the reference.  Same arguments and results as intra_llm_bwd
 * without `workspace`: the kernels use an array of INTRA_NOALLOC_SCRATCH_FLOATS floats (16 MiB)
 * that is part of the library's device image, one copy per GPU, held until the process ends.
 * Calls whose intra_llm_bwd_workspace(...) exceeds that size return INTRA_ERR_UNSUPPORTED.  The
 * entry point calls no hipMalloc / hipFree and no allocating library routine.  All calls on one
 * GPU share that GPU's array: calls that overlap in time on one GPU (different streams or
 * threads) race; calls on one stream, or otherwise ordered, are fine.  Nothing in the array has
 * to survive between calls or start at zero: every value a launch reads was written by an earlier
 * launch of the same call. */
#define INTRA_NOALLOC_SCRATCH_FLOATS (4 * 1024 * 1024)
int intra_llm_bwd_noalloc(const void* q, const void* k, const void* v, const void* o,
                          const float* lse, const void* dout, void* dq, void* dk, void* dv, int B,
                          int S, int H, int Hkv, const int64_t q_strides[3],
                          const int64_t k_strides[3], const int64_t v_strides[3],
                          const int64_t o_strides[3], const int64_t dout_strides[3],
                          const int64_t dq_strides[3], const int64_t dk_strides[3],
                          const int64_t dv_strides[3], const int64_t lse_strides[3], int pattern,
                          int group_num, int window, int block, int offset, int n_sink,
                          float softmax_scale, void* hip_stream);

/* The same for intra_image_fwd: dq, dk, dv of image Scatter and Gather 0 (arguments as in
 * intra_llm_bwd; pattern, width, text_len as in intra_image_fwd).  dq in one launch; the grid keys'
 * dk / dv against the queries that see them (Scatter: their group's; Gather 0: the query patches
 * around them, then their group's text queries added to the rows already written, both rounded to
 * bf16); the text keys' dk / dv against all queries in chunks, as the sink keys of intra_llm_bwd.
 * No counterpart in the reference (its FLUX training differentiates masked SDPA,
 * experiments/flux/intra_processor.py:138-142). */
int intra_image_bwd(const void* q, const void* k, const void* v, const void* o, const float* lse,
                    const void* dout, void* dq, void* dk, void* dv, float* workspace, int B, int S,
                    int H, int Hkv, const int64_t q_strides[3], const int64_t k_strides[3],
                    const int64_t v_strides[3], const int64_t o_strides[3],
                    const int64_t dout_strides[3], const int64_t dq_strides[3],
                    const int64_t dk_strides[3], const int64_t dv_strides[3],
                    const int64_t lse_strides[3], int pattern, int width, int text_len,
                    float softmax_scale, void* hip_stream);
int64_t intra_image_bwd_workspace(int B, int S, int H, int Hkv, int pattern, int width,
                                  int text_len);

/* ------------------------------------------------------------------ host-only helpers (no GPU)
 * How a call would be launched; mirrors the grid / per-set length derivation of the reference
 * launchers (csrc/flash_attn/src/flash_fwd_launch_template.h:401-565, flash_api.cpp:408-411,
 * 611-612, 703-714). */
typedef struct IntraPlan {
  int kind;            /* internal pattern kind 0..6 */
  int heads_per_block; /* query heads of one kv head packed into a workgroup (main launch) */
  int waves;           /* wavefronts per workgroup (main launch) */
  int pos_per_block;   /* in-set queries per workgroup (main launch) */
  int n_sets;          /* sets per (batch, kv head) (main launch) */
  int n_mblocks;       /* row blocks of the largest set (main launch) */
  int work_items;      /* row blocks to process, all launches (a multiple of 8: padded per XCD) */
  int grid;            /* upper bound of workgroups launched; a launch uses min(work_items, what the
                          device holds at once: one workgroup of 8 wavefronts, or two of 4, per CU) */
  int lds_bytes;       /* LDS per workgroup */
  int launches;        /* kernel launches per forward call: 1 for every pattern */
  int64_t pairs_per_head; /* unmasked (query, key) pairs per query head and batch */
} IntraPlan;

/* domain 0 = LLM (arg0 = group_num, arg1 = window), 1 = image (arg0 = width, arg1 = text_len). */
int intra_plan(int domain, int pattern, int B, int S, int H, int Hkv, int arg0, int arg1,
               IntraPlan* plan);

/* Walks the exact set / row-block / wavefront / 32-key-block decomposition the kernel uses
 * (same index maps and block classification, compiled for the host) and adds 1 to
 * count[q_pos * S + k_pos] for every score the kernel would compute and keep.  `count` is an
 * S*S byte array the caller zeroed.  heads_per_block <= 0 means 1; waves: 8 (or <= 0), or 4 where that
 * shape exists (half-size workgroups). */
int intra_model_mask(int domain, int pattern, int S, int arg0, int arg1, int heads_per_block,
                     int waves, uint8_t* count);

/* Enumerates how the forward launch of a request deals its work items (row blocks) to a grid of
 * `grid` workgroups of `waves` wavefronts (8, or 4 where that shape exists; grid a multiple of 8 up
 * to plan.work_items), with the kernels' own code compiled for the host: visits[item] += 1 for every
 * item a workgroup is dealt, item = ((pair * n_mblocks + row block) * head groups + head group),
 * pair = (set * B + batch) * Hkv + kv head.  `visits` holds n_visits >= plan.work_items bytes the
 * caller zeroed.  Every row block that exists must come out as 1, whatever the grid.  (No
 * counterpart in the reference: it launches one thread block per row block.) */
int intra_model_deal(int domain, int pattern, int B, int S, int H, int Hkv, int arg0, int arg1,
                     int waves, int grid, uint8_t* visits, int64_t n_visits);

/* intra_plan / intra_model_mask for the arguments of intra_llm_fwd_ex (the walk: row blocks of 8
 * wavefronts). */
int intra_plan_llm_ex(int pattern, int B, int S, int H, int Hkv, int group_num, int window,
                      int block, int offset, int n_sink, IntraPlan* plan);
int intra_model_mask_llm_ex(int pattern, int S, int group_num, int window, int block, int offset,
                            int n_sink, int heads_per_block, uint8_t* count);
/* The same for the dk / dv launches of intra_llm_bwd: count[q * S + k] += 1 for every (query, key)
 * pair that the key-row decomposition (inverse index maps, sink pass) multiplies; must equal the
 * dense mask. */
int intra_model_mask_llm_bwd(int pattern, int S, int group_num, int window, int block, int offset,
                             int n_sink, uint8_t* count);
int intra_model_mask_image_bwd(int pattern, int S, int width, int text_len, uint8_t* count);

/* ------------------------------------------------------------------ measurement aids
 * None of these has a counterpart in the reference; they exist so that the numbers quoted for the
 * kernels can be reproduced from this library.
 *
 * intra_diag_set_buffer: libraries built with -DINTRA_DIAG_TIMERS (python -m intra_amd.build --diag
 * makes intra_amd/libintra_hip_diag.so) time the phases of a work item inside the forward kernel.
 * `counters` is device memory for 16 int64 values per workgroup of the largest launch to come,
 * zeroed by the caller; every forward launch whose grid fits ADDS per workgroup: 100 MHz wall-clock
 * ticks of [0] item set-up, [1] the first barrier, [2] the first key block, [3] the tile loop,
 * [4] look-up of the next item, its Q request, normalisation and stores; [5] work items, [6] key
 * tiles, [7] shader cycles of the tile loops; [8]..[15] shader cycles at the barriers in front of
 * the Q slots, of the first key block, of tile 0 and between tiles, each as a pair {waiting for the
 * wavefront's own requests and LDS reads, waiting for the other wavefronts}.  Launches of workgroups
 * of 4 wavefronts have no barriers at the item boundary: [1] stays 0, and [8]..[11] are WRITTEN with
 * the hardware id of wavefronts 0..3 (HW_ID register in the low half, XCC_ID above it), from which a
 * reader sees which workgroups share a CU.  NULL switches it off.  A production build returns
 * INTRA_ERR_UNSUPPORTED and never touches such a buffer.
 *
 * intra_diag_mfma_ceiling: one launch of `workgroups` x 8 wavefronts that issue nothing but bf16
 * MFMAs on independent accumulators: `shape` 16 = v_mfma_f32_16x16x32_bf16 (the kernels'
 * instruction, 32 per iteration and wavefront), 32 = v_mfma_f32_32x32x16_bf16 (the alternative
 * shape, 16 per iteration), on
 * operands read once from `table` (131072 bytes the caller fills: constant or random bf16 bits).
 * `sink` takes workgroups * 512 floats, `clocks` per workgroup {shader cycles, 100 MHz ticks} of
 * the loop.  Work per launch: workgroups * 8 * iters * 16 * 32768 flop.  Allocates nothing.
 *
 * intra_diag_ablation: 0 for every library whose results are meant to be used.  Measurement builds can
 * be compiled with -DINTRA_ABLATE=<n> (python -m intra_amd.build --ablate <n>), which removes or doubles
 * one ingredient of the forward kernel's inner step (1: V^T operand reads, 2: K operand re-reads, 3: the
 * barrier between tiles, 4: exponentials, packing and row sums; 5: those issued twice; 6: the loader's
 * rows: the same 64 for every tile, so no address arithmetic and only L2 hits) so that its cost shows
 * in the phase timers; such a library computes wrong results on purpose and reports <n> here. */
int intra_diag_set_buffer(long long* counters, int64_t n_values);
int intra_diag_ablation(void);
int intra_diag_mfma_ceiling(const void* table, float* sink, long long* clocks, int workgroups,
                            int iters, int shape, void* hip_stream);

#ifdef __cplusplus
}
#endif
#endif /* INTRA_HIP_H */
