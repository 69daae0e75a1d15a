"""CPU restatement of INTRA's dense-mask specification.  TEST INFRASTRUCTURE ONLY.

Nothing under intra_amd/ may import this package: it is the checker that tests/,
__graft_entry__.smoke() and bench.py's cpu_baseline leg compare the HIP kernels with, never a
code path of the product.

What it restates (reference file:line) and what pins each function (tests/test_oracle.py):

  masks.llm_scatter_mask     intra_attn/reference.py:14-17   brute-force loops; known answers
  masks.llm_gather1_mask     intra_attn/reference.py:20-24   brute-force loops
  masks.llm_window_mask      intra_attn/reference.py:27-32   known answers of reference.py:93-94;
                                                              per-block loop construction
  masks.image_scatter_mask   intra_attn/reference.py:36-53   invariants of reference.py:95-98;
                                                              loop construction; density 22.22 %
  masks.image_gather0_mask   intra_attn/reference.py:56-74   invariants / known answers of
                                                              reference.py:99-102; loop construction;
                                                              density 17.28 %
  masks.llm_block_scatter_mask   experiments/llm/llama_intra.py:98-110
                                                              equals llm_scatter_mask at block 1 and
                                                              llm_gather1_mask at block G (offset 0);
                                                              the reference's other construction of
                                                              the same pattern (gathered per-group
                                                              attention with appended sinks,
                                                              llama_intra.py:124-165) restated in the
                                                              test; offsets 0..G-1 partition the
                                                              earlier blocks; brute-force loops
  masks.llm_window_sink_mask     experiments/llm/llama_intra.py:62-72
                                                              tril at window >= S; closed-form row
                                                              counts; brute-force loops
  attention.masked_lse_rows  flash_api.cpp:470,670 (softmax_lse)  float64 loop; consistency with
                                                              masked_attention
  attention.masked_attention intra_attn/reference.py:78-83   float64 triple loop on tiny inputs;
                                                              torch SDPA (the library routine the
                                                              reference calls) incl. GQA
  attention.masked_attention_grads   experiments/llm/llama_intra.py:26 (autograd of masked SDPA)
                                                              central finite differences in float64;
                                                              hand-written softmax-Jacobian formulas in
                                                              loops; closed form for one-key rows
  pairs.*                    closed forms                     mask.sum() of the masks above

Every function has at least one such independent check, so no part is "parity unpinned".
The reference's Python file was read, not imported or run.
"""
from .attention import masked_attention, masked_attention_grads, masked_attention_rows, masked_lse_rows  # noqa: F401
from .masks import (TEXT_LEN, image_gather0_mask, image_scatter_mask, llm_block_scatter_mask,  # noqa: F401
                    llm_gather1_mask, llm_scatter_mask, llm_window_mask, llm_window_sink_mask, mask_rows)
from .pairs import pairs_per_head  # noqa: F401
