"""Drop-in name: `from intra_attn import intra_llm_attn, intra_image_attn` keeps working for code
written against the reference package; the implementation lives in intra_amd."""
from intra_amd import (__version__, intra_image_attn, intra_image_attn_bwd, intra_image_attn_func,  # noqa: F401
                       intra_llm_attn, intra_llm_attn_bwd, intra_llm_attn_func)
