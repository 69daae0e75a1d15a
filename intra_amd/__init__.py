"""MI355X-native INTRA sparse attention (forward kernels of the reference, plus a backward pass).  Mirrors intra_attn/__init__.py:1-9 of the
reference: if the native library is missing, both entry points raise ImportError when called."""
try:
    from .interface import (get_softmax_mode, intra_image_attn, intra_image_attn_bwd, intra_image_attn_func,
                            intra_llm_attn, intra_llm_attn_bwd, intra_llm_attn_func, set_softmax_mode)
except ImportError as _err:
    def _missing(*args, _err=_err, **kwargs):
        raise ImportError(f"libintra_hip.so is not built ({_err}); run `python -m intra_amd.build`")

    intra_image_attn = intra_image_attn_bwd = intra_image_attn_func = _missing
    intra_llm_attn = intra_llm_attn_bwd = intra_llm_attn_func = _missing
    get_softmax_mode = set_softmax_mode = _missing

__version__ = "0.3.0"  # intra_version() of the library: 300
