"""Alias of intra_amd.interface under the reference's module path."""
from intra_amd.interface import *  # noqa: F401,F403
from intra_amd.interface import IMAGE_PATTERNS, LLM_PATTERNS, TEXT_LEN  # noqa: F401
