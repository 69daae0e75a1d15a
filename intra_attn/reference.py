"""Dense boolean masks of the INTRA patterns and masked fp32 attention, under the names and
signatures of the reference's intra_attn/reference.py:10-83, so that its callers import them
unchanged: the parity test (tests/test_kernel.py:9-11), the benchmark
(benchmarks/bench_kernel.py:19-20) and the FLUX processor, which builds its masked-SDPA fallback
from the two image masks (experiments/flux/intra_processor.py:23,38-47).

`mask[i, j]` is True where query token i may attend to key token j.  Every builder returns the full
S x S matrix, so these are for checking and for short sequences.  The kernels never use them.
"""
import torch

TEXT_LEN = 512  # text tokens in front of the latent grid of a FLUX sequence


def _pairs(n, device):
    """Query index as a column, key index as a row: broadcasting them spans all (i, j)."""
    idx = torch.arange(n, device=device)
    return idx.unsqueeze(1), idx.unsqueeze(0)


# --------------------------------------------------------------------------- causal, language
def llm_scatter_mask(S, group_num=8, device=None):
    """Tokens are dealt round-robin into group_num groups; attention is causal inside a group."""
    i, j = _pairs(S, device)
    return ((i - j) % group_num == 0) & (j <= i)


def llm_gather1_mask(S, group_num=8, device=None):
    """Runs of group_num consecutive tokens are dealt round-robin into group_num groups; causal
    inside a group."""
    i, j = _pairs(S, device)
    run_i = torch.div(i, group_num, rounding_mode="floor")
    run_j = torch.div(j, group_num, rounding_mode="floor")
    return ((run_i - run_j) % group_num == 0) & (j <= i)


def llm_window_mask(S, window=576, block=64, device=None):
    """Queries come in blocks of `block`; a block sees itself and the window - block tokens before
    its first query (so a query looks back between window - block and window - 1 tokens)."""
    i, j = _pairs(S, device)
    first_of_block = i - i % block
    return (j <= i) & (j >= first_of_block - (window - block))


# ------------------------------------------------------------------------ bidirectional, image
def _image_group(width, text_len, device):
    """Group 0..7 of every token: the text is cut into eight equal chunks, chunk n in group n;
    grid token (row, col) is in group 4 * (row % 2) + col % 4."""
    text = torch.arange(text_len, device=device) * 8 // text_len
    cell = torch.arange(width * width, device=device)
    row, col = torch.div(cell, width, rounding_mode="floor"), cell % width
    return torch.cat((text, 4 * (row % 2) + col % 4))


def image_scatter_mask(width, text_len=TEXT_LEN, device=None):
    """Every query sees the whole text and the grid tokens of its own group."""
    group = _image_group(width, text_len, device)
    key_is_text = torch.arange(text_len + width * width, device=device) < text_len
    same_group = group.unsqueeze(1) == group.unsqueeze(0)
    return key_is_text.unsqueeze(0) | same_group


def image_gather0_mask(width, text_len=TEXT_LEN, patch=8, window=16, device=None):
    """A grid query sees the whole text and a window x window square of grid keys around its
    patch x patch tile, pushed inwards where it would cross the border of the grid.  Text queries
    see what image_scatter_mask shows them."""
    mask = image_scatter_mask(width, text_len, device)
    cell = torch.arange(width * width, device=device)
    row, col = torch.div(cell, width, rounding_mode="floor"), cell % width
    margin = (window - patch) // 2

    def origin(coord):  # first grid line of the window of the tile that holds `coord`
        tile_start = coord - coord % patch
        return (tile_start - margin).clamp(0, width - window)

    top, left = origin(row), origin(col)
    dr = row.unsqueeze(0) - top.unsqueeze(1)
    dc = col.unsqueeze(0) - left.unsqueeze(1)
    mask[text_len:, text_len:] = (dr >= 0) & (dr < window) & (dc >= 0) & (dc < window)
    return mask


# ------------------------------------------------------------------------------- specification
def masked_attention(q, k, v, mask, softmax_scale=None):
    """softmax(scale * q k^T) v over the keys `mask` allows, computed in fp32 and returned in
    q's dtype.  q: (B, S, H, D); k, v: (B, S, Hkv, D) with H a multiple of Hkv (query head h reads
    kv head h // (H / Hkv)); mask: (S, S) bool."""
    heads_first = [t.float().permute(0, 2, 1, 3) for t in (q, k, v)]
    grouped = heads_first[0].shape[1] != heads_first[1].shape[1]
    out = torch.nn.functional.scaled_dot_product_attention(*heads_first, attn_mask=mask, scale=softmax_scale,
                                                           enable_gqa=grouped)
    return out.permute(0, 2, 1, 3).to(q.dtype)
