"""Dense boolean masks of every INTRA pattern; mask[q, k] == True means q may attend to k.

Restates intra_attn/reference.py:14-74.  Each builder takes an optional `rows` tensor of query
positions and then returns only those rows (len(rows), S), so long sequences can be checked on a
subset of queries without materialising S x S.
"""
import torch

TEXT_LEN = 512  # reference.py:10


def _qk(S, rows, device):
    k = torch.arange(S, device=device)
    q = k if rows is None else torch.as_tensor(rows, device=device, dtype=torch.long)
    return q[:, None], k[None, :]


def llm_scatter_mask(S, group_num=8, device=None, rows=None):
    """reference.py:14-17: causal attention among tokens with equal position % group_num."""
    q, k = _qk(S, rows, device)
    return (k <= q) & (q % group_num == k % group_num)


def llm_gather1_mask(S, group_num=8, device=None, rows=None):
    """reference.py:20-24: segments of G consecutive tokens, segment s in group s % G; causal."""
    q, k = _qk(S, rows, device)
    return (k <= q) & ((q // group_num) % group_num == (k // group_num) % group_num)


def llm_window_mask(S, window=576, block=64, device=None, rows=None):
    """reference.py:27-32: a query block of `block` tokens sees itself plus the window - block
    tokens before the block."""
    q, k = _qk(S, rows, device)
    start = ((q // block) * block - (window - block)).clamp(min=0)
    return (k <= q) & (k >= start)


def llm_block_scatter_mask(S, group_num=2, block=256, offset=0, n_sink=0, device=None, rows=None):
    """experiments/llm/llama_intra.py:98-110 (mask_mod of _scatter_block_mask): blocks of `block`
    tokens, block b in group b % G; a query block qb reads, causally, the key blocks of group
    (qb + offset) % G, with offset != 0 also its own block, and the first n_sink tokens."""
    q, k = _qk(S, rows, device)
    qb, kb = q // block, k // block
    vis = (kb % group_num) == ((qb + offset) % group_num)
    if offset:
        vis = vis | (kb == qb)
    if n_sink:
        vis = vis | (k < n_sink)
    return (k <= q) & vis


def llm_window_sink_mask(S, window=575, n_sink=0, device=None, rows=None):
    """experiments/llm/llama_intra.py:62-72 (mask_mod of _sliding_block_mask): causal, and the key
    is among the last `window` positions up to the query or among the first n_sink tokens."""
    q, k = _qk(S, rows, device)
    return (k <= q) & ((q - k < window) | (k < n_sink))


def _image_group(pos, width, text_len):
    """reference.py:36-46: text token t -> t // (text_len/8); grid token (r, c) -> (r%2)*4 + c%4."""
    p = (pos - text_len).clamp(min=0)
    r, c = p // width, p % width
    return torch.where(pos < text_len, pos // (text_len // 8), (r % 2) * 4 + c % 4)


def image_scatter_mask(width, text_len=TEXT_LEN, device=None, rows=None):
    """reference.py:49-53: every query sees all text keys plus the grid keys of its own group."""
    q, k = _qk(text_len + width * width, rows, device)
    return (k < text_len) | (_image_group(q, width, text_len) == _image_group(k, width, text_len))


def image_gather0_mask(width, text_len=TEXT_LEN, patch=8, window=16, device=None, rows=None):
    """reference.py:56-74: grid queries of an 8x8 patch see all text plus a 16x16 grid window
    centred on the patch, moved inwards at the borders; text queries keep their scatter rows."""
    q, k = _qk(text_len + width * width, rows, device)
    n_patch = width // patch

    def start(idx):
        s = idx * patch - (window - patch) // 2
        s = torch.where(idx == 0, torch.zeros_like(s), s)
        return torch.where(idx == n_patch - 1, idx * patch - (window - patch), s)

    pq, pk = (q - text_len).clamp(min=0), (k - text_len).clamp(min=0)
    rq, cq, rk, ck = pq // width, pq % width, pk // width, pk % width
    r0, c0 = start(rq // patch), start(cq // patch)
    inside = (rk >= r0) & (rk < r0 + window) & (ck >= c0) & (ck < c0 + window)
    grid_rows = (k < text_len) | inside
    return torch.where(q < text_len, image_scatter_mask(width, text_len, device, rows), grid_rows)


def mask_rows(kind, S, rows=None, device=None, **kw):
    """Dispatch by the API's names: kind in {"llm/scatter", "llm/gather1", "llm/window",
    "llm/block_scatter", "llm/window_sink", "image/scatter", "image/gather0"}."""
    if kind == "llm/scatter":
        return llm_scatter_mask(S, kw.get("group_num", 8), device, rows)
    if kind == "llm/gather1":
        return llm_gather1_mask(S, kw.get("group_num", 8), device, rows)
    if kind == "llm/window":
        return llm_window_mask(S, kw.get("window", 576), 64, device, rows)
    if kind == "llm/block_scatter":
        return llm_block_scatter_mask(S, kw.get("group_num", 2), kw.get("block", 256), kw.get("offset", 0),
                                      kw.get("n_sink", 0), device, rows)
    if kind == "llm/window_sink":
        return llm_window_sink_mask(S, kw.get("window", 575), kw.get("n_sink", 0), device, rows)
    width = kw.get("width", 64)
    text_len = kw.get("text_len", TEXT_LEN)
    assert S == text_len + width * width
    if kind == "image/scatter":
        return image_scatter_mask(width, text_len, device, rows)
    if kind == "image/gather0":
        return image_gather0_mask(width, text_len, device=device, rows=rows)
    raise KeyError(kind)
