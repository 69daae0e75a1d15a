"""Closed-form counts of unmasked (query, key) pairs per head; the algorithmic work of a call is
4 * 128 * pairs * heads * batch flops (QK^T and PV, 2*128 flops each per pair)."""


def pairs_per_head(kind, S, group_num=8, window=576, width=64, text_len=512):
    if kind in ("llm/scatter", "llm/gather1"):
        G = group_num
        if kind == "llm/scatter":
            sizes = [(S - g + G - 1) // G if S > g else 0 for g in range(G)]
        else:
            full, rem = divmod(S, G * G)
            sizes = [full * G + max(0, min(G, rem - G * g)) for g in range(G)]
        return sum(n * (n + 1) // 2 for n in sizes)
    if kind == "llm/window":
        total = 0
        for b0 in range(0, S, 64):  # one 64-query block at a time
            start = max(b0 - (window - 64), 0)
            n = min(64, S - b0)
            total += n * (b0 - start) + n * (n + 1) // 2
        return total
    grid = width * width
    assert S == text_len + grid
    if kind == "image/scatter":
        return S * (text_len + grid // 8)
    if kind == "image/gather0":
        return text_len * (text_len + grid // 8) + grid * (text_len + 256)
    raise KeyError(kind)
