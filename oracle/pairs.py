"""Closed-form counts of unmasked (query, key) pairs per head; the algorithmic work of a call is
4 * 128 * pairs * heads * batch flops (QK^T and PV, 2*128 flops each per pair)."""


def pairs_per_head(kind, S, group_num=8, window=576, width=64, text_len=512, block=256, offset=0, n_sink=0):
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
    if kind == "llm/window_sink":
        # window part min(i + 1, window) keys, plus the sinks the window no longer reaches
        return sum(min(i + 1, window) + max(0, min(n_sink, i + 1 - window)) for i in range(S))
    if kind == "llm/block_scatter":
        G, total = group_num, 0
        for qb in range((S + block - 1) // block):
            n = min(block, S - qb * block)             # queries of this block
            tgt = (qb + offset) % G
            earlier = [kb for kb in range(qb) if kb % G == tgt]
            cls = len(earlier) * block * n             # whole earlier blocks of the target group
            own = n * (n + 1) // 2 if (offset or qb % G == tgt) else 0
            # sinks not already counted: block 0 is counted if it is an earlier target block or the own block
            sink = 0 if (0 in earlier or qb == 0) else min(n_sink, S) * n
            total += cls + own + sink
        return total
    grid = width * width
    assert S == text_len + grid
    if kind == "image/scatter":
        return S * (text_len + grid // 8)
    if kind == "image/gather0":
        return text_len * (text_len + grid // 8) + grid * (text_len + 256)
    raise KeyError(kind)
