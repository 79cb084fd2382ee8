"""CPU restatement of the reference's slice planner (latency_model.py:97-152) in plain Python loops.
TEST INFRASTRUCTURE ONLY (see oracle/__init__.py).  Pinned in tests/test_planner.py by exhaustive enumeration
of every batch grouping and every slicing on tiny grids."""
import itertools
import math


def planning(latency_grid, total_batch_size, total_nslices, pipelinelen, max_latency):
    """Returns (final_time, [(batch_size, [slice steps, last slice first]), ...]) or (inf, None); same loops
    and tie-breaking (strict '<' in increasing order) as latency_model.py:101-150."""
    B, N = total_batch_size, total_nslices
    inf = math.inf
    f = [[0.0] * (N + 1) for _ in range(B + 1)]
    f_step = [[0] * (N + 1) for _ in range(B + 1)]
    f_max = [[0.0] * (N + 1) for _ in range(B + 1)]
    for bs in range(1, B + 1):                                               # :105-116
        for acc in range(1, N + 1):
            f[bs][acc] = inf
            for step in range(1, acc + 1):
                lat = latency_grid[bs][step][acc - step]
                tot = f[bs][acc - step] + lat
                if lat <= max_latency and tot < f[bs][acc]:
                    f[bs][acc] = tot
                    f_step[bs][acc] = step
                    f_max[bs][acc] = max(f_max[bs][acc - step], lat)
    g, g_step, g_max = [0.0] * (B + 1), [0] * (B + 1), [0.0] * (B + 1)
    for acc in range(1, B + 1):                                              # :125-133
        g[acc] = inf
        for bs in range(1, acc + 1):
            tot = g[acc - bs] + f[bs][N]
            if tot < g[acc]:
                g[acc] = tot
                g_step[acc] = bs
                g_max[acc] = max(g_max[acc - bs], f_max[bs][N])
    final = (pipelinelen - 1) * g_max[B] + g[B]                              # :135
    if final == inf:
        return final, None
    scheme, cur_b = [], B
    while cur_b > 0:                                                         # :138-150
        bs = g_step[cur_b]
        sl, cur = [], N
        while cur > 0:
            st = f_step[bs][cur]
            sl.append(st)
            cur -= st
        scheme.append((bs, sl))
        cur_b -= bs
    return final, scheme


def compositions(n):
    """All ordered ways to write n as a sum of positive integers."""
    for cuts in itertools.product([0, 1], repeat=n - 1):
        parts, cur = [], 1
        for c in cuts:
            if c:
                parts.append(cur)
                cur = 1
            else:
                cur += 1
        parts.append(cur)
        yield parts


def brute_force_best(latency_grid, total_batch_size, total_nslices, pipelinelen, max_latency):
    """min over every batch grouping (as a multiset in the DP's sense: ordered compositions of the batch) and
    every slicing per group of  sum(latencies) + (pipelinelen - 1) * max(latency), all latencies <= max_latency."""
    best = math.inf
    for groups in compositions(total_batch_size):
        per_group = []
        for bs in groups:
            opts = []
            for sl in compositions(total_nslices):
                ctx, lats = 0, []
                for s in sl:
                    lats.append(latency_grid[bs][s][ctx])
                    ctx += s
                if max(lats) <= max_latency:
                    opts.append((sum(lats), max(lats)))
            per_group.append(opts)
        if any(not o for o in per_group):
            continue
        for choice in itertools.product(*per_group):
            tot = sum(c[0] for c in choice) + (pipelinelen - 1) * max(c[1] for c in choice)
            best = min(best, tot)
    return best
