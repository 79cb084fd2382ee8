"""The GEMM plan (tile configuration + k splits) that tp_gemm picks, asked through tp_gemm_plan: host code, so these
run without a GPU.  The measured table must give every shape of the four benchmark geometries exactly its entry, and
the rules for slice GEMMs outside the table must give plans that are valid and that follow the stated principles
(one round of workgroups when k is split, no split that leaves less than 1536 of k)."""
import ctypes
import os
import re

import pytest

from terapipe_amd import _lib

OPS = {"NT": _lib.TP_GEMM_NT, "NN": _lib.TP_GEMM_NN, "TN": _lib.TP_GEMM_TN}
# tile configuration -> (rows, columns, workgroups that fit a CU)
TILES = {0: (64, 64, 2), 2: (256, 256, 1), 6: (192, 160, 1), 7: (160, 160, 1), 3: (128, 256, 1), 5: (128, 128, 2), 8: (64, 64, 2), 10: (128, 128, 2), 11: (64, 256, 1),
         12: (64, 64, 2), 13: (128, 128, 1), 14: (192, 128, 1), 15: (256, 128, 1), 16: (128, 128, 1), 17: (256, 160, 1), 18: (256, 128, 1), 19: (256, 256, 1), 20: (256, 256, 1),
         31: (192, 128, 1), 33: (192, 256, 1), 41: (224, 128, 1), 42: (160, 128, 1), 43: (224, 160, 1)}


def plan(op, M, N, K, dtype=_lib.TP_F16):
    d = _lib.GemmDesc()
    d.op, d.dtype, d.epilogue, d.M, d.N, d.K = OPS[op], dtype, _lib.TP_EPI_STORE, M, N, K
    d.A = d.B = d.C = 4096          # never dereferenced: the plan is host arithmetic on the extents
    d.lda = M if op == "TN" else K
    d.ldb = K if op == "NT" else N
    d.ldc = N
    c, n = ctypes.c_int(), ctypes.c_int()
    rc = _lib.load().tp_gemm_plan(ctypes.byref(d), ctypes.byref(c), ctypes.byref(n))
    assert rc == 0, _lib.load().tp_last_error()
    assert n.value == _lib.load().tp_gemm_splits(ctypes.byref(d))
    return c.value, n.value


def _table():
    path = os.path.join(os.path.dirname(_lib.__file__), "csrc", "gemm_tuned.inc")
    out = []
    for line in open(path):
        m = re.match(r"\{TP_GEMM_(\w+), (\d+), (\d+), (\d+), (\d+), (\d+)\}", line)
        if m:
            out.append((m.group(1),) + tuple(int(v) for v in m.groups()[1:]))
    return out


def test_every_table_entry_is_the_plan_of_its_shape():
    entries = _table()
    assert len(entries) >= 90
    for op, M, N, K, cfg, ns in entries:
        assert plan(op, M, N, K) == (cfg, ns), (op, M, N, K)
        assert plan(op, M, N, K, _lib.TP_BF16) == (cfg, ns), (op, M, N, K)


def test_the_baseline_geometries_are_covered_by_exact_entries():
    """Every 16-bit GEMM of benchmark configs 2-5 (slice linears at each slice length, parameter gradients of a step)
    has its own entry, so that a revision of the rules cannot move a benchmark shape."""
    have = {e[:4] for e in _table()}
    geos = [(2048, 8192, [256], 2048), (5120, 20480, [512, 384, 320, 256, 224, 192, 160], 2048),
            (12288, 49152, [128], 2048), (6144, 24576, [64], 4096)]
    for E, F, rows, step in geos:
        for N, K in ((3 * E, E), (E, E), (F, E), (E, F)):
            for M in rows:
                assert ("NT", M, N, K) in have and ("NN", M, K, N) in have, (M, N, K)
            assert ("TN", N, K, step) in have, (N, K, step)


@pytest.mark.parametrize("E,F", [(1024, 4096), (3072, 12288), (4096, 16384), (7168, 28672), (8192, 32768), (10240, 40960)])
def test_rules_for_slice_gemms_outside_the_table(E, F):
    for M in (8, 40, 64, 96, 128, 160, 200, 256, 320, 384, 448, 512):
        for N, K in ((3 * E, E), (E, E), (F, E), (E, F)):
            for op, n, k in (("NT", N, K), ("NN", K, N)):
                cfg, ns = plan(op, M, n, k)
                assert cfg in TILES, (op, M, n, k, cfg)
                bm, bn, per_cu = TILES[cfg]
                tiles = -(-M // bm) * -(-n // bn)
                assert 1 <= ns <= 8
                if ns > 1:
                    assert k // ns >= 1536, "split too thin: %s" % ((op, M, n, k, cfg, ns),)
                    assert tiles * ns <= 256 * per_cu, "more than one round of workgroups: %s" % ((op, M, n, k, cfg, ns),)
                # a tile is never taller than twice the slice
                assert bm < 2 * max(M, 64), (op, M, n, k, cfg)


def test_rule_examples():
    """Shapes from the sweeps the rules were drawn from (measured best or within a few percent of it)."""
    assert plan("NT", 64, 16384, 4096) == (8, 1)           # 256 tiles of 64 x 64
    assert plan("NN", 64, 4096, 16384) == (8, 4)           # 64 tiles, k split to 256 workgroups
    assert plan("NT", 128, 4096, 4096) == (12, 1)          # small weight: 64 x 64 x 128 tiles, unsplit
    assert plan("NN", 128, 4096, 12288) == (16, 8)         # 32 tiles of 128 x 128 (the pipelined tile)
    assert plan("NT", 256, 32768, 8192) == (3, 1)          # 256 tiles of 128 x 256
    assert plan("NN", 256, 8192, 32768) == (3, 4)          # 64 of them on a long k
    assert plan("NT", 256, 12288, 4096) == (16, 1)         # 192 tiles of 128 x 128, k too short to split
    assert plan("NT", 320, 30720, 10240) == (33, 1)        # two row tiles of 192: the weight-streaming kernel
    assert plan("NT", 512, 20480, 4096) == (19, 1)         # two rows of 256 x 256 tiles
    assert plan("NN", 512, 4096, 16384) == (15, 4)         # 2 x 32 pipelined tiles of 256 x 128 on a long k
    assert plan("NT", 384, 16384, 4096) == (14, 1)         # two row tiles of 192 x 128
    assert plan("NT", 224, 16384, 8192) == (41, 2)         # one row of 224 x 128 tiles: nothing of a tile beyond the slice
    assert plan("NN", 448, 8192, 32768) == (41, 2)         # two of them
    assert plan("NT", 320, 16384, 8192) == (42, 1)         # two row tiles of 160 x 128
    assert plan("NT", 160, 32768, 8192) == (42, 1)         # one
    # fp32 keeps its own plan (64 x 64 register-staged tiles)
    assert plan("NT", 128, 4096, 4096, _lib.TP_F32)[0] == 0


def _forced_plan(op, M, N, K, cfg, nsplit=0):
    d = _lib.GemmDesc()
    d.op, d.dtype, d.epilogue, d.M, d.N, d.K = OPS[op], _lib.TP_F16, _lib.TP_EPI_STORE, M, N, K
    d.A = d.B = d.C = 4096
    d.lda = M if op == "TN" else K
    d.ldb = K if op == "NT" else N
    d.ldc = N
    d.reserved = (cfg + 1) | (nsplit << 8)
    c, n = ctypes.c_int(), ctypes.c_int()
    assert _lib.load().tp_gemm_plan(ctypes.byref(d), ctypes.byref(c), ctypes.byref(n)) == 0
    return c.value, n.value


def test_forced_tiles_that_load_whole_k_tiles_fall_back_on_a_ragged_k():
    """A tile configuration forced through the descriptor's reserved field is replaced by the 128 x 128 register-
    free tile (5) when the kernel behind it cannot run the shape: the weight-streaming, pipelined and tall tiles
    load whole 64-wide k-tiles only, the weight-streaming tiles have no TN form."""
    for cfg in (21, 26, 33, 40, 14, 15, 16, 19, 2, 41, 42, 43):
        assert _forced_plan("NT", 128, 1024, 1024, cfg)[0] == cfg, cfg          # K % 64 == 0: taken as forced
        assert _forced_plan("NT", 128, 1024, 72, cfg)[0] == 5, cfg              # K = 72: would drop the k tail
        assert _forced_plan("NN", 128, 1024, 1096, cfg)[0] == 5, cfg
    for cfg in (21, 33, 41, 42, 43):
        assert _forced_plan("TN", 1024, 1024, 1024, cfg)[0] == 5, cfg
    assert _forced_plan("NN", 128, 1024, 1024, 24)[0] == 5                      # 80-wide tiles: NT only
    assert _forced_plan("NN", 224, 1024, 1024, 43)[0] == 5                      # 160-wide pipelined tile: NT only
