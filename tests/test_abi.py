"""CPU-side checks of the boundary: the shared library loads and exports every symbol that
include/terapipe_hip.h declares, the ctypes mirrors match the C struct sizes, and argument errors are
reported without touching a GPU.  No compute calls."""
import ctypes
import os
import re
import subprocess
import sys
import tempfile

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "terapipe_hip.h")


def _declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(tp_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported_and_bound(lib):
    from terapipe_amd import _lib
    names = _declared_symbols()
    assert len(names) >= 13
    for n in names:
        assert hasattr(lib, n), "library does not export %s" % n
        assert n in _lib.SYMBOLS, "ctypes binding misses %s" % n
    assert sorted(_lib.SYMBOLS) == names


def test_struct_sizes_match_c_compiler(lib):
    """Compiles a 10-line C program against the header with gcc and compares sizeof/offsetof."""
    from terapipe_amd import _lib
    src = r'''
#include <stdio.h>
#include <stddef.h>
#include "terapipe_hip.h"
int main(void) {
  printf("%zu %zu %zu %zu %zu %zu\n", sizeof(tp_gemm_desc), offsetof(tp_gemm_desc, colsum_acc),
         offsetof(tp_gemm_desc, q_scale), sizeof(tp_attn_desc), offsetof(tp_attn_desc, q_scale),
         offsetof(tp_attn_desc, colsum_dqkv_acc));
  printf("%zu %zu %zu %zu %zu %zu\n", offsetof(tp_gemm_desc, defer_reduce), offsetof(tp_attn_desc, dq_only),
         offsetof(tp_attn_desc, stat_bh_rows), sizeof(tp_attn_suffix_desc), offsetof(tp_attn_suffix_desc, q_all),
         offsetof(tp_attn_suffix_desc, dqkv));
  printf("%zu %zu %zu %zu\n", sizeof(tp_adam_tensor), offsetof(tp_adam_tensor, n), sizeof(tp_adam_desc),
         offsetof(tp_adam_desc, tensors));
  printf("%zu %zu %zu\n", sizeof(tp_vecgrad_desc), offsetof(tp_vecgrad_desc, ld), offsetof(tp_vecgrad_desc, N));
  return 0;
}'''
    with tempfile.TemporaryDirectory() as d:
        c = os.path.join(d, "t.c")
        open(c, "w").write(src)
        exe = os.path.join(d, "t")
        subprocess.check_call(["gcc", "-I", os.path.join(ROOT, "include"), c, "-o", exe])
        got = [int(v) for v in subprocess.check_output([exe]).split()]
    G, A, S = _lib.GemmDesc, _lib.AttnDesc, _lib.AttnSuffixDesc
    assert got == [ctypes.sizeof(G), G.colsum_acc.offset, G.q_scale.offset, ctypes.sizeof(A), A.q_scale.offset,
                   A.colsum_dqkv_acc.offset, G.defer_reduce.offset, A.dq_only.offset, A.stat_bh_rows.offset,
                   ctypes.sizeof(S), S.q_all.offset, S.dqkv.offset,
                   ctypes.sizeof(_lib.AdamTensor), _lib.AdamTensor.n.offset, ctypes.sizeof(_lib.AdamDesc),
                   _lib.AdamDesc.tensors.offset,
                   ctypes.sizeof(_lib.VecGradDesc), _lib.VecGradDesc.ld.offset, _lib.VecGradDesc.N.offset]


def test_argument_errors_without_gpu(lib):
    from terapipe_amd import _lib
    assert lib.tp_version() >= 100
    d = _lib.GemmDesc()
    assert lib.tp_gemm(ctypes.byref(d), None, 0, None) == 1          # TP_ERR_ARG
    assert b"shape" in lib.tp_last_error()
    d.M, d.N, d.K, d.dtype = 8, 8, 12, _lib.TP_F16                   # K not a multiple of 8
    d.A = d.B = d.C = 256
    d.lda = d.ldb = 12
    d.ldc = 8
    assert lib.tp_gemm(ctypes.byref(d), None, 0, None) == 2          # TP_ERR_UNSUPPORTED
    assert lib.tp_gemm_workspace_bytes(ctypes.byref(d)) == 0
    a = _lib.AttnDesc()
    a.head_dim = 72
    assert lib.tp_attn_prefix_fwd(ctypes.byref(a), None, 0, None) != 0
    assert b"head_dim" in lib.tp_last_error()
    assert lib.tp_layernorm_fwd(None, None, None, None, None, None, 4, 64, 1e-5, 0, None) == 1
    assert lib.tp_zero_words(None, 4, None) == 1
    assert lib.tp_fill_probe(None, 8192, None, 8192, 0, 1, 1, 0, None) == 1
    assert lib.tp_fill_probe(4096, 8192, 4096, 100, 0, 1, 1, 0, None) == 1   # region not a multiple of 8192 bytes
    assert lib.tp_fill_probe(4096, 8192, 4096, 8192, 0, 1, 1, 1024, None) == 1   # 64 rows of that pitch do not fit


def test_every_head_dimension_of_the_model_table_is_accepted(lib):
    """The attention entry points take the head dimension of every entry of MODEL_CONFIGS (reference
    transformer_models.py:17-59): a descriptor that is otherwise empty gets past the head-dimension check and is
    refused for its geometry instead."""
    from terapipe_amd import _lib, transformer_models as tm
    dims = sorted({e // h for (_, e, _, h) in tm.MODEL_CONFIGS.values()})
    assert dims == [16, 64, 80, 96, 128]
    for hd in dims + [32]:
        a = _lib.AttnDesc()
        a.head_dim = hd
        assert lib.tp_attn_prefix_fwd(ctypes.byref(a), None, 0, None) == 1      # TP_ERR_ARG
        assert b"geometry" in lib.tp_last_error()
    for hd in (8, 48, 72, 112, 256):
        a = _lib.AttnDesc()
        a.head_dim = hd
        assert lib.tp_attn_prefix_bwd(ctypes.byref(a), None, 0, None) == 2      # TP_ERR_UNSUPPORTED
    s = _lib.AttnSuffixDesc()
    s.dtype, s.head_dim = _lib.TP_F16, 96
    assert lib.tp_attn_suffix_dkdv(ctypes.byref(s), None) == 2                  # the one-pass kernel: 64 and 128 only
    assert b"head_dim" in lib.tp_last_error()


def test_failed_replayed_launch_raises_the_library_error():
    """A recorded launch that returns a status on replay surfaces as TeraPipeHipError."""
    from terapipe_amd import _lib, terapipe
    ran = []
    with pytest.raises(_lib.TeraPipeHipError, match="replayed launch failed"):
        terapipe._run_program([(lambda a: ran.append(a) or 0, 1), (lambda a: 4, 2), (lambda a: ran.append(a) or 0, 3)])
    assert ran == [1]


def test_hip_graph_with_slice_streams_is_refused():
    """use_hip_graph with more than one slice stream is switched off (constructor and later attribute changes)."""
    import terapipe_amd as ta
    layers = ta.TransformerLayers(1, 128, 256, 2, dtype=torch.float16, device="cpu")
    with pytest.raises(ValueError, match="slice_streams=1"):
        ta.TeraPipe(layers, 1, 64, [1], [32, 32], use_hip_graph=True, slice_streams=3)
    r = ta.TeraPipe(layers, 1, 64, [1], [32, 32], use_hip_graph=True)
    assert r.slice_streams == 1 and not r.launch_replay
    r.slice_streams = 2
    with pytest.raises(ValueError):
        r._check_mode()
    r = ta.TeraPipe(layers, 1, 64, [1], [32, 32])
    assert r.slice_streams == 3 and r.launch_replay


def _delta_reads_are_ordered(seq_slices, n_lanes, plan):
    """Happens-before check of one layer of the reverse-order backward as the runner issues it: slice i runs on
    lane i mod n_lanes; a two-launch slice issues dQ (writes its delta), waits for slice i+1's event, records its own,
    then issues the one-pass dK/dV (reads delta of every later position from memory); a fused slice waits, records,
    then issues one launch that writes its delta and reads delta from its own_end on.  Returns the first
    (reader, writer) pair that nothing orders, or None."""
    ns = len(seq_slices)
    n = max(n_lanes, 1)
    ends = [sum(seq_slices[:i + 1]) for i in range(ns)]
    before_lane = {l: set() for l in range(n)}      # launches that precede the lane's next operation
    event = {}                                       # slice -> launches its event stands for
    for i in reversed(range(ns)):
        lane = i % n
        own_end, fused = plan[i]
        if not fused:
            before_lane[lane] = before_lane[lane] | {("w", i)}            # dQ launch leaves delta_i
        if i + 1 in event:
            before_lane[lane] = before_lane[lane] | event[i + 1]
        event[i] = set(before_lane[lane])
        first_read = own_end if fused else ends[i]
        for j in range(i + 1, ns):
            if ends[j] > first_read and ("w", j) not in before_lane[lane]:
                return (i, j)
        if fused:
            before_lane[lane] = before_lane[lane] | {("w", i)}
    return None


def test_fused_backward_plan_orders_every_delta_read():
    """Several lanes: no two-launch slice may come before a fused one (the fused slice's event is recorded before
    the launch that writes its delta).  The rule decides once per step there; on one stream per slice."""
    from terapipe_amd import ops
    from terapipe_amd.terapipe import fused_backward_slices
    W = ops.FUSED_BWD_WINDOW
    cases = [[128] * 16, [64] * 32, [32] * 64, [512, 384, 320, 256, 224, 192, 160], [256] * 8, [16] * 8,
             [40, 200, 24, 64, 32, 16, 8], [128, 64, 32, 32], [32, 32, 200, 32, 32], [2048]]
    for ss in cases:
        for n in (1, 2, 3, 4):
            plan = fused_backward_slices(ss, n)
            assert len(plan) == len(ss)
            assert _delta_reads_are_ordered(ss, n, plan) is None, (ss, n)
            for i, (own_end, fused) in enumerate(plan):
                assert own_end == min(sum(ss), sum(ss[:i]) + sum(ss[i:i + n]))
                if fused:
                    assert own_end - sum(ss[:i]) <= W
    # uniform 32-token slices on three lanes stay fused (96 positions), 128-token ones are not (384)
    assert all(f for _, f in fused_backward_slices([32] * 64, 3))
    assert not any(f for _, f in fused_backward_slices([128] * 16, 3))
    assert all(f for _, f in fused_backward_slices([128] * 16, 1))
    # the check has teeth: deciding per slice on three lanes (windows shrink at the sequence end, so the last slice
    # of a 128-token slicing would be fused and the one before it not) leaves a read unordered
    L = 2048
    per_slice = [(e, e - 128 * i <= W) for i, (e, _) in enumerate(fused_backward_slices([128] * 16, 3))]
    assert per_slice[15][1] and not per_slice[14][1]
    assert _delta_reads_are_ordered([128] * 16, 3, per_slice) == (14, 15)


def test_ops_refuse_cpu_tensors():
    """There is no CPU fallback: host tensors raise instead of computing."""
    from terapipe_amd import _lib, ops
    with pytest.raises(_lib.TeraPipeHipError):
        ops.layernorm_fwd(torch.zeros(4, 64), torch.ones(64), torch.zeros(64))
    with pytest.raises(_lib.TeraPipeHipError):
        ops.gemm(_lib.TP_GEMM_NT, torch.zeros(8, 8), torch.zeros(8, 8), 8, 8, 8, C=torch.zeros(8, 8))


def test_package_does_not_import_the_oracle():
    """The shipped package must not reach into oracle/ (test infrastructure only)."""
    for dirpath, _, files in os.walk(os.path.join(ROOT, "terapipe_amd")):
        for f in files:
            if f.endswith(".py"):
                text = open(os.path.join(dirpath, f)).read()
                assert not re.search(r"^\s*(import|from)\s+oracle\b", text, flags=re.M), f
    code = "import sys; sys.path.insert(0, %r); import terapipe_amd; assert 'oracle' not in sys.modules" % ROOT
    subprocess.check_call([sys.executable, "-c", code])


def test_host_side_surface_mirrors_reference_names():
    import terapipe_amd as ta
    from terapipe_amd import transformer_models as tm
    layer = ta.ModelParallelTransformerLayer(64, 256, 1, device="cpu")
    keys = set(layer.state_dict().keys())
    assert keys == {"attn_ln.weight", "attn_ln.bias", "attn.in_proj.weight", "attn.in_proj.bias",
                    "attn.out_proj.weight", "attn.out_proj.bias", "fc_ln.weight", "fc_ln.bias",
                    "fc1.weight", "fc1.bias", "fc2.weight", "fc2.bias"}
    assert layer.attn.in_proj.weight.shape == (192, 64) and layer.fc1.weight.shape == (256, 64)
    assert not layer.fc1.bias.abs().any() and not layer.attn.out_proj.bias.abs().any()   # zero-init biases
    k, v = layer.attn.create_attn_cache(2, 16, device="cpu", dtype=torch.float16)
    assert k.shape == (2, 16, 64) and k.dtype == torch.float16 and not k.abs().any()
    with pytest.raises(AssertionError):
        tm.MultiheadLMAttentionWithCache(100, 3)              # embed_dim not divisible by heads
    with pytest.raises(AssertionError):
        layer(torch.zeros(4, 1, 32))                          # wrong embedding dim
    with pytest.raises(AssertionError):
        layer(torch.zeros(4, 1, 64), None, 3)                 # cache_len without a cache
    assert ta.uniform_slice(10, 4) == [3, 3, 2, 2]
    assert tm.MODEL_CONFIGS["gpt3-13b"] == (40, 5120, 2048, 40) and tm.BATCH_CONFIGS["gpt3-175b"] == 2
    cfg = tm.TransformerConfig.from_predefined_model("gpt3-1b")
    assert (cfg.n_layers, cfg.embedding_dim, cfg.ffn_embedding_dim, cfg.attention_heads_dim) == (24, 2048, 8192, 128)
    with pytest.raises(AssertionError):
        ta.TeraPipe(None, 2, 16, [2], [8, 4])                 # slices must sum to the sequence length


def test_slicers_and_loss_on_cpu_tensors():
    """uniform_slice_x, grid_slice_batch_and_sequence and loss_func are plain tensor code: checked on CPU tensors
    against index arithmetic (reference transformer_models.py:368-377, :393-409, terapipe.py:48-49)."""
    import terapipe_amd as ta
    x = torch.arange(11 * 4 * 3, dtype=torch.float32).view(11, 4, 3)
    parts = ta.uniform_slice_x(x, 4)                           # 11 = 3 + 3 + 3 + 2: the first 11 % 4 slices get one more
    assert [p.size(0) for p in parts] == [3, 3, 3, 2] == ta.uniform_slice(11, 4)
    assert torch.equal(torch.cat(parts), x)
    assert parts[1].data_ptr() == x[3:].data_ptr()             # views, as in the reference
    g = ta.grid_slice_batch_and_sequence(x, [1, 3], [5, 2, 4], requires_grad=True)
    assert g.shape == (2, 3) and g.dtype == object
    assert torch.equal(g[1, 2], x[7:11, 1:4]) and g[1, 2].is_contiguous() and g[1, 2].requires_grad and g[1, 2].is_leaf
    assert torch.equal(g[0, 1], x[5:7, 0:1])
    with pytest.raises(AssertionError):
        ta.grid_slice_batch_and_sequence(x, [1, 3], [5, 2])    # slices must cover the sequence
    with pytest.raises(AssertionError):
        ta.grid_slice_batch_and_sequence(x, [1, 2], [5, 2, 4])
    assert ta.loss_func(x).item() == pytest.approx(x.mean().item())


def test_adam_table_validation_without_gpu(lib):
    from terapipe_amd import _lib
    t = (_lib.AdamTensor * 2)()
    for i in range(2):
        t[i].master, t[i].grad, t[i].exp_avg, t[i].exp_avg_sq, t[i].model, t[i].n = 256, 512, 768, 1024, 1280, 100
    assert lib.tp_adam_check_table(ctypes.cast(t, ctypes.c_void_p), 2, _lib.TP_F16) == 0
    t[1].grad = 520                                                   # 8-byte aligned only
    assert lib.tp_adam_check_table(ctypes.cast(t, ctypes.c_void_p), 2, _lib.TP_F16) == 2      # TP_ERR_UNSUPPORTED
    assert b"tensor 1" in lib.tp_last_error()
    t[1].grad, t[0].model = 512, None
    assert lib.tp_adam_check_table(ctypes.cast(t, ctypes.c_void_p), 2, -1) == 0               # model unused
    assert lib.tp_adam_check_table(ctypes.cast(t, ctypes.c_void_p), 2, _lib.TP_BF16) == 1
    d = _lib.AdamDesc()
    assert lib.tp_adam_step(ctypes.byref(d), None) == 1
    d.n_tensors, d.tensors, d.model_dtype, d.step = 1, 256, -1, 0
    assert lib.tp_adam_step(ctypes.byref(d), None) == 1 and b"step" in lib.tp_last_error()


def test_measured_gemm_plans_are_looked_up_without_gpu(lib):
    """plan_gemm consults csrc/gemm_tuned.inc before its heuristics: the weight extents match exactly and the
    nearest measured M at or above the slice's (within a factor of two) is taken.  tp_gemm_splits exposes the
    planned k-split, which is enough to see which rule fired."""
    import re
    from terapipe_amd import _lib
    root = os.path.join(ROOT, "terapipe_amd", "csrc", "gemm_tuned.inc")
    entries = [tuple(m.groups()) for m in re.finditer(r"\{TP_GEMM_(NT|NN), (\d+), (\d+), (\d+), (\d+), (\d+)\}", open(root).read())]
    assert entries, "the table holds measured plans"
    ops_ = {"NT": _lib.TP_GEMM_NT, "NN": _lib.TP_GEMM_NN}
    by_weight = {}
    for op, M, N, K, cfg, ns in entries:
        by_weight.setdefault((op, int(N), int(K)), []).append((int(M), int(ns)))

    def splits(op, M, N, K):
        d = _lib.GemmDesc()
        d.op, d.dtype, d.M, d.N, d.K = ops_[op], _lib.TP_F16, M, N, K
        d.A = d.B = d.C = 256                              # planning only: nothing is dereferenced
        d.lda, d.ldb, d.ldc = K, (K if op == "NT" else N), N
        return lib.tp_gemm_splits(ctypes.byref(d))

    checked = 0
    for (op, N, K), rows in by_weight.items():
        rows.sort()
        for M, ns in rows:
            assert splits(op, M, N, K) == min(ns, K // 8), (op, M, N, K)          # the entry itself
            lower = [m for m, _ in rows if m < M]
            probe = M - 8                                                          # a slightly shorter slice
            if probe > (lower[-1] if lower else 0) and 2 * probe >= M:
                assert splits(op, probe, N, K) == ns, (op, probe, N, K)
                checked += 1
    assert checked > 10
