"""CPU tests of the C-ABI shared library: it loads, exports every symbol the header
declares, and its host-only entry points (schedule builder, argument checks) behave."""
import ctypes as C
import os
import re

import pytest
import torch

from flame_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    if not os.path.exists(_lib.LIB_PATH):
        import __graft_entry__
        __graft_entry__.build()
    return _lib.load()


def test_exports_every_declared_symbol(lib):
    header = open(os.path.join(ROOT, "include", "sba_mi355x.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(sba_[a-z_]+)\s*\(", header))
    assert declared == set(_lib.EXPORTED_SYMBOLS)
    for name in declared:
        assert getattr(lib, name) is not None


def test_abi_version_and_struct_size(lib):
    assert lib.sba_abi_version() == 6
    p = _lib.SbaParams()
    p.struct_size = C.sizeof(_lib.SbaParams) - 8
    assert lib.sba_fwd(C.byref(p)) == -7          # SBA_ERR_ABI, before anything touches a GPU
    assert b"struct_size" in lib.sba_error_string(-7)


def test_argument_checks_without_gpu(lib):
    p = _lib.SbaParams()
    p.struct_size = C.sizeof(_lib.SbaParams)
    p.dtype = 7
    assert lib.sba_fwd(C.byref(p)) == -3          # dtype
    p.dtype = _lib.SBA_DTYPE_BF16
    assert lib.sba_fwd(C.byref(p)) == -2          # shape (all zero)
    p.n_seq, p.n_heads, p.seq_len, p.total_tokens, p.head_dim = 1, 2, 64, 64, 257
    assert lib.sba_fwd(C.byref(p)) == -2          # head_dim > 256
    assert lib.sba_workspace_bytes(C.byref(p)) == 0 and lib.sba_bwd_scratch_bytes(C.byref(p)) == 0
    p.head_dim = 64
    assert lib.sba_fwd(C.byref(p)) == -1          # NULL q/k/v
    p.dtype = _lib.SBA_DTYPE_F16                  # float16: every head dim, like bf16
    assert lib.sba_fwd(C.byref(p)) == -1
    p.head_dim = 96
    assert lib.sba_fwd(C.byref(p)) == -1
    p.dtype, p.head_dim = _lib.SBA_DTYPE_BF16, 64
    assert lib.sba_attention_weights(C.byref(p), None) == -1      # NULL q/k/v come first
    p.q.ptr = p.k.ptr = p.v.ptr = 256                             # never dereferenced: the checks below come before any launch
    assert lib.sba_attention_weights(C.byref(p), None) == -1      # no output
    p.q.ptr = p.k.ptr = p.v.ptr = None
    assert lib.sba_fwd(None) == -1
    assert lib.sba_row_block() == 128


def test_error_codes_of_the_call_sequence_without_gpu(lib):
    # every check below fails before anything is launched
    p = _lib.SbaParams()
    p.struct_size = C.sizeof(_lib.SbaParams)
    p.dtype = _lib.SBA_DTYPE_BF16
    p.n_seq, p.n_heads, p.seq_len, p.total_tokens, p.head_dim = 1, 2, 256, 256, 64
    for t in ("q", "k", "v", "o", "d_o", "dq", "dk", "dv"):
        getattr(p, t).ptr = 256
        getattr(p, t).stride_h, getattr(p, t).stride_t = 256 * 64, 64
    p.rem.ptr = 256
    p.save_for_backward = 1
    assert lib.sba_fwd(C.byref(p)) == -4                      # SBA_ERR_WORKSPACE: no workspace given
    p.workspace, p.workspace_bytes = 256, lib.sba_workspace_bytes(C.byref(p)) - 1
    assert lib.sba_fwd(C.byref(p)) == -4                      # one byte short
    assert lib.sba_bwd(C.byref(p)) == -4                      # the backward checks it too
    p.workspace_bytes += 1
    assert lib.sba_bwd(C.byref(p)) == -4                      # and its own scratch
    assert b"sba_bwd_scratch_bytes" in lib.sba_error_string(-4)
    p.q.ptr = 264                                             # not 16-byte aligned
    assert lib.sba_fwd(C.byref(p)) == -2
    p.q.ptr, p.k.stride_t = 256, 68                           # stride not a multiple of 8 elements
    assert lib.sba_fwd(C.byref(p)) == -2
    p.k.stride_t = 1 << 23                                    # beyond the 32-bit tile addressing
    assert lib.sba_fwd(C.byref(p)) == -2
    assert b"token stride" in lib.sba_error_string(-2)
    p.k.stride_t = 64
    p.cu_seqlens = 256                                        # packed layout ...
    assert lib.sba_fwd(C.byref(p)) == -5                      # ... without a schedule: SBA_ERR_SCHEDULE
    p.schedule, p.n_schedule = 256, 2
    assert lib.sba_fwd(C.byref(p)) == -5                      # ... without the table size
    assert b"sba_build_schedule" in lib.sba_error_string(-5)


def test_workspace_bytes(lib):
    p = _lib.SbaParams()
    p.struct_size = C.sizeof(_lib.SbaParams)
    p.dtype = _lib.SBA_DTYPE_BF16
    p.n_seq, p.n_heads, p.seq_len, p.total_tokens, p.head_dim = 1, 16, 4096, 4096, 64
    # one carry table: per head, row block qb keeps 128 queries x its 2*qb + 2 visible 64-key blocks:
    # 32 * 33 columns of 128 floats at T = 4096 (half of a full [T/64][T] rectangle, plus the diagonal)
    table = 16 * 32 * 33 * 128 * 4
    # bf16: the forward hands two tables to the backward (the carries entering the right and the left half of every 64-key step)
    assert lib.sba_workspace_bytes(C.byref(p)) == 2 * table
    scaled_q = 16 * 4096 * 64 * 2                   # head_dim 64: the dQ pass's copy of q times the logit scale, for the dK/dV stream
    assert lib.sba_bwd_scratch_bytes(C.byref(p)) == 4 * table + scaled_q + 256    # no workspace: the backward recomputes those tables (+ error word)
    p.workspace = 1
    assert lib.sba_bwd_scratch_bytes(C.byref(p)) == 2 * table + scaled_q + 256    # what the backward needs for itself
    p.workspace = None
    p.dtype = _lib.SBA_DTYPE_F32                    # fp32 at head_dim 64 runs on the matrix cores too: one table from the forward
    assert lib.sba_workspace_bytes(C.byref(p)) == table
    assert lib.sba_bwd_scratch_bytes(C.byref(p)) == 2 * table      # the forward's table again and the dQ pass's; no bounded waits, no error word
    p.workspace = 1
    assert lib.sba_bwd_scratch_bytes(C.byref(p)) == table
    p.workspace = None
    p.head_dim = 128                                # and at head_dim 128
    assert lib.sba_workspace_bytes(C.byref(p)) == table
    p.head_dim = 96                                 # generic kernels: nothing kept, fp32 dk|dv accumulators
    assert lib.sba_workspace_bytes(C.byref(p)) == 0
    assert lib.sba_bwd_scratch_bytes(C.byref(p)) == 2 * 4096 * 16 * 128 * 4
    p.head_dim = 256                                # fp32 above 128: generic kernels
    assert lib.sba_workspace_bytes(C.byref(p)) == 0
    assert lib.sba_bwd_scratch_bytes(C.byref(p)) == 2 * 4096 * 16 * 256 * 4
    p.dtype = _lib.SBA_DTYPE_BF16                   # bf16 at 256: matrix cores, two tables each way, the error word, no copy of q
    assert lib.sba_workspace_bytes(C.byref(p)) == 2 * table
    assert lib.sba_bwd_scratch_bytes(C.byref(p)) == 4 * table + 256
    p.dtype = _lib.SBA_DTYPE_F16                    # float16 is sized like bf16
    assert lib.sba_workspace_bytes(C.byref(p)) == 2 * table
    assert lib.sba_bwd_scratch_bytes(C.byref(p)) == 4 * table + 256
    p.head_dim = 64
    assert lib.sba_bwd_scratch_bytes(C.byref(p)) == 4 * table + scaled_q + 256
    p.dtype, p.head_dim = _lib.SBA_DTYPE_BF16, 256
    p.dtype, p.head_dim = _lib.SBA_DTYPE_F16, 200   # float16 on the generic kernels: sized like bf16 there too
    assert lib.sba_workspace_bytes(C.byref(p)) == 0
    assert lib.sba_bwd_scratch_bytes(C.byref(p)) == 2 * 4096 * 16 * 256 * 4
    p.dtype = _lib.SBA_DTYPE_BF16
    p.head_dim = 200                                # bf16 in between: generic kernels unless the caller pads to 256
    assert lib.sba_workspace_bytes(C.byref(p)) == 0
    assert lib.sba_bwd_scratch_bytes(C.byref(p)) == 2 * 4096 * 16 * 256 * 4


def test_static_backward_refuses_oversize_without_gpu(lib):
    # the size check of sba_bwd_static() comes before anything touches a GPU
    p = _lib.SbaParams()
    p.struct_size = C.sizeof(_lib.SbaParams)
    p.dtype = _lib.SBA_DTYPE_BF16
    p.n_seq, p.n_heads, p.seq_len, p.total_tokens, p.head_dim = 1, 16, 16384, 16384, 128
    for t in ("q", "k", "v", "d_o", "dq", "dk", "dv"):
        getattr(p, t).ptr = 256                     # never dereferenced
    p.workspace = 256
    assert lib.sba_bwd_scratch_bytes(C.byref(p)) > _lib.STATIC_SCRATCH_BYTES
    assert lib.sba_bwd_static(C.byref(p)) == -8
    assert b"sba_bwd_static" in lib.sba_error_string(-8)


def test_gave_up_helper_without_gpu(lib):
    # argument checks come first; problems without bounded waits (fp32, generic kernels) report 0 without a copy
    flag = C.c_int(7)
    assert lib.sba_bwd_gave_up(None, 0, C.byref(flag)) == -1
    p = _lib.SbaParams()
    p.struct_size = C.sizeof(_lib.SbaParams)
    p.dtype = _lib.SBA_DTYPE_F32
    p.n_seq, p.n_heads, p.seq_len, p.total_tokens, p.head_dim = 1, 2, 256, 256, 64
    for t in ("q", "k", "v"):
        getattr(p, t).ptr = 256
        getattr(p, t).stride_h, getattr(p, t).stride_t = 256 * 64, 64
    assert lib.sba_bwd_gave_up(C.byref(p), 0, None) == -1
    assert lib.sba_bwd_gave_up(C.byref(p), 0, C.byref(flag)) == 0 and flag.value == 0
    p.dtype, p.head_dim = _lib.SBA_DTYPE_BF16, 96          # generic kernels
    flag.value = 7
    assert lib.sba_bwd_gave_up(C.byref(p), 0, C.byref(flag)) == 0 and flag.value == 0
    p.head_dim = 64                                        # bf16 matrix-core path: needs the scratch it is to read
    assert lib.sba_bwd_gave_up(C.byref(p), 0, C.byref(flag)) == -4


def test_python_raises_when_the_error_word_is_set(lib, monkeypatch):
    # the Python side of the check, with the library call replaced (no test makes a kernel's wait expire)
    calls = []

    class Fake:
        def sba_bwd_gave_up(self, p, static_used, flag):
            calls.append(static_used)
            flag._obj.value = 1
            return 0
    monkeypatch.setattr(_lib, "load", lambda: Fake())
    monkeypatch.setattr(torch.cuda, "is_current_stream_capturing", lambda: False)
    with pytest.raises(RuntimeError, match="abandoned a bounded internal wait"):
        _lib.raise_if_gave_up(_lib.SbaParams(), static_scratch_used=True)
    assert calls == [1]


def test_workspace_budget_switch(monkeypatch):
    monkeypatch.delenv("SBA_RECOMPUTE_CARRIES", raising=False)
    monkeypatch.delenv("SBA_WORKSPACE_BUDGET_MB", raising=False)
    _lib.set_workspace_budget(None)
    assert _lib.workspace_budget() == 256 << 20
    assert not _lib.recompute_carries(17 << 20)            # B=1, H=16, T=4096: kept
    assert _lib.recompute_carries(270 << 20)               # T=16384: recomputed
    monkeypatch.setenv("SBA_WORKSPACE_BUDGET_MB", "512")
    assert not _lib.recompute_carries(270 << 20)
    _lib.set_workspace_budget(0)
    assert _lib.recompute_carries(16)
    _lib.set_workspace_budget(float("inf"))
    assert not _lib.recompute_carries(1 << 40)
    monkeypatch.setenv("SBA_RECOMPUTE_CARRIES", "1")
    assert _lib.recompute_carries(0)
    _lib.set_workspace_budget(None)


def test_schedule_builder(lib):
    cu = torch.tensor([0, 100, 400, 401, 1000, 1000], dtype=torch.int32)   # last doc empty
    s = _lib.build_schedule(cu)
    jobs = [tuple(r[:4]) for r in s.tolist()]
    # every (doc, row_block) exactly once, none for the empty document; the fourth int is the
    # document's first carry-table column: documents of 1, 3, 1, 5 row blocks take 2, 12, 2, 30 columns
    doc_of_col = {0: 0, 2: 1, 14: 2, 16: 3}
    expect = {(0, 100, 0, 0), (100, 300, 0, 2), (100, 300, 1, 2), (100, 300, 2, 2), (400, 1, 0, 14)}
    expect |= {(401, 599, rb, 16) for rb in range(5)}
    assert lib.sba_table_columns(C.cast(cu.data_ptr(), C.POINTER(C.c_int32)), 5) == 46
    assert _lib.table_columns(cu) == 46
    assert set(jobs) == expect and len(jobs) == len(expect)
    rbs = [j[2] for j in jobs]
    assert rbs == sorted(rbs, reverse=True)       # longest sweeps first
    # ints 4-7: the same jobs again, longest key-owner sweeps (blocks of the doc - rb) first
    key_jobs = [tuple(r[4:8]) for r in s.tolist()]
    assert sorted(key_jobs) == sorted(jobs)
    key_len = [(j[1] + 127) // 128 - j[2] for j in key_jobs]
    assert key_len == sorted(key_len, reverse=True) and key_len[0] == 5
    # capacity too small: returns the count needed and writes nothing
    out = torch.full((2, 8), -1, dtype=torch.int32)
    n = lib.sba_build_schedule(C.cast(cu.data_ptr(), C.POINTER(C.c_int32)), 5, 0,
                               C.cast(out.data_ptr(), C.POINTER(C.c_int32)), 2)
    assert n == len(expect) and bool((out == -1).all())
    # a launch of SBA_DOC_MAJOR_GRID workgroups or more: same jobs, document-major (longest
    # document first; row blocks descending for the row owners, ascending for the key owners)
    heads = -(-_lib.DOC_MAJOR_GRID // len(jobs))
    d = _lib.build_schedule(cu, heads)
    assert sorted(tuple(r[:4]) for r in d.tolist()) == sorted(jobs)
    assert sorted(tuple(r[4:8]) for r in d.tolist()) == sorted(jobs)
    row_order = [(doc_of_col[r[3]], r[2]) for r in d.tolist()]
    assert row_order == [(3, 4), (3, 3), (3, 2), (3, 1), (3, 0), (1, 2), (1, 1), (1, 0), (0, 0), (2, 0)]
    key_order = [(doc_of_col[r[7]], r[6]) for r in d.tolist()]
    assert key_order == [(3, 0), (3, 1), (3, 2), (3, 3), (3, 4), (1, 0), (1, 1), (1, 2), (0, 0), (2, 0)]
    assert _lib.build_schedule(cu, heads - 1).tolist() == s.tolist()      # just below: the usual order


def test_op_refuses_cpu_tensors():
    from flame_amd import sb_attn
    q = torch.zeros(1, 1, 4, 8)
    with pytest.raises(RuntimeError, match="GPU only"):
        sb_attn(q, q, q)


def test_python_workspace_bound_covers_the_library(lib):
    for dtype in (_lib.SBA_DTYPE_BF16, _lib.SBA_DTYPE_F32, _lib.SBA_DTYPE_F16):
        for (B, H, T, D) in [(1, 16, 4096, 64), (2, 3, 129, 128), (1, 2, 77, 80), (4, 1, 1, 8), (2, 3, 300, 256), (1, 2, 77, 200)]:
            p = _lib.SbaParams()
            p.struct_size = C.sizeof(_lib.SbaParams)
            p.dtype = dtype
            p.n_seq, p.n_heads, p.seq_len, p.total_tokens, p.head_dim = B, H, T, T, D
            cols = _lib.dense_columns(B, T)
            assert _lib.workspace_upper_bound(H, cols) >= lib.sba_workspace_bytes(C.byref(p))
            assert _lib.bwd_scratch_upper_bound(H, cols, B * T, D) >= lib.sba_bwd_scratch_bytes(C.byref(p))
    # packed: the bound from shapes alone (what a torch.compile trace can see) covers the exact count
    for lens in ([1, 130, 500, 64, 205], [4096] * 3 + [16] * 40, [127, 128, 129], [1]):
        cu = torch.tensor([0] + list(torch.tensor(lens).cumsum(0)), dtype=torch.int32)
        assert _lib.packed_columns_bound(sum(lens), len(lens), max(lens)) >= _lib.table_columns(cu)


def test_head_dim_routing_of_the_python_layer(monkeypatch):
    # which head dim a problem runs with: matrix-core sizes as they are, everything else zero-padded up to the next one
    # (16-bit types up to 256, float32 up to 128); the generic kernels keep every head dim
    monkeypatch.delenv("SBA_FORCE_GENERIC", raising=False)
    monkeypatch.delenv("SBA_FORCE_GENERIC_BWD", raising=False)
    expect = {torch.bfloat16: {8: 64, 64: 64, 80: 128, 128: 128, 129: 256, 200: 256, 256: 256},
              torch.float16: {8: 64, 64: 64, 80: 128, 128: 128, 129: 256, 200: 256, 256: 256},
              torch.float32: {8: 64, 64: 64, 80: 128, 128: 128, 129: 129, 200: 200, 256: 256}}
    for dtype, table in expect.items():
        for D, Dp in table.items():
            assert _lib.matrix_core_head_dim(torch.empty(1, 1, 1, D, dtype=dtype)) == Dp, (dtype, D)
    assert _lib.dtype_code(torch.float16) == _lib.SBA_DTYPE_F16 == 2
    with pytest.raises(ValueError, match="head_dim"):
        _lib.check_supported(torch.empty(1, 1, 1, 257, dtype=torch.bfloat16))
    with pytest.raises(TypeError, match="float16"):
        _lib.check_supported(torch.empty(1, 1, 1, 64, dtype=torch.float64))
    monkeypatch.setenv("SBA_FORCE_GENERIC", "1")
    assert _lib.matrix_core_head_dim(torch.empty(1, 1, 1, 80, dtype=torch.bfloat16)) == 80
