"""ctypes binding of libsba_mi355x.so (the C ABI declared in include/sba_mi355x.h).

The library is the only compute path: if it is missing, loading raises and every
operator call fails loudly.  There is no PyTorch or CPU fallback.
"""
from __future__ import annotations

import ctypes as C
import os
import threading

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "libsba_mi355x.so")

SBA_DTYPE_F32, SBA_DTYPE_BF16, SBA_DTYPE_F16 = 0, 1, 2
SBA_ABI_VERSION = 6


class SbaTensor(C.Structure):
    _fields_ = [("ptr", C.c_void_p), ("stride_b", C.c_int64), ("stride_h", C.c_int64),
                ("stride_t", C.c_int64)]


class SbaVector(C.Structure):
    _fields_ = [("ptr", C.c_void_p), ("stride_b", C.c_int64), ("stride_h", C.c_int64)]


class SbaParams(C.Structure):
    _fields_ = [
        ("struct_size", C.c_uint32), ("dtype", C.c_int32), ("n_seq", C.c_int32),
        ("n_heads", C.c_int32), ("seq_len", C.c_int32), ("total_tokens", C.c_int32),
        ("head_dim", C.c_int32), ("attend_current", C.c_int32), ("scale", C.c_float),
        ("save_for_backward", C.c_int32), ("bwd_phases", C.c_int32),
        ("cu_seqlens", C.c_void_p), ("schedule", C.c_void_p), ("n_schedule", C.c_int32),
        ("table_cols", C.c_int64),
        ("q", SbaTensor), ("k", SbaTensor), ("v", SbaTensor), ("o", SbaTensor),
        ("rem", SbaVector), ("d_o", SbaTensor), ("d_rem", SbaVector),
        ("dq", SbaTensor), ("dk", SbaTensor), ("dv", SbaTensor),
        ("workspace", C.c_void_p), ("workspace_bytes", C.c_size_t),
        ("bwd_scratch", C.c_void_p), ("bwd_scratch_bytes", C.c_size_t), ("stream", C.c_void_p),
    ]


_lib = None
_lock = threading.Lock()


def load() -> C.CDLL:
    """Load the shared library once; raise if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is not None:
            return _lib
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with `make -C {os.path.dirname(LIB_PATH)}` "
                "(or __graft_entry__.build()). There is no fallback path.")
        lib = C.CDLL(LIB_PATH)
        lib.sba_abi_version.restype = C.c_int
        lib.sba_error_string.restype = C.c_char_p
        lib.sba_error_string.argtypes = [C.c_int]
        lib.sba_workspace_bytes.restype = C.c_size_t
        lib.sba_workspace_bytes.argtypes = [C.POINTER(SbaParams)]
        lib.sba_bwd_scratch_bytes.restype = C.c_size_t
        lib.sba_bwd_scratch_bytes.argtypes = [C.POINTER(SbaParams)]
        lib.sba_build_schedule.restype = C.c_int
        lib.sba_build_schedule.argtypes = [C.POINTER(C.c_int32), C.c_int, C.c_int, C.POINTER(C.c_int32), C.c_int]
        lib.sba_row_block.restype = C.c_int
        lib.sba_table_columns.restype = C.c_int64
        lib.sba_table_columns.argtypes = [C.POINTER(C.c_int32), C.c_int]
        lib.sba_fwd.restype = C.c_int
        lib.sba_fwd.argtypes = [C.POINTER(SbaParams)]
        lib.sba_bwd.restype = C.c_int
        lib.sba_bwd.argtypes = [C.POINTER(SbaParams)]
        lib.sba_attention_weights.restype = C.c_int
        lib.sba_attention_weights.argtypes = [C.POINTER(SbaParams), C.c_void_p]
        lib.sba_bwd_static.restype = C.c_int
        lib.sba_bwd_static.argtypes = [C.POINTER(SbaParams)]
        lib.sba_bwd_gave_up.restype = C.c_int
        lib.sba_bwd_gave_up.argtypes = [C.POINTER(SbaParams), C.c_int, C.POINTER(C.c_int)]
        if lib.sba_abi_version() != SBA_ABI_VERSION:
            raise RuntimeError("libsba_mi355x.so ABI version mismatch; rebuild it")
        _lib = lib
    return _lib


EXPORTED_SYMBOLS = ("sba_abi_version", "sba_error_string", "sba_workspace_bytes", "sba_bwd_scratch_bytes",
                    "sba_build_schedule", "sba_row_block", "sba_table_columns", "sba_fwd", "sba_bwd",
                    "sba_bwd_static", "sba_bwd_gave_up", "sba_attention_weights")

STATIC_SCRATCH_BYTES = 64 << 20     # SBA_STATIC_SCRATCH_BYTES: what sba_bwd_static() holds per GPU


def check(rc: int, what: str) -> None:
    if rc != 0:
        raise RuntimeError(f"{what} failed: {load().sba_error_string(rc).decode()} (code {rc})")


MAX_HEAD_DIM = 256     # the reference pads the head dim to the next power of two (sb_attn/sb_fwd.py:199); here up to 256


def dtype_code(dt: torch.dtype) -> int:
    if dt == torch.float32:
        return SBA_DTYPE_F32
    if dt == torch.bfloat16:
        return SBA_DTYPE_BF16
    if dt == torch.float16:
        return SBA_DTYPE_F16
    raise TypeError(f"stick-breaking attention supports float32, bfloat16 and float16, got {dt}")


def check_supported(q: torch.Tensor) -> None:
    """Say up front what the kernels do not cover instead of failing inside the library."""
    if q.dtype not in (torch.float32, torch.bfloat16, torch.float16):
        raise TypeError(f"stick-breaking attention supports float32, bfloat16 and float16, got {q.dtype}")
    if q.shape[-1] > MAX_HEAD_DIM:
        raise ValueError(f"head_dim {q.shape[-1]} is not supported (at most {MAX_HEAD_DIM})")


_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def current_stream_handle(device: torch.device) -> int:
    """hipStream_t of torch's current stream on `device` (the stream the kernels are launched on)."""
    if _raw_stream is not None and device.index is not None:
        return _raw_stream(device.index)          # the same handle, without building a torch.cuda.Stream object
    return torch.cuda.current_stream(device).cuda_stream


def tensor4(t: torch.Tensor) -> SbaTensor:
    """[B, H, T, D] view -> descriptor."""
    return SbaTensor(t.data_ptr(), t.stride(0), t.stride(1), t.stride(2))


def tensor3(t: torch.Tensor) -> SbaTensor:
    """[H, T, D] view -> descriptor (no batch stride)."""
    return SbaTensor(t.data_ptr(), 0, t.stride(0), t.stride(1))


def usable(t: torch.Tensor) -> torch.Tensor:
    """Kernels need unit stride along D and 16-byte aligned rows; copy otherwise."""
    if torch.compiler.is_compiling():
        return t.contiguous()            # no data_ptr() on traced tensors
    ok = t.stride(-1) == 1 and t.data_ptr() % 16 == 0
    if ok:
        per16 = 16 // t.element_size()
        ok = all(s % per16 == 0 for s in t.stride()[:-1])
    return t if ok else t.contiguous()


def empty_grads_like(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor):
    """Uninitialised dq, dk, dv.  When q, k and v are the three column slices of one [.., 3*H*D] tensor (the
    output of a stacked q/k/v projection), the gradients are laid out the same way in ONE allocation, so that
    the caller's backward can hand the whole of it to the projection without concatenating."""
    # (three tensors at the same offset of their storages cannot be slices of one buffer: the usual case, decided first)
    if (not torch.compiler.is_compiling() and k.storage_offset() != q.storage_offset()
            and q.shape == k.shape == v.shape and q.stride() == k.stride() == v.stride()):
        n = q.numel()
        span = sum((sz - 1) * st for sz, st in zip(q.shape, q.stride())) + 1      # elements from q's first to its last
        base = q.untyped_storage().data_ptr()
        if (k.untyped_storage().data_ptr() == base and v.untyped_storage().data_ptr() == base and n > 0
                and q.stride(-1) == 1):
            step = k.storage_offset() - q.storage_offset()
            # interleaved thirds of one dense buffer: q's span plus the two slices to its right is exactly 3n
            if step > 0 and v.storage_offset() - k.storage_offset() == step and span + 2 * step == 3 * n:
                buf = torch.empty(3 * n, dtype=q.dtype, device=q.device)
                return tuple(buf.as_strided(q.shape, q.stride(), i * step) for i in range(3))
    return torch.empty_like(q), torch.empty_like(k), torch.empty_like(v)


# What a layer may keep from its forward to its backward (the forward's carry tables) before the operator
# switches to the memory-lean mode by itself: the forward then keeps nothing and the backward repeats the
# forward's sweep for the carries alone (bit-identical gradients, 12-13 % more time per forward + backward).
# The reference keeps one float per query (sb_fwd.py:146); the tables grow with the square of the sequence
# length: 17 MB at B=1, H=16, T=4096, 270 MB at T=16384, 4.3 GB for a dense 65 536-token row.
DEFAULT_WORKSPACE_BUDGET = 256 << 20
_workspace_budget = None            # set_workspace_budget(); None: SBA_WORKSPACE_BUDGET_MB or the default


def set_workspace_budget(nbytes) -> None:
    """Largest carry-table workspace (bytes) a forward may keep for its backward; larger ones are
    recomputed in the backward instead.  None restores the default (SBA_WORKSPACE_BUDGET_MB megabytes if
    that is set, else 256 MiB); 0 never keeps anything; float('inf') always keeps the tables."""
    global _workspace_budget
    _workspace_budget = nbytes


def workspace_budget():
    if _workspace_budget is not None:
        return _workspace_budget
    e = os.environ.get("SBA_WORKSPACE_BUDGET_MB")
    return float(e) * (1 << 20) if e else DEFAULT_WORKSPACE_BUDGET


def recompute_carries(workspace_nbytes: int = 0) -> bool:
    """Whether the forward keeps nothing for the backward (which then recomputes the carries):
    under SBA_RECOMPUTE_CARRIES=1 always, otherwise when the tables would exceed workspace_budget()."""
    if os.environ.get("SBA_RECOMPUTE_CARRIES") == "1":
        return True
    return workspace_nbytes > workspace_budget()


# Error word of the bf16 matrix-core backward (set if a kernel abandoned one of its bounded internal waits,
# see sba_bwd_gave_up in include/sba_mi355x.h).  Reading it waits for the stream, so it is off by default:
# SBA_CHECK_GAVE_UP=1 or check_gave_up(True) (the test-suite's GPU tests) make every backward read it and raise.
_check_gave_up = None


def check_gave_up(on) -> None:
    global _check_gave_up
    _check_gave_up = on


def gave_up_checked() -> bool:
    if _check_gave_up is not None:
        return bool(_check_gave_up)
    return os.environ.get("SBA_CHECK_GAVE_UP") == "1"


def raise_if_gave_up(p, static_scratch_used: bool = False) -> None:
    """Reads the error word of the backward just launched with `p` (waits for its stream) and raises if set."""
    if torch.compiler.is_compiling() or torch.cuda.is_current_stream_capturing():
        return
    flag = C.c_int(0)
    check(load().sba_bwd_gave_up(C.byref(p), int(static_scratch_used), C.byref(flag)), "sba_bwd_gave_up")
    if flag.value != 0:
        raise RuntimeError("stick-breaking attention backward: a kernel abandoned a bounded internal wait "
                           "(error word set); the gradients of this call are invalid")


def matrix_core_head_dim(t: torch.Tensor) -> int:
    """Head dim that a problem runs with.  The matrix-core kernels exist for bf16, float16 and fp32 at 64
    and 128 and for the two 16-bit types at 256; any other head dim below those rides them zero-padded (zero columns add
    nothing to q.k and give zero output columns), which is far faster than the generic kernels
    (float32 above 128 has only those).  Everything keeps its head dim under SBA_FORCE_GENERIC=1
    (generic kernels)."""
    D = t.shape[-1]
    if D > MAX_HEAD_DIM or os.environ.get("SBA_FORCE_GENERIC") == "1":
        return D
    if t.dtype not in (torch.bfloat16, torch.float16, torch.float32) or D in (64, 128):
        return D
    if D > 128:
        return 256 if t.dtype != torch.float32 else D
    return 64 if D < 64 else 128


def pad_head_dim(t: torch.Tensor, D: int) -> torch.Tensor:
    return t if t.shape[-1] == D else torch.nn.functional.pad(t, (0, D - t.shape[-1]))


def cut_head_dim(t: torch.Tensor, D: int) -> torch.Tensor:
    return t if t.shape[-1] == D else t[..., :D].contiguous()


SCHEDULE_INTS = 8      # int32 per row: {first_token, doc_len, row_block, first table column of the document} of job i, then of the i-th job in key-owner order


DOC_MAJOR_GRID = 8192  # workgroups (jobs x heads) from which the schedule is document-major


def build_schedule(cu_host: torch.Tensor, n_heads: int = 0) -> torch.Tensor:
    """Host int32 cu_seqlens (leading 0) -> host int32 [n_jobs, 8] schedule for launches with
    `n_heads` heads (the job order depends on the launch size)."""
    lib = load()
    cu = cu_host.to(torch.int32).contiguous()
    n_seq = cu.numel() - 1
    ptr = C.cast(cu.data_ptr(), C.POINTER(C.c_int32))
    n = lib.sba_build_schedule(ptr, n_seq, n_heads, None, 0)
    out = torch.empty((max(n, 1), SCHEDULE_INTS), dtype=torch.int32)
    got = lib.sba_build_schedule(ptr, n_seq, n_heads, C.cast(out.data_ptr(), C.POINTER(C.c_int32)), n)
    assert got == n
    return out[:n]


def table_columns(cu_host: torch.Tensor) -> int:
    """Carry-table columns (of 128 floats, per head) of a packed batch: SbaParams.table_cols."""
    cu = cu_host.to(torch.int32).contiguous()
    return int(load().sba_table_columns(C.cast(cu.data_ptr(), C.POINTER(C.c_int32)), cu.numel() - 1))


# Pure-Python bounds on the library's sizes, usable while torch.compile traces (no ctypes call,
# no look at cu_seqlens' values there).  Always >= what the library asks for.
def dense_columns(n_seq: int, seq_len: int) -> int:
    n = (seq_len + 127) // 128
    return n_seq * n * (n + 1)


def packed_columns_bound(total_tokens: int, n_docs: int, max_len: int) -> int:
    """sum over documents of n*(n+1) <= (n_max + 1) * sum n <= (n_max + 1) * (tokens/128 + n_docs)."""
    n_max = (max_len + 127) // 128
    return (n_max + 1) * (total_tokens // 128 + n_docs)


def table_bytes(n_heads: int, columns: int) -> int:
    """One carry table."""
    return (n_heads * columns * 128 * 4 + 255) & ~255


def workspace_upper_bound(n_heads: int, columns: int) -> int:
    """What the forward hands to the backward (sba_workspace_bytes): two carry tables in bf16, one in fp32."""
    return 2 * table_bytes(n_heads, columns)


def bwd_scratch_upper_bound(n_heads: int, columns: int, tab_tokens: int, head_dim: int) -> int:
    """Four tables (the recompute mode's count) or the generic path's fp32 dk|dv accumulators."""
    dp = 32 if head_dim <= 32 else (64 if head_dim <= 64 else (128 if head_dim <= 128 else 256))
    acc = (2 * tab_tokens * n_heads * dp * 4 + 255) & ~255
    scaled_q = (tab_tokens * n_heads * 64 * 2 + 255) & ~255      # bf16 at head_dim 64: the dQ pass's scaled copy of q
    return max(4 * table_bytes(n_heads, columns) + scaled_q + 256, acc)      # + the backward's error word
