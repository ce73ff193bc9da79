"""ctypes binding of libpbs_hip.so, the C-ABI HIP library behind the three block-sparse matmuls.

This takes the place of the reference's pybind11 module ``block_sparse_native``
(native/block_sparse_native.cpp:31-34): tensors are passed as raw device pointers plus
sizes, kernels are launched on torch's current stream, and a non-zero return code raises
(the reference drops the code, block_sparse.py:565, :640).

There is no fallback: if the library is missing or the tensors are not on a GPU the calls
raise.
"""
import ctypes
import os

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "libpbs_hip.so")

DTYPE_CODES = {torch.float32: 0, torch.bfloat16: 1}
SUPPORTED_DTYPES = tuple(DTYPE_CODES)

_lib = None

_vp = ctypes.c_void_p
_i32 = ctypes.c_int
_i64 = ctypes.c_int64

_PROTOTYPES = {
    "pbs_abi_version": (ctypes.c_int, []),
    "pbs_error_string": (ctypes.c_char_p, [_i32]),
    "pbs_build_indices": (_i32, [_vp, _vp, _i32, _i32, _i32, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "pbs_blocksparse_matmul_plan_bytes": (ctypes.c_size_t, [_i32, _i32]),
    "pbs_blocksparse_matmul_plan": (_i32, [_vp, _vp, _i32, _i32, _i32, _vp, ctypes.c_size_t, _vp]),
    "pbs_blocksparse_matmul": (_i32, [_vp, _vp, _vp, _vp, _vp, _i64, _i32, _i32, _i32, _i32, _i32, _vp]),
    "pbs_blocksparse_matmul_workspace_bytes": (ctypes.c_size_t, [_i64, _i32, _i32, _i32, _i32, _i32]),
    "pbs_blocksparse_matmul_ws": (
        _i32,
        [_vp, _vp, _vp, _vp, _vp, _i64, _i32, _i32, _i32, _i32, _i32, _vp, ctypes.c_size_t, _vp],
    ),
    "pbs_blocksparse_matmul_back_workspace_bytes": (ctypes.c_size_t, [_i64, _i32, _i32, _i32, _i32]),
    "pbs_blocksparse_matmul_back": (
        _i32,
        [_vp, _vp, _vp, _vp, _vp, _i64, _i32, _i32, _i32, _i32, _vp, ctypes.c_size_t, _vp],
    ),
    "pbs_blocksparse_matmul_back_blocks_workspace_bytes": (ctypes.c_size_t, [_i64, _i32, _i32, _i32, _i32, _i32, _i32]),
    "pbs_blocksparse_matmul_back_blocks": (
        _i32,
        [_vp, _i32, _vp, _i32, _vp, _i64, _i32, _i32, _vp, _i32, _i32, _vp, ctypes.c_size_t, _vp],
    ),
    "pbs_blocksparse_matmul_back_noalloc_max_bytes": (ctypes.c_size_t, []),
    "pbs_blocksparse_matmul_back_noalloc_init": (_i32, []),
    "pbs_protocol_failures": (_i32, [ctypes.POINTER(ctypes.c_uint)]),
    "pbs_blocksparse_matmul_kernel_name": (ctypes.c_char_p, [_i64, _i32, _i32, _i32, _i32, _i32, _i32]),
    "pbs_blocksparse_matmul_back_kernel_name": (ctypes.c_char_p, [_i64, _i32, _i32, _i32, _i32]),
    "pbs_blocksparse_matmul_back_noalloc": (_i32, [_vp, _vp, _vp, _vp, _vp, _i64, _i32, _i32, _i32, _i32, _vp]),
}

EXPORTED_SYMBOLS = tuple(_PROTOTYPES)


class NativeLibraryMissing(ImportError):
    pass


def load():
    """Load libpbs_hip.so (once) and declare the prototypes of its entry points."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise NativeLibraryMissing(
            f"{LIB_PATH} is not built. Run `python -m pytorch_block_sparse_amd.csrc.build` "
            f"(or `make -C {os.path.dirname(LIB_PATH)}`); there is no non-HIP path for the matmuls."
        )
    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in _PROTOTYPES.items():
        fn = getattr(lib, name)
        fn.restype = restype
        fn.argtypes = argtypes
    _lib = lib
    return lib


def error_string(code):
    return load().pbs_error_string(int(code)).decode()


def _check(code, what):
    if code != 0:
        raise RuntimeError(f"{what} failed with code {code}: {error_string(code)}")


_failures_seen = {}


def check_protocol(what):
    """With PBS_DEBUG set: raise if a bounded wait of a barrier-free kernel has run out since the last check
    (the kernel marks the affected results NaN and counts the event; without this the call reports success)."""
    if not os.environ.get("PBS_DEBUG"):
        return
    count = ctypes.c_uint(0)
    _check(load().pbs_protocol_failures(ctypes.byref(count)), "pbs_protocol_failures")
    dev = torch.cuda.current_device()
    before = _failures_seen.get(dev, 0)
    _failures_seen[dev] = count.value
    if count.value != before:
        raise RuntimeError(
            f"{what}: {count.value - before} wait(s) of the kernel's progress protocol ran into their bound; "
            "the results of the affected tiles are NaN"
        )


def matmul_kernel_name(tokens, n, k, nnz, transpose, dtype, with_workspace=True):
    """Which kernel pbs_blocksparse_matmul_ws runs for these sizes (for benchmark labels)."""
    return load().pbs_blocksparse_matmul_kernel_name(
        tokens, n, k, nnz, 1 if transpose else 0, DTYPE_CODES[dtype], 1 if with_workspace else 0).decode()


def matmul_back_kernel_name(tokens, out_features, in_features, nnz, dtype):
    return load().pbs_blocksparse_matmul_back_kernel_name(tokens, out_features, in_features, nnz, DTYPE_CODES[dtype]).decode()


def _stream(index=None):
    """The current stream of device `index` (default: the current device) as a hipStream_t."""
    if index is None:
        index = torch.cuda.current_device()
    raw = getattr(torch._C, "_cuda_getCurrentRawStream", None)   # the handle without a Stream object around it
    return ctypes.c_void_p(raw(index) if raw is not None else torch.cuda.current_stream(index).cuda_stream)


class _on_device:
    """`with torch.cuda.device(d)` only when d is not the current device already (the context manager costs
    several microseconds, which is most of a small product's host time)."""

    def __init__(self, device):
        self.index = device.index if device.index is not None else torch.cuda.current_device()
        self.ctx = None if self.index == torch.cuda.current_device() else torch.cuda.device(self.index)

    def __enter__(self):
        if self.ctx is not None:
            self.ctx.__enter__()
        return self.index

    def __exit__(self, *exc):
        if self.ctx is not None:
            self.ctx.__exit__(*exc)
        return False


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None and t.numel() > 0 else ctypes.c_void_p(0)


def _require_cuda(*tensors):
    for t in tensors:
        if t is not None and not t.is_cuda:
            raise RuntimeError(
                "pytorch_block_sparse_amd: the block-sparse matmuls run only on a GPU through libpbs_hip.so; "
                f"got a tensor on {t.device}"
            )


def build_indices(block_mask, block_ptr, nnz):
    """Device build of (blocks, cols_a, row_start_ends_a, rows_b, col_start_ends_b) for a CUDA mask."""
    lib = load()
    _require_cuda(block_mask, block_ptr)
    X, Y = block_mask.shape
    dev = block_mask.device
    mask_u8 = block_mask.contiguous().view(torch.uint8) if block_mask.dtype == torch.bool else (
        block_mask != 0
    ).contiguous().view(torch.uint8)
    if block_ptr is not None:
        block_ptr = block_ptr.to(device=dev, dtype=torch.int64).contiguous()
        if block_ptr.numel() != nnz:
            raise RuntimeError(f"block_ptr has {block_ptr.numel()} entries for {nnz} blocks")
    i32 = dict(dtype=torch.int32, device=dev)
    cols_a = torch.empty((nnz, 2), **i32)
    rows_b = torch.empty((nnz, 2), **i32)
    blocks = torch.empty((2 * nnz,), **i32)
    row_ptr = torch.empty((X + 1,), **i32)
    col_ptr = torch.empty((Y + 1,), **i32)
    status = torch.zeros((2,), **i32)
    with torch.cuda.device(dev):
        code = lib.pbs_build_indices(
            _ptr(mask_u8), _ptr(block_ptr), X, Y, nnz, _ptr(cols_a), _ptr(row_ptr), _ptr(rows_b), _ptr(col_ptr),
            _ptr(blocks), _ptr(status), _stream(),
        )
    _check(code, "pbs_build_indices")
    counted, err = status.tolist()
    if err == 1:
        raise RuntimeError(f"block mask holds {counted} blocks but {nnz} were expected")
    if err == 2:
        raise RuntimeError("block_ptr holds an entry outside [0, n_blocks)")
    return blocks, cols_a, row_ptr, rows_b, col_ptr


def blocksparse_matmul_plan(ptr, indices, n, k):
    """Schedule buffer of the dense x block-sparse product for (ptr, indices); depends on the pattern only."""
    lib = load()
    _require_cuda(ptr, indices)
    nbytes = lib.pbs_blocksparse_matmul_plan_bytes(n, k)
    plan = torch.empty((nbytes // 4,), dtype=torch.int32, device=ptr.device)
    with torch.cuda.device(ptr.device):
        code = lib.pbs_blocksparse_matmul_plan(
            _ptr(ptr), _ptr(indices), n, k, indices.shape[0], _ptr(plan), nbytes, _stream()
        )
    _check(code, "pbs_blocksparse_matmul_plan")
    return plan


def blocksparse_matmul(dense_a, data, plan, n, k, nnz, transpose, bias=None, out=None):
    """out[tokens, n] = dense_a[tokens, k] . W^T (transpose) or . W (not transpose)."""
    lib = _lib or load()
    dtype = dense_a.dtype
    if not (dense_a.is_cuda and data.is_cuda and plan.is_cuda and (bias is None or bias.is_cuda)):
        _require_cuda(dense_a, data, plan, bias)
    code_dtype = DTYPE_CODES.get(dtype)
    if code_dtype is None:
        raise RuntimeError(f"unsupported dtype {dtype}; supported: {SUPPORTED_DTYPES}")
    if data.dtype != dtype:
        raise RuntimeError(f"dense operand is {dtype} but the block data is {data.dtype}")
    if bias is not None and bias.dtype != dtype:
        raise RuntimeError(f"bias is {bias.dtype}, expected {dtype}")
    tokens = dense_a.shape[0]
    if out is None:
        out = torch.empty((tokens, n), dtype=dtype, device=dense_a.device)
    tr = 1 if transpose else 0
    # the transposed copy of the blocks that the forward bf16 kernel for dense patterns works from (made by the library)
    ws, ws_bytes = None, 0
    if tr and code_dtype == 1:
        ws_bytes = lib.pbs_blocksparse_matmul_workspace_bytes(tokens, n, k, nnz, tr, code_dtype)
        if ws_bytes:
            ws = torch.empty((ws_bytes,), dtype=torch.uint8, device=dense_a.device)
    with _on_device(dense_a.device) as index:
        code = lib.pbs_blocksparse_matmul_ws(
            _ptr(dense_a), _ptr(data), _ptr(plan), _ptr(bias), _ptr(out), tokens, n, k, nnz, tr, code_dtype,
            _ptr(ws), ws_bytes, _stream(index),
        )
    if code != 0:
        _check(code, "pbs_blocksparse_matmul_ws")
    check_protocol("pbs_blocksparse_matmul_ws")
    return out


def blocksparse_matmul_back(dense_a, dense_b, row_start_ends_a, cols_a, out):
    """out (packed [nnz*32, 32]) = blocks of dense_a^T . dense_b on the pattern's support."""
    lib = load()
    _require_cuda(dense_a, dense_b, row_start_ends_a, cols_a, out)
    if dense_a.dtype not in DTYPE_CODES:
        raise RuntimeError(f"unsupported dtype {dense_a.dtype}; supported: {SUPPORTED_DTYPES}")
    if dense_b.dtype != dense_a.dtype or out.dtype != dense_a.dtype:
        raise RuntimeError("operands and result must share one dtype")
    tokens, out_features = dense_a.shape
    in_features = dense_b.shape[1]
    nnz = cols_a.shape[0]
    code_dtype = DTYPE_CODES[dense_a.dtype]
    ws_bytes = lib.pbs_blocksparse_matmul_back_workspace_bytes(tokens, out_features, in_features, nnz, code_dtype)
    ws = torch.empty((ws_bytes,), dtype=torch.uint8, device=dense_a.device) if ws_bytes else None
    with _on_device(dense_a.device) as index:
        code = lib.pbs_blocksparse_matmul_back(
            _ptr(dense_a), _ptr(dense_b), _ptr(row_start_ends_a), _ptr(cols_a), _ptr(out), tokens, out_features,
            in_features, nnz, code_dtype, _ptr(ws), ws_bytes, _stream(index),
        )
    _check(code, "pbs_blocksparse_matmul_back")
    return out
