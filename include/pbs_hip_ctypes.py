"""ctypes binding of libpbs_hip.so as a maintainer of the reference would add it.

It imports nothing from this repository: plain ``ctypes.CDLL`` plus torch tensors, the way the
reference's ``BlockSparseMatrixBase`` would call the library instead of its pybind11 module
``block_sparse_native`` (reference native/block_sparse_native.cpp:6-29; call sites
block_sparse.py:562-574 for the dense x sparse product and :637-652 for the sparse-output one).
Prototypes are those of ``pbs_hip.h`` next to this file.

    lib = PbsHip("/path/to/libpbs_hip.so")
    plan = lib.make_plan(row_start_ends_a, cols_a, n=out_features, k=in_features)        # once per pattern
    y = lib.matmul(x, data, plan, n=out_features, k=in_features, nnz=nnz, transpose=True)
    dw = lib.matmul_back(grad_out, x, row_start_ends_a, cols_a, torch.empty_like(data))

``nnz`` is the number of stored blocks: ``cols_a.shape[0]`` (equivalently ``data.shape[0] // 32``), not
``blocks_count()``, which in the reference is the (X, Y) size of the block grid (block_sparse.py:78-83).
"""
import ctypes

import torch

_p, _i, _l, _z = ctypes.c_void_p, ctypes.c_int, ctypes.c_int64, ctypes.c_size_t

PROTOTYPES = {
    "pbs_abi_version": (_i, []),
    "pbs_error_string": (ctypes.c_char_p, [_i]),
    "pbs_build_indices": (_i, [_p, _p, _i, _i, _i, _p, _p, _p, _p, _p, _p, _p]),
    "pbs_blocksparse_matmul_plan_bytes": (_z, [_i, _i]),
    "pbs_blocksparse_matmul_plan": (_i, [_p, _p, _i, _i, _i, _p, _z, _p]),
    "pbs_blocksparse_matmul": (_i, [_p, _p, _p, _p, _p, _l, _i, _i, _i, _i, _i, _p]),
    "pbs_blocksparse_matmul_workspace_bytes": (_z, [_l, _i, _i, _i, _i, _i]),
    "pbs_blocksparse_matmul_ws": (_i, [_p, _p, _p, _p, _p, _l, _i, _i, _i, _i, _i, _p, _z, _p]),
    "pbs_blocksparse_matmul_back_workspace_bytes": (_z, [_l, _i, _i, _i, _i]),
    "pbs_blocksparse_matmul_back": (_i, [_p, _p, _p, _p, _p, _l, _i, _i, _i, _i, _p, _z, _p]),
    "pbs_blocksparse_matmul_back_blocks_workspace_bytes": (_z, [_l, _i, _i, _i, _i, _i, _i]),
    "pbs_blocksparse_matmul_back_blocks": (_i, [_p, _i, _p, _i, _p, _l, _i, _i, _p, _i, _i, _p, _z, _p]),
}

DTYPES = {torch.float32: 0, torch.bfloat16: 1}


class PbsHip:
    def __init__(self, path):
        self.lib = ctypes.CDLL(path)
        for name, (restype, argtypes) in PROTOTYPES.items():
            fn = getattr(self.lib, name)
            fn.restype, fn.argtypes = restype, argtypes

    def _check(self, rc, what):
        if rc != 0:
            raise RuntimeError("%s: %s" % (what, self.lib.pbs_error_string(rc).decode()))

    @staticmethod
    def _stream():
        return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)

    def make_plan(self, ptr, indices, n, k):
        """Schedule of one pattern and direction: (row_start_ends_a, cols_a, out, in) for ``a @ W^T``,
        (col_start_ends_b, rows_b, in, out) for ``a @ W``.  Build it again whenever the index arrays change
        (the reference's rebuild(), block_sparse.py:33-76, is the place to drop a cached plan)."""
        nnz = indices.shape[0]
        nbytes = self.lib.pbs_blocksparse_matmul_plan_bytes(n, k)
        plan = torch.empty(max(nbytes, 16) // 4, dtype=torch.int32, device=ptr.device)
        with torch.cuda.device(ptr.device):
            self._check(self.lib.pbs_blocksparse_matmul_plan(ptr.data_ptr(), indices.data_ptr(), n, k, nnz,
                                                             plan.data_ptr(), nbytes, self._stream()), "plan")
        return plan

    def matmul(self, dense_a, data, plan, n, k, nnz, transpose, bias=None):
        """dense_a [tokens, k] row-major contiguous -> [tokens, n]; replaces the reference's call at block_sparse.py:562-574."""
        tokens, tr, dt = dense_a.shape[0], int(bool(transpose)), DTYPES[dense_a.dtype]
        out = torch.empty(tokens, n, dtype=dense_a.dtype, device=dense_a.device)
        # room for the transposed copy of the blocks that the reference makes itself at block_sparse.py:541-544
        nws = self.lib.pbs_blocksparse_matmul_workspace_bytes(tokens, n, k, nnz, tr, dt)
        ws = torch.empty(max(nws, 16), dtype=torch.uint8, device=dense_a.device)
        with torch.cuda.device(dense_a.device):
            self._check(self.lib.pbs_blocksparse_matmul_ws(
                dense_a.data_ptr(), data.data_ptr(), plan.data_ptr(), None if bias is None else bias.data_ptr(),
                out.data_ptr(), tokens, n, k, nnz, tr, dt, ws.data_ptr(), nws, self._stream()), "matmul")
        return out

    def matmul_back(self, grad_out, inp, row_start_ends_a, cols_a, data_out):
        """Packed blocks of grad_out^T @ inp on the pattern; replaces the reference's call at block_sparse.py:637-652."""
        tokens, out_f, in_f = grad_out.shape[0], grad_out.shape[1], inp.shape[1]
        nnz, dt = cols_a.shape[0], DTYPES[grad_out.dtype]
        nws = self.lib.pbs_blocksparse_matmul_back_workspace_bytes(tokens, out_f, in_f, nnz, dt)
        ws = torch.empty(max(nws, 16), dtype=torch.uint8, device=inp.device)
        with torch.cuda.device(inp.device):
            self._check(self.lib.pbs_blocksparse_matmul_back(
                grad_out.data_ptr(), inp.data_ptr(), row_start_ends_a.data_ptr(), cols_a.data_ptr(),
                data_out.data_ptr(), tokens, out_f, in_f, nnz, dt, ws.data_ptr(), nws, self._stream()), "matmul_back")
        return data_out

    def matmul_back_blocks(self, dense_a, a_row_major, dense_b, b_row_major, blocks, data_out):
        """The reference's own call (block_sparse.py:637-652) with its arguments: ``dense_a`` is [tokens, out] when
        ``a_row_major`` else [out, tokens] (likewise ``dense_b`` with in_features), ``blocks`` is the module's buffer."""
        tokens = dense_a.shape[0] if a_row_major else dense_a.shape[1]
        out_f = dense_a.shape[1] if a_row_major else dense_a.shape[0]
        in_f = dense_b.shape[1] if b_row_major else dense_b.shape[0]
        nnz, dt = blocks.shape[0] // 2, DTYPES[dense_a.dtype]
        nws = self.lib.pbs_blocksparse_matmul_back_blocks_workspace_bytes(tokens, out_f, in_f, nnz, dt, int(a_row_major),
                                                                          int(b_row_major))
        ws = torch.empty(max(nws, 16), dtype=torch.uint8, device=dense_a.device)
        with torch.cuda.device(dense_a.device):
            self._check(self.lib.pbs_blocksparse_matmul_back_blocks(
                dense_a.data_ptr(), int(a_row_major), dense_b.data_ptr(), int(b_row_major), data_out.data_ptr(), tokens,
                out_f, in_f, blocks.data_ptr(), nnz, dt, ws.data_ptr(), nws, self._stream()), "matmul_back_blocks")
        return data_out
