"""The entry point that allocates nothing (pbs_blocksparse_matmul_back_noalloc) against the workspace entry
point it is a variant of: same kernels, so the packed weight gradients must be bit-identical.  Two calls in
a row share the library's built-in scratch array; the second is smaller than the first.
"""
import ctypes

import numpy as np
import pytest
import torch

from oracle import block_sparse_oracle as O
from pytorch_block_sparse_amd import native

pytestmark = pytest.mark.gpu

ERR_SCRATCH = -7


def _problem(out_f, in_f, tokens, density, dtype, seed, dev):
    X, Y = out_f // 32, in_f // 32
    rng = np.random.RandomState(seed)
    mask = rng.rand(X, Y) < density
    mask[0, 0] = True
    idx = O.build_indices(mask)
    g = torch.Generator().manual_seed(seed)
    dy = torch.randn(tokens, out_f, generator=g).to(dtype).to(dev)
    x = torch.randn(tokens, in_f, generator=g).to(dtype).to(dev)
    ptr = torch.from_numpy(idx["row_start_ends_a"]).to(dev)
    cols = torch.from_numpy(idx["cols_a"]).to(dev)
    return dy, x, ptr, cols


def _both(lib, dy, x, ptr, cols, dtype):
    tokens, out_f = dy.shape
    in_f, nnz, code = x.shape[1], cols.shape[0], native.DTYPE_CODES[dtype]
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    need = lib.pbs_blocksparse_matmul_back_workspace_bytes(tokens, out_f, in_f, nnz, code)
    ws = torch.empty(max(need, 16), dtype=torch.uint8, device=dy.device)
    ref = torch.full((nnz * 32, 32), 7.0, dtype=dtype, device=dy.device)
    got = torch.full((nnz * 32, 32), -7.0, dtype=dtype, device=dy.device)
    rc = lib.pbs_blocksparse_matmul_back(p(dy), p(x), p(ptr), p(cols), p(ref), tokens, out_f, in_f, nnz, code, p(ws), need, stream)
    assert rc == 0, native.error_string(rc)
    rc = lib.pbs_blocksparse_matmul_back_noalloc(p(dy), p(x), p(ptr), p(cols), p(got), tokens, out_f, in_f, nnz, code, stream)
    assert rc == 0, native.error_string(rc)
    torch.cuda.synchronize()
    return need, ref, got


def test_no_alloc_entry_point_under_graph_capture(cuda):
    """The caller this entry point is for: a stream under HIP graph capture.  The address of the scratch array is
    looked up by pbs_blocksparse_matmul_back_noalloc_init() before the capture begins (this test comes first in the
    file, so in a fresh process that lookup is the library's first); the captured call, whose partial sums go
    through the array, is replayed several times with eager calls that use the same array in between, and every
    replay must give the eager result of the workspace entry point."""
    lib = native.load()
    assert lib.pbs_blocksparse_matmul_back_noalloc_init() == 0
    dtype = torch.bfloat16
    dy, x, ptr, cols = _problem(1024, 1024, 4096, 0.5, dtype, 1, cuda)
    need, ref, got = _both(lib, dy, x, ptr, cols, dtype)   # eager: also raises the kernel's LDS limit before the capture
    assert need > 0 and torch.equal(ref, got)
    tokens, out_f = dy.shape
    in_f, nnz, code = x.shape[1], cols.shape[0], native.DTYPE_CODES[dtype]
    p = lambda t: ctypes.c_void_p(t.data_ptr())
    out = torch.full((nnz * 32, 32), -3.0, dtype=dtype, device=cuda)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        rc = lib.pbs_blocksparse_matmul_back_noalloc(p(dy), p(x), p(ptr), p(cols), p(out), tokens, out_f, in_f, nnz, code, stream)
    assert rc == 0, native.error_string(rc)
    dy2, x2, ptr2, cols2 = _problem(512, 768, 1000, 0.3, dtype, 2, cuda)
    for replay in range(3):
        out.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(out, ref), f"replay {replay}"
        _, ref2, got2 = _both(lib, dy2, x2, ptr2, cols2, dtype)   # eager work on the same scratch array in between
        assert torch.equal(ref2, got2)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_no_alloc_entry_point_matches_workspace_entry_point(cuda, dtype):
    lib = native.load()
    limit = lib.pbs_blocksparse_matmul_back_noalloc_max_bytes()
    assert limit == 64 << 20
    # first call: the token range is split, so the scratch array carries partial sums
    dy, x, ptr, cols = _problem(1024, 1024, 4096, 0.5, dtype, 1, cuda)
    print("first call", dtype, tuple(dy.shape), tuple(x.shape), flush=True)
    need, ref, got = _both(lib, dy, x, ptr, cols, dtype)
    assert 0 < need <= limit
    assert torch.equal(ref, got)
    # second call, smaller, right behind the first: the array still holds the first call's partial sums
    dy2, x2, ptr2, cols2 = _problem(512, 768, 1000, 0.3, dtype, 2, cuda)
    print("second call", dtype, tuple(dy2.shape), tuple(x2.shape), flush=True)
    need2, ref2, got2 = _both(lib, dy2, x2, ptr2, cols2, dtype)
    assert 0 < need2 < need
    assert torch.equal(ref2, got2)
    # and the first problem again gives the first result again
    _, _, again = _both(lib, dy, x, ptr, cols, dtype)
    assert torch.equal(again, ref)


def test_no_alloc_entry_point_rejects_what_does_not_fit(cuda):
    lib = native.load()
    limit = lib.pbs_blocksparse_matmul_back_noalloc_max_bytes()
    code = native.DTYPE_CODES[torch.bfloat16]
    tokens, out_f, in_f, nnz = 16384, 4096, 4096, 8192   # density 0.5: twice the blocks of the benchmark layer
    assert lib.pbs_blocksparse_matmul_back_workspace_bytes(tokens, out_f, in_f, nnz, code) > limit
    p = ctypes.c_void_p(0x1000)   # never dereferenced: the size check comes first
    rc = lib.pbs_blocksparse_matmul_back_noalloc(p, p, p, p, p, tokens, out_f, in_f, nnz, code, None)
    assert rc == ERR_SCRATCH
    assert "scratch" in native.error_string(rc)
    # the benchmark's weight-gradient problem needs exactly the array
    assert lib.pbs_blocksparse_matmul_back_workspace_bytes(16384, 4096, 4096, 4096, code) == limit
