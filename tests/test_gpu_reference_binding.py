"""The drop-in boundary used the way a maintainer of the reference would: ``include/pbs_hip_ctypes.py``
(plain ctypes + torch tensors) against the oracle, without importing the ``pytorch_block_sparse_amd``
package.  Index arrays come from the oracle's restatement of ``build_indices`` (they are what the
reference's own BlockSparseMatrix holds: block_sparse.py:125-153), including the state after a
``block_replace`` (:167-219), where the cached plan has to be rebuilt.
"""
import importlib.util
import os
import sys

import numpy as np
import pytest
import torch

from oracle import block_sparse_oracle as O
from tests.helpers import assert_close

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB = os.path.join(ROOT, "pytorch_block_sparse_amd", "csrc", "libpbs_hip.so")


def _binding():
    spec = importlib.util.spec_from_file_location("pbs_hip_ctypes", os.path.join(ROOT, "include", "pbs_hip_ctypes.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def _device_indices(idx, dev):
    return {k: torch.from_numpy(np.ascontiguousarray(v)).to(dev) for k, v in idx.items()}


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_reference_side_binding_against_oracle(cuda, dtype):
    if not os.path.exists(LIB):
        pytest.fail("libpbs_hip.so is not built")
    loaded_before = "pytorch_block_sparse_amd" in sys.modules
    binding = _binding()
    lib = binding.PbsHip(LIB)
    assert lib.lib.pbs_abi_version() >= 2
    if not loaded_before:
        assert "pytorch_block_sparse_amd" not in sys.modules   # the binding stands on its own

    out_f, in_f, tokens = 256, 192, 333
    X, Y = out_f // 32, in_f // 32
    rng = np.random.RandomState(7)
    mask = rng.rand(X, Y) < 0.4
    mask[2, :] = False           # an empty block row
    nnz = int(mask.sum())
    idx = O.build_indices(mask)
    g = torch.Generator().manual_seed(11)
    data = (torch.randn(nnz * 32, 32, generator=g) / 8).to(dtype)
    x = torch.randn(tokens, in_f, generator=g).to(dtype)
    dy = torch.randn(tokens, out_f, generator=g).to(dtype)
    bias = torch.randn(out_f, generator=g).to(dtype)
    f64 = lambda t: t.double().numpy()

    def check(idx, what):
        coo = O.build_coo_block_index(idx["row_start_ends_a"], idx["cols_a"])
        y_ref, dx_ref, dw_ref = O.linear_fwd_bwd(f64(x), f64(dy), f64(data), coo, (out_f, in_f))
        d = _device_indices(idx, cuda)
        n = d["cols_a"].shape[0]
        plan_fwd = lib.make_plan(d["row_start_ends_a"], d["cols_a"], out_f, in_f)
        plan_dx = lib.make_plan(d["col_start_ends_b"], d["rows_b"], in_f, out_f)
        dd, xd, dyd = data.to(cuda), x.to(cuda), dy.to(cuda)
        y = lib.matmul(xd, dd, plan_fwd, out_f, in_f, n, True, bias=bias.to(cuda))
        assert_close(y, y_ref + f64(bias), dtype, what + " fwd")
        assert_close(lib.matmul(dyd, dd, plan_dx, in_f, out_f, n, False), dx_ref, dtype, what + " dx")
        dw = lib.matmul_back(dyd, xd, d["row_start_ends_a"], d["cols_a"], torch.empty_like(dd))
        assert_close(dw, dw_ref, dtype, what + " dw")
        return plan_fwd, y

    plan_old, y_old = check(idx, "initial pattern")

    # block_replace: move two data blocks to free positions; block_ptr keeps every other block where it is
    coo = O.build_coo_block_index(idx["row_start_ends_a"], idx["cols_a"])   # [2, nnz] (row, col) by data block
    free = np.argwhere(~mask)
    pos = coo.copy().astype(np.int64)
    pos[:, 0] = free[0]
    pos[:, 5] = free[-1]
    mask2 = np.zeros_like(mask)
    mask2[pos[0], pos[1]] = True
    block_ptr = np.argsort(pos[0] * Y + pos[1])
    idx2 = O.build_indices(mask2, block_ptr)
    plan_new, y_new = check(idx2, "after block_replace")
    # the plan belongs to the pattern: the old one gives the old pattern's product, not the new one's
    assert not torch.equal(plan_old, plan_new)
    assert not torch.allclose(y_old.float(), y_new.float())


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_reference_signature_of_the_sparse_output_product(cuda, dtype):
    """pbs_blocksparse_matmul_back_blocks takes what the reference's blocksparse_matmul_back_cutlass takes
    (native/block_sparse_native.cpp:18-29): each dense operand in either memory order with its flag, and the `blocks`
    list instead of the CSR pair.  All four flag combinations (the four kernels of
    native/block_sparse_cutlass_kernel_back.cu:145-157) against the oracle, on a pattern whose data blocks are not in
    row-major order (the state after a block_replace) and with a token count that splits the token range."""
    binding = _binding()
    lib = binding.PbsHip(LIB)
    out_f, in_f, tokens = 384, 320, 4099
    X, Y = out_f // 32, in_f // 32
    rng = np.random.RandomState(3)
    mask = rng.rand(X, Y) < 0.35
    mask[5, :] = False
    nnz = int(mask.sum())
    block_ptr = rng.permutation(nnz)            # data block of the i-th nonzero in row-major order
    idx = O.build_indices(mask, block_ptr)
    coo = O.build_coo_block_index(idx["row_start_ends_a"], idx["cols_a"])
    g = torch.Generator().manual_seed(5)
    x = torch.randn(tokens, in_f, generator=g).to(dtype)
    dy = torch.randn(tokens, out_f, generator=g).to(dtype)
    data = torch.zeros(nnz * 32, 32).to(dtype)
    _, _, dw_ref = O.linear_fwd_bwd(x.double().numpy(), dy.double().numpy(), data.double().numpy(), coo, (out_f, in_f))
    blocks = torch.from_numpy(np.ascontiguousarray(idx["blocks"])).to(cuda)
    xd, dyd = x.to(cuda), dy.to(cuda)
    xt, dyt = xd.t().contiguous(), dyd.t().contiguous()    # [features, tokens]: "the transpose is contiguous"
    results = []
    for a_rm in (True, False):
        for b_rm in (True, False):
            print(f"memory orders a_row_major={a_rm} b_row_major={b_rm} {dtype}", flush=True)
            out = torch.full((nnz * 32, 32), float("nan"), dtype=dtype, device=cuda)
            lib.matmul_back_blocks(dyd if a_rm else dyt, a_rm, xd if b_rm else xt, b_rm, blocks, out)
            assert_close(out, dw_ref, dtype, f"a_row_major={a_rm} b_row_major={b_rm}")
            results.append(out)
    for r in results[1:]:
        assert torch.equal(r, results[0])       # the memory order of an operand does not change a bit of the result
    # and it is the result of the entry point that takes the CSR pair
    d = _device_indices(idx, cuda)
    ref = lib.matmul_back(dyd, xd, d["row_start_ends_a"], d["cols_a"], torch.empty_like(results[0]))
    assert torch.equal(ref, results[0])
