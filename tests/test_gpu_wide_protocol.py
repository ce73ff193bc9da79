"""The progress protocol of the two barrier-free bf16 kernels against its conservative variant.

In the product build a copying wave publishes "the operands of step t have landed" with one more 4-byte
LDS-DMA load issued behind the step's operand loads, which relies on one wave's LDS-DMA loads landing in
issue order.  libpbs_hip_check.so is the same library compiled with -DPBS_DDS16_PUBLISH_AFTER_WAIT
-DPBS_DDSC_PUBLISH_AFTER_WAIT: there
the copy wave waits for all its loads (s_waitcnt vmcnt(0)) and then writes the number itself, which relies
on nothing.  If the ordering assumption failed, compute waves of the product build would multiply operands
that had not arrived yet and the two libraries would disagree; they must agree bit for bit.
"""
import importlib.util
import os

import numpy as np
import pytest
import torch

from pytorch_block_sparse_amd import BlockSparseMatrix, native, workloads

pytestmark = pytest.mark.gpu

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
CHECK_LIB = os.path.join(os.path.dirname(native.LIB_PATH), "libpbs_hip_check.so")


def _binding(path):
    spec = importlib.util.spec_from_file_location("pbs_hip_ctypes", os.path.join(ROOT, "include", "pbs_hip_ctypes.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod.PbsHip(path)


@pytest.mark.parametrize("kernel", ["wide", "column"])
@pytest.mark.parametrize("case", ["c4", "ragged"])
def test_product_and_conservative_protocol_agree_bitwise(cuda, monkeypatch, case, kernel):
    # which of the two kernels serves the calls below (both libraries read the variable at every call)
    monkeypatch.setenv("PBS_COLUMN_KERNEL", "1" if kernel == "column" else "0")
    assert os.path.exists(CHECK_LIB), "libpbs_hip_check.so is not built (python -m pytorch_block_sparse_amd.csrc.build)"
    if case == "c4":
        w = workloads.WORKLOADS["c4_4096x4096_d0.25_bf16"]
        blocks, data, x, dy = workloads.make_inputs(w)
        m = BlockSparseMatrix.zeros((w.out_features, w.in_features), blocks=blocks, device="cpu", dtype=w.dtype)
        with torch.no_grad():
            m.data.copy_(data)
        m = m.to(cuda)
    else:   # token tail, a last column group with four columns, several tiles per workgroup, both contractions a multiple of 128
        np.random.seed(5)
        torch.manual_seed(5)
        m = BlockSparseMatrix.randn((1152, 512), 36 * 16 // 3, device=cuda, dtype=torch.bfloat16)
        x = torch.randn(33000 + 7, 512).to(torch.bfloat16)
        dy = torch.randn(33000 + 7, 1152).to(torch.bfloat16)
    xd, dyd = x.to(cuda), dy.to(cuda)
    product, check = _binding(native.LIB_PATH), _binding(CHECK_LIB)
    out_f, in_f = m.shape
    nnz = m.cols_a.shape[0]
    for transpose, a in ((True, xd), (False, dyd)):
        if transpose:
            ptr, idx, n, k = m.row_start_ends_a, m.cols_a, out_f, in_f
        else:
            ptr, idx, n, k = m.col_start_ends_b, m.rows_b, in_f, out_f
        results = []
        for lib in (product, check):
            plan = lib.make_plan(ptr, idx, n, k)
            for rep in range(3):   # the protocol's timing differs from run to run; the values must not
                results.append(lib.matmul(a, m.data, plan, n, k, nnz, transpose))
            torch.cuda.synchronize()
        for r in results[1:]:
            assert torch.equal(r, results[0]), f"{case}: transpose={transpose}: the two protocols disagree"
        assert torch.isfinite(results[0].float()).all()


def test_no_wait_runs_into_its_bound(cuda, monkeypatch):
    """With PBS_DEBUG set the Python layer reads the library's count of protocol waits that ran out after every
    product and raises if it has grown: both barrier-free kernels, both directions, on the benchmark layer."""
    import ctypes

    monkeypatch.setenv("PBS_DEBUG", "1")
    w = workloads.WORKLOADS["c4_4096x4096_d0.25_bf16"]
    blocks, data, x, dy = workloads.make_inputs(w, tokens=8192)
    m = BlockSparseMatrix.zeros((w.out_features, w.in_features), blocks=blocks, device="cpu", dtype=w.dtype)
    with torch.no_grad():
        m.data.copy_(data)
    m = m.to(cuda)
    xd, dyd = x.to(cuda), dy.to(cuda)
    for kernel in ("0", "1"):
        monkeypatch.setenv("PBS_COLUMN_KERNEL", kernel)
        for _ in range(3):
            m.reverse_matmul(xd, True)     # raises if a wait ran out
            m.reverse_matmul(dyd, False)
    count = ctypes.c_uint(123)
    assert native.load().pbs_protocol_failures(ctypes.byref(count)) == 0
    assert count.value == 0
