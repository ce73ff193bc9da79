"""The bf16 weight-gradient kernel without barriers in the token loop (PBS_DW_KERNEL=1) against the oracle and against
the kernel with a barrier per chunk.

Both kernels cut the work the same way (rectangles, token slices, blocks per wave) and add a block's products in token
order, 16 tokens per matrix instruction, so their results must be the same to the last bit; the oracle check is
the parity bar of every other test.  Shapes: ragged token counts (a last chunk of one token, fewer tokens than one
chunk), density 0.5 (two passes over the tokens), a Zipf pattern (row bands regrouped, rectangles of very different
block counts, waves without blocks), empty block rows, the benchmark layer.
"""
import numpy as np
import pytest
import torch

from oracle import block_sparse_oracle as O
from pytorch_block_sparse_amd import BlockSparseMatrix, workloads
from tests.helpers import assert_close, to64

pytestmark = pytest.mark.gpu
BF16 = torch.bfloat16


def _both_kernels(m, dy, x, monkeypatch):
    monkeypatch.setenv("PBS_DW_KERNEL", "0")
    ref = m.matmul_with_output_sparse_support(dy, x)
    monkeypatch.setenv("PBS_DW_KERNEL", "1")
    got = m.matmul_with_output_sparse_support(dy, x)
    again = m.matmul_with_output_sparse_support(dy, x)
    torch.cuda.synchronize()
    monkeypatch.delenv("PBS_DW_KERNEL", raising=False)
    return ref, got, again


@pytest.mark.parametrize("in_f,out_f,tokens,density", [
    (128, 96, 1, 0.5),
    (256, 512, 77, 0.3),
    (512, 512, 1000 + 17, 0.5),
    (1024, 1024, 4096 + 1, 0.5),       # rectangles of about 128 blocks: two passes; a last chunk of one token
    (768, 3072, 2048, 0.25),
    (2048, 544, 3000, 0.05),           # sparse: rectangles with a few blocks, waves without any
])
def test_shapes(cuda, monkeypatch, in_f, out_f, tokens, density):
    print(f"dw {in_f}->{out_f} tokens={tokens} d={density}", flush=True)
    np.random.seed(3)
    torch.manual_seed(3)
    n_blocks = max(1, int(density * (in_f // 32) * (out_f // 32)))
    m = BlockSparseMatrix.randn((out_f, in_f), n_blocks, device="cpu", dtype=BF16).to(cuda)
    g = torch.Generator().manual_seed(5)
    x = torch.randn((tokens, in_f), generator=g).to(BF16)
    dy = torch.randn((tokens, out_f), generator=g).to(BF16)
    coo = m.build_coo_block_index().cpu().numpy()
    _, _, dw_ref = O.linear_fwd_bwd(to64(x), to64(dy), to64(m.data), coo, tuple(m.shape))
    ref, got, again = _both_kernels(m, dy.to(cuda), x.to(cuda), monkeypatch)
    assert_close(got, dw_ref, BF16, "barrier-free dw")
    assert torch.equal(got, again)
    assert torch.equal(got, ref), "the two weight-gradient kernels differ"


def test_zipf_pattern_and_empty_rows(cuda, monkeypatch):
    w = workloads.WORKLOADS["c3_3072x768_d0.25_zipf_fp32"]
    blocks = [b for b in workloads.make_pattern(w) if b[0] not in (3, 4)]    # two empty block rows on top
    np.random.seed(1)
    torch.manual_seed(1)
    m = BlockSparseMatrix.randn((w.out_features, w.in_features), None, blocks=blocks, device="cpu", dtype=BF16).to(cuda)
    g = torch.Generator().manual_seed(9)
    tokens = 2500
    x = torch.randn((tokens, w.in_features), generator=g).to(BF16)
    dy = torch.randn((tokens, w.out_features), generator=g).to(BF16)
    coo = m.build_coo_block_index().cpu().numpy()
    _, _, dw_ref = O.linear_fwd_bwd(to64(x), to64(dy), to64(m.data), coo, tuple(m.shape))
    ref, got, again = _both_kernels(m, dy.to(cuda), x.to(cuda), monkeypatch)
    assert_close(got, dw_ref, BF16, "zipf dw")
    assert torch.equal(got, again) and torch.equal(got, ref)


@pytest.mark.parametrize("name", ["c4_4096x4096_d0.25_bf16", "c4_4096x4096_d0.5_bf16"])
def test_benchmark_layer_full_size(cuda, monkeypatch, name):
    w = workloads.WORKLOADS[name]
    blocks, data, x, dy = workloads.make_inputs(w)
    m = BlockSparseMatrix.zeros((w.out_features, w.in_features), blocks=blocks, device="cpu", dtype=w.dtype)
    with torch.no_grad():
        m.data.copy_(data)
    m = m.to(cuda)
    ref, got, again = _both_kernels(m, dy.to(cuda), x.to(cuda), monkeypatch)
    assert torch.isfinite(got.float()).all()
    assert torch.equal(got, again) and torch.equal(got, ref)
