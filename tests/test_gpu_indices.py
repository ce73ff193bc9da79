"""Device build of the index arrays: bit-exact against the CPU oracle and the reference's golden vectors."""
import numpy as np
import pytest
import torch

from oracle import block_sparse_oracle as O
from pytorch_block_sparse_amd import BlockSparseMatrix, native
from tests.helpers import load_golden

pytestmark = pytest.mark.gpu
NAMES = ["blocks", "cols_a", "row_start_ends_a", "rows_b", "col_start_ends_b"]


def _device_indices(mask, block_ptr, cuda):
    nnz = int(mask.sum())
    bp = None if block_ptr is None else torch.from_numpy(np.asarray(block_ptr)).to(cuda)
    out = native.build_indices(torch.from_numpy(mask).to(cuda), bp, nnz)
    return dict(zip(NAMES, out))


def test_golden_vectors(cuda):
    """reference tests/test_basic.py:13-25 and tests/test_replace.py:23-43, on the device."""
    g = load_golden()
    b, r = g["build"], g["replace"]
    m = BlockSparseMatrix.randn(tuple(b["size"]), None, blocks=[tuple(x) for x in b["blocks_row_col"]], device=cuda,
                                positive=True)
    assert m.cols_a.is_cuda and m.cols_a.dtype == torch.int32
    for name in ("row_start_ends_a", "cols_a", "col_start_ends_b", "rows_b", "blocks"):
        assert getattr(m, name).tolist() == b[name], name
    m.check_ = True
    m.block_replace(torch.tensor(r["replacements"]))
    assert m.row_start_ends_a.tolist() == r["row_start_ends_a"]
    assert m.cols_a.tolist() == r["cols_a"]
    assert m.block_mask_build(None).long().tolist() == r["block_mask"]
    m.check_with_dense(m.to_dense())


@pytest.mark.parametrize("grid,density", [((1, 1), 1.0), ((4, 7), 0.3), ((8, 32), 0.1), ((24, 96), 0.25),
                                          ((128, 128), 0.25), ((96, 24), 0.5), ((33, 65), 1.0), ((16, 16), 0.0),
                                          ((300, 70), 0.05), ((512, 512), 0.02)])
def test_random_masks_bit_exact(cuda, grid, density):
    rng = np.random.RandomState(grid[0] * 1000 + grid[1])
    mask = rng.rand(*grid) < density
    nnz = int(mask.sum())
    for bp in (None, rng.permutation(nnz)):
        ref = O.build_indices(mask, bp)
        got = _device_indices(mask, bp, cuda)
        for name in NAMES:
            g = got[name].cpu().numpy()
            assert g.dtype == np.int32 and g.shape == ref[name].shape, name
            assert np.array_equal(g, ref[name]), f"{name} grid={grid} d={density} block_ptr={'given' if bp is not None else 'default'}"


def test_benchmark_patterns_match_host_build(cuda):
    from pytorch_block_sparse_amd import workloads

    for name, w in workloads.WORKLOADS.items():
        blocks = workloads.make_pattern(w)
        host = BlockSparseMatrix.zeros((w.out_features, w.in_features), blocks=blocks, device="cpu")
        dev = BlockSparseMatrix.zeros((w.out_features, w.in_features), blocks=blocks, device=cuda)
        for n in NAMES:
            assert torch.equal(getattr(host, n), getattr(dev, n).cpu()), (name, n)


def test_error_reports(cuda):
    mask = torch.zeros((4, 4), dtype=torch.bool, device=cuda)
    mask[0, 1] = mask[2, 2] = True
    with pytest.raises(RuntimeError, match="holds 2 blocks but 3 were expected"):
        native.build_indices(mask, None, 3)
    with pytest.raises(RuntimeError, match="outside"):
        native.build_indices(mask, torch.tensor([0, 5], device=cuda), 2)
    # data sized for 3 blocks, mask with 2
    with pytest.raises(Exception, match="holds 2 blocks but 3 were expected"):
        BlockSparseMatrix((128, 128), mask, torch.zeros((96, 32), device=cuda))
