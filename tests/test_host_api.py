"""CPU tests of the host-side mirror of the reference interface (no GPU, no matmul kernels).

They follow the reference's CPU-runnable tests (tests/test_emulate.py) and the host-only parts of
tests/test_basic.py, test_replace.py, test_save.py, test_sparse_optimizer.py and test_integration.py
(parameter counts of a patched model).
"""
import io

import numpy as np
import pytest
import torch

import pytorch_block_sparse_amd as pbs
from oracle import block_sparse_oracle as O
from pytorch_block_sparse_amd import (
    BlockSparseLinear,
    BlockSparseMatrix,
    BlockSparseMatrixEmulator,
    BlockSparseModelPatcher,
    SparseOptimizer,
    workloads,
)
from pytorch_block_sparse_amd.block_sparse_linear import PseudoBlockSparseLinear

INDEX_NAMES = ["blocks", "cols_a", "row_start_ends_a", "rows_b", "col_start_ends_b"]


def test_public_names():
    assert set(pbs.__all__) == {
        "BlockSparseMatrix", "BlockSparseMatrixEmulator", "BlockSparseLinear", "BlockSparseModelPatcher",
        "SparseOptimizer",
    }


def test_index_arrays_golden_and_against_oracle():
    m = BlockSparseMatrix.randn((128, 64), None, blocks=[(0, 0), (1, 0), (2, 0), (0, 1)], device="cpu")
    assert m.row_start_ends_a.tolist() == [0, 2, 3, 4, 4]
    assert m.cols_a.tolist() == [[0, 0], [1, 1], [0, 2], [0, 3]]
    assert m.col_start_ends_b.tolist() == [0, 3, 4]
    assert m.rows_b.tolist() == [[0, 0], [1, 2], [2, 3], [0, 1]]
    rng = np.random.RandomState(0)
    for X, Y, d in [(1, 1, 1.0), (4, 7, 0.3), (24, 96, 0.25), (9, 3, 0.8)]:
        mask = rng.rand(X, Y) < d
        nnz = int(mask.sum())
        for bp in (None, rng.permutation(nnz)):
            data = torch.zeros((nnz * 32, 32))
            mat = BlockSparseMatrix((X * 32, Y * 32), torch.from_numpy(mask), data)
            if bp is not None:
                mat.rebuild(torch.from_numpy(mask), torch.from_numpy(bp))
            ref = O.build_indices(mask, bp)
            for name in INDEX_NAMES:
                got = getattr(mat, name)
                assert got.dtype == torch.int32
                assert np.array_equal(got.numpy(), ref[name]), name


def test_block_replace_golden_and_error():
    m = BlockSparseMatrix.randn((128, 64), None, blocks=[(0, 0), (1, 0), (2, 0), (0, 1)], device="cpu", positive=True)
    m.check_ = True
    before = m.to_dense().clone()
    pos_before = m.build_coo_block_index().t().tolist()
    assert pos_before == [[0, 0], [0, 1], [1, 0], [2, 0]]
    m.block_replace(torch.tensor([(3, 1, 0), (2, 1, 2), (1, 1, 1)]))
    assert m.row_start_ends_a.tolist() == [0, 0, 1, 3, 4]
    assert m.cols_a.tolist() == [[1, 1], [0, 3], [1, 2], [1, 0]]
    assert m.block_mask_build(None).long().tolist() == [[0, 0], [0, 1], [1, 1], [0, 1]]
    after = m.to_dense()
    m.check_with_dense(after)
    # data moved with its block (reference tests/test_replace.py:104-129)
    for (r, c, b) in [(3, 1, 0), (2, 1, 2), (1, 1, 1)]:
        r0, c0 = pos_before[b]
        assert torch.equal(after[r * 32 : r * 32 + 32, c * 32 : c * 32 + 32], before[r0 * 32 : r0 * 32 + 32, c0 * 32 : c0 * 32 + 32])
    assert torch.equal(after[64:96, 0:32], before[64:96, 0:32])  # block 3 untouched
    mask = m.block_mask_build(None).repeat_interleave(32, 0).repeat_interleave(32, 1)
    assert (after[~mask] == 0).all()
    m2 = BlockSparseMatrix.randn((128, 64), None, blocks=[(0, 0), (1, 0), (2, 0), (0, 1)], device="cpu")
    m2.check_ = True
    with pytest.raises(Exception, match=r"Block position \(0,1\) was already used"):
        m2.block_replace(torch.tensor([(0, 1, 0)]))


@pytest.mark.parametrize("size", [(32, 32), (64, 32), (32, 64), (64, 64), (256, 64)])
def test_dense_round_trip(size):
    """reference tests/test_basic.py:48-67."""
    n = size[0] * size[1] // 1024
    m = BlockSparseMatrix.randn(size, n, device="cpu")
    a = m.to_dense()
    m.check_with_dense(a)
    m2 = BlockSparseMatrix.from_dense(a, (32, 32), block_count=None)
    m2.check_with_dense(a)
    assert torch.equal(m2.to_dense(), a)
    coo = m.build_coo_block_index().numpy()
    assert np.array_equal(O.to_dense(m.data.detach().numpy(), coo, size), a.numpy())
    assert torch.equal(m.to_sparse().to_dense().transpose(1, 2).reshape(size), a)


def test_from_dense_variants():
    """slow == fast (reference tests/test_emulate.py:44-69); prefix-copy branch (block_sparse.py:345-350)."""
    torch.manual_seed(0)
    dense = torch.randn(96, 64)
    blocks = [(0, 1), (2, 0), (1, 1)]
    fast = BlockSparseMatrix.from_dense(dense, blocks=blocks)
    slow = BlockSparseMatrix.from_dense(dense, blocks=blocks, slow=True)
    assert torch.equal(fast.data, slow.data)
    coo = fast.build_coo_block_index().numpy()
    assert np.array_equal(fast.data.detach().numpy(), O.from_dense(dense.numpy(), coo))
    np.random.seed(1)
    part = BlockSparseMatrix.from_dense(dense, block_count=2)
    assert torch.equal(part.data.flatten(), dense.flatten()[: 2 * 1024])


def test_emulator_on_cpu():
    """reference tests/test_emulate.py:10-42: constructors and products of the dense-masked twin."""
    np.random.seed(0)
    torch.manual_seed(0)
    for shape, bs, n in [((64, 48), (4, 8), 20), ((8, 8), (4, 1), 5), ((64, 64), (32, 32), 3)]:
        m = BlockSparseMatrixEmulator.randn(shape, n, block_shape=bs, device="cpu")
        d = m.to_dense()
        mask = m._mask
        assert (d[~mask] == 0).all() and int(mask.sum()) == n * bs[0] * bs[1]
        a = torch.randn(5, shape[1])
        b = torch.randn(5, shape[0])
        assert torch.allclose(m.reverse_matmul(a, transpose=True), a @ d.t())
        assert torch.allclose(m.reverse_matmul(b, transpose=False), b @ d)
        assert torch.allclose(m.matmul_with_output_sparse_support(b, a), (b.t() @ a) * mask)


def test_constructor_errors_and_block_count():
    with pytest.raises(Exception, match="invalid in_features"):
        BlockSparseLinear(100, 64, device="cpu")
    with pytest.raises(Exception, match="invalid out_features"):
        BlockSparseLinear(64, 100, device="cpu")
    with pytest.raises(Exception, match="invalid density"):
        BlockSparseLinear(64, 64, density=1.5, device="cpu")
    with pytest.raises(Exception, match="multiples of 32"):
        BlockSparseMatrix((100, 64), torch.zeros(3, 2, dtype=torch.bool), torch.zeros(0, 32))
    with pytest.raises(Exception, match="float32 or bfloat16"):
        BlockSparseMatrix((32, 32), torch.ones(1, 1, dtype=torch.bool), torch.zeros(32, 32, dtype=torch.float64))
    with pytest.raises(Exception, match="Too many blocks"):
        BlockSparseMatrix.zeros((32, 32), n_blocks=2, device="cpu")
    np.random.seed(0)
    layer = BlockSparseLinear(1024, 256, density=0.1, device="cpu")  # int(25.6) == 25: truncation
    assert layer.block_count == 25 and layer.weight.data.shape == (25 * 32, 32)
    assert layer.weight.shape == (256, 1024) and layer.bias.shape == (256,)
    hash(layer.weight)  # reference tests/test_basic.py:69-71


def test_matmul_needs_gpu_and_library():
    """There is no CPU path for the three products: a CPU tensor raises instead of silently computing."""
    np.random.seed(0)
    m = BlockSparseMatrix.randn((64, 64), 2, device="cpu")
    with pytest.raises(RuntimeError, match="only on a GPU"):
        m.reverse_matmul(torch.randn(4, 64), transpose=True)
    with pytest.raises(RuntimeError, match="only on a GPU"):
        m.matmul_with_output_sparse_support(torch.randn(4, 64), torch.randn(4, 64))
    with pytest.raises(Exception, match="Invalid matrices sizes"):
        m.reverse_matmul(torch.randn(4, 32), transpose=True)


def test_state_dict_round_trip():
    """reference tests/test_save.py:37-51: the index buffers travel in the state dict."""
    np.random.seed(0)
    torch.manual_seed(0)
    a = BlockSparseLinear(64, 128, True, density=0.5, device="cpu")
    keys = set(a.state_dict().keys())
    assert keys == {"bias"} | {f"weight.{k}" for k in ["data"] + INDEX_NAMES}
    for k in INDEX_NAMES:
        assert a.state_dict()[f"weight.{k}"].dtype == torch.int32
    buf = io.BytesIO()
    torch.save(a.state_dict(), buf)
    buf.seek(0)
    b = BlockSparseLinear(64, 128, True, density=0.5, device="cpu")  # a different random pattern
    assert not torch.equal(a.weight.cols_a, b.weight.cols_a)
    b.load_state_dict(torch.load(buf, weights_only=True))
    assert torch.equal(a.weight.to_dense(), b.weight.to_dense())
    for k in INDEX_NAMES:
        assert torch.equal(getattr(a.weight, k), getattr(b.weight, k))


def test_corrupt_index_buffers_are_rejected():
    """Index buffers are validated where they enter (the reference runs sanity_check on both compressed
    lists in every rebuild, block_sparse.py:67-73, :431-463): a checkpoint whose lists are inconsistent
    raises from load_state_dict instead of reaching a kernel."""
    np.random.seed(0)
    torch.manual_seed(0)
    a = BlockSparseLinear(64, 128, True, density=0.75, device="cpu")
    good = {k: v.clone() for k, v in a.state_dict().items()}
    nnz = a.weight.cols_a.shape[0]

    def corrupt(key, fn):
        sd = {k: v.clone() for k, v in good.items()}
        fn(sd["weight." + key])
        return sd

    cases = {
        "row list runs past the entries": corrupt("row_start_ends_a", lambda t: t.__setitem__(-1, nnz + 5)),
        "row list decreases": corrupt("row_start_ends_a", lambda t: t.__setitem__(1, nnz + 1)),
        "column list does not start at 0": corrupt("col_start_ends_b", lambda t: t.__setitem__(0, 1)),
        "block column out of range": corrupt("cols_a", lambda t: t.__setitem__((0, 0), 99)),
        "negative block row": corrupt("rows_b", lambda t: t.__setitem__((0, 0), -1)),
        "data block id out of range": corrupt("cols_a", lambda t: t.__setitem__((0, 1), nnz)),
        "data block id used twice": corrupt("rows_b", lambda t: t.__setitem__((0, 1), int(t[1, 1]))),
        "block position outside the grid": corrupt("blocks", lambda t: t.__setitem__(0, 1000)),
    }
    # a block row of this pattern that holds two blocks: its two entries, in turn, repeated (a duplicate
    # position), swapped (unsorted), and given each other's data blocks (the lists disagree)
    ends = a.weight.row_start_ends_a.tolist()
    e0 = next(ends[r] for r in range(len(ends) - 1) if ends[r + 1] - ends[r] >= 2)

    def swap_coords(t):
        t[e0, 0], t[e0 + 1, 0] = int(t[e0 + 1, 0]), int(t[e0, 0])

    def swap_blocks(t):
        t[e0, 1], t[e0 + 1, 1] = int(t[e0 + 1, 1]), int(t[e0, 1])

    cases["the same block column twice in a row"] = corrupt("cols_a", lambda t: t.__setitem__((e0 + 1, 0), int(t[e0, 0])))
    cases["a row's block columns out of order"] = corrupt("cols_a", swap_coords)
    cases["the two lists disagree about a block"] = corrupt("cols_a", swap_blocks)
    for what, sd in cases.items():
        b = BlockSparseLinear(64, 128, True, density=0.75, device="cpu")
        mine = {k: getattr(b.weight, k).clone() for k in INDEX_NAMES}
        with pytest.raises(RuntimeError, match="index buffers are inconsistent"):
            b.load_state_dict(sd)
        # the module is left with the index buffers it had before the load, which are consistent
        for k in INDEX_NAMES:
            assert torch.equal(getattr(b.weight, k), mine[k]), (what, k)
        b.weight.validate_indices()
        # direct use of the check on bad buffers
        for k in INDEX_NAMES:
            getattr(b.weight, k).copy_(sd["weight." + k])
        with pytest.raises(Exception):
            b.weight.validate_indices()
    b = BlockSparseLinear(64, 128, True, density=0.75, device="cpu")
    b.load_state_dict(good)   # the untouched state dict still loads
    b.weight.validate_indices()
    # sanity_check keeps the reference's signature and conditions
    w = b.weight
    w.sanity_check(w.cols_a, w.row_start_ends_a, w.shape, w.block_shape)
    w.sanity_check(w.rows_b, w.col_start_ends_b, (w.shape[1], w.shape[0]), (32, 32))
    with pytest.raises(Exception, match="row_end last element"):
        w.sanity_check(w.cols_a[:-1], w.row_start_ends_a, w.shape, w.block_shape)


class _Tiny(torch.nn.Module):
    def __init__(self):
        super().__init__()
        self.embed = torch.nn.Embedding(10, 64)
        self.layer = torch.nn.ModuleList()
        for _ in range(2):
            blk = torch.nn.Module()
            blk.intermediate = torch.nn.Module()
            blk.intermediate.dense = torch.nn.Linear(64, 256)
            blk.output = torch.nn.Module()
            blk.output.dense = torch.nn.Linear(256, 64)
            blk.norm = torch.nn.LayerNorm(64)
            self.layer.append(blk)


def test_patcher_counts_and_errors(capsys):
    """reference tests/test_integration.py:37-64 (parameter counts) and util.py semantics."""
    np.random.seed(0)
    model = _Tiny()
    dense_params = sum(p.numel() for p in model.parameters())
    mp = BlockSparseModelPatcher()
    names = [d["regexp"] for d in mp.get_patchable_layers(model)]
    assert names == [r"layer\.0\.intermediate\.dense", r"layer\.0\.output\.dense", r"layer\.1\.intermediate\.dense",
                     r"layer\.1\.output\.dense"]
    mp.add_pattern(r"layer\.[0-9]+\.intermediate\.dense", {"density": 0.5})
    mp.add_pattern(r"layer\.[0-9]+\.output\.dense", {"density": 0.25})
    mp.patch_model(model)
    out = capsys.readouterr().out
    assert out.count("Patching with BlockSparseLinear") == 4
    for blk in model.layer:
        assert isinstance(blk.intermediate.dense, BlockSparseLinear) and blk.intermediate.dense.block_count == 8
        assert isinstance(blk.output.dense, BlockSparseLinear) and blk.output.dense.block_count == 4
    sparse_params = sum(p.numel() for p in model.parameters())
    assert dense_params - sparse_params == 2 * (64 * 256 // 2 + 64 * 256 * 3 // 4)
    # from_dense prefix copy scaled by 1/sqrt(density) (reference block_sparse_linear.py:207-210)
    torch.manual_seed(1)
    lin = torch.nn.Linear(64, 64)
    sp = BlockSparseLinear(0, 0, False, torch_nn_linear=lin, density=0.5)
    assert torch.allclose(sp.weight.data.flatten(), lin.weight.detach().flatten()[: 2 * 1024] / 0.5 ** 0.5)
    assert torch.equal(sp.bias, lin.bias)
    # not a Linear -> raises; nothing matched -> warning
    mp2 = BlockSparseModelPatcher()
    mp2.add_pattern(r"layer\.0\.norm", {"density": 0.5})
    with pytest.raises(Exception, match="Cannot patch layer.0.norm"):
        mp2.patch_model(_Tiny())
    mp3 = BlockSparseModelPatcher()
    mp3.add_pattern("nothing", {"density": 0.5})
    mp3.patch_model(_Tiny())
    assert "did not patch anything" in capsys.readouterr().out
    # pseudo_linear twin
    mp4 = BlockSparseModelPatcher()
    mp4.add_pattern(r"layer\.0\.output\.dense", {"density": 0.5, "pseudo_linear": True})
    t = _Tiny()
    mp4.patch_model(t)
    pl = t.layer[0].output.dense
    assert isinstance(pl, PseudoBlockSparseLinear) and abs(pl.density - 0.5) < 1e-9
    x = torch.randn(3, 256)
    assert torch.allclose(pl(x), torch.nn.functional.linear(x, pl.weight * pl.mask, pl.bias))


def test_sparse_optimizer_moves_blocks():
    """reference tests/test_sparse_optimizer.py:39-40: 2 * int(ratio * nnz) positions change."""
    np.random.seed(0)
    torch.manual_seed(0)
    layer = BlockSparseLinear(256, 256, True, density=0.5, device="cpu")
    objs = SparseOptimizer.sparse_objects(layer)
    assert objs == [layer.weight]
    adam = torch.optim.Adam(layer.parameters())
    # give Adam a state for the data without running the (GPU-only) forward
    layer.weight.data.grad = torch.ones_like(layer.weight.data)
    layer.bias.grad = torch.ones_like(layer.bias)
    adam.step()
    so = SparseOptimizer(objs, lr=0.25)
    so.attach_optimizer(adam)
    before = layer.weight.block_mask_build(None).clone()
    so.step()
    after = layer.weight.block_mask_build(None)
    nnz = layer.block_count
    assert int((before != after).sum()) == 2 * int(0.25 * nnz)
    assert int(after.sum()) == nnz
    state = adam.state[layer.weight.data]
    moved = (state["exp_avg"].reshape(nnz, -1) == 0).all(1)
    assert int(moved.sum()) == int(0.25 * nnz)
    layer.weight.check_with_dense(layer.weight.to_dense())
    with pytest.raises(Exception):
        SparseOptimizer(objs, lr=0.1, method="nope")


def test_workload_generators():
    w = workloads.WORKLOADS["c1_1024x256_d0.1_fp32"]
    assert w.nnz == 25 and w.grid == (8, 32)
    a = workloads.uniform_positions(8, 32, 25)
    b = workloads.uniform_positions(8, 32, 25)
    assert (a == b).all() and len(set(a.tolist())) == 25
    w3 = workloads.WORKLOADS["c3_3072x768_d0.25_zipf_fp32"]
    counts = workloads.zipf_row_counts(*w3.grid, w3.nnz)
    assert counts.sum() == 576 and counts.max() == 96 and counts.min() >= 1
    blocks = workloads.make_pattern(w3)
    assert len(set(blocks)) == 576 and blocks == sorted(blocks)
    w4 = workloads.WORKLOADS["c4_4096x4096_d0.25_bf16"]
    assert w4.nnz == 4096 and abs(w4.flops_per_gemm * 3 - 412.3e9) < 0.1e9
