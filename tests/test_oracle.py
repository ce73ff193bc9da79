"""Pins of the CPU oracle (oracle/block_sparse_oracle.py).

Each check is chosen so that a plausible mistake in the oracle (a transposed block, a swapped
(row, col) pair, an off-by-one in a start/end array, the wrong operand order in dW) fails it:
golden vectors held by the reference's own tests, an independent per-element statement of the
layout, algebraic identities and special cases that reduce to a plain GEMM.
"""
import itertools

import numpy as np
import pytest

from oracle import block_sparse_oracle as O
from tests.helpers import load_golden

# ---- golden vectors held by the reference: tests/test_basic.py:13-25, tests/test_replace.py:23-43 ----
_G = load_golden()
GOLD_SIZE = tuple(_G["build"]["size"])
GOLD_BLOCKS = [tuple(b) for b in _G["build"]["blocks_row_col"]]
GOLD = {k: _G["build"][k] for k in ("row_start_ends_a", "cols_a", "col_start_ends_b", "rows_b")}
GOLD_REPLACE = [tuple(r) for r in _G["replace"]["replacements"]]
GOLD_AFTER = {k: _G["replace"][k] for k in ("row_start_ends_a", "cols_a", "block_mask")}


def _gold_indices():
    X, Y = O.blocks_count(GOLD_SIZE)
    return O.build_indices(O.mask_from_blocks(X, Y, GOLD_BLOCKS))


def test_build_indices_golden():
    idx = _gold_indices()
    for k, v in GOLD.items():
        assert idx[k].dtype == np.int32
        assert idx[k].tolist() == v, k
    # blocks: (col, row) of data block b; data blocks are in row-major order of the mask
    assert idx["blocks"].tolist() == _G["build"]["blocks"]


def test_block_info_golden():
    """tests/test_replace.py:29 block_info: position of every data block."""
    idx = _gold_indices()
    coo = O.build_coo_block_index(idx["row_start_ends_a"], idx["cols_a"])
    assert coo.T.tolist() == _G["build"]["block_info_row_col"]


def test_block_replace_golden():
    idx = _gold_indices()
    mask, block_ptr = O.block_replace(idx["row_start_ends_a"], idx["cols_a"], (4, 2), GOLD_REPLACE, check=True)
    assert mask.astype(int).tolist() == GOLD_AFTER["block_mask"]
    after = O.build_indices(mask, block_ptr)
    assert after["row_start_ends_a"].tolist() == GOLD_AFTER["row_start_ends_a"]
    assert after["cols_a"].tolist() == GOLD_AFTER["cols_a"]
    # data block b now sits where the replacement put it; block 3 stayed at (2, 0)
    coo = O.build_coo_block_index(after["row_start_ends_a"], after["cols_a"])
    assert coo.T.tolist() == _G["replace"]["block_info_row_col"]


def test_block_replace_rejects_used_position():
    """tests/test_replace.py:56: error text of the reference."""
    idx = _gold_indices()
    with pytest.raises(Exception, match=r"Block position \(0,1\) was already used"):
        O.block_replace(idx["row_start_ends_a"], idx["cols_a"], (4, 2), [(0, 1, 0)], check=True)


def _invariants(mask, block_ptr=None):
    X, Y = mask.shape
    idx = O.build_indices(mask, block_ptr)
    nnz = int(mask.sum())
    rp, cp = idx["row_start_ends_a"], idx["col_start_ends_b"]
    assert rp.shape == (X + 1,) and cp.shape == (Y + 1,)
    assert rp[0] == 0 and cp[0] == 0 and rp[-1] == nnz and cp[-1] == nnz
    assert (np.diff(rp) == mask.sum(1)).all() and (np.diff(cp) == mask.sum(0)).all()
    assert sorted(idx["cols_a"][:, 1].tolist()) == list(range(nnz))
    assert sorted(idx["rows_b"][:, 1].tolist()) == list(range(nnz))
    # CSR and CSC describe the same (row, col, block) triples
    rows_of_entry = np.repeat(np.arange(X), np.diff(rp))
    csr = {(int(r), int(c), int(b)) for r, (c, b) in zip(rows_of_entry, idx["cols_a"])}
    cols_of_entry = np.repeat(np.arange(Y), np.diff(cp))
    csc = {(int(r), int(c), int(b)) for c, (r, b) in zip(cols_of_entry, idx["rows_b"])}
    assert csr == csc and len(csr) == nnz
    assert {(r, c) for r, c, _ in csr} == {tuple(p) for p in np.argwhere(mask).tolist()}
    # columns sorted inside a row, rows sorted inside a column
    for r in range(X):
        seg = idx["cols_a"][rp[r] : rp[r + 1], 0]
        assert (np.diff(seg) > 0).all()
    for c in range(Y):
        seg = idx["rows_b"][cp[c] : cp[c + 1], 0]
        assert (np.diff(seg) > 0).all()
    # blocks[b] = (col, row) of data block b; build_coo_block_index inverts build_indices
    blocks = idx["blocks"].reshape(-1, 2)
    for r, c, b in csr:
        assert blocks[b].tolist() == [c, r]
    coo = O.build_coo_block_index(rp, idx["cols_a"])
    assert (coo[0] == blocks[:, 1]).all() and (coo[1] == blocks[:, 0]).all()
    return idx


def test_build_indices_all_3x3_masks():
    """Brute force: every mask of a 3 x 3 grid, default block order."""
    for bits in itertools.product([0, 1], repeat=9):
        _invariants(np.array(bits, dtype=bool).reshape(3, 3))


def test_build_indices_random_masks_with_block_ptr():
    rng = np.random.RandomState(0)
    for X, Y, d in [(1, 1, 1.0), (4, 7, 0.3), (8, 8, 0.5), (24, 96, 0.25), (33, 5, 0.9), (6, 6, 0.0)]:
        mask = rng.rand(X, Y) < d
        _invariants(mask)
        nnz = int(mask.sum())
        _invariants(mask, rng.permutation(nnz))


def test_layout_element_formula():
    """dense[32r + i, 32c + j] == data[32b + j, i] (reference block_sparse.py:465-476), element by element."""
    rng = np.random.RandomState(1)
    X, Y = 3, 4
    mask = rng.rand(X, Y) < 0.5
    idx = O.build_indices(mask, rng.permutation(int(mask.sum())))
    coo = O.build_coo_block_index(idx["row_start_ends_a"], idx["cols_a"])
    nnz = coo.shape[1]
    data = rng.randn(nnz * 32, 32).astype(np.float32)
    dense = O.to_dense(data, coo, (X * 32, Y * 32))
    for b in range(nnz):
        r, c = coo[:, b]
        for i in (0, 1, 17, 31):
            for j in (0, 5, 30, 31):
                assert dense[32 * r + i, 32 * c + j] == data[32 * b + j, i]
    assert (dense[~np.kron(mask, np.ones((32, 32), dtype=bool))] == 0).all()
    assert (O.block_mask_dense(coo, dense.shape) == np.kron(mask, np.ones((32, 32), dtype=bool))).all()
    # exact round trip (reference tests/test_basic.py:48-67)
    assert (O.from_dense(dense, coo) == data).all()


@pytest.mark.parametrize("size", [(32, 32), (64, 32), (32, 64), (64, 64), (256, 64)])
def test_full_round_trip(size):
    rng = np.random.RandomState(2)
    X, Y = O.blocks_count(size)
    mask = np.ones((X, Y), dtype=bool)
    idx = O.build_indices(mask)
    coo = O.build_coo_block_index(idx["row_start_ends_a"], idx["cols_a"])
    a = rng.randn(*size).astype(np.float32)
    data = O.from_dense(a, coo)
    assert (O.to_dense(data, coo, size) == a).all()


def test_from_dense_prefix():
    """reference block_sparse.py:345-350: first n*1024 scalars of the flattened dense matrix."""
    a = np.arange(64 * 96, dtype=np.float32).reshape(64, 96)
    d = O.from_dense_prefix(a, 3)
    assert d.shape == (96, 32) and (d.reshape(-1) == np.arange(3 * 1024)).all()


def _random_problem(rng, X, Y, d, tokens, full=False):
    mask = np.ones((X, Y), bool) if full else rng.rand(X, Y) < d
    if not mask.any():
        mask[0, 0] = True
    idx = O.build_indices(mask)
    coo = O.build_coo_block_index(idx["row_start_ends_a"], idx["cols_a"])
    data = rng.randn(coo.shape[1] * 32, 32)
    x = rng.randn(tokens, Y * 32)
    dy = rng.randn(tokens, X * 32)
    return mask, coo, data, x, dy


def test_matmuls_density_one_is_plain_gemm():
    rng = np.random.RandomState(3)
    mask, coo, data, x, dy = _random_problem(rng, 3, 2, 1.0, 5, full=True)
    w = O.to_dense(data, coo, (96, 64))
    y, dx, dw = O.linear_fwd_bwd(x, dy, data, coo, (96, 64))
    assert np.allclose(y, x @ w.T) and np.allclose(dx, dy @ w)
    assert np.allclose(O.to_dense(dw, coo, (96, 64)), dy.T @ x)


def test_matmuls_single_block():
    """One block at (1, 2): Y[:, 32:64] = X[:, 64:96] @ Wblk^T with Wblk = data.T (reference tests/test_matmul.py:141-229)."""
    rng = np.random.RandomState(4)
    X, Y = 3, 4
    mask = np.zeros((X, Y), bool)
    mask[1, 2] = True
    idx = O.build_indices(mask)
    coo = O.build_coo_block_index(idx["row_start_ends_a"], idx["cols_a"])
    data = rng.randn(32, 32)
    x = rng.randn(7, 128)
    dy = rng.randn(7, 96)
    y, dx, dw = O.linear_fwd_bwd(x, dy, data, coo, (96, 128))
    wblk = data.T
    exp_y = np.zeros((7, 96))
    exp_y[:, 32:64] = x[:, 64:96] @ wblk.T
    exp_dx = np.zeros((7, 128))
    exp_dx[:, 64:96] = dy[:, 32:64] @ wblk
    assert np.allclose(y, exp_y) and np.allclose(dx, exp_dx)
    # packed gradient block, transposed, equals the dense product at rows blocks[2b+1]*32, cols blocks[2b]*32
    # (reference tests/test_matmul_back.py:188-196)
    assert np.allclose(dw.T, dy[:, 32:64].T @ x[:, 64:96])


def test_adjoint_identities():
    """<dY, X W^T> == <dY W, X> == <dW, W>: ties the three products and the packed layout together."""
    rng = np.random.RandomState(5)
    mask, coo, data, x, dy = _random_problem(rng, 5, 6, 0.4, 11)
    y, dx, dw = O.linear_fwd_bwd(x, dy, data, coo, (160, 192))
    a = (dy * y).sum()
    assert np.isclose(a, (dx * x).sum()) and np.isclose(a, (dw * data).sum())


def test_leading_dims_and_fp32_timing_path():
    import torch

    rng = np.random.RandomState(6)
    mask, coo, data, x, dy = _random_problem(rng, 2, 3, 0.6, 12)
    y3 = O.reverse_matmul(x.reshape(3, 4, -1), data, coo, (64, 96), True)
    assert y3.shape == (3, 4, 64) and np.allclose(y3.reshape(12, 64), O.reverse_matmul(x, data, coo, (64, 96), True))
    w = torch.from_numpy(O.to_dense(data.astype(np.float32), coo, (64, 96)))
    m = torch.from_numpy(O.block_mask_dense(coo, (64, 96))).float()
    yt, dxt, dwt = O.linear_fwd_bwd_torch_fp32(torch.from_numpy(x).float(), torch.from_numpy(dy).float(), w, m)
    y, dx, dw = O.linear_fwd_bwd(x, dy, data, coo, (64, 96))
    assert np.allclose(yt.numpy(), y, atol=1e-4) and np.allclose(dxt.numpy(), dx, atol=1e-4)
    assert np.allclose(O.from_dense(dwt.numpy(), coo), dw, atol=1e-4)


def test_sample_positions_is_numpy_choice():
    np.random.seed(7)
    got = O.sample_positions(8, 32, 25)
    np.random.seed(7)
    assert (got == np.sort(np.random.choice(256, size=25, replace=False))).all()
    assert len(set(got.tolist())) == 25
