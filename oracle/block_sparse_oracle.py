"""CPU oracle for the block-sparse linear hot path.  TEST INFRASTRUCTURE ONLY.

This module restates, in numpy, the algorithms of the reference library
(huggingface/pytorch_block_sparse) for the path behind ``BlockSparseLinear``:
the five int32 index arrays, the packed-block <-> dense conversion and the three
matmuls (forward, input gradient, sparse-support weight gradient) in their
dense-equivalent form (``to_dense()`` followed by a plain matmul), which is what
every reference test compares the native kernels with.

Only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import it, and only as the checker.  Nothing under
``pytorch_block_sparse_amd/`` imports it: the product path is the HIP library.

Pins (what stops a plausible mistake in this file from going unnoticed; all of
them are exercised by ``tests/test_oracle.py``):

* ``build_indices`` (default block_ptr): the golden index vectors held by the
  reference's ``tests/test_basic.py:13-25``.
* ``build_indices`` with an explicit block_ptr / ``block_replace``: the golden
  after-state held by ``tests/test_replace.py:23-43``; ``build_coo_block_index``
  inverts it; ``cols_a[:,1]`` / ``rows_b[:,1]`` are permutations of 0..nnz-1.
* ``to_dense`` / ``from_dense``: the element formula stated by the reference's
  ``check_with_dense`` (``block_sparse.py:465-476``) evaluated by an independent
  per-element loop, exact round trips (``tests/test_basic.py:48-67``) and
  mask == to_dense(ones).
* the three matmuls: they *are* numpy matmul on the densified weight; special
  cases (density 1.0 == plain GEMM, single block == one 32x32 GEMM), the
  adjoint identity <dY, X W^T> == <dY W, X> == <dW, W> and a per-block loop.

No function here is "parity unpinned".
"""
import numpy as np

INT = np.int32


# --------------------------------------------------------------------------------------
# pattern sampling
# --------------------------------------------------------------------------------------
def blocks_count(shape, block_shape=(32, 32)):
    """Block grid (X, Y) of a matrix.  reference: block_sparse.py:78-83."""
    return shape[0] // block_shape[0], shape[1] // block_shape[1]


def sample_positions(X, Y, n_blocks):
    """Flat row-major positions of n_blocks random blocks, sorted.

    reference: block_sparse.py:250-251 (numpy global RandomState, choice without
    replacement, then sort).  Seed with ``numpy.random.seed`` beforehand.
    """
    pos = np.random.choice(X * Y, size=n_blocks, replace=False)
    return np.sort(pos.astype(np.int64))


def mask_from_positions(X, Y, positions):
    """Boolean [X, Y] mask with the listed flat positions set.  reference: block_sparse.py:253-255."""
    mask = np.zeros(X * Y, dtype=bool)
    mask[np.asarray(positions, dtype=np.int64)] = True
    return mask.reshape(X, Y)


def mask_from_blocks(X, Y, blocks):
    """Mask from a list of (block_row, block_col).  reference: block_sparse.py:247-248."""
    return mask_from_positions(X, Y, [b[0] * Y + b[1] for b in blocks])


# --------------------------------------------------------------------------------------
# index arrays
# --------------------------------------------------------------------------------------
def _build_indices_one(mask, block_ptr, nnz_rc, transpose_indices):
    """One compressed list (CSR if not transpose_indices, else CSC).

    reference: block_sparse.py:85-123.  ``nnz_rc`` is [nnz, 2] (row, col) of the
    nonzeros in row-major order, ``block_ptr[i]`` the data-block id of the i-th.
    """
    X, Y = mask.shape
    rows = nnz_rc[:, 0]
    cols = nnz_rc[:, 1]
    if transpose_indices:
        # :92-110 -- scatter (block_ptr + 1) to the row-major grid, read it back
        # column-major, keep the nonzero entries.
        grid = np.zeros(X * Y, dtype=np.int64)
        grid[rows * Y + cols] = block_ptr + 1
        grid = grid.reshape(X, Y).T.reshape(X * Y)
        block_ptr = grid[grid != 0] - 1
        nnz_t = np.argwhere(mask.T)  # (col, row), sorted by col then row
        X, Y = Y, X
        rows = nnz_t[:, 0]
        cols = nnz_t[:, 1]
    # :112-119 -- counts per row, exclusive scan
    counts = np.zeros(X + 1, dtype=np.int64)
    np.add.at(counts, rows + 1, 1)
    start_ends = np.cumsum(counts).astype(INT)
    # :121
    pairs = np.stack([cols, block_ptr], axis=1).astype(INT).reshape(-1, 2)
    return pairs, start_ends


def build_indices(mask, block_ptr=None):
    """The five index arrays of a block mask.

    reference: block_sparse.py:125-153.  Returns a dict with int32 arrays
    ``blocks [2*nnz]``, ``cols_a [nnz,2]``, ``row_start_ends_a [X+1]``,
    ``rows_b [nnz,2]``, ``col_start_ends_b [Y+1]``.
    """
    mask = np.asarray(mask, dtype=bool)
    nnz_rc = np.argwhere(mask)  # row-major order, like torch.nonzero (:131)
    if block_ptr is None:
        block_ptr = np.arange(nnz_rc.shape[0], dtype=np.int64)  # :133-134
    block_ptr = np.asarray(block_ptr, dtype=np.int64)
    order = np.argsort(block_ptr, kind="stable")  # :138
    blocks = nnz_rc[order][:, ::-1].reshape(-1).astype(INT)  # :139-141 (flip -> (col,row))
    cols_a, row_start_ends_a = _build_indices_one(mask, block_ptr, nnz_rc, False)
    rows_b, col_start_ends_b = _build_indices_one(mask, block_ptr, nnz_rc, True)
    return dict(
        blocks=blocks,
        cols_a=cols_a,
        row_start_ends_a=row_start_ends_a,
        rows_b=rows_b,
        col_start_ends_b=col_start_ends_b,
    )


def build_coo_block_index(row_start_ends_a, cols_a):
    """[2, nnz] (block_row, block_col) indexed by data-block id.

    reference: block_sparse.py:371-403 (row id of every CSR entry from the row
    ends, then reorder by the block pointer column).
    """
    nnz = cols_a.shape[0]
    rows = np.zeros(nnz + 1, dtype=np.int64)
    np.add.at(rows, np.asarray(row_start_ends_a[1:], dtype=np.int64), 1)
    rows = np.cumsum(rows)[:-1]
    summary = np.concatenate([rows[:, None], np.asarray(cols_a, dtype=np.int64)], axis=1)
    order = np.argsort(summary[:, 2], kind="stable")
    summary = summary[order]
    return summary[:, :2].T.astype(INT)


def block_replace(row_start_ends_a, cols_a, grid, block_replacements, check=False):
    """New (mask, block_ptr) after moving data blocks to new positions.

    reference: block_sparse.py:167-219.  ``block_replacements`` rows are
    (block_row, block_col, data_block_id); ``grid`` is (X, Y).
    """
    X, Y = grid
    pos = build_coo_block_index(row_start_ends_a, cols_a).astype(np.int64)
    rep = np.asarray(block_replacements, dtype=np.int64).reshape(-1, 3)
    if check:  # :175-199
        ref = np.zeros(X * Y, dtype=np.int64)
        ref[pos[0] * Y + pos[1]] = 1
        np.add.at(ref, rep[:, 0] * Y + rep[:, 1], 1)
        am = int(ref.argmax())
        if ref[am] > 1:
            raise Exception(f"Block position ({am // Y},{am % Y}) was already used")
    pos[:, rep[:, 2]] = rep[:, :2].T  # :202-204
    mask = np.zeros((X, Y), dtype=bool)
    mask[pos[0], pos[1]] = True  # :207
    block_ptr = np.argsort(pos[0] * Y + pos[1], kind="stable")  # :210-216
    return mask, block_ptr


# --------------------------------------------------------------------------------------
# packed data <-> dense
# --------------------------------------------------------------------------------------
def to_dense(data, coo, shape, block_shape=(32, 32)):
    """Dense [shape] matrix of packed data: block b holds W_block transposed.

    reference: block_sparse.py:405-429 and the element statement :465-476:
    ``dense[r*bs0:(r+1)*bs0, c*bs1:(c+1)*bs1] == data[b*bs0:(b+1)*bs0, :].T``.
    """
    bs0, bs1 = block_shape
    data = np.asarray(data)
    out = np.zeros(shape, dtype=data.dtype)
    blocks = data.reshape(-1, bs1, bs0)  # :412
    for b in range(coo.shape[1]):
        r, c = int(coo[0, b]), int(coo[1, b])
        out[r * bs0 : (r + 1) * bs0, c * bs1 : (c + 1) * bs1] = blocks[b].T  # :413
    return out


def from_dense(dense, coo, block_shape=(32, 32)):
    """Packed data gathered from a dense matrix at the listed blocks.

    reference: block_sparse.py:323-331 (the "slow" statement of from_dense).
    """
    bs0, bs1 = block_shape
    dense = np.asarray(dense)
    nnz = coo.shape[1]
    data = np.zeros((nnz * bs0, bs1), dtype=dense.dtype)
    for b in range(nnz):
        r, c = int(coo[0, b]), int(coo[1, b])
        part = dense[r * bs0 : (r + 1) * bs0, c * bs1 : (c + 1) * bs1]
        data[b * bs0 : (b + 1) * bs0] = part.T.reshape(bs0, bs1)
    return data


def from_dense_prefix(dense, n_blocks, block_shape=(32, 32)):
    """Packed data filled with the first n_blocks*bs0*bs1 scalars of the dense matrix.

    reference: block_sparse.py:345-350 (branch taken when block_count < full).
    """
    bs0, bs1 = block_shape
    n = n_blocks * bs0 * bs1
    return np.asarray(dense).reshape(-1)[:n].reshape(n_blocks * bs0, bs1).copy()


def block_mask_dense(coo, shape, block_shape=(32, 32)):
    """Dense 0/1 mask of the pattern.  reference: to_dense(data_replace=ones) == 1 (block_sparse.py:705)."""
    nnz = coo.shape[1]
    ones = np.ones((nnz * block_shape[0], block_shape[1]), dtype=np.float32)
    return to_dense(ones, coo, shape, block_shape) == 1


# --------------------------------------------------------------------------------------
# the three matmuls, dense-equivalent
# --------------------------------------------------------------------------------------
def reverse_matmul(dense_a, data, coo, shape, transpose, block_shape=(32, 32), dtype=np.float64):
    """a @ W.T if transpose else a @ W, W = to_dense(data).

    reference: block_sparse.py:496-497 docstring; emulator :707-710; every native
    test compares with ``a.matmul(dense.t())`` (tests/test_matmul.py:64-70).
    """
    w = to_dense(np.asarray(data, dtype=dtype), coo, shape, block_shape)
    a = np.asarray(dense_a, dtype=dtype)
    lead = a.shape[:-1]
    a2 = a.reshape(-1, a.shape[-1])
    out = a2 @ (w.T if transpose else w)
    return out.reshape(*lead, out.shape[-1])


def matmul_with_output_sparse_support(dense_a, dense_b, coo, shape, block_shape=(32, 32), dtype=np.float64):
    """Packed (a.T @ b) restricted to the pattern's blocks.

    reference: block_sparse.py:606-607 docstring, emulator :712-714, packed result
    layout tests/test_matmul_back.py:188-196 (block b of the result, transposed,
    equals the dense product at rows blocks[2b+1]*32, cols blocks[2b]*32).
    """
    a = np.asarray(dense_a, dtype=dtype)
    b = np.asarray(dense_b, dtype=dtype)
    a2 = a.reshape(-1, a.shape[-1])
    b2 = b.reshape(-1, b.shape[-1])
    full = a2.T @ b2
    assert full.shape == tuple(shape)
    return from_dense(full, coo, block_shape)


def linear_fwd_bwd(x, dy, data, coo, shape, dtype=np.float64):
    """(Y, dX, dW_packed) of BlockSparseLinear without bias.

    reference: block_sparse_linear.py:40 (Y), :80 (dX), :123 (dW).
    """
    y = reverse_matmul(x, data, coo, shape, True, dtype=dtype)
    dx = reverse_matmul(dy, data, coo, shape, False, dtype=dtype)
    dw = matmul_with_output_sparse_support(dy, x, coo, shape, dtype=dtype)
    return y, dx, dw


def linear_fwd_bwd_torch_fp32(x, dy, w_dense, mask_dense):
    """The reference's CPU dense-equivalent path with torch fp32, for timing.

    ``Y = X @ W.T; dX = dY @ W; dW = (dY.T @ X) * mask`` -- what the reference's
    emulator and PseudoBlockSparseLinear do (block_sparse.py:707-714,
    block_sparse_linear.py:255-257).  Arguments are torch CPU tensors.
    """
    y = x @ w_dense.t()
    dx = dy @ w_dense
    dw = (dy.t() @ x) * mask_dense
    return y, dx, dw
