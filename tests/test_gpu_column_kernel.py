"""The bf16 dense x block-sparse kernel with one block column per wave, against the CPU oracle.

The library picks that kernel by itself only for large, fairly dense problems (many blocks per column, at least
256 tiles); the environment variable PBS_COLUMN_KERNEL=1 makes it run wherever it can, so that small shapes the
oracle does in seconds reach all of its paths: token tails, groups with empty places, empty columns, lists of
more than 64 items (density 1), very uneven columns, the fused bias, several token tiles per workgroup.  The
forward direction goes through the transposed copy of the blocks that the library makes in the caller's
workspace; the input gradient reads the data as stored.
"""
import numpy as np
import pytest
import torch

from oracle import block_sparse_oracle as O
from pytorch_block_sparse_amd import BlockSparseMatrix, native, workloads
from tests.helpers import assert_close, to64

pytestmark = pytest.mark.gpu
BF16 = torch.bfloat16


@pytest.fixture
def column_kernel(monkeypatch):
    monkeypatch.setenv("PBS_COLUMN_KERNEL", "1")
    yield
    monkeypatch.delenv("PBS_COLUMN_KERNEL", raising=False)


def _matrix(out_f, in_f, blocks, n_blocks, device, seed):
    np.random.seed(seed)
    torch.manual_seed(seed)
    return BlockSparseMatrix.randn((out_f, in_f), n_blocks, blocks=blocks, device="cpu", dtype=BF16).to(device)


def _runs_column_kernel(m, tokens):
    """The forward product of m asks for a workspace exactly when the column kernel is going to run it."""
    out_f, in_f = m.shape
    nnz = m.cols_a.shape[0]
    return native.load().pbs_blocksparse_matmul_workspace_bytes(tokens, out_f, in_f, nnz, 1, 1) == nnz * 2048


def _check_both_directions(m, tokens, device, seed, what, bias=False):
    out_f, in_f = m.shape
    g = torch.Generator().manual_seed(seed)
    x = torch.randn((tokens, in_f), generator=g).to(BF16)
    dy = torch.randn((tokens, out_f), generator=g).to(BF16)
    b = torch.randn((out_f,), generator=g).to(BF16) if bias else None
    coo = m.build_coo_block_index().cpu().numpy()
    w_dense = O.to_dense(to64(m.data), coo, (out_f, in_f))
    y_ref = to64(x) @ w_dense.T + (to64(b)[None, :] if bias else 0.0)
    dx_ref = to64(dy) @ w_dense
    print(f"{what}: {in_f}->{out_f} tokens={tokens} nnz={m.cols_a.shape[0]} bias={bias}", flush=True)
    assert _runs_column_kernel(m, tokens), what + ": the column kernel does not take this shape"
    y = m.reverse_matmul(x.to(device), transpose=True, bias=None if b is None else b.to(device))
    assert_close(y, y_ref, BF16, what + " fwd")
    dx = m.reverse_matmul(dy.to(device), transpose=False)
    assert_close(dx, dx_ref, BF16, what + " dx")
    return y, dx


@pytest.mark.parametrize("in_f,out_f,tokens,density,bias", [
    (128, 96, 300, 0.5, False),          # 3 block columns: 13 of the 16 places of the only group are empty
    (256, 1024, 1000 + 7, 0.3, True),    # token tail, bias
    (64, 512, 5000, 1.0, True),          # one step per tile, 40 tiles
    (4096, 128, 200, 1.0, False),        # lists of 128 items: more than the two item registers hold
    (1024, 544, 2048 + 1, 0.05, False),  # sparse: columns with no block, steps most columns skip
    (448, 2080, 777, 0.4, True),         # k / 64 = 7 steps, a last group with one column
    (64, 2048, 128 * 64 * 3 + 50, 0.6, False),   # one step per tile and four tiles per workgroup (steps are numbered across tiles)
    (192, 4096, 128 * 32 * 2 + 1, 0.3, True),    # three steps per tile, three tiles per workgroup, the last one a single token
])
def test_shapes_against_oracle(cuda, column_kernel, in_f, out_f, tokens, density, bias):
    n_blocks = max(1, int(density * (in_f // 32) * (out_f // 32)))
    m = _matrix(out_f, in_f, None, n_blocks, cuda, seed=31)
    _check_both_directions(m, tokens, cuda, 37, f"column d={density}", bias=bias)


def test_empty_columns_and_empty_group(cuda, column_kernel):
    """Blocks only in the first 8 block rows of W: every other result column is the bias, bit for bit."""
    in_f, out_f, tokens = 256, 1024, 1500
    rng = np.random.RandomState(5)
    blocks = sorted({(int(r), int(c)) for r, c in zip(rng.randint(0, 8, 40), rng.randint(0, 8, 40))})
    m = _matrix(out_f, in_f, blocks, None, cuda, seed=9)
    y, dx = _check_both_directions(m, tokens, cuda, 4, "empty group", bias=True)
    g = torch.Generator().manual_seed(4)
    torch.randn((tokens, in_f), generator=g), torch.randn((tokens, out_f), generator=g)
    b = torch.randn((out_f,), generator=g).to(BF16).to(cuda)
    assert torch.equal(y[:, 256:], b[None, 256:].expand(tokens, -1))


def test_very_uneven_columns(cuda, column_kernel):
    """Zipf-distributed blocks per row of W (the 3072 -> 768 benchmark pattern, in bf16): the forward product's
    columns range from 1 to 96 blocks, which the kernel deals to its waves by rank."""
    w = workloads.WORKLOADS["c3_3072x768_d0.25_zipf_fp32"]
    blocks = workloads.make_pattern(w)
    m = _matrix(w.out_features, w.in_features, blocks, None, cuda, seed=3)
    _check_both_directions(m, 1024 + 33, cuda, 41, "zipf", bias=True)


def test_agrees_with_wide_kernel_and_is_chosen_at_density_half(cuda, monkeypatch):
    """4096 -> 4096 at density 0.5, 4096 tokens, oracle-checked in full: the library takes the column kernel for
    this problem by itself; with PBS_COLUMN_KERNEL=0 the wide kernel runs instead and the two must agree to bf16
    rounding (same fp32 products, summed in a different order)."""
    w = workloads.WORKLOADS["c4_4096x4096_d0.5_bf16"]
    tokens = 4096
    blocks, data, x, dy = workloads.make_inputs(w, tokens=tokens)
    m = BlockSparseMatrix.zeros((w.out_features, w.in_features), blocks=blocks, device="cpu", dtype=w.dtype)
    with torch.no_grad():
        m.data.copy_(data)
    coo = m.build_coo_block_index().numpy()
    y_ref, dx_ref, dw_ref = O.linear_fwd_bwd(to64(x), to64(dy), to64(data), coo, tuple(m.shape))
    m = m.to(cuda)
    xd, dyd = x.to(cuda), dy.to(cuda)
    monkeypatch.delenv("PBS_COLUMN_KERNEL", raising=False)
    assert _runs_column_kernel(m, tokens)
    y, dx = m.reverse_matmul(xd, True), m.reverse_matmul(dyd, False)
    assert_close(y, y_ref, BF16, "d0.5 fwd")
    assert_close(dx, dx_ref, BF16, "d0.5 dx")
    assert_close(m.matmul_with_output_sparse_support(dyd, xd), dw_ref, BF16, "d0.5 dw")
    monkeypatch.setenv("PBS_COLUMN_KERNEL", "0")
    assert not _runs_column_kernel(m, tokens)
    y_w, dx_w = m.reverse_matmul(xd, True), m.reverse_matmul(dyd, False)
    monkeypatch.delenv("PBS_COLUMN_KERNEL", raising=False)
    for a, b, what in ((y, y_w, "fwd"), (dx, dx_w, "dx")):
        diff = (a.float() - b.float()).abs()
        # one bf16 rounding step apart at most
        assert (diff <= 2.0 ** -7 * torch.maximum(a.float().abs(), b.float().abs()) + 1e-6).all(), what
        assert (diff == 0).float().mean().item() > 0.9, what


def test_without_workspace_the_forward_product_still_runs(cuda, column_kernel):
    """pbs_blocksparse_matmul (no workspace) stays a complete entry point: the forward product then comes from a
    kernel that reads the data as stored."""
    import ctypes

    m = _matrix(512, 256, None, 60, cuda, seed=2)
    out_f, in_f = m.shape
    nnz = m.cols_a.shape[0]
    tokens = 700
    g = torch.Generator().manual_seed(8)
    x = torch.randn((tokens, in_f), generator=g).to(BF16).to(cuda)
    lib = native.load()
    plan = native.blocksparse_matmul_plan(m.row_start_ends_a, m.cols_a, out_f, in_f)
    out = torch.empty((tokens, out_f), dtype=BF16, device=cuda)
    vp = lambda t: ctypes.c_void_p(t.data_ptr())
    rc = lib.pbs_blocksparse_matmul(vp(x), vp(m.data), vp(plan), None, vp(out), tokens, out_f, in_f, nnz, 1, 1,
                                    ctypes.c_void_p(torch.cuda.current_stream().cuda_stream))
    assert rc == 0
    y = m.reverse_matmul(x, True)   # with workspace: the column kernel
    coo = m.build_coo_block_index().cpu().numpy()
    y_ref = to64(x) @ O.to_dense(to64(m.data), coo, (out_f, in_f)).T
    assert_close(out, y_ref, BF16, "no workspace")
    assert_close(y, y_ref, BF16, "workspace")


def test_sparse_wide_layer_takes_the_column_kernel_by_itself(cuda, monkeypatch):
    """2048 -> 2048 at density 0.06 (4 blocks per column), 8229 tokens: a result of 2048 columns and a contraction of
    32 k-pairs go to the column kernel without being forced, in both directions; checked against the oracle in full."""
    monkeypatch.delenv("PBS_COLUMN_KERNEL", raising=False)
    out_f = in_f = 2048
    tokens = 8192 + 37
    m = _matrix(out_f, in_f, None, int(0.06 * 64 * 64), cuda, seed=12)
    name = native.matmul_kernel_name(tokens, out_f, in_f, m.cols_a.shape[0], True, BF16)
    assert "ddsc" in name, name
    name = native.matmul_kernel_name(tokens, in_f, out_f, m.cols_a.shape[0], False, BF16)
    assert "ddsc" in name, name
    _check_both_directions(m, tokens, cuda, 5, "sparse wide layer", bias=True)
    # a result of 1024 columns at the same density stays with the other kernels
    assert "ddsc" not in native.matmul_kernel_name(16384, 1024, 4096, int(0.06 * 32 * 128), True, BF16)
