"""GPU parity of the three block-sparse matmuls against the dense-equivalent CPU oracle.

Layouts and shapes follow the reference's tests/test_matmul.py (:141-244 tiny layouts, 1 token,
3-D/4-D leading dims; :246-305 1024 -> 2048 at density 0.42 and 1.0) and tests/test_matmul_back.py
(:205-277), plus the benchmark configurations.  Operands are signed N(0,1) (the reference uses
positive operands so that isclose has no cancellation; here the absolute floor in assert_close
plays that role).
"""
import numpy as np
import pytest
import torch

from oracle import block_sparse_oracle as O
from pytorch_block_sparse_amd import BlockSparseMatrix, workloads
from tests.helpers import assert_close, to64

pytestmark = pytest.mark.gpu

TINY = [
    # (lead dims of a, in_features, out_features, blocks)
    ((32,), 32, 32, [(0, 0)]),
    ((32,), 64, 32, [(0, 0)]),
    ((64,), 32, 32, [(0, 0)]),
    ((128,), 32, 32, [(0, 0)]),
    ((128,), 64, 32, [(0, 0)]),
    ((128,), 64, 32, [(0, 1)]),
    ((128,), 64, 32, [(0, 0), (0, 1)]),
    ((32,), 32, 64, [(0, 0)]),
    ((32,), 32, 64, [(1, 0)]),
    ((32,), 32, 64, [(0, 0), (1, 0)]),
    ((64, 32), 32, 64, [(0, 0), (1, 0)]),
    ((4, 8, 32), 128, 256, [(0, 0), (1, 0)]),
    ((32,), 64, 64, [(0, 0), (1, 0), (0, 1)]),
    ((32,), 64, 128, [(0, 0), (1, 0), (0, 1), (2, 0)]),
    ((1,), 32, 32, [(0, 0)]),
    ((1,), 64, 128, [(0, 0), (1, 0), (0, 1), (2, 0)]),
    ((33,), 64, 128, [(0, 0), (1, 0), (0, 1), (2, 0)]),
    ((77,), 96, 64, [(1, 2), (0, 0)]),
]


def _matrix(out_f, in_f, blocks, n_blocks, dtype, device, seed):
    np.random.seed(seed)
    torch.manual_seed(seed)
    m = BlockSparseMatrix.randn((out_f, in_f), n_blocks, blocks=blocks, device="cpu", dtype=dtype)
    return m.to(device)


def _check_all(m, lead, dtype, device, seed, what):
    out_f, in_f = m.shape
    g = torch.Generator().manual_seed(seed + 1)
    x = torch.randn(lead + (in_f,), generator=g).to(dtype)
    dy = torch.randn(lead + (out_f,), generator=g).to(dtype)
    coo = m.build_coo_block_index().cpu().numpy()
    y_ref, dx_ref, dw_ref = O.linear_fwd_bwd(to64(x), to64(dy), to64(m.data), coo, tuple(m.shape))
    xd, dyd = x.to(device), dy.to(device)
    y = m.reverse_matmul(xd, transpose=True)
    assert y.shape == lead + (out_f,)
    assert_close(y, y_ref, dtype, what + " fwd")
    dx = m.reverse_matmul(dyd, transpose=False)
    assert dx.shape == lead + (in_f,)
    assert_close(dx, dx_ref, dtype, what + " dx")
    dw = m.matmul_with_output_sparse_support(dyd, xd)
    assert dw.shape == m.data.shape
    assert_close(dw, dw_ref, dtype, what + " dw")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_tiny_layouts(cuda, dtype):
    for i, (lead, in_f, out_f, blocks) in enumerate(TINY):
        print(f"tiny[{i}] lead={lead} {in_f}->{out_f} blocks={blocks} {dtype}", flush=True)
        m = _matrix(out_f, in_f, blocks, None, dtype, cuda, seed=i)
        _check_all(m, lead, dtype, cuda, i, f"tiny[{i}]")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("density", [0.42, 1.0, 0.05])
@pytest.mark.parametrize("tokens", [1, 200, 1024])
def test_1024_to_2048(cuda, dtype, density, tokens):
    """reference: tests/test_matmul.py:246-305 shape (1024 -> 2048), tokens reduced to what the oracle does in seconds."""
    print(f"1024->2048 d={density} tokens={tokens} {dtype}", flush=True)
    n_blocks = int(density * 32 * 64)
    m = _matrix(2048, 1024, None, n_blocks, dtype, cuda, seed=7)
    _check_all(m, (tokens,), dtype, cuda, 11, f"d={density} t={tokens}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_empty_rows_and_columns(cuda, dtype):
    """Block rows / columns without any block must come out as exact zeros (no pre-zeroed output)."""
    m = _matrix(256, 192, [(1, 0), (1, 5), (6, 5)], None, dtype, cuda, seed=3)
    x = torch.randn((100, 192), device=cuda).to(dtype)
    y = m.reverse_matmul(x, transpose=True)
    assert (y[:, :32] == 0).all() and (y[:, 64:192] == 0).all() and (y[:, 224:] == 0).all()
    dy = torch.randn((100, 256), device=cuda).to(dtype)
    dx = m.reverse_matmul(dy, transpose=False)
    assert (dx[:, 32:160] == 0).all()
    _check_all(m, (100,), dtype, cuda, 5, "empty rows")


@pytest.mark.parametrize("name", ["c1_1024x256_d0.1_fp32", "c2_768x3072_d0.5_fp32", "c3_3072x768_d0.25_zipf_fp32"])
def test_benchmark_configs_fp32(cuda, name):
    w = workloads.WORKLOADS[name]
    print(name, flush=True)
    blocks, data, x, dy = workloads.make_inputs(w)
    assert len(blocks) == w.nnz
    m = BlockSparseMatrix.zeros((w.out_features, w.in_features), blocks=blocks, device="cpu", dtype=w.dtype)
    with torch.no_grad():
        # make_inputs lists blocks in row-major order, which is the data-block order
        m.data.copy_(data)
    m = m.to(cuda)
    coo = m.build_coo_block_index().cpu().numpy()
    y_ref, dx_ref, dw_ref = O.linear_fwd_bwd(to64(x), to64(dy), to64(data), coo, tuple(m.shape))
    xd, dyd = x.to(cuda), dy.to(cuda)
    assert_close(m.reverse_matmul(xd, True), y_ref, w.dtype, name + " fwd")
    assert_close(m.reverse_matmul(dyd, False), dx_ref, w.dtype, name + " dx")
    assert_close(m.matmul_with_output_sparse_support(dyd, xd), dw_ref, w.dtype, name + " dw")


def test_benchmark_config_bf16_reduced_tokens(cuda):
    """4096 -> 4096, density 0.25, bf16: oracle-checked on the first 2048 tokens of the workload."""
    w = workloads.WORKLOADS["c4_4096x4096_d0.25_bf16"]
    blocks, data, x, dy = workloads.make_inputs(w, tokens=2048)
    m = BlockSparseMatrix.zeros((w.out_features, w.in_features), blocks=blocks, device="cpu", dtype=w.dtype)
    with torch.no_grad():
        m.data.copy_(data)
    m = m.to(cuda)
    coo = m.build_coo_block_index().cpu().numpy()
    y_ref, dx_ref, dw_ref = O.linear_fwd_bwd(to64(x), to64(dy), to64(data), coo, tuple(m.shape))
    xd, dyd = x.to(cuda), dy.to(cuda)
    assert_close(m.reverse_matmul(xd, True), y_ref, w.dtype, "c4 fwd")
    assert_close(m.reverse_matmul(dyd, False), dx_ref, w.dtype, "c4 dx")
    assert_close(m.matmul_with_output_sparse_support(dyd, xd), dw_ref, w.dtype, "c4 dw")


def test_benchmark_config_bf16_full_size_properties(cuda):
    """Full 16384-token bf16 workload through size-independent properties.

    * adjoint identity: <dY, X W^T> == <dY W, X> == <dW, W> (all three kernels tie together);
    * token additivity of dW: dW(all tokens) == dW(first half) + dW(second half);
    * row independence of fwd: rows of Y computed in the full call equal those of a call on a shifted token range bit for
      bit, and those of a 512-token call (another kernel) to one bf16 rounding step.
    """
    w = workloads.WORKLOADS["c4_4096x4096_d0.25_bf16"]
    blocks, data, x, dy = workloads.make_inputs(w)
    m = BlockSparseMatrix.zeros((w.out_features, w.in_features), blocks=blocks, device="cpu", dtype=w.dtype)
    with torch.no_grad():
        m.data.copy_(data)
    m = m.to(cuda)
    xd, dyd = x.to(cuda), dy.to(cuda)
    y = m.reverse_matmul(xd, True)
    dx = m.reverse_matmul(dyd, False)
    dw = m.matmul_with_output_sparse_support(dyd, xd)
    a = (dyd.double() * y.double()).sum().item()
    b = (dx.double() * xd.double()).sum().item()
    c = (dw.double() * m.data.double()).sum().item()
    scale = (dyd.double().norm() * y.double().norm()).item()
    print("adjoint", a, b, c, scale, flush=True)
    # each side carries bf16 output rounding (2^-9 relative per element, random sign)
    assert abs(a - b) < 2e-3 * scale and abs(a - c) < 2e-3 * scale
    half = w.tokens // 2
    dw1 = m.matmul_with_output_sparse_support(dyd[:half], xd[:half])
    dw2 = m.matmul_with_output_sparse_support(dyd[half:], xd[half:])
    ref = dw1.double() + dw2.double()
    err = (dw.double() - ref).abs().max().item()
    assert err < 3 * 2.0 ** -8 * ref.abs().max().item(), err
    # rows do not depend on where they sit in a call: the same kernel on a token range shifted by 96 rows (other tiles,
    # other places in them) gives the same bits ...
    y_shift = m.reverse_matmul(xd[96:], True)
    assert torch.equal(y_shift, y[96:])
    # ... and a 512-token call, which another kernel serves (other summation order of the same fp32 products), agrees
    # to one bf16 rounding step
    y_small = m.reverse_matmul(xd[1024:1536], True)
    a_, b_ = y_small.float(), y[1024:1536].float()
    assert ((a_ - b_).abs() <= 2.0 ** -7 * torch.maximum(a_.abs(), b_.abs()) + 1e-6).all()
    assert (a_ == b_).float().mean().item() > 0.9


# Shapes that the wide-tile persistent bf16 kernel serves (at least 256 tiles of 128 tokens x 512
# result columns, contraction size a multiple of 64): one k-pair per tile, token tail, a last column
# group with a single block column, full density (every step fills the block ring), persistence over
# several token tiles.
@pytest.mark.parametrize("in_f,out_f,tokens,density", [
    (64, 512, 32768 + 5, 0.5),
    (128, 1056, 11011, 1.0),
    (512, 2048, 8192 + 77, 0.3),
    (320, 512, 33000, 0.07),
])
def test_wide_tile_kernel_shapes(cuda, in_f, out_f, tokens, density):
    print(f"wide {in_f}->{out_f} d={density} tokens={tokens}", flush=True)
    n_blocks = max(1, int(density * (in_f // 32) * (out_f // 32)))
    m = _matrix(out_f, in_f, None, n_blocks, torch.bfloat16, cuda, seed=21)
    _check_all(m, (tokens,), torch.bfloat16, cuda, 23, f"wide {in_f}->{out_f} d={density}")


def test_wide_tile_kernel_empty_group_and_bias(cuda):
    """Blocks only in the first 8 block rows of W: the second group of 16 result columns has no block."""
    in_f, out_f, tokens = 256, 1024, 16384 + 130
    rng = np.random.RandomState(5)
    blocks = sorted({(int(r), int(c)) for r, c in zip(rng.randint(0, 8, 40), rng.randint(0, 8, 40))})
    m = _matrix(out_f, in_f, blocks, None, torch.bfloat16, cuda, seed=9)
    g = torch.Generator().manual_seed(4)
    x = torch.randn((tokens, in_f), generator=g).to(torch.bfloat16)
    bias = torch.randn((out_f,), generator=g).to(torch.bfloat16)
    coo = m.build_coo_block_index().cpu().numpy()
    w_dense = O.to_dense(to64(m.data), coo, (out_f, in_f))
    y_ref = to64(x) @ w_dense.T
    xd = x.to(cuda)
    y = m.reverse_matmul(xd, True)
    assert (y[:, 256:] == 0).all()
    assert_close(y, y_ref, torch.bfloat16, "empty group fwd")
    yb = m.reverse_matmul(xd, True, bias=bias.to(cuda))
    assert_close(yb, y_ref + to64(bias)[None, :], torch.bfloat16, "empty group fwd + bias")
    assert torch.equal(yb[:, 256:], bias.to(cuda)[None, 256:].expand(tokens, -1))


def test_benchmark_config_bf16_4096_tokens(cuda):
    """4096 -> 4096, density 0.25, bf16 at 4096 tokens: the smallest token count of this layer that runs
    the wide-tile kernel in both directions; oracle-checked in full."""
    w = workloads.WORKLOADS["c4_4096x4096_d0.25_bf16"]
    blocks, data, x, dy = workloads.make_inputs(w, tokens=4096)
    m = BlockSparseMatrix.zeros((w.out_features, w.in_features), blocks=blocks, device="cpu", dtype=w.dtype)
    with torch.no_grad():
        m.data.copy_(data)
    coo = m.build_coo_block_index().numpy()
    y_ref, dx_ref, dw_ref = O.linear_fwd_bwd(to64(x), to64(dy), to64(data), coo, tuple(m.shape))
    m = m.to(cuda)
    xd, dyd = x.to(cuda), dy.to(cuda)
    assert_close(m.reverse_matmul(xd, True), y_ref, w.dtype, "c4/4096 fwd")
    assert_close(m.reverse_matmul(dyd, False), dx_ref, w.dtype, "c4/4096 dx")
    assert_close(m.matmul_with_output_sparse_support(dyd, xd), dw_ref, w.dtype, "c4/4096 dw")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_uneven_rows_use_balanced_column_groups(cuda, dtype):
    """Very uneven block counts per row of W (and, transposed, per column): the result's block columns
    are regrouped by count.  Values, the fused bias and untouched columns must not notice."""
    out_f, in_f, tokens = 13 * 32, 10 * 32, 300
    blocks = [(0, c) for c in range(10)] + [(1, c) for c in range(0, 10, 2)] + [(r, (3 * r) % 10) for r in range(2, 12)]
    m = _matrix(out_f, in_f, blocks, None, dtype, cuda, seed=13)   # block row 12 of W is empty
    _check_all(m, (tokens,), dtype, cuda, 17, "uneven rows")
    g = torch.Generator().manual_seed(6)
    x = torch.randn((tokens, in_f), generator=g).to(dtype)
    bias = torch.randn((out_f,), generator=g).to(dtype)
    coo = m.build_coo_block_index().cpu().numpy()
    w_dense = O.to_dense(to64(m.data), coo, (out_f, in_f))
    yb = m.reverse_matmul(x.to(cuda), True, bias=bias.to(cuda))
    assert_close(yb, to64(x) @ w_dense.T + to64(bias)[None, :], dtype, "uneven rows fwd + bias")
    assert torch.equal(yb[:, 12 * 32:], bias.to(cuda)[None, 12 * 32:].expand(tokens, -1))


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_long_contraction(cuda, dtype):
    """A contraction of 32768 features (a 4096 -> 32000-class layer's input gradient): the schedule records of a
    column group no longer fit in LDS beside the larger tile shapes' rings, and the library has to fall
    through to a shape that fits instead of refusing (the reference has no such limit)."""
    big, small, tokens = 32768, 64, 40
    np.random.seed(17)
    # out = big: the input gradient contracts over 32768; in = big: the forward does
    for out_f, in_f in ((big, small), (small, big)):
        n_blocks = 96
        print(f"long contraction {in_f}->{out_f} {dtype}", flush=True)
        m = _matrix(out_f, in_f, None, n_blocks, dtype, cuda, seed=17)
        _check_all(m, (tokens,), dtype, cuda, 17, f"{in_f}->{out_f}")


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("cols,tokens", [(24, 4096), (24, 16384), (40, 4096), (50, 4096), (13, 16384), (5, 2048)])
def test_column_groups_of_fewer_than_eight(cuda, dtype, cols, tokens):
    """Results with few block columns against many tokens: the library regroups the block columns 7, 6 or 5 to
    a tile (24 columns in 4 groups of 6, 40 in 8 groups of 5, 50 in 8 groups of 7 minus a ragged last one) when
    that gives every CU a tile.  Values, bias and ragged last groups must not notice which grouping ran;
    both directions, so the regrouped side is once the output features and once the input features."""
    wide, narrow = cols * 32, 8 * 32
    for out_f, in_f in ((wide, narrow), (narrow, wide)):
        print(f"column groups {in_f}->{out_f} tokens {tokens} {dtype}", flush=True)
        m = _matrix(out_f, in_f, None, max(1, (out_f // 32) * (in_f // 32) // 2), dtype, cuda, seed=cols)
        _check_all(m, (tokens,), dtype, cuda, cols + 1, f"{in_f}->{out_f}@{tokens}")
    g = torch.Generator().manual_seed(cols)
    x = torch.randn((tokens, narrow), generator=g).to(dtype)
    bias = torch.randn((wide,), generator=g).to(dtype)
    m = _matrix(wide, narrow, None, cols * 4, dtype, cuda, seed=cols + 2)
    coo = m.build_coo_block_index().cpu().numpy()
    w_dense = O.to_dense(to64(m.data), coo, (wide, narrow))
    yb = m.reverse_matmul(x.to(cuda), True, bias=bias.to(cuda))
    assert_close(yb, to64(x) @ w_dense.T + to64(bias)[None, :], dtype, "fwd + bias")


def test_weight_gradient_equal_shares_on_uneven_patterns(cuda):
    """The fp32 weight-gradient kernel cuts each band of 16 block rows into shares of equal block count and sizes
    the shares for a uniform pattern.  Patterns that are far from uniform take its slow paths, which must still be
    exact: (a) a share that spans more block columns than its X panel holds is done in several column windows;
    (b) a band much denser than the average gives shares with more blocks than a workgroup has accumulators
    for, done in several passes; (c) a share boundary inside a block column splits that column between two
    workgroups.  Ragged token counts on top (the last chunk is padded with zeros in LDS)."""
    dtype = torch.float32
    # (a) 16 x 256 block positions: 8 full columns, then one block in every other column
    blocks_a = [(r, c) for c in range(8) for r in range(16)] + [((c * 7) % 16, c) for c in range(8, 256, 2)]
    # (b) 64 x 32: the first band full, one block per row below it
    blocks_b = [(r, c) for r in range(16) for c in range(32)] + [(r, (5 * r) % 32) for r in range(16, 64)]
    # (c) 16 x 6, every position present, 96 blocks: shares cut columns in the middle
    blocks_c = [(r, c) for r in range(16) for c in range(6)]
    for name, grid, blocks, tokens in (("windows", (16, 256), blocks_a, 209), ("passes", (64, 32), blocks_b, 333),
                                       ("split columns", (16, 6), blocks_c, 4099)):
        print(f"equal shares: {name}", flush=True)
        m = _matrix(grid[0] * 32, grid[1] * 32, blocks, None, dtype, cuda, seed=len(blocks))
        _check_all(m, (tokens,), dtype, cuda, 23, name)


def test_benchmark_shape_fp32_4096(cuda):
    """4096 -> 4096, density 0.25, fp32 (the headline shape in the reference's dtype): oracle-checked on the first
    3072 tokens (the oracle is three dense fp64 products), and at the full 16384 tokens through the adjoint identity
    <dY, X W^T> == <dY W, X> == <dW, W> and token additivity of dW, which tie the three kernels together."""
    w = workloads.WORKLOADS["c4_4096x4096_d0.25_fp32"]
    blocks, data, x, dy = workloads.make_inputs(w)
    m = BlockSparseMatrix.zeros((w.out_features, w.in_features), blocks=blocks, device="cpu", dtype=w.dtype)
    with torch.no_grad():
        m.data.copy_(data)
    m = m.to(cuda)
    coo = m.build_coo_block_index().cpu().numpy()
    part = 3072
    y_ref, dx_ref, dw_ref = O.linear_fwd_bwd(to64(x[:part]), to64(dy[:part]), to64(data), coo, tuple(m.shape))
    xd, dyd = x.to(cuda), dy.to(cuda)
    assert_close(m.reverse_matmul(xd[:part], True), y_ref, w.dtype, "fwd")
    assert_close(m.reverse_matmul(dyd[:part], False), dx_ref, w.dtype, "dx")
    assert_close(m.matmul_with_output_sparse_support(dyd[:part], xd[:part]), dw_ref, w.dtype, "dw")
    y = m.reverse_matmul(xd, True)
    dx = m.reverse_matmul(dyd, False)
    dw = m.matmul_with_output_sparse_support(dyd, xd)
    a = (dyd.double() * y.double()).sum().item()
    b = (dx.double() * xd.double()).sum().item()
    c = (dw.double() * m.data.double()).sum().item()
    scale = (dyd.double().norm() * y.double().norm()).item()
    print("adjoint", a, b, c, scale, flush=True)
    assert abs(a - b) < 1e-5 * scale and abs(a - c) < 1e-5 * scale
    half = w.tokens // 2
    ref = (m.matmul_with_output_sparse_support(dyd[:half], xd[:half]).double()
           + m.matmul_with_output_sparse_support(dyd[half:], xd[half:]).double())
    assert (dw.double() - ref).abs().max().item() < 1e-4 * ref.abs().max().item()
    assert torch.equal(m.reverse_matmul(xd[1024:1536], True), y[1024:1536])


def test_skewed_pattern_with_thousands_of_block_columns(cuda):
    """A result of 3500 block columns with very uneven block counts: the slot tables of all four group widths (8, 7, 6
    and 5 columns to a group; 3500 columns in groups of 5 are 700 groups = 5600 places) must each hold every block
    column exactly once, and the product must be right whichever width the launch takes."""
    out_f, in_f, tokens = 3500 * 32, 96, 40
    X, Y = out_f // 32, in_f // 32
    rng = np.random.RandomState(2)
    kind = rng.rand(X)
    blocks = []
    for r in range(X):
        if kind[r] < 0.05:
            blocks += [(r, c) for c in range(Y)]          # three blocks
        elif kind[r] < 0.75:
            blocks.append((r, int(rng.randint(Y))))       # one
    counts = np.bincount([r for r, _ in blocks], minlength=X)
    assert counts.max() * X > 2 * counts.sum()            # what the library calls skewed
    m = _matrix(out_f, in_f, blocks, None, torch.float32, cuda, seed=4)
    from pytorch_block_sparse_amd import native

    plan = native.blocksparse_matmul_plan(m.row_start_ends_a, m.cols_a, out_f, in_f).cpu().numpy()
    # the plan buffer of a contraction that is not a multiple of 64: [records, width 8][slots 8][records 7][slots 7] ...
    off = 0
    for width in (8, 7, 6, 5):
        groups = (X + width - 1) // width
        off += groups * (Y + 2) * 16          # records: header + one per k-block + sentinel, 16 ints each
        n_slots = groups * 8
        slots = plan[off:off + n_slots]
        off += (n_slots * 4 + 63) // 64 * 16
        held = np.sort(slots[slots >= 0])
        assert np.array_equal(held, np.arange(X)), f"width {width}: the slot table loses or repeats block columns"
    assert off * 4 == native.load().pbs_blocksparse_matmul_plan_bytes(out_f, in_f)
    # forward and weight gradient (the input gradient of this layer contracts over 112000 features, beyond what the
    # kernels' plan records hold in LDS)
    g = torch.Generator().manual_seed(6)
    x = torch.randn((tokens, in_f), generator=g)
    dy = torch.randn((tokens, out_f), generator=g)
    coo = m.build_coo_block_index().cpu().numpy()
    y_ref, _, dw_ref = O.linear_fwd_bwd(to64(x), to64(dy), to64(m.data), coo, tuple(m.shape))
    assert_close(m.reverse_matmul(x.to(cuda), True), y_ref, torch.float32, "3500 block columns fwd")
    assert_close(m.matmul_with_output_sparse_support(dy.to(cuda), x.to(cuda)), dw_ref, torch.float32, "3500 block columns dw")
