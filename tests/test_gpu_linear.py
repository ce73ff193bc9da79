"""BlockSparseLinear, the patcher and the pattern tools on the GPU, against dense twins.

Procedure of the reference's tests/test_linear_nn.py (:16-134): train the sparse layer and a
dense-masked twin side by side with Adam and compare outputs, input gradients and weight
gradients at every step; plus save/load (tests/test_save.py), block_replace followed by products
(tests/test_replace.py:140-161), the patcher (tests/test_integration.py) and SparseOptimizer.
"""
import io

import numpy as np
import pytest
import torch

from oracle import block_sparse_oracle as O
from pytorch_block_sparse_amd import (
    BlockSparseLinear,
    BlockSparseMatrix,
    BlockSparseModelPatcher,
    SparseOptimizer,
)
from pytorch_block_sparse_amd.block_sparse_linear import PseudoBlockSparseLinear
from tests.helpers import assert_close, to64

pytestmark = pytest.mark.gpu


# 40 steps in fp32 as in the reference (tests/test_linear_nn.py:16-134)
@pytest.mark.parametrize("dtype,steps", [(torch.float32, 40), (torch.bfloat16, 3)])
def test_training_matches_dense_twin(cuda, dtype, steps):
    np.random.seed(0)
    torch.manual_seed(0)
    layer = BlockSparseLinear(256, 192, True, density=0.4, device=cuda, dtype=dtype)
    with torch.no_grad():
        layer.bias.normal_()
    twin = PseudoBlockSparseLinear(layer).to(cuda)  # dense weight * mask, plain torch
    twin.weight.data = twin.weight.data.float()
    twin.bias.data = twin.bias.data.float()
    opt_s = torch.optim.Adam(layer.parameters(), lr=1e-2)
    opt_d = torch.optim.Adam(twin.parameters(), lr=1e-2)
    for step in range(steps):
        g = torch.Generator().manual_seed(step)
        x = torch.randn((4, 33, 256), generator=g).to(cuda)
        target = torch.randn((4, 33, 192), generator=g).to(cuda)
        xs = x.to(dtype).requires_grad_(True)
        xd = x.to(dtype).float().requires_grad_(True)
        ys = layer(xs)
        with torch.no_grad():
            # the twin follows the sparse layer's (possibly bf16-rounded) parameters exactly
            twin.weight.copy_(layer.weight.to_dense().float())
            twin.bias.copy_(layer.bias.float())
        yd = twin(xd)
        assert ys.shape == (4, 33, 192) and ys.dtype == dtype
        assert_close(ys, to64(yd), dtype, f"step {step} output")
        (ys.float() - target).pow(2).mean().backward()
        (yd - target).pow(2).mean().backward()
        if dtype == torch.float32:
            assert_close(xs.grad, to64(xd.grad), dtype, f"step {step} grad_input")
            gw = layer.weight.to_dense(data_replace=layer.weight.data.grad)
            assert_close(gw, to64(twin.weight.grad * twin.mask), dtype, f"step {step} grad_weight")
            assert_close(layer.bias.grad, to64(twin.bias.grad), dtype, f"step {step} grad_bias")
        else:
            # bf16: the upstream gradient is rounded differently in the two graphs, so the gradients are
            # only checked for sanity here; test_autograd_function_against_oracle checks them exactly
            assert torch.isfinite(xs.grad.float()).all() and torch.isfinite(layer.weight.data.grad.float()).all()
        opt_s.step()
        opt_d.step()
        opt_s.zero_grad()
        opt_d.zero_grad()


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_autograd_function_against_oracle(cuda, dtype):
    np.random.seed(1)
    torch.manual_seed(1)
    layer = BlockSparseLinear(320, 96, True, density=0.3, device=cuda, dtype=dtype)
    with torch.no_grad():
        layer.bias.normal_()
    x = torch.randn(2, 3, 37, 320, device=cuda).to(dtype).requires_grad_(True)
    y = layer(x)
    dy = torch.randn_like(y)
    y.backward(dy)
    coo = layer.weight.build_coo_block_index().cpu().numpy()
    y_ref, dx_ref, dw_ref = O.linear_fwd_bwd(to64(x), to64(dy), to64(layer.weight.data), coo, (96, 320))
    assert_close(y, y_ref + to64(layer.bias), dtype, "y")
    assert_close(x.grad, dx_ref, dtype, "dx")
    assert_close(layer.weight.data.grad, dw_ref, dtype, "dw")
    assert_close(layer.bias.grad, to64(dy).reshape(-1, 96).sum(0), dtype, "dbias")
    # no grad for the input -> no dX product, still a weight gradient
    layer.zero_grad()
    y2 = layer(x.detach())
    y2.backward(dy)
    assert_close(layer.weight.data.grad, dw_ref, dtype, "dw without dx")


def test_non_contiguous_operands(cuda):
    """reference tests/test_matmul_back.py:32-36, :226-227: every memory order of the two operands."""
    np.random.seed(2)
    torch.manual_seed(2)
    m = BlockSparseMatrix.randn((128, 96), 5, device=cuda)
    coo = m.build_coo_block_index().cpu().numpy()
    a = torch.randn(70, 96, device=cuda)
    b = torch.randn(70, 128, device=cuda)
    ref = O.matmul_with_output_sparse_support(to64(b), to64(a), coo, (128, 96))
    for nca in (False, True):
        for ncb in (False, True):
            aa = a.t().contiguous().t() if nca else a
            bb = b.t().contiguous().t() if ncb else b
            assert aa.is_contiguous() != nca and bb.is_contiguous() != ncb
            assert_close(m.matmul_with_output_sparse_support(bb, aa), ref, torch.float32, f"dw nc={nca},{ncb}")
    y_ref = O.reverse_matmul(to64(a), to64(m.data), coo, (128, 96), True)
    assert_close(m.reverse_matmul(a.t().contiguous().t(), True), y_ref, torch.float32, "fwd strided")
    # overwrite_data=True writes into the matrix itself (reference :626-629)
    m.matmul_with_output_sparse_support(b, a, overwrite_data=True)
    assert_close(m.data, ref, torch.float32, "overwrite")


def test_block_replace_then_products(cuda):
    """reference tests/test_replace.py:140-161."""
    torch.manual_seed(3)
    m = BlockSparseMatrix.randn((128, 64), None, blocks=[(0, 0), (1, 0), (2, 0), (0, 1)], device=cuda, positive=True)
    a = torch.randn((1, 64), device=cuda).abs()
    y0 = m.reverse_matmul(a, transpose=True)           # builds the plan of the old pattern
    m.block_replace(torch.tensor([(3, 1, 0), (2, 1, 2), (1, 1, 1)]))
    d = m.to_dense()
    y = m.reverse_matmul(a, transpose=True)             # must use a plan of the new pattern
    assert torch.allclose(y, a @ d.t(), rtol=1e-5, atol=1e-6)
    assert not torch.allclose(y, y0)
    b = torch.randn((1, 128), device=cuda).abs()
    m.matmul_with_output_sparse_support(b, a, overwrite_data=True)
    back = m.to_dense()
    expect = (b.t() @ a) * m.to_dense(data_replace=torch.ones_like(m.data))
    assert torch.allclose(back, expect, rtol=1e-5, atol=1e-6)


def test_save_load_and_device_moves(cuda):
    np.random.seed(4)
    torch.manual_seed(4)
    a = BlockSparseLinear(64, 128, True, density=0.5, device=cuda)
    x = torch.randn(9, 64, device=cuda)
    ya = a(x)
    buf = io.BytesIO()
    torch.save(a.state_dict(), buf)
    buf.seek(0)
    b = BlockSparseLinear(64, 128, True, density=0.5, device=cuda)
    yb0 = b(x)  # plan of b's own pattern is now cached
    b.load_state_dict(torch.load(buf, weights_only=True))
    assert torch.equal(b(x), ya) and not torch.equal(yb0, ya)
    # built on the host, moved to the GPU afterwards
    c = BlockSparseLinear(64, 128, True, density=0.5, device="cpu")
    c.load_state_dict({k: v.cpu() for k, v in a.state_dict().items()})
    c = c.to(cuda)
    assert torch.equal(c(x), ya)


def test_patched_model_trains_and_sparse_optimizer(cuda, capsys):
    np.random.seed(5)
    torch.manual_seed(5)
    model = torch.nn.Sequential()
    model.add_module("inp", torch.nn.Linear(64, 128))
    model.add_module("act", torch.nn.GELU())
    model.add_module("mid", torch.nn.Linear(128, 256))
    model.add_module("act2", torch.nn.GELU())
    model.add_module("out", torch.nn.Linear(256, 32))
    model = model.to(cuda)
    mp = BlockSparseModelPatcher()
    mp.add_pattern("mid", {"density": 0.5})
    mp.patch_model(model)
    assert isinstance(model.mid, BlockSparseLinear) and model.mid.weight.data.is_cuda
    opt = torch.optim.Adam(model.parameters(), lr=1e-3)
    so = SparseOptimizer(SparseOptimizer.sparse_objects(model), lr=0.25)
    so.attach_optimizer(opt)
    x = torch.randn(50, 64, device=cuda)
    t = torch.randn(50, 32, device=cuda)
    losses = []
    for step in range(6):
        loss = (model(x) - t).pow(2).mean()
        loss.backward()
        opt.step()
        opt.zero_grad()
        losses.append(loss.item())
        if step == 2:
            before = model.mid.weight.block_mask_build(None).clone()
            so.step()
            after = model.mid.weight.block_mask_build(None)
            assert int((before != after).sum()) == 2 * int(0.25 * model.mid.block_count)
            d = model.mid.weight.to_dense()
            y = model.mid.weight.reverse_matmul(x @ model.inp.weight.t(), True)
            assert torch.allclose(y, (x @ model.inp.weight.t()) @ d.t(), rtol=1e-4, atol=1e-4)
    assert all(np.isfinite(losses)) and losses[-1] < losses[0]


def test_magnitude_strategy_on_the_device(cuda):
    """MagnitudeSparseOptimizerStrategy.run with the matrix on the GPU (reference sparse_optimizer.py:38-87): the
    blocks it drops are exactly the lowest-norm ones, the positions it fills were empty and are distinct, the blocks it
    keeps stay where they were with their values, the regrown blocks get the new values, and the choice of
    positions is random under the device generator's seed."""
    from pytorch_block_sparse_amd.sparse_optimizer import MagnitudeSparseOptimizerStrategy

    def one(seed, distribution):
        np.random.seed(11)
        torch.manual_seed(11)
        m = BlockSparseMatrix.randn((512, 384), 70, device=cuda)
        with torch.no_grad():   # distinct block norms
            m.data.mul_(torch.linspace(0.5, 2.0, 70, device=cuda).repeat_interleave(32).unsqueeze(1))
        norms = m.block_norm().clone()
        pos0 = m.build_coo_block_index().t().clone()    # (row, column) by data block
        data0 = m.data.detach().clone()
        mask0 = m.block_mask_build(None).clone()
        torch.manual_seed(seed)
        keep = MagnitudeSparseOptimizerStrategy(0.2, distribution, 0.1).run(m)
        return m, norms, pos0, data0, mask0, keep

    m, norms, pos0, data0, mask0, keep = one(1, "gaussian")
    k = int(70 * 0.2)
    dropped = norms.sort()[1][:k]
    kept = norms.sort()[1][k:]
    pos1 = m.build_coo_block_index().t()
    assert torch.equal(pos1[kept], pos0[kept])                       # kept blocks did not move
    new_pos = pos1[dropped]
    assert not mask0[new_pos[:, 0], new_pos[:, 1]].any()             # regrown where nothing was
    assert torch.unique(new_pos[:, 0] * 12 + new_pos[:, 1]).numel() == k
    assert int(m.block_mask_build(None).sum()) == 70
    d0, d1 = data0.view(70, -1), m.data.detach().view(70, -1)
    assert torch.equal(d1[kept], d0[kept])                           # nor did their values change
    fresh = d1[dropped]
    assert abs(fresh.std().item() / (0.1 * data0.std().item()) - 1.0) < 0.05
    assert torch.equal(keep.view(70, -1)[:, 0] == 0, torch.isin(torch.arange(70, device=cuda), dropped))
    m.check_with_dense(m.to_dense())
    # the reference's "uniform" is the constant -std * scale (random_(0, 1) only draws 0)
    mu, _, _, data0u, _, _ = one(1, "uniform")
    assert torch.allclose(mu.data.detach().view(70, -1)[dropped], (-0.1 * data0u.std()).expand(k, 1024), rtol=1e-5)
    # same seed, same choice; another seed, another choice
    again = one(1, "gaussian")[0].build_coo_block_index().t()[dropped]
    other = one(2, "gaussian")[0].build_coo_block_index().t()[dropped]
    assert torch.equal(again, new_pos) and not torch.equal(other, new_pos)


def test_roberta_patched_at_full_density_keeps_outputs(cuda):
    """reference tests/test_integration.py:66-113 (test1), two encoder layers instead of six: patching the
    feed-forward linears of a RoBERTa masked-LM model at density 1.0 keeps parameter count and logits;
    at density 0.5 the patched weights halve."""
    transformers = pytest.importorskip("transformers")
    torch.manual_seed(3)
    np.random.seed(3)
    config = transformers.RobertaConfig(vocab_size=52_000, max_position_embeddings=514, num_attention_heads=12,
                                        num_hidden_layers=2, type_vocab_size=1)
    patterns = [r"roberta\.encoder\.layer\.[0-9]+.intermediate\.dense", r"roberta\.encoder\.layer\.[0-9]+.output\.dense"]

    def patch(model, density):
        mp = BlockSparseModelPatcher()
        for p in patterns:
            mp.add_pattern(p, {"density": density})
        mp.patch_model(model)
        return model

    model = transformers.RobertaForMaskedLM(config=config).to(cuda).eval()
    n0 = model.num_parameters()
    input_ids = torch.tensor([[4, 5, 6, 7] * 8], device=cuda)
    with torch.no_grad():
        out0 = model(input_ids)[0]
        patch(model, 1.0)
        out1 = model(input_ids)[0]
    assert sum(isinstance(m, BlockSparseLinear) for m in model.modules()) == 4
    assert model.num_parameters() == n0
    assert torch.isclose(out0, out1, atol=1e-3).all()
    model2 = patch(transformers.RobertaForMaskedLM(config=config).to(cuda).eval(), 0.5)
    with torch.no_grad():
        assert torch.isfinite(model2(input_ids)[0]).all()
    assert model2.num_parameters() == n0 - 4 * (768 * 3072 // 2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_hip_graph_capture_and_replay(cuda, dtype):
    """The three products launch on the current stream and use no memset or host synchronisation, so a
    forward + backward of the layer can be captured in a HIP graph.  Every replay, with new inputs copied
    into the static buffers and eager work in between, must reproduce the eager result."""
    torch.manual_seed(2)
    np.random.seed(2)
    layer = BlockSparseLinear(256, 384, True, 0.4, device=cuda, dtype=dtype)
    x_static = torch.randn(200, 256, device=cuda).to(dtype).requires_grad_(True)
    gy_static = torch.randn(200, 384, device=cuda).to(dtype)

    def run(x, gy):
        y = layer(x)
        gx, gw, gb = torch.autograd.grad(y, [x, layer.weight.data, layer.bias], gy)
        return y, gx, gw, gb

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        for _ in range(3):   # warm-up on the side stream: plans are built, allocator pools are primed
            run(x_static, gy_static)
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        outs_static = run(x_static, gy_static)
    for i in range(4):
        g = torch.Generator().manual_seed(100 + i)
        x_new = torch.randn(200, 256, generator=g).to(dtype).to(cuda)
        gy_new = torch.randn(200, 384, generator=g).to(dtype).to(cuda)
        with torch.no_grad():
            x_static.copy_(x_new)
            gy_static.copy_(gy_new)
        graph.replay()
        torch.cuda.synchronize()
        got = [o.clone() for o in outs_static]
        ref = run(x_new.clone().requires_grad_(True), gy_new)   # eager, between the replays
        torch.cuda.synchronize()
        for a, b in zip(got, ref):
            assert torch.equal(a, b)
