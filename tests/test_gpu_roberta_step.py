"""The RoBERTa-base-shaped training step with block-sparse linears (12 layers, 32 x 512 tokens, fp32).

Two parts, following the reference's tests/test_integration.py (:66-113 builds RoBERTa and patches
``intermediate.dense`` / ``output.dense``; :37-64 checks parameter counts of patched models):

* the three patched layer shapes (768 -> 768, 768 -> 3072, 3072 -> 768 at density 0.5) at the step's
  16384 tokens, all three products against the fp64 dense-equivalent oracle;
* the whole model: one forward + backward + AdamW step of the model whose ``attention.output.dense``,
  ``intermediate.dense`` and ``output.dense`` are block-sparse at density 0.5, against the same model
  patched with ``{"pseudo_linear": True}`` (dense weight x block mask in plain torch) holding identical
  weights and patterns: loss, the weight gradient of every patched layer on its support, bias gradients.
"""
import copy

import numpy as np
import pytest
import torch

from oracle import block_sparse_oracle as O
from pytorch_block_sparse_amd import BlockSparseLinear, BlockSparseMatrix, BlockSparseModelPatcher, workloads
from pytorch_block_sparse_amd.block_sparse_linear import PseudoBlockSparseLinear
from tests.helpers import assert_close, to64

pytestmark = pytest.mark.gpu

PATTERNS = (
    r"roberta\.encoder\.layer\.[0-9]+\.attention\.output\.dense",
    r"roberta\.encoder\.layer\.[0-9]+\.intermediate\.dense",
    r"roberta\.encoder\.layer\.[0-9]+\.output\.dense",
)


@pytest.mark.parametrize("name", workloads.ROBERTA_LAYER_WORKLOADS)
def test_roberta_layer_shapes_full_tokens(cuda, name):
    w = workloads.WORKLOADS[name]
    print(name, flush=True)
    assert w.tokens == 32 * 512 and w.dtype == torch.float32
    blocks, data, x, dy = workloads.make_inputs(w)
    assert len(blocks) == w.nnz == (w.in_features // 32) * (w.out_features // 32) // 2
    m = BlockSparseMatrix.zeros((w.out_features, w.in_features), blocks=blocks, device="cpu", dtype=w.dtype)
    with torch.no_grad():
        m.data.copy_(data)
    m = m.to(cuda)
    coo = m.build_coo_block_index().cpu().numpy()
    y_ref, dx_ref, dw_ref = O.linear_fwd_bwd(to64(x), to64(dy), to64(data), coo, tuple(m.shape))
    xd, dyd = x.to(cuda), dy.to(cuda)
    assert_close(m.reverse_matmul(xd, True), y_ref, w.dtype, name + " fwd")
    assert_close(m.reverse_matmul(dyd, False), dx_ref, w.dtype, name + " dx")
    assert_close(m.matmul_with_output_sparse_support(dyd, xd), dw_ref, w.dtype, name + " dw")


def _patched(base, pseudo, seed):
    """A copy of `base` with the three linears of every layer replaced; the numpy seed fixes the patterns."""
    model = copy.deepcopy(base)
    np.random.seed(seed)
    mp = BlockSparseModelPatcher()
    info = {"density": 0.5, "pseudo_linear": True} if pseudo else {"density": 0.5}
    for p in PATTERNS:
        mp.add_pattern(p, info)
    mp.patch_model(model)
    return model


def test_roberta_base_training_step_matches_pseudo_linear_twin(cuda, capsys):
    transformers = pytest.importorskip("transformers")
    batch, seq, layers, hidden, ffn, vocab = 32, 512, 12, 768, 3072, 50265
    cfg = transformers.RobertaConfig(vocab_size=vocab, hidden_size=hidden, num_hidden_layers=layers,
                                     num_attention_heads=12, intermediate_size=ffn,
                                     max_position_embeddings=seq + 2, type_vocab_size=1,
                                     hidden_dropout_prob=0.0, attention_probs_dropout_prob=0.0)
    torch.manual_seed(1)
    base = transformers.RobertaForMaskedLM(cfg).to(cuda)
    n_dense = sum(p.numel() for p in base.parameters())
    g = torch.Generator().manual_seed(0)
    ids = torch.randint(0, vocab, (batch, seq), generator=g)
    labels = ids.clone()
    labels[torch.rand((batch, seq), generator=g) >= 0.15] = -100   # 15 % of the positions are predicted
    ids, labels = ids.to(cuda), labels.to(cuda)

    sparse = _patched(base, pseudo=False, seed=5)
    twin = _patched(base, pseudo=True, seed=5)
    del base
    capsys.readouterr()   # the patcher prints one line per layer

    sparse_layers = {n: m for n, m in sparse.named_modules() if isinstance(m, BlockSparseLinear)}
    twin_layers = {n: m for n, m in twin.named_modules() if isinstance(m, PseudoBlockSparseLinear)}
    assert len(sparse_layers) == 3 * layers and sparse_layers.keys() == twin_layers.keys()
    # parameter count: every patched weight keeps half of its blocks (reference tests/test_integration.py:48-64)
    n_sparse = sum(p.numel() for p in sparse.parameters())
    assert n_sparse == n_dense - layers * (hidden * hidden + 2 * hidden * ffn) // 2
    for name, lay in sparse_layers.items():
        tw = twin_layers[name]
        assert torch.equal(lay.weight.to_dense(), tw.weight.detach() * tw.mask), name   # same weights, same pattern

    def step(model):
        model.train()
        opt = torch.optim.AdamW(model.parameters(), lr=1e-4)
        loss = model(input_ids=ids, labels=labels).loss
        loss.backward()
        grads = {}
        for name, mod in model.named_modules():
            if isinstance(mod, BlockSparseLinear):
                grads[name] = (mod.weight.to_dense(data_replace=mod.weight.data.grad).detach().clone(),
                               mod.bias.grad.detach().clone())
            elif isinstance(mod, PseudoBlockSparseLinear):
                grads[name] = ((mod.weight.grad * mod.mask).detach().clone(), mod.bias.grad.detach().clone())
        opt.step()
        opt.zero_grad(set_to_none=True)
        return float(loss.detach()), grads

    print("twin step", flush=True)
    loss_twin, g_twin = step(twin)
    print("sparse step", flush=True)
    loss_sparse, g_sparse = step(sparse)
    torch.cuda.synchronize()
    assert np.isfinite(loss_sparse)
    assert abs(loss_sparse - loss_twin) <= 1e-4 * abs(loss_twin), (loss_sparse, loss_twin)
    for name in sparse_layers:
        assert_close(g_sparse[name][0], to64(g_twin[name][0]), torch.float32, name + " weight gradient")
        assert_close(g_sparse[name][1], to64(g_twin[name][1]), torch.float32, name + " bias gradient")
    # the optimizer step moved the packed weights and kept them finite
    for name, lay in sparse_layers.items():
        tw = twin_layers[name]
        assert torch.isfinite(lay.weight.data).all()
        assert not torch.equal(lay.weight.to_dense(), tw.weight.detach() * 0)
    # after the step the two models still agree on the loss of the same batch (AdamW moved both the same way)
    with torch.no_grad():
        l2s = float(sparse(input_ids=ids, labels=labels).loss)
        l2t = float(twin(input_ids=ids, labels=labels).loss)
    assert l2s < loss_sparse and abs(l2s - l2t) <= 2e-3 * abs(l2t), (l2s, l2t, loss_sparse)
