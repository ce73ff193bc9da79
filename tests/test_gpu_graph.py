"""The three products recorded into a HIP graph and replayed.

The library allocates nothing, keeps nothing between calls and launches only on the stream it is given
(its zero fill is a kernel, not a memset), so a caller may capture forward + input gradient + weight
gradient into a graph once the pattern's plans exist.  Every replay is compared with the eager result;
eager work and synchronisations run between the replays, and the inputs are changed in place before the
last one.
"""
import numpy as np
import pytest
import torch

from pytorch_block_sparse_amd import BlockSparseMatrix

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype,out_f,in_f,tokens", [
    (torch.float32, 256, 1024, 2048),     # the 1024 -> 256 forward shape, with its gradients
    (torch.float32, 768, 768, 4096),      # several token slices in the weight gradient (partial sums + reduce)
    (torch.bfloat16, 512, 2048, 33000),   # the wide-tile persistent kernel
])
def test_graph_replay_matches_eager(cuda, dtype, out_f, in_f, tokens):
    np.random.seed(3)
    torch.manual_seed(3)
    m = BlockSparseMatrix.randn((out_f, in_f), (out_f // 32) * (in_f // 32) // 4, device=cuda, dtype=dtype)
    x = torch.randn(tokens, in_f, device=cuda).to(dtype)
    dy = torch.randn(tokens, out_f, device=cuda).to(dtype)

    def step():
        return m.reverse_matmul(x, True), m.reverse_matmul(dy, False), m.matmul_with_output_sparse_support(dy, x)

    eager = [t.clone() for t in step()]          # also builds the plans and raises the kernels' LDS limits
    torch.cuda.synchronize()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):                # a few eager runs on the capturing stream first
        for _ in range(2):
            step()
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        captured = step()
    for replay in range(3):
        for t in captured:
            t.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        for got, want, name in zip(captured, eager, ("fwd", "dx", "dw")):
            assert torch.equal(got, want), f"replay {replay}: {name} differs from the eager result"
        other = step()                            # eager work between the replays
        torch.cuda.synchronize()
        for got, want in zip(other, eager):
            assert torch.equal(got, want)
    # new operand values in the same buffers: the graph computes with what is there now
    x.mul_(-0.5)
    dy.add_(0.25)
    graph.replay()
    torch.cuda.synchronize()
    for got, want, name in zip(captured, step(), ("fwd", "dx", "dw")):
        assert torch.equal(got, want), f"after changing the operands: {name}"
