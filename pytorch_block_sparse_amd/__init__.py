"""MI355X-native block-sparse linear layers: the public names of ``pytorch_block_sparse`` (its __init__.py:1-6)."""
from .block_sparse import BlockSparseMatrix, BlockSparseMatrixBase, BlockSparseMatrixEmulator
from .block_sparse_linear import BlockSparseLinear, BlockSparseLinearFunction, PseudoBlockSparseLinear
from .util import BlockSparseModelPatcher, ModelPatcher
from .sparse_optimizer import SparseOptimizer

__all__ = [
    "BlockSparseMatrix",
    "BlockSparseMatrixEmulator",
    "BlockSparseLinear",
    "BlockSparseModelPatcher",
    "SparseOptimizer",
]
__version__ = "0.1.0"
