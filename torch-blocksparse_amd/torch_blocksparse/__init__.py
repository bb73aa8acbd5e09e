"""torch_blocksparse for AMD MI355X: block-sparse MatMul (sdd / dsd / dds) and Softmax (plus the package's two dense
utility ops, ReLU and Permute) as HIP kernels behind the reference package's API."""
from .softmax import Softmax
from .matmul import MatMul, Linear
from .attention import MultiheadAttention, make_layout, replace_mha
from .deepspeedsparseselfattention import DeepSpeedSparseSelfAttention, SparseSelfAttention, SparsityConfig
from .layouts import fixed_layout, bigbird_layout, sparse_transformer_layout
from .permute import _permute, Permute
from .relu import ReLU

__all__ = ['Softmax', 'MatMul', 'Linear', 'MultiheadAttention', 'make_layout', 'replace_mha',
           'DeepSpeedSparseSelfAttention', 'SparseSelfAttention', 'SparsityConfig', 'fixed_layout', 'bigbird_layout', 'sparse_transformer_layout',
           'Permute', 'ReLU']
