"""PyTorch-ROCm wrappers for the int8 inference path, with the names of cpm_kernels/torch
(torch/__init__.py:1-14 of the reference) for everything on that path."""
from .gelu import gelu, geluTH, gelu_inplace
from .gemm import bmm
from .mask import mask, mask_inplace, maskTH
from .arith import ln_mul_add, ln_mul_add_inplace, ln_mul_addTH, ln_mul, ln_mul_inplace, ln_mulTH, \
    element_add, element_add_inplace, element_addTH
from .layernorm import LayerNorm, LayerNormTH, normalize_inplace, normalizeTH
from .position_embedding import PositionEmbedding, PositionEmbeddingTH
from .softmax import softmax, softmaxTH, softmax_inplace
