"""PyTorch-ROCm wrappers with the names of cpm_kernels/torch (torch/__init__.py:1-14 of the reference)."""
from .embedding import OpEmbedding, Embedding, EmbeddingTH
from .gelu import gelu, geluTH, gelu_inplace
from .gemm import bmm
from .mask import mask, mask_inplace, maskTH
from .arith import ln_div, ln_div_inplace, ln_divTH, ln_mul_add, ln_mul_add_inplace, \
    ln_mul_addTH, ln_mul, ln_mul_inplace, ln_mulTH, ln_sub_div, \
    ln_sub_divTH, ln_sub_div_inplace, element_add, element_add_inplace, \
    element_addTH, batched_add, batched_add_inplace, batched_addTH, \
    element_mul, element_mul_inplace, element_mulTH, \
    ln_add, ln_add_inplace, ln_addTH, global_scale, global_scale_inplace, global_scaleTH
from .layernorm import LayerNorm, LayerNormTH, normalize_inplace, normalizeTH
from .position_embedding import PositionEmbedding, PositionEmbeddingTH
from .softmax import softmax, softmaxTH, softmax_inplace
from .transpose import transpose, transposeTH
from .utils import has_nan_inf
