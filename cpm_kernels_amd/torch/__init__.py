"""PyTorch-ROCm operators under the names a user of cpm_kernels.torch imports (the reference's
export list is torch/__init__.py:1-14).  One import per module, names in alphabetical order;
`__all__` is that public surface."""
from .arith import (
    batched_add, batched_add_inplace, batched_addTH,
    element_add, element_add_inplace, element_addTH,
    element_mul, element_mul_inplace, element_mulTH,
    global_scale, global_scale_inplace, global_scaleTH,
    ln_add, ln_add_inplace, ln_addTH,
    ln_div, ln_div_inplace, ln_divTH,
    ln_mul, ln_mul_inplace, ln_mulTH,
    ln_mul_add, ln_mul_add_inplace, ln_mul_addTH,
    ln_sub_div, ln_sub_div_inplace, ln_sub_divTH,
)
from .embedding import Embedding, EmbeddingTH, OpEmbedding
from .gelu import gelu, gelu_inplace, geluTH
from .gemm import bmm
from .layernorm import LayerNorm, LayerNormTH, normalize_inplace, normalizeTH
from .mask import mask, mask_inplace, maskTH
from .position_embedding import PositionEmbedding, PositionEmbeddingTH
from .softmax import softmax, softmax_inplace, softmaxTH
from .transpose import transpose, transposeTH
from .utils import has_nan_inf

# (gelu, mask, softmax and transpose name a function here and a submodule: the function wins)
__all__ = sorted(n for n, v in list(globals().items()) if not n.startswith("_") and type(v).__name__ != "module")
