"""Same export list as cpm_kernels/kernels/__init__.py:1-14 of the reference, plus the fused
launchers this build adds (gemm_int8_scale, gemm_quantize, gemm_quantize_cols, gemm_quantize_pair,
layernorm_affine_forward)."""
from .embedding import embedding_forward, embedding_backward_stage1, embedding_backward_stage2, embedding_step
from .gelu import gelu_forward, gelu_backward, gelu_inplace_forward
from .gemm import gemm_calc_scale, gemm_calc_scale_transpose, gemm_round, gemm_round_transpose, gemm_scale, \
    gemm_fp16, gemm_int8, gemm_backward_round_scale, gemm_backward_scale_round, gemm_scale_x, gemm_scale_y, \
    gemm_int8_scale, gemm_quantize, gemm_quantize_cols, gemm_quantize_pair
from .gemv import gemv_fp16, gemv_broadcast_mat_int8, gemv_fp16_transpose, gemv_broadcast_mat_fp16, \
    gemv_calc_scale, gemv_round, gemv_broadcast_mat_fp16_light, gemv_fp16_light, gemv_fp16_transpose_light
from .mask import mask
from .arith import arith_batch_add_backward, arith_batch_add_forward, arith_element_add, arith_ln_add_backward, \
    arith_ln_div, arith_ln_mul, arith_ln_mul_add, arith_ln_mul_backward, arith_ln_sub_div, arith_element_mul, \
    arith_ln_add, arith_batch_mul, arith_batch_mul_add, arith_global_scale
from .layernorm import layernorm_forward, layernorm_inplace_forward, layernorm_forward_v, layernorm_forward_mv, \
    layernorm_backward_v, layernorm_backward_mv, layernorm_step, layernorm_step_inplace, layernorm_affine_forward
from .position_bucket import position_embedding_init, position_embedding_forward, position_embedding_backward, \
    position_embedding_step
from .softmax import softmax_forward, softmax_backward, softmax_inplace_forward, softmax_step_inplace
from .transpose import transpose, transpose_i8
from .utils import copy_data_to_kv, has_nan_inf
from . import utils
