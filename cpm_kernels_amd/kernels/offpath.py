"""Names exported by cpm_kernels.kernels (kernels/__init__.py:1-14 of the reference) that are
outside the int8 inference path: token embedding, fp16 transpose and decode-loop utilities.
They exist so that code written against the reference imports; calling one raises."""
from .base import not_on_path

_e = "token embedding, kernels/embedding.py"
embedding_forward = not_on_path("embedding_forward", _e)
embedding_backward_stage1 = not_on_path("embedding_backward_stage1", _e)
embedding_backward_stage2 = not_on_path("embedding_backward_stage2", _e)
embedding_step = not_on_path("embedding_step", _e)
transpose = not_on_path("transpose", "kernels/transpose.py")
_u = "decode-loop utilities, kernels/utils.py"
copy_data_to_kv = not_on_path("copy_data_to_kv", _u)
has_nan_inf = not_on_path("has_nan_inf", _u)
array_add = not_on_path("array_add", _u)
adjustify_logits = not_on_path("adjustify_logits", _u)
copy_extend_buffer = not_on_path("copy_extend_buffer", _u)
copy_pos_hidden = not_on_path("copy_pos_hidden", _u)
