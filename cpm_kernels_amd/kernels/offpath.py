"""Names exported by cpm_kernels.kernels (kernels/__init__.py:1-14 of the reference) that are
outside the int8 inference path: fp16 transpose and decode-loop utilities.
They exist so that code written against the reference imports; calling one raises."""
from .base import not_on_path

transpose = not_on_path("transpose", "kernels/transpose.py")
_u = "decode-loop utilities, kernels/utils.py"
has_nan_inf = not_on_path("has_nan_inf", _u)
array_add = not_on_path("array_add", _u)
adjustify_logits = not_on_path("adjustify_logits", _u)
copy_extend_buffer = not_on_path("copy_extend_buffer", _u)
copy_pos_hidden = not_on_path("copy_pos_hidden", _u)
