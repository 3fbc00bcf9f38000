"""``cpm_kernels.kernels.utils`` of the reference holds decode-loop utilities that are not on
the int8 inference path; the names resolve, calls raise NotImplementedError."""
from .offpath import copy_data_to_kv, has_nan_inf, array_add, adjustify_logits, copy_extend_buffer, copy_pos_hidden  # noqa: F401
