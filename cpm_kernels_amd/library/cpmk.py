"""ctypes binding of libcpmk_hip.so (include/cpmk.h).

Replaces cpm_kernels/library/{cuda,cudart,cublaslt}.py of the reference: instead of a CUDA
driver launch (library/cuda.py:249-267) or a cuBLASLt call (library/cublaslt.py:113-150)
per kernel, every kernel has one ``extern "C"`` launcher.  A non-zero status raises
``RuntimeError`` like the reference's check*Status helpers (library/cudart.py:325-327).
"""
import ctypes
from .base import Lib

lib = Lib("cpmk_hip")

# launchers: name -> argument ctypes (all return int status)
_LAUNCHERS = {
    "cpmk_gemm_calc_scale": [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p],
    "cpmk_gemm_calc_scale_transpose": [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p],
    "cpmk_gemm_round": [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p],
    "cpmk_gemm_round_transpose": [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p],
    "cpmk_gemm_scale": [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p],
    "cpmk_gemm_scale_x": [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p],
    "cpmk_gemm_scale_y": [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p],
    "cpmk_gemm_int8": [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p],
    "cpmk_gemm_int8_scale": [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p],
    "cpmk_gemm_quantize": [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p],
    "cpmk_gemm_quantize_pair": [ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int32, ctypes.c_void_p],
    "cpmk_gemm_quantize_cols": [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p],
    "cpmk_gemm_fp16": [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_int, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p],
    "cpmk_gemv_fp16": [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p],
    "cpmk_gemv_fp16_transpose": [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p],
    "cpmk_gemv_broadcast_mat_fp16": [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p],
    "cpmk_embedding_forward": [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p],
    "cpmk_embedding_step": [ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p],
    "cpmk_copy_data_to_kv": [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int32, ctypes.c_void_p],
    "cpmk_gemv_calc_scale": [ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p],
    "cpmk_gemv_round": [ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p],
    "cpmk_gemv_broadcast_mat_int8": [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p],
    "cpmk_layernorm_forward": [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_float, ctypes.c_int, ctypes.c_void_p],
    "cpmk_layernorm_forward_noalloc": [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_float, ctypes.c_int, ctypes.c_void_p],
    "cpmk_layernorm_step": [ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_float, ctypes.c_int, ctypes.c_void_p],
    "cpmk_layernorm_affine_forward": [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_float, ctypes.c_int, ctypes.c_void_p],
    "cpmk_softmax_forward": [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p],
    "cpmk_softmax_step_inplace": [ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p],
    "cpmk_gelu_forward": [ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p],
    "cpmk_position_embedding_init": [ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p],
    "cpmk_position_embedding_forward": [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p],
    "cpmk_position_embedding_step": [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p],
    "cpmk_arith_ln_mul_add": [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p],
    "cpmk_arith_ln_mul": [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p],
    "cpmk_arith_element_add": [ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p],
    "cpmk_mask": [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_float, ctypes.c_void_p, ctypes.c_void_p],
    "cpmk_arith_global_scale": [ctypes.c_int64, ctypes.c_void_p, ctypes.c_float, ctypes.c_void_p, ctypes.c_void_p],
    "cpmk_arith_element_mul": [ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p],
    "cpmk_arith_batch_add_forward": [ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p],
    "cpmk_arith_batch_add_backward": [ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p],
    "cpmk_arith_ln_add": [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p],
    "cpmk_arith_ln_div": [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p],
    "cpmk_arith_ln_sub_div": [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p],
    "cpmk_arith_ln_mul_backward": [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p],
    "cpmk_arith_ln_add_backward": [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p],
    "cpmk_arith_batch_mul_add": [ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p],
    "cpmk_arith_batch_mul": [ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p],
    "cpmk_gelu_backward": [ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p],
    "cpmk_softmax_backward": [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p],
    "cpmk_layernorm_forward_v": [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_float, ctypes.c_void_p],
    "cpmk_layernorm_forward_mv": [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_float, ctypes.c_void_p],
    "cpmk_layernorm_backward_v": [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p],
    "cpmk_layernorm_backward_mv": [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p],
    "cpmk_gemm_backward_round_scale": [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p],
    "cpmk_gemm_backward_scale_round": [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p],
    "cpmk_position_embedding_backward": [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p],
    "cpmk_embedding_backward_stage1": [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p],
    "cpmk_embedding_backward_stage2": [ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p],
    "cpmk_transpose": [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p],
    "cpmk_transpose_i8": [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p],
    "cpmk_array_add": [ctypes.c_void_p, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p],
    "cpmk_adjustify_logits": [ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_float, ctypes.c_float, ctypes.c_float, ctypes.c_void_p, ctypes.c_void_p],
    "cpmk_copy_extend_buffer": [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p],
    "cpmk_has_nan_inf": [ctypes.c_int64, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p],
    "cpmk_copy_pos_hidden": [ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p, ctypes.c_void_p, ctypes.c_void_p],
    "cpmk_async_status": [],
    "cpmk_selftest_exchange_timeout": [ctypes.c_int32, ctypes.c_void_p],
}

EXPORTED_SYMBOLS = sorted(list(_LAUNCHERS) + [
    "cpmk_version", "cpmk_error_string", "cpmk_device_count", "cpmk_get_device",
    "cpmk_set_device", "cpmk_device_props", "cpmk_exchange_capture_slots_left",
])


@lib.bind("cpmk_error_string", [ctypes.c_int], ctypes.c_char_p)
def error_string(code: int) -> str:
    return lib.cpmk_error_string(code).decode()


@lib.bind("cpmk_version", [], ctypes.c_int)
def _version() -> int:
    return lib.cpmk_version()


def checkStatus(status: int) -> None:
    if status != 0:
        raise RuntimeError("HIP Error: %s" % error_string(status))


def _make(name, argtypes):
    @lib.bind(name, argtypes, ctypes.c_int)
    def call(*args):
        checkStatus(getattr(lib, name)(*args))
    call.__name__ = name[len("cpmk_"):]
    call.__doc__ = "Launch %s (see include/cpmk.h)." % name
    return call


for _name, _argtypes in _LAUNCHERS.items():
    globals()[_name[len("cpmk_"):]] = _make(_name, _argtypes)


def check() -> None:
    """Raise ``RuntimeError`` if a kernel launched on the current device has failed while it ran (a
    team of workgroups whose partial results did not arrive in time: the outputs then hold NaN, or 0
    in int8 tensors), and clear the condition.  Blocks like a device-to-host copy, so it sees all work
    queued before it on the blocking streams; synchronise non-blocking streams first.  Until it is
    called, every other call into the library raises the same error (the reference raises pending
    failures from the status check of whichever call comes next, library/cudart.py:325-327)."""
    globals()["async_status"]()


@lib.bind("cpmk_exchange_capture_slots_left", [ctypes.POINTER(ctypes.c_int32)], ctypes.c_int)
def exchange_capture_slots_left() -> int:
    n = ctypes.c_int32(0)
    checkStatus(lib.cpmk_exchange_capture_slots_left(ctypes.byref(n)))
    return n.value


@lib.bind("cpmk_device_count", [ctypes.POINTER(ctypes.c_int)], ctypes.c_int)
def device_count() -> int:
    n = ctypes.c_int(0)
    checkStatus(lib.cpmk_device_count(ctypes.byref(n)))
    return n.value


@lib.bind("cpmk_get_device", [ctypes.POINTER(ctypes.c_int)], ctypes.c_int)
def get_device() -> int:
    d = ctypes.c_int(0)
    checkStatus(lib.cpmk_get_device(ctypes.byref(d)))
    return d.value


@lib.bind("cpmk_set_device", [ctypes.c_int], ctypes.c_int)
def set_device(device: int) -> None:
    checkStatus(lib.cpmk_set_device(device))


@lib.bind("cpmk_device_props", [ctypes.c_int, ctypes.c_char_p, ctypes.c_int] +
          [ctypes.POINTER(ctypes.c_int)] * 7 + [ctypes.POINTER(ctypes.c_uint64)], ctypes.c_int)
def device_props(device: int) -> dict:
    name = ctypes.create_string_buffer(64)
    ints = [ctypes.c_int(0) for _ in range(7)]
    mem = ctypes.c_uint64(0)
    checkStatus(lib.cpmk_device_props(device, name, 64, *[ctypes.byref(i) for i in ints],
                                      ctypes.byref(mem)))
    keys = ["compute_units", "lds_bytes", "wavefront", "clock_khz", "mem_clock_khz",
            "mem_bus_bits", "l2_bytes"]
    props = {k: v.value for k, v in zip(keys, ints)}
    props["name"] = name.value.decode()
    props["global_mem_bytes"] = mem.value
    return props


try:
    version = _version()
except RuntimeError:      # library not built / not loadable on this host
    version = 0
