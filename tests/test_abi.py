"""CPU-only checks of the drop-in boundary: the C-ABI library loads and exports every symbol
include/cpmk.h declares, the Python layers keep the reference's names and error behaviour, and
nothing in the product path imports the oracle.  No compute calls (no GPU here)."""
import ctypes
import json
import os
import re
import subprocess
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_symbols():
    text = open(os.path.join(ROOT, "include", "cpmk.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(cpmk_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from cpm_kernels_amd.build import library_path, build_library
    if not os.path.exists(library_path()):
        build_library(verbose=False)
    lib = ctypes.CDLL(library_path())
    syms = header_symbols()
    assert len(syms) >= 30
    for s in syms:
        assert hasattr(lib, s), "libcpmk_hip.so does not export %s" % s
    from cpm_kernels_amd.library import cpmk
    assert sorted(cpmk.EXPORTED_SYMBOLS) == syms, "python binding and header disagree"
    assert cpmk.version == 10000
    assert "divisibility" in cpmk.error_string(10002) and cpmk.error_string(0) == "success"


# cpm_kernels/kernels/__init__.py:1-14 of the reference exports these names
REFERENCE_KERNEL_NAMES = """
embedding_forward embedding_backward_stage1 embedding_backward_stage2 embedding_step
gelu_forward gelu_backward gelu_inplace_forward
gemm_calc_scale gemm_calc_scale_transpose gemm_round gemm_round_transpose gemm_scale gemm_fp16 gemm_int8
gemm_backward_round_scale gemm_backward_scale_round gemm_scale_x gemm_scale_y
gemv_fp16 gemv_broadcast_mat_int8 gemv_fp16_transpose gemv_broadcast_mat_fp16 gemv_calc_scale gemv_round
gemv_broadcast_mat_fp16_light gemv_fp16_light gemv_fp16_transpose_light
mask
arith_batch_add_backward arith_batch_add_forward arith_element_add arith_ln_add_backward arith_ln_div arith_ln_mul
arith_ln_mul_add arith_ln_mul_backward arith_ln_sub_div arith_element_mul arith_ln_add arith_batch_mul
arith_batch_mul_add arith_global_scale
layernorm_forward layernorm_inplace_forward layernorm_forward_v layernorm_forward_mv layernorm_backward_v
layernorm_backward_mv layernorm_step layernorm_step_inplace
position_embedding_init position_embedding_forward position_embedding_backward position_embedding_step
softmax_forward softmax_backward softmax_inplace_forward softmax_step_inplace
transpose copy_data_to_kv has_nan_inf
""".split()


def test_kernel_layer_keeps_reference_names_and_signatures():
    import inspect
    import cpm_kernels.kernels as ck
    import cpm_kernels_amd.kernels as ck2
    assert ck is ck2
    for name in REFERENCE_KERNEL_NAMES:
        assert callable(getattr(ck, name)), name
    for name in ("array_add", "adjustify_logits", "copy_extend_buffer", "copy_pos_hidden"):
        assert callable(getattr(ck.utils, name))
    sig = lambda f: list(inspect.signature(f).parameters)   # noqa: E731
    assert sig(ck.gemm_int8) == ["m", "k", "n", "batchA", "batchB", "aT", "bT", "A", "B", "out", "stream"]
    assert sig(ck.gemm_scale) == ["batch", "n", "m", "mat", "scale_x", "scale_y", "out", "broad_cast_x", "broad_cast_y", "stream"]
    assert sig(ck.gemm_round) == ["batch", "n", "m", "mat", "scale", "out", "stream"]
    assert sig(ck.gemm_calc_scale) == ["batch", "n", "m", "mat", "out", "stream"]
    assert sig(ck.gemv_broadcast_mat_int8) == ["batch", "dim_out", "dim_in", "scale_mat", "mat", "scale_vec", "vec", "out", "stream"]
    assert sig(ck.layernorm_forward) == ["batch", "n", "m", "mat", "out", "eps", "rd_mean", "stream"]
    assert sig(ck.softmax_forward) == ["batch", "n", "m", "inp", "out", "stream"]
    assert sig(ck.gelu_forward) == ["batch", "n", "mat", "out", "stream"]
    assert sig(ck.position_embedding_forward) == ["query_len", "key_len", "num_buckets", "max_distance", "num_heads",
                                                  "position_mapping", "weight", "out", "bidirectional", "stream"]
    assert sig(ck.mask) == ["batch", "n", "m", "inp", "mask", "value", "out", "stream"]
    assert sig(ck.arith_ln_mul_add) == ["batch", "n", "m", "inp", "alpha", "beta", "out", "stream"]
    assert sig(ck.embedding_forward) == ["batch", "hidden_size", "seq_len", "ids", "weights", "out", "stream"]
    assert sig(ck.embedding_step) == ["batch", "embedding_size", "ids", "weights", "out", "stream"]
    assert sig(ck.copy_data_to_kv) == ["batch", "buffer_len", "n", "inp", "out", "pos", "stream"]
    assert ck.utils.copy_data_to_kv is ck.copy_data_to_kv
    # every public function of the reference's kernels/*.py: same parameter names in the same order
    # (tests/golden/kernel_signatures.json lists them as read from the reference's def lines)
    with open(os.path.join(os.path.dirname(__file__), "golden", "kernel_signatures.json")) as f:
        table = json.load(f)
    assert set(REFERENCE_KERNEL_NAMES) <= set(table)
    for name, params in table.items():
        fn = getattr(ck, name, None) or getattr(ck.utils, name)
        assert sig(fn) == params, name


def test_reference_asserts_are_kept():
    import cpm_kernels_amd.kernels as ck
    with pytest.raises(AssertionError):          # kernels/gemm.py:139
        ck.gemm_int8(6, 4, 4, 1, 1, False, False, 0, 0, 0, None)
    with pytest.raises(AssertionError):          # kernels/gemm.py:140
        ck.gemm_int8(4, 4, 4, 2, 3, False, False, 0, 0, 0, None)
    with pytest.raises(AssertionError):          # kernels/gemv.py:65
        ck.gemv_broadcast_mat_int8(1, 4, 6, 0, 0, 0, 0, 0, None)
    with pytest.raises(AssertionError):          # kernels/arith.py:53
        ck.arith_element_add(1, 3, 0, 0, 0, None)
    with pytest.raises(AssertionError):          # kernels/arith.py:146
        ck.arith_ln_mul_add(1, 2, 3, 0, 0, 0, 0, None)


def test_argument_errors_from_the_c_abi_without_a_gpu():
    """Argument checks happen before any launch, so they can be exercised on a GPU-less host."""
    from cpm_kernels_amd.library import cpmk
    with pytest.raises(RuntimeError, match="HIP Error: cpmk: invalid argument"):
        cpmk.gemm_calc_scale(-1, 4, 4, None, None, None)
    with pytest.raises(RuntimeError, match="divisibility"):
        cpmk.gemv_broadcast_mat_int8(1, 4, 6, None, None, None, None, None, None)
    with pytest.raises(RuntimeError, match="invalid argument"):
        cpmk.gemm_int8(4, 4, 4, 2, 3, 0, 0, None, None, None, None)
    # empty problems return before touching the device
    cpmk.gemm_round(0, 4, 4, None, None, None, None)
    cpmk.softmax_forward(1, 0, 4, None, None, None)
    cpmk.position_embedding_forward(0, 4, 32, 128, 2, None, None, None, 1, None)


def test_null_buffers_are_refused_before_any_launch():
    """A null buffer in a call that has work to do would be a memory fault on the device; every launcher
    answers it with CPMK_EBADARG on the host instead (so this runs on a GPU-less host too)."""
    from cpm_kernels_amd.library import cpmk
    N = None
    calls = [
        lambda: cpmk.gemm_calc_scale(1, 4, 8, N, N, N),
        lambda: cpmk.gemm_calc_scale_transpose(1, 4, 8, N, N, N),
        lambda: cpmk.gemm_round(1, 4, 16, N, N, N, N),
        lambda: cpmk.gemm_round_transpose(1, 4, 16, N, N, N, N),
        lambda: cpmk.gemm_scale(1, 4, 8, N, N, N, N, 0, 0, N),
        lambda: cpmk.gemm_scale_x(1, 4, 8, N, N, N, N),
        lambda: cpmk.gemm_scale_y(1, 4, 8, N, N, N, N),
        lambda: cpmk.gemm_int8(4, 4, 4, 1, 1, 0, 0, N, N, N, N),
        lambda: cpmk.gemm_int8_scale(4, 4, 4, 1, 1, 0, 0, N, N, N, N, 0, 0, N, N),
        lambda: cpmk.gemm_fp16(4, 4, 4, 1, 1, 0, 0, N, N, N, N),
        lambda: cpmk.gemm_quantize(1, 4, 8, N, N, N, 0, N),
        lambda: cpmk.gemm_quantize(1, 4, 8, N, N, N, 1, N),
        lambda: cpmk.gemm_quantize_pair(4, N, N, N, 4, N, N, N, 8, N),
        lambda: cpmk.gemm_quantize_cols(1, 4, 8, N, N, N, 0, N),
        lambda: cpmk.gemv_calc_scale(2, 8, N, N, N),
        lambda: cpmk.gemv_round(2, 8, N, N, N, N),
        lambda: cpmk.gemv_broadcast_mat_int8(1, 4, 8, N, N, N, N, N, N),
        lambda: cpmk.gemv_fp16(1, 4, 8, N, N, N, N),
        lambda: cpmk.gemv_fp16_transpose(1, 4, 8, N, N, N, N),
        lambda: cpmk.gemv_broadcast_mat_fp16(1, 4, 8, N, N, N, N),
        lambda: cpmk.layernorm_forward(1, 4, 8, N, N, 1e-5, 1, N),
        lambda: cpmk.layernorm_step(1, 8, N, N, 1e-5, 1, N),
        lambda: cpmk.softmax_forward(1, 4, 8, N, N, N),
        lambda: cpmk.softmax_step_inplace(1, 8, N, N),
        lambda: cpmk.gelu_forward(1, 8, N, N, N),
        lambda: cpmk.arith_ln_mul(1, 4, 8, N, N, N, N),
        lambda: cpmk.arith_element_add(1, 8, N, N, N, N),
        lambda: cpmk.mask(1, 4, 8, N, N, 0.0, N, N),
        lambda: cpmk.position_embedding_init(32, 128, N, 1, N),
        lambda: cpmk.position_embedding_forward(4, 4, 32, 128, 2, N, N, N, 1, N),
        lambda: cpmk.position_embedding_step(1, 4, 32, 128, 2, N, N, N, 1, N),
        lambda: cpmk.embedding_forward(1, 8, 4, N, N, N, N),
        lambda: cpmk.embedding_step(1, 8, N, N, N, N),
        lambda: cpmk.copy_data_to_kv(1, 4, 8, N, N, 0, N),
        lambda: cpmk.transpose(1, 4, 8, N, N, N),
        lambda: cpmk.has_nan_inf(8, N, N, N),
        lambda: cpmk.arith_global_scale(8, N, 1.0, N, N),
        lambda: cpmk.arith_element_mul(1, 8, N, N, N, N),
        lambda: cpmk.arith_batch_add_backward(2, 8, N, N, N),
        lambda: cpmk.arith_ln_mul_backward(1, 4, 8, N, N, N, N),
        lambda: cpmk.gelu_backward(1, 8, N, N, N, N),
        lambda: cpmk.softmax_backward(1, 4, 8, N, N, N, N),
        lambda: cpmk.layernorm_forward_mv(1, 4, 8, N, N, N, N, 1e-5, N),
        lambda: cpmk.layernorm_backward_v(1, 4, 8, N, N, N, N, N),
        lambda: cpmk.gemm_backward_round_scale(1, 4, 8, N, N, N, N, 0, N),
        lambda: cpmk.gemm_backward_scale_round(1, 4, 8, N, N, N, N, 0, N),
        lambda: cpmk.position_embedding_backward(4, 4, 32, 128, 2, N, N, N, 1, N),
        lambda: cpmk.embedding_backward_stage2(2, 8, N, N, N, N),
    ]
    for i, call in enumerate(calls):
        with pytest.raises(RuntimeError, match="invalid argument"):
            call()
            pytest.fail(f"call {i} accepted a null buffer")


def test_missing_library_gives_stubs_not_import_errors():
    """cpm_kernels/library/base.py:67-74 of the reference: an absent library leaves the package
    importable and every bound call raises RuntimeError('Library ... is not initialized')."""
    code = ("import cpm_kernels_amd.kernels as ck\n"
            "from cpm_kernels_amd.library import cpmk\n"
            "from cpm_kernels_amd.device import num_devices\n"
            "assert cpmk.version == 0 and not cpmk.lib.loaded and num_devices() == 0\n"
            "try:\n    ck.gemm_calc_scale(1, 4, 4, 0, 0, None)\n"
            "except RuntimeError as e:\n    assert 'is not initialized' in str(e); print('STUB-OK')\n")
    env = dict(os.environ, CPMK_LIBRARY="/nonexistent/libcpmk_hip.so", PYTHONPATH=ROOT)
    out = subprocess.run([sys.executable, "-c", code], env=env, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    assert "STUB-OK" in out.stdout, out.stdout


def test_product_code_never_touches_the_oracle():
    bad = []
    for base, _, files in os.walk(os.path.join(ROOT, "cpm_kernels_amd")):
        for f in files:
            if f.endswith((".py", ".hip", ".h", ".cpp")):
                text = open(os.path.join(base, f)).read()
                if re.search(r"^\s*(from|import)\s+oracle\b", text, flags=re.M) or "cpmk_oracle" in text:
                    bad.append(os.path.join(base, f))
    assert not bad, bad
    for f in os.listdir(os.path.join(ROOT, "cpm_kernels")):
        if f.endswith(".py"):
            assert "oracle" not in open(os.path.join(ROOT, "cpm_kernels", f)).read()


def test_torch_layer_imports_and_exports():
    import cpm_kernels.torch as ct
    for name in ("bmm", "LayerNorm", "LayerNormTH", "normalize_inplace", "normalizeTH", "softmax", "softmaxTH",
                 "softmax_inplace", "gelu", "geluTH", "gelu_inplace", "PositionEmbedding", "PositionEmbeddingTH",
                 "mask", "mask_inplace", "maskTH", "ln_mul_add", "ln_mul", "element_add"):
        assert hasattr(ct, name), name


def test_device_module_without_gpu():
    from cpm_kernels_amd import device
    n = device.num_devices()
    assert n >= 0
    with pytest.raises(ValueError):
        device.Device(n)          # one past the end is out of range (the reference accepts it by an off-by-one)


def test_single_hip_runtime_whichever_is_imported_first():
    """libcpmk_hip.so must bind to the HIP runtime PyTorch ships, also when this package is
    imported before torch: two copies of libamdhip64 in one process do not share streams,
    pointers or the device."""
    code = ("import cpm_kernels_amd, torch\n"
            "libs = sorted(set(l.split()[-1] for l in open('/proc/self/maps') if 'libamdhip64' in l))\n"
            "print('HIPLIBS', len(libs), libs)\n")
    out = subprocess.run([sys.executable, "-c", code], env=dict(os.environ, PYTHONPATH=ROOT), stdout=subprocess.PIPE,
                         stderr=subprocess.STDOUT, text=True)
    assert "HIPLIBS 1 " in out.stdout, out.stdout


def test_torch_surface_through_the_alias_package():
    """`import cpm_kernels.torch as ct` must give every operator name of the reference's
    torch/__init__.py:1-14 -- including gelu, mask, softmax and transpose, which are also the
    names of submodules (a star import that listed the modules instead would hide the functions)."""
    import types
    import cpm_kernels.torch as ct
    names = """OpEmbedding Embedding EmbeddingTH gelu geluTH gelu_inplace bmm mask mask_inplace maskTH
        ln_div ln_div_inplace ln_divTH ln_mul_add ln_mul_add_inplace ln_mul_addTH ln_mul ln_mul_inplace ln_mulTH
        ln_sub_div ln_sub_divTH ln_sub_div_inplace element_add element_add_inplace element_addTH
        batched_add batched_add_inplace batched_addTH element_mul element_mul_inplace element_mulTH
        ln_add ln_add_inplace ln_addTH global_scale global_scale_inplace global_scaleTH
        LayerNorm LayerNormTH normalize_inplace normalizeTH PositionEmbedding PositionEmbeddingTH
        softmax softmaxTH softmax_inplace transpose transposeTH has_nan_inf""".split()
    for n in names:
        obj = getattr(ct, n, None)
        assert obj is not None and not isinstance(obj, types.ModuleType) and callable(obj), n


def test_torch_submodules_through_the_alias_package():
    """Every submodule of the reference's torch package imports under the drop-in name and is the
    implementation's module object (not the function of the same name), and the classes a user
    imports from them are there (torch/*.py of the reference)."""
    import importlib
    import types
    wanted = {
        "arith": ["OpGlobalScale", "OpElementAdd", "OpElementMul", "OpBatchedAdd", "OpLnMulAdd", "OpLnMul", "OpLnAdd",
                  "ln_sub_div", "ln_div"],
        "embedding": ["OpEmbedding", "Embedding", "EmbeddingTH"],
        "gelu": ["OpGeLU", "gelu", "gelu_impl", "geluTH", "gelu_inplace"],
        "gemm": ["calc_scale", "round_i8", "gemm_and_scale", "GEMMInt8", "gemm_pth_fp16", "GEMMFloat", "bmm"],
        "layernorm": ["OpLayerNormMean", "OpLayerNormNoMean", "LayerNorm", "LayerNormTH", "normalize_inplace", "normalizeTH"],
        "mask": ["OpMask", "mask", "mask_inplace", "maskTH"],
        "position_embedding": ["OpPositionEmbedding", "PositionEmbedding", "PositionEmbeddingTH"],
        "softmax": ["OpSoftmax", "softmax", "softmax_inplace", "softmaxTH"],
        "transpose": ["OpTranspose", "transpose", "transposeTH"],
        "utils": ["has_nan_inf"],
    }
    import cpm_kernels.torch as ct
    for sub, names in wanted.items():
        mod = importlib.import_module("cpm_kernels.torch." + sub)
        assert isinstance(mod, types.ModuleType), sub
        assert mod is importlib.import_module("cpm_kernels_amd.torch." + sub), sub
        assert sys.modules["cpm_kernels.torch." + sub] is mod
        for n in names:
            assert callable(getattr(mod, n, None)), "%s.%s" % (sub, n)
    from cpm_kernels.torch.softmax import OpSoftmax      # noqa: F401
    import cpm_kernels.torch.embedding, cpm_kernels.torch.transpose, cpm_kernels.torch.utils      # noqa: F401,E401
    # in the package namespace the function wins where both exist, as in the reference
    for n in ("gelu", "mask", "softmax", "transpose"):
        assert not isinstance(getattr(ct, n), types.ModuleType), n
    assert isinstance(ct.utils, types.ModuleType) and isinstance(ct.gemm, types.ModuleType)


def test_yardstick_library_is_separate_from_the_product():
    """bench.py's yardstick kernels live in a library of their own: it builds, exports the entry points
    the bench binds, rejects bad arguments without a GPU, and the product library neither exports nor
    needs any of them."""
    from cpm_kernels_amd.build import bench_library_path, build_bench_library, library_path
    if not os.path.exists(bench_library_path()):
        build_bench_library(verbose=False)
    lib = ctypes.CDLL(bench_library_path())
    for s in ("ceil_mfma_i8", "ceil_read", "ceil_write", "ceil_copy", "ceil_copy_segments"):
        assert hasattr(lib, s), s
    lib.ceil_copy_segments.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int64, ctypes.c_int32, ctypes.c_int32, ctypes.c_void_p]
    assert lib.ceil_copy_segments(None, None, 1024, 1024, 48, None) == 1        # segment width not a power of two
    assert lib.ceil_copy_segments(None, None, 1000, 1024, 128, None) == 1       # rows not whole tiles
    prod = ctypes.CDLL(library_path())
    assert not hasattr(prod, "ceil_mfma_i8")
    out = subprocess.run(["nm", "-D", "--undefined-only", library_path()], capture_output=True, text=True).stdout
    assert "ceil_" not in out
    # the async status and the allocation-free entry point are part of the product ABI
    assert "gave up waiting" in __import__("cpm_kernels_amd.library.cpmk", fromlist=["x"]).error_string(10004)
