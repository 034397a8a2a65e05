"""Host-side checks that need no GPU: the C-ABI library loads, exports every function its public
header declares, and rejects bad arguments before touching the device."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_functions():
    text = open(os.path.join(ROOT, "include", "inferspore_amd.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(isp_[a-z0-9_]+)\s*\(", text)))


@pytest.fixture(scope="module")
def lib():
    from inferspore_amd import capi
    return capi.lib()


def test_header_declares_the_expected_entry_points():
    names = declared_functions()
    for n in ("isp_embedding_f16", "isp_rmsnorm_f32", "isp_fused_add_bias_residual_rmsnorm_f16",
              "isp_qkv_bias_rope_transpose_f16", "isp_swiglu_f16", "isp_cal_padding_offset"):
        assert n in names


def test_library_exports_every_declared_symbol(lib):
    from inferspore_amd import capi
    for name in declared_functions():
        assert hasattr(lib, name), "libinferspore_amd.so does not export " + name
        assert name in capi.SIGNATURES, "no ctypes signature for " + name


def test_version_and_error_strings(lib):
    assert b"gfx950" in lib.isp_version()
    for code in (0, -1, -2, -3, -4, -5):
        assert lib.isp_strerror(code)
    assert lib.isp_strerror(-99) == b"unknown status"


def test_argument_validation_returns_before_any_launch(lib):
    from inferspore_amd import capi
    p = ctypes.c_void_p(16)  # a non-NULL placeholder; validation fails before it is dereferenced
    # zero work is OK whatever the pointers are
    assert lib.isp_swiglu_f16(None, None, 0, 11008, None) == capi.OK
    assert lib.isp_embedding_f16(None, None, None, 0, 4096, 0, None) == capi.OK
    assert lib.isp_rmsnorm_f32(None, None, 1e-5, 0, 4096, None) == capi.OK
    # NULL required operands
    assert lib.isp_swiglu_f16(None, p, 4, 8, None) == capi.ERR_NULL_POINTER
    assert lib.isp_embedding_f32(p, None, p, 4, 8, 0, None) == capi.ERR_NULL_POINTER
    assert lib.isp_rmsnorm_f16(p, None, 1e-5, 4, 8, None) == capi.ERR_NULL_POINTER
    assert lib.isp_fused_add_bias_residual_rmsnorm_f16(None, None, None, p, 1e-5, 4, 8, 0, None) == capi.ERR_NULL_POINTER
    assert lib.isp_cal_padding_offset(p, None, p, 2, 4, None) == capi.ERR_NULL_POINTER
    # negative extents
    assert lib.isp_swiglu_f32(p, p, -1, 8, None) == capi.ERR_BAD_SHAPE
    assert lib.isp_embedding_f16(p, p, p, 4, -8, 0, None) == capi.ERR_BAD_SHAPE
    assert lib.isp_rmsnorm_f32(p, p, 1e-5, -4, 8, None) == capi.ERR_BAD_SHAPE
    assert lib.isp_cal_padding_offset(p, p, p, -2, 4, None) == capi.ERR_BAD_SHAPE
    qkv = lib.isp_qkv_bias_rope_transpose_f16
    args = dict(batch=1, seq=4, tok=3, hn=2, kvn=2, hs=128, rot=128)

    def call(q=p, k=p, v=p, x=p, po=p, hist=p, **kw):
        a = dict(args, **kw)
        return qkv(q, k, v, x, None, po, hist, p, a["batch"], a["seq"], a["tok"], a["hn"], a["kvn"], a["hs"],
                   a["rot"], 10000.0, 2048, 0, None)

    assert call(tok=0) == capi.OK
    assert call(x=None) == capi.ERR_NULL_POINTER
    assert call(po=None) == capi.ERR_NULL_POINTER
    assert call(q=None) == capi.ERR_NULL_POINTER
    assert call(hs=127) == capi.ERR_BAD_SHAPE          # odd head size cannot be split in halves
    assert call(rot=130) == capi.ERR_BAD_SHAPE         # rotary dim larger than the head
    assert call(seq=0) == capi.ERR_BAD_SHAPE
    assert call(hs=1024, rot=1024) == capi.ERR_UNSUPPORTED


def test_norm_launch_queries_need_no_device(lib):
    """isp_norm_launch_config / isp_norm_launch_variant only describe what a call would launch: they work without
    a GPU (device facts fall back to the MI355X's) and reject what the norm entry points reject."""
    from inferspore_amd import capi
    out = [ctypes.c_int() for _ in range(4)]
    refs = [ctypes.byref(x) for x in out]
    assert lib.isp_norm_launch_config(2, 2048, 4096, 1, *refs) == capi.OK
    assert out[0].value in (1, 2, 4, 8, 16) and out[1].value in (1, 2, 4, 8) and out[2].value in (256, 512, 1024)
    assert lib.isp_norm_launch_config(2, 0, 4096, 1, *refs) == capi.ERR_BAD_SHAPE
    assert lib.isp_norm_launch_config(3, 8, 4096, 1, *refs) == capi.ERR_BAD_SHAPE          # no such element size
    assert lib.isp_norm_launch_config(2, 8, 4095, 1, *refs) == capi.ERR_UNSUPPORTED        # not whole vectors: scalar kernel
    # a decode-step norm takes the few-rows kernel, a prefill-sized one the general kernel; the reference's literal
    # residual order and a bias without a residual are outside the few-rows kernels
    assert lib.isp_norm_launch_variant(2, 16, 4096, 1, 0, 0) == 1
    assert lib.isp_norm_launch_variant(4, 64, 4096, 0, 0, 0) == 1
    assert lib.isp_norm_launch_variant(2, 4096, 4096, 1, 0, 0) == 0
    assert lib.isp_norm_launch_variant(2, 16, 4096, 1, 1, capi.NORM_RESIDUAL_EXCLUDES_BIAS) == 0
    assert lib.isp_norm_launch_variant(2, 16, 4096, 0, 1, 0) == 0
    assert lib.isp_norm_launch_variant(2, -1, 4096, 1, 0, 0) == capi.ERR_BAD_SHAPE
    assert lib.isp_norm_launch_variant(8, 16, 4096, 1, 0, 0) == capi.ERR_BAD_SHAPE
    assert lib.isp_norm_launch_variant(4, 16, 4098, 1, 0, 0) == capi.ERR_UNSUPPORTED


def test_python_layer_refuses_cpu_tensors():
    import torch
    from inferspore_amd import ops
    with pytest.raises(RuntimeError, match="GPU"):
        ops.act(torch.ones((2, 2, 8)), torch.empty((2, 8)))


def test_python_layer_refuses_mismatched_dtypes():
    import torch
    from inferspore_amd import ops
    # dtype checks come after the device check, so fake "cuda-ness" is not needed: use meta-free CPU tensors
    # and confirm the device check fires first, then the dtype helper on its own
    with pytest.raises(TypeError):
        ops._same_dtype(torch.ones(2, dtype=torch.float16), torch.ones(2, dtype=torch.float32))
    with pytest.raises(TypeError):
        ops._int32(torch.ones(2, dtype=torch.int64))


def test_argument_validation_of_the_neighbour_entry_points(lib):
    from inferspore_amd import capi
    p = ctypes.c_void_p(16)
    rope = lib.isp_rope_decode_f16
    assert rope(None, 0, 32, 32, 128, 5, 128, 10000.0, None) == capi.OK            # no rows: nothing to do
    assert rope(None, 1, 32, 32, 128, 5, 128, 10000.0, None) == capi.ERR_NULL_POINTER
    assert rope(p, 1, 32, 32, 127, 5, 126, 10000.0, None) == capi.ERR_BAD_SHAPE    # odd head size
    assert rope(p, 1, 32, 32, 128, 5, 130, 10000.0, None) == capi.ERR_BAD_SHAPE    # rotary dim > head size
    assert rope(p, -1, 32, 32, 128, 5, 128, 10000.0, None) == capi.ERR_BAD_SHAPE
    tr = lib.isp_transpose_remove_padding_f32
    assert tr(None, None, None, 2, 4, 8, 16, 0, None) == capi.OK
    assert tr(p, None, p, 2, 4, 8, 16, 5, None) == capi.ERR_NULL_POINTER
    assert tr(p, p, p, 0, 4, 8, 16, 5, None) == capi.ERR_BAD_SHAPE                 # tokens but no batch
    assert tr(p, p, p, 2, -4, 8, 16, 5, None) == capi.ERR_BAD_SHAPE
    cat = lib.isp_concat_kv_cache_f16
    assert cat(None, None, None, None, 0, None, None, 0, 4, 8, 16, 128, None) == capi.OK
    assert cat(p, p, p, None, 0, p, p, 2, 4, 8, 16, 128, None) == capi.ERR_NULL_POINTER
    assert cat(p, p, p, p, -1, p, p, 2, 4, 8, 16, 128, None) == capi.ERR_BAD_SHAPE  # negative layer
    assert cat(p, p, p, p, 0, p, p, 1 << 20, 4096, 8, 16, 128, None) == capi.ERR_UNSUPPORTED  # 2^32 workgroups
    assert cat(p, p, p, p, 0, p, p, 70000, 4, 8, 16, 126, None) == capi.ERR_UNSUPPORTED  # row-per-workgroup form: 65535 rows
    rep = lib.isp_repeat_kv_cache_f32
    assert rep(None, None, None, None, 0, None, 0, 8, 2, 16, 8, 128, None) == capi.OK
    assert rep(p, p, p, p, 0, None, 2, 8, 2, 16, 8, 128, None) == capi.ERR_NULL_POINTER
    assert rep(p, p, p, p, 0, p, 2, 8, 3, 16, 8, 128, None) == capi.ERR_BAD_SHAPE   # heads not a multiple of kv heads
    assert lib.isp_calibration_copy(p, p, 24, None) == capi.ERR_BAD_SHAPE           # not a multiple of 16 bytes
    assert lib.isp_calibration_copy(None, None, 0, None) == capi.OK
    assert lib.isp_tuning_set(99, 1) == capi.ERR_BAD_SHAPE
    assert lib.isp_tuning_set(capi.TUNE_NORM_STORE, 0) >= 0


def test_build_flags_for_the_kernel_files():
    """Every HIP compile switches packed-fp32 formation off; every kernel file of the C-ABI library is built with
    preloaded kernel arguments except the general norm kernel, and the few-rows norm kernels -- the ones that
    need the preloading most -- live in a file that gets it."""
    from inferspore_amd import build
    flags = build.HIPCC_FLAGS
    i = flags.index("-packed-fp32-ops")
    assert flags[i - 3:i] == ["-Xclang", "-target-feature", "-Xclang"]
    assert "--offload-arch=gfx950" in flags
    assert build.KERNARG_PRELOAD == ["-mllvm", "-amdgpu-kernarg-preload-count=16"]
    kernel_files = sorted(f for f in os.listdir(build.CSRC) if f.endswith(".hip"))
    assert "norm_few_rows.hip" in kernel_files and "norm.hip" in kernel_files
    assert build.NO_KERNARG_PRELOAD == {"norm.hip"}
    few = open(os.path.join(build.CSRC, "norm_few_rows.hip")).read()
    assert "__global__" in few and "void fused_norm_few_rows(" in few
    assert "void fused_norm_few_rows(" not in open(os.path.join(build.CSRC, "norm.hip")).read()
