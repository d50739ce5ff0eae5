"""The C-ABI library loads and exports exactly what include/tokenweave_amd.h
declares; argument errors are reported as codes, never as crashes.  None of
these calls launches a kernel, so they run without a GPU."""
import ctypes
import os
import re

import pytest

from tokenweave_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "tokenweave_amd.h")


def declared_symbols():
    text = open(HEADER).read()
    return re.findall(r"TW_API\s+[\w\s\*]+?\b(tw_\w+)\s*\(", text)


def test_header_declares_the_expected_entry_points():
    syms = declared_symbols()
    assert len(syms) == len(set(syms)) >= 11
    for must in ("tw_fused_add_rms_norm", "tw_rms_norm", "tw_rms_norm_inplace",
                 "tw_fused_add_rms_norm_cta", "tw_reduce_add_rms_norm", "tw_fused_rs_ln_cta",
                 "tw_fused_rs_ln_ag_cta", "tw_gemm_bf16_nt", "tw_last_error"):
        assert must in syms


def test_library_exports_every_declared_symbol():
    assert os.path.exists(_lib.LIB_PATH), "build with make -C tokenweave_amd/csrc"
    L = ctypes.CDLL(_lib.LIB_PATH)
    for s in declared_symbols():
        assert hasattr(L, s), f"{s} declared in the header but not exported"
    assert set(declared_symbols()) == set(_lib.PROTOTYPES), "ctypes prototypes out of sync with header"


def test_header_cites_the_reference_interface_for_each_op():
    text = re.sub(r"\s*\n\s*\*\s*", "", open(HEADER).read())  # undo comment line wraps
    for cite in ("csrc/layernorm_kernels.cu:194-231", "csrc/torch_bindings.cpp:141-144",
                 "csrc/tokenweave_fused_kernels.cu:220-261", "csrc/torch_bindings.cpp:152-157",
                 "csrc/tokenweave_artifact_kernels.cu:717-754", "csrc/tokenweave_artifact_kernels.cu:772-813",
                 "csrc/tokenweave_fused_kernels.cu:186-202", "vllm/model_executor/layers/linear.py:203-228",
                 "1310-1321", "csrc/tokenweave_fused_kernels.cu:241-244"):
        assert cite in text, cite


def test_version_and_empty_error():
    L = _lib.lib()
    assert L.tw_version() >= 100


BUF = ctypes.create_string_buffer(4096 + 64)
ALIGNED = (ctypes.addressof(BUF) + 63) & ~63   # host memory: never dereferenced by these calls


def test_zero_tokens_is_ok_without_touching_the_gpu():
    L = _lib.lib()
    assert L.tw_fused_add_rms_norm(None, None, None, 0, 8192, 1e-5, _lib.TW_DTYPE_BF16, None) == _lib.TW_OK
    assert L.tw_rms_norm(None, None, None, 0, 64, 1e-5, _lib.TW_DTYPE_F32, None) == _lib.TW_OK
    assert L.tw_gemm_bf16_nt(None, None, None, 0, 128, 64, 128, 0, None) == _lib.TW_OK


def test_invalid_arguments_return_codes_and_messages():
    L = _lib.lib()
    assert L.tw_fused_add_rms_norm(None, ALIGNED, ALIGNED, 4, 64, 1e-5, 0, None) == _lib.TW_ERR_INVALID_ARGUMENT
    assert "null" in _lib.last_error()
    assert L.tw_fused_add_rms_norm(ALIGNED, None, ALIGNED, 4, 64, 1e-5, 0, None) == _lib.TW_ERR_INVALID_ARGUMENT
    assert L.tw_rms_norm(ALIGNED, ALIGNED, ALIGNED, -1, 64, 1e-5, 0, None) == _lib.TW_ERR_INVALID_ARGUMENT
    assert L.tw_rms_norm(ALIGNED, ALIGNED, ALIGNED, 4, 0, 1e-5, 0, None) == _lib.TW_ERR_INVALID_ARGUMENT
    assert L.tw_rms_norm(ALIGNED, ALIGNED, ALIGNED, 4, 64, 1e-5, 7, None) == _lib.TW_ERR_DTYPE
    assert L.tw_rms_norm_inplace(ALIGNED, ALIGNED, ALIGNED, 4, 64, 1e-5, 0, None) == _lib.TW_ERR_INVALID_ARGUMENT
    assert "alias" in _lib.last_error()
    ptrs = (ctypes.c_void_p * 17)(*([ALIGNED] * 17))
    assert L.tw_reduce_add_rms_norm(ptrs, 17, ALIGNED, ALIGNED, ALIGNED, 4, 64, 0, 1e-5, None) == _lib.TW_ERR_INVALID_ARGUMENT
    assert L.tw_reduce_add_rms_norm(ptrs, 0, ALIGNED, ALIGNED, ALIGNED, 4, 64, 0, 1e-5, None) == _lib.TW_ERR_INVALID_ARGUMENT
    ptrs[1] = None
    assert L.tw_reduce_add_rms_norm(ptrs, 2, ALIGNED, ALIGNED, ALIGNED, 4, 64, 0, 1e-5, None) == _lib.TW_ERR_INVALID_ARGUMENT
    assert "partial 1" in _lib.last_error()


def test_cta_entry_points_refuse_misaligned_or_odd_hidden_like_the_reference():
    """TORCH_CHECK(false, ...) at csrc/tokenweave_fused_kernels.cu:257-260."""
    L = _lib.lib()
    msg = "must be 16-byte aligned and hidden_size must be divisible by 8"
    assert L.tw_fused_add_rms_norm_cta(ALIGNED, ALIGNED, ALIGNED, 4, 12, 8, 1e-5, None) == _lib.TW_ERR_ALIGNMENT
    assert msg in _lib.last_error()
    assert L.tw_fused_add_rms_norm_cta(ALIGNED + 2, ALIGNED, ALIGNED, 4, 64, 8, 1e-5, None) == _lib.TW_ERR_ALIGNMENT
    ptrs = (ctypes.c_void_p * 2)(ALIGNED, ALIGNED + 8)
    assert L.tw_reduce_add_rms_norm(ptrs, 2, ALIGNED, ALIGNED, ALIGNED, 4, 64, 0, 1e-5, None) == _lib.TW_ERR_ALIGNMENT
    assert L.tw_fused_rs_ln_ag_cta(ALIGNED, ALIGNED, ALIGNED, ALIGNED, 24, 0, 2, 8, 1e-5, 4, 64, None) == _lib.TW_ERR_ALIGNMENT
    assert L.tw_fused_rs_ln_cta(ALIGNED, ALIGNED, ALIGNED, ALIGNED, 1024, 2, 2, 8, 1e-5, 4, 64, None) == _lib.TW_ERR_INVALID_ARGUMENT
    assert "Invalid rank 2" in _lib.last_error()
    assert L.tw_fused_rs_ln_cta(ALIGNED, ALIGNED, ALIGNED, 0, 1024, 0, 2, 8, 1e-5, 4, 64, None) == _lib.TW_ERR_INVALID_ARGUMENT
    assert L.tw_fused_rs_ln_cta(ALIGNED, ALIGNED, ALIGNED, ALIGNED, 1024, 0, 17, 8, 1e-5, 4, 64, None) == _lib.TW_ERR_INVALID_ARGUMENT


def test_workspace_and_static_workspace_entry_points_check_before_they_launch():
    L = _lib.lib()
    ptrs = (ctypes.c_void_p * 2)(ALIGNED, ALIGNED)
    args = (ptrs, 2, ALIGNED, ALIGNED, ALIGNED, 4, 64, 0, 1e-5)
    assert L.tw_reduce_add_rms_norm_ws(*args, ALIGNED, 100, None) == _lib.TW_ERR_INVALID_ARGUMENT
    assert "workspace" in _lib.last_error() and str(_lib.TW_SPLIT_WORKSPACE_BYTES) in _lib.last_error()
    assert L.tw_fused_rs_ln_ag_cta_ws(ALIGNED, ALIGNED, ALIGNED, ALIGNED, 1024, 0, 2, 0, 1e-5, 4, 64, ALIGNED, 100,
                                      None) == _lib.TW_ERR_INVALID_ARGUMENT
    assert L.tw_reduce_add_rms_norm_ws(ptrs, 2, ALIGNED, None, ALIGNED, 4, 64, 0, 1e-5, None, 0, None) == \
        _lib.TW_ERR_INVALID_ARGUMENT
    assert L.tw_reduce_add_rms_norm_ws(ptrs, 2, None, None, None, 0, 64, 0, 1e-5, None, 0, None) == _lib.TW_OK
    # the static workspace holds TW_SPLIT_MAX_TOKENS rows: larger batches are refused up front
    too_many = _lib.TW_SPLIT_MAX_TOKENS + 1
    assert L.tw_reduce_add_rms_norm_noalloc(ptrs, 2, ALIGNED, ALIGNED, ALIGNED, too_many, 64, 0, 1e-5, None) == \
        _lib.TW_ERR_INVALID_ARGUMENT
    assert "exceeds" in _lib.last_error()
    assert _lib.TW_SPLIT_WORKSPACE_BYTES == 256 * 384
    text = open(HEADER).read()
    assert "#define TW_SPLIT_MAX_TOKENS 256" in text and "(TW_SPLIT_MAX_TOKENS * 384)" in text


def test_partials_producer_argument_checks():
    L = _lib.lib()
    vp = ctypes.c_void_p
    three = (vp * 3)(ALIGNED, ALIGNED, ALIGNED)
    assert L.tw_gemm_bf16_nt_partials(three, three, three, 0, 16, 64, 64, 64, 0, None) == _lib.TW_ERR_INVALID_ARGUMENT
    assert L.tw_gemm_bf16_nt_partials(three, three, three, 17, 16, 64, 64, 64, 0, None) == _lib.TW_ERR_INVALID_ARGUMENT
    assert L.tw_gemm_bf16_nt_partials(three, three, three, 3, 0, 64, 64, 64, 0, None) == _lib.TW_OK
    assert L.tw_gemm_bf16_nt_partials(three, three, three, 3, 16, 64, 12, 64, 0, None) == _lib.TW_ERR_ALIGNMENT
    bad = (vp * 3)(ALIGNED, None, ALIGNED)
    assert L.tw_gemm_bf16_nt_partials(three, bad, three, 3, 16, 64, 64, 64, 0, None) == _lib.TW_ERR_INVALID_ARGUMENT
    odd = (vp * 3)(ALIGNED, ALIGNED + 4, ALIGNED)
    assert L.tw_gemm_bf16_nt_partials(odd, three, three, 3, 16, 64, 64, 64, 0, None) == _lib.TW_ERR_ALIGNMENT
    assert L.tw_gemm_bf16_nt_partials(None, three, three, 3, 16, 64, 64, 64, 0, None) == _lib.TW_ERR_INVALID_ARGUMENT


def test_gemm_argument_checks():
    L = _lib.lib()
    assert L.tw_gemm_bf16_nt(ALIGNED, ALIGNED, ALIGNED, 16, 64, 12, 64, 0, None) == _lib.TW_ERR_ALIGNMENT
    assert L.tw_gemm_bf16_nt(ALIGNED, ALIGNED, ALIGNED, 16, 64, 64, 32, 0, None) == _lib.TW_ERR_INVALID_ARGUMENT
    assert L.tw_gemm_bf16_nt(None, ALIGNED, ALIGNED, 16, 64, 64, 64, 0, None) == _lib.TW_ERR_INVALID_ARGUMENT


def test_check_maps_codes_to_the_reference_exception_types():
    L = _lib.lib()
    rc = L.tw_rms_norm(ALIGNED, ALIGNED, ALIGNED, 4, 64, 1e-5, 9, None)
    with pytest.raises(NotImplementedError):
        _lib.check(rc)
    rc = L.tw_fused_add_rms_norm_cta(ALIGNED, ALIGNED, ALIGNED, 4, 12, 8, 1e-5, None)
    with pytest.raises(RuntimeError, match="16-byte aligned"):
        _lib.check(rc)
