"""The C-ABI library loads, exports every symbol include/planmoe_hip.h declares, and its
argument checks (which run before anything touches a GPU) report errors as the header says."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "planmoe_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(planmoe_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_surface():
    names = declared_symbols()
    for must in ("planmoe_route_topk", "planmoe_dispatch_fwd", "planmoe_combine_fwd", "planmoe_bwd_gate",
                 "planmoe_int8_compress", "planmoe_int8_decompress", "planmoe_zfp_compress",
                 "planmoe_zfp_decompress", "planmoe_cumsum_sub_one", "planmoe_gate_logits",
                 "planmoe_dispatch_int8"):
        assert must in names


def test_library_exports_every_declared_symbol():
    from planmoe_amd import _lib
    raw = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared_symbols():
        assert hasattr(raw, name), name
    assert set(_lib.SIGNATURES) == set(declared_symbols())
    assert _lib.lib.planmoe_abi_version() == 1


def test_capacity_is_host_only_arithmetic():
    from planmoe_amd import ops
    assert ops.capacity(16384, 8, 2, 1.25, 4) == 5120
    assert ops.capacity(32768, 64, 1, 1.0, 4) == 512
    assert ops.capacity(10, 3, 5, 1.0, 1) == 12          # top_k clamps to the expert count
    from planmoe_amd._lib import PlanMoEError
    with pytest.raises(PlanMoEError):
        ops.capacity(10, 3, 2, 0.0, 1)


def test_argument_errors_are_reported_without_a_gpu():
    from planmoe_amd._lib import lib
    # zfp extents must be multiples of 4 -> the reference's "zfp fails." assertion
    rc = lib.planmoe_zfp_compress(None, 2, 6, 8, 8.0, None, 0, None)
    assert rc != 0 and b"zfp fails." in lib.planmoe_last_error()
    rc = lib.planmoe_zfp_compress(None, 3, 8, 8, 8.0, None, 0, None)
    assert rc != 0 and b"dims" in lib.planmoe_last_error()
    rc = lib.planmoe_zfp_compress(None, 2, 8, 8, 7.0, None, 0, None)
    assert rc != 0 and b"bits per block" in lib.planmoe_last_error()
    rc = lib.planmoe_int8_compress(None, 7, 4, 4, None, None, None, None)
    assert rc != 0 and b"dtype" in lib.planmoe_last_error()
    rc = lib.planmoe_route_topk(None, 0, 0, None, 4, 4096, 1, 1, None, None, None, 4, None, None, None, None, 0, None)
    assert rc != 0 and b"experts" in lib.planmoe_last_error()
    # sizes that would overflow the 32-bit slot / offset arithmetic are refused, not wrapped
    p16 = ctypes.c_void_p(16)
    rc = lib.planmoe_dispatch_fwd(p16, 0, None, p16, p16, 8, 1, 8, 64, 70000, 70000, p16, p16, 1 << 40, None)
    assert rc != 0 and b"overflows int32" in lib.planmoe_last_error()
    rc = lib.planmoe_lz_compress(p16, 1 << 31, p16, p16, p16, p16, p16, 1 << 40, None)
    assert rc != 0 and b"too large" in lib.planmoe_last_error()
    rc = lib.planmoe_lz_compress(p16, 6, p16, p16, p16, p16, p16, 1 << 40, None)
    assert rc != 0 and b"multiple of 4" in lib.planmoe_last_error()
    rc = lib.planmoe_dispatch_zfp(p16, None, p16, p16, 8, 1, 8, 64, 3, 2, 8.0, p16, 1 << 40, p16, 1 << 40, None)
    assert rc != 0 and b"zfp fails." in lib.planmoe_last_error()          # 6 slot rows
    rc = lib.planmoe_forward_int8(p16, p16, 1, 1, None, 64, 512, 65, 2, 1, 16, p16, p16, p16, 64, None, None, None,
                                  None, p16, p16, p16, p16, 1 << 40, None)
    assert rc != 0 and b"64 experts" in lib.planmoe_last_error()
    # the GEMM forms that read an operand along its slow index take the reduction in steps of 64
    rc = lib.planmoe_gemm_nn_bf16(p16, p16, None, 0, 1, 64, 64, 96, 96, 64, 64, 0, 0, 0, p16, None)
    assert rc != 0 and b"multiple of 64" in lib.planmoe_last_error()
    rc = lib.planmoe_gemm_tn_bf16(p16, p16, 1, 64, 64, 96, 64, 64, 64, 0, 0, 0, p16, None)
    assert rc != 0 and b"multiple of 64" in lib.planmoe_last_error()
    rc = lib.planmoe_gemm_tn_bf16(p16, p16, 1, 60, 64, 64, 64, 64, 64, 0, 0, 0, p16, None)
    assert rc != 0 and b"multiples of 8" in lib.planmoe_last_error()
    rc = lib.planmoe_gemm_nn_bf16(p16, p16, None, 2, 1, 64, 64, 64, 64, 64, 64, 0, 0, 0, p16, None)
    assert rc != 0 and b"activation" in lib.planmoe_last_error()
    assert lib.planmoe_gemm_tn_bf16(None, None, 0, 64, 64, 64, 64, 64, 64, 0, 0, 0, None, None) == 0
    # empty inputs are a successful no-op
    assert lib.planmoe_int8_compress(None, 0, 0, 8, None, None, None, None) == 0
    assert lib.planmoe_lz_blocks(0) == 0 and lib.planmoe_lz_blocks(2049) == 2
    assert lib.planmoe_lz_decompress(None, 0, None, None, None, None, None) == 0
    assert lib.planmoe_combine_fwd(None, 0, None, ctypes.c_void_p(16), ctypes.c_void_p(16), 0, 1, 0, 8, 4, None, None) == 0


def test_size_queries():
    from planmoe_amd import ops
    assert ops.zfp_stream_bytes(2, 1024, 131072) == 1024 * 131072          # 8 bits per value
    assert ops.zfp_stream_bytes(1, 1024, 131072) == 1024 * 131072
    assert ops.zfp_max_bytes(2, 64, 32) == 2072 and ops.zfp_max_bytes(1, 64, 32) == 2072
    assert ops.zfp_stream_bytes(1, 12, 1) == 16                            # 3 blocks -> 2 words
