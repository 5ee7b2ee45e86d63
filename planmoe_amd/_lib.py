"""ctypes binding of libplanmoe_hip.so (the C ABI declared in include/planmoe_hip.h).

The library is the only compute back end of this package: there is no CPU or eager
fall-back.  Importing this module raises if the shared object has not been built
(``python -c "import __graft_entry__ as g; g.build()"`` or ``make -C planmoe_amd/csrc``).
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "libplanmoe_hip.so")

ABI_VERSION = 1

c_void_p, c_int, c_int64, c_size_t, c_double = (ctypes.c_void_p, ctypes.c_int, ctypes.c_int64,
                                                ctypes.c_size_t, ctypes.c_double)

# name -> (restype, argtypes): one entry per function declared in include/planmoe_hip.h
SIGNATURES = {
    "planmoe_abi_version": (c_int, []),
    "planmoe_last_error": (ctypes.c_char_p, []),
    "planmoe_cumsum_workspace_bytes": (c_size_t, [c_int, c_int]),
    "planmoe_cumsum_sub_one": (c_int, [c_void_p, c_void_p, c_int, c_int, c_void_p, c_size_t, c_void_p]),
    "planmoe_capacity": (c_int, [c_int, c_int, c_int, c_double, c_int, ctypes.POINTER(c_int)]),
    "planmoe_route_workspace_bytes": (c_size_t, [c_int, c_int, c_int]),
    "planmoe_route_topk": (c_int, [c_void_p, c_int, c_int, c_void_p, c_int, c_int, c_int, c_int,
                                   c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_void_p,
                                   c_void_p, c_void_p, c_size_t, c_void_p]),
    "planmoe_route_locations": (c_int, [c_void_p, c_int64, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p,
                                        c_void_p, c_size_t, c_void_p]),
    "planmoe_route_bwd": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_int64, c_int, c_int, c_int, c_int,
                                  c_void_p, c_void_p, c_int, c_void_p, c_void_p]),
    "planmoe_gate_logits": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int,
                                    c_void_p]),
    "planmoe_dispatch_workspace_bytes": (c_size_t, [c_int, c_int]),
    "planmoe_dispatch_fwd": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int64, c_int,
                                     c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_size_t,
                                     c_void_p]),
    "planmoe_combine_fwd": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int64, c_int,
                                    c_int, c_int, c_int, c_void_p, c_void_p]),
    "planmoe_bwd_gate": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int64, c_int,
                                 c_int, c_int, c_int, c_void_p, c_void_p]),
    "planmoe_int8_compress": (c_int, [c_void_p, c_int, c_int64, c_int, c_void_p, c_void_p, c_void_p,
                                      c_void_p]),
    "planmoe_int8_decompress": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int,
                                        c_void_p, c_void_p]),
    "planmoe_dispatch_int8": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int64, c_int,
                                      c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p,
                                      c_void_p, c_size_t, c_void_p]),
    "planmoe_combine_bwd_int8": (c_int, [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int64, c_int,
                                         c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p,
                                         c_void_p, c_size_t, c_void_p]),
    "planmoe_combine_bwd_int8_coded": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p,
                                               c_void_p, c_int64, c_int, c_int, c_int, c_int, c_int, c_void_p,
                                               c_void_p, c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "planmoe_combine_int8": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int64,
                                     c_int, c_int, c_int, c_int, c_void_p, c_void_p]),
    "planmoe_forward_workspace_bytes": (c_size_t, [c_int, c_int, c_int]),
    "planmoe_gate_route": (c_int, [c_void_p, c_void_p, c_int, c_int, c_void_p, c_int, c_int, c_int, c_int,
                                   c_int, c_void_p, c_void_p, c_void_p, c_int64, c_void_p, c_void_p,
                                   c_void_p, c_void_p, c_void_p, c_size_t, c_void_p]),
    "planmoe_forward_plain": (c_int, [c_void_p, c_void_p, c_int, c_int, c_void_p, c_int, c_int, c_int, c_int,
                                      c_int, c_int, c_void_p, c_void_p, c_void_p, c_int64, c_void_p,
                                      c_void_p, c_void_p, c_void_p, c_void_p,
                                      c_void_p, c_size_t, c_void_p]),
    "planmoe_forward_int8": (c_int, [c_void_p, c_void_p, c_int, c_int, c_void_p, c_int, c_int, c_int, c_int,
                                     c_int, c_int, c_void_p, c_void_p, c_void_p, c_int64, c_void_p,
                                     c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                     c_void_p, c_size_t, c_void_p]),
    "planmoe_forward_int8_single_serves": (c_int, [c_int, c_int, c_int, c_int, c_int, c_int]),
    "planmoe_forward_int8_single": (c_int, [c_void_p, c_void_p, c_int, c_int, c_void_p, c_int, c_int, c_int, c_int,
                                            c_int, c_int, c_void_p, c_void_p, c_void_p, c_int64, c_void_p,
                                            c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                            c_void_p, c_size_t, c_int, c_void_p, c_void_p]),
    "planmoe_forward_int8_single_ceiling": (c_int, [c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p,
                                                    c_void_p, c_void_p, c_size_t, c_int, c_int, c_void_p, c_void_p]),
    "planmoe_gemm_nt_bf16": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
                                     c_int64, c_int64, c_int64, c_void_p, c_void_p]),
    "planmoe_gemm_nn_bf16": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int,
                                     c_int64, c_int64, c_int64, c_void_p, c_void_p]),
    "planmoe_gemm_tn_bf16": (c_int, [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_int64,
                                     c_int64, c_int64, c_void_p, c_void_p]),
    "planmoe_transpose_bf16": (c_int, [c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_void_p]),
    "planmoe_forward_int8_static": (c_int, [c_void_p, c_void_p, c_int, c_int, c_void_p, c_int, c_int, c_int, c_int,
                                            c_int, c_int, c_void_p, c_void_p, c_void_p, c_int64, c_void_p,
                                            c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                            c_void_p]),
    "planmoe_forward_int8_redispatch": (c_int, [c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p,
                                                c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p,
                                                c_size_t, c_void_p]),
    "planmoe_ffn_fc1_int8": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int,
                                     c_int, c_void_p, c_void_p]),
    "planmoe_ffn_fc1_int8_affine": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_int, c_int,
                                            c_int, c_int, c_void_p, c_void_p]),
    "planmoe_zfp_max_bytes": (c_size_t, [c_int, c_int64, c_int64, c_double]),
    "planmoe_zfp_stream_bytes": (c_size_t, [c_int, c_int64, c_int64, c_double]),
    "planmoe_zfp_compress": (c_int, [c_void_p, c_int, c_int64, c_int64, c_double, c_void_p, c_size_t,
                                     c_void_p]),
    "planmoe_zfp_decompress": (c_int, [c_void_p, c_int, c_int64, c_int64, c_double, c_void_p,
                                       c_void_p]),
    "planmoe_dispatch_zfp_workspace_bytes": (c_size_t, [c_int, c_int]),
    "planmoe_dispatch_zfp": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_int64, c_int, c_int, c_int, c_int,
                                     c_int, c_double, c_void_p, c_size_t, c_void_p, c_size_t, c_void_p]),
    "planmoe_combine_zfp_workspace_bytes": (c_size_t, [c_int, c_int]),
    "planmoe_combine_zfp": (c_int, [c_void_p, c_double, c_void_p, c_void_p, c_void_p, c_int64, c_int, c_int, c_int,
                                    c_int, c_int, c_void_p, c_void_p, c_size_t, c_void_p]),
    "planmoe_gate_dx_accumulate": (c_int, [c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]),
    "planmoe_bwd_gate_zfp": (c_int, [c_void_p, c_double, c_void_p, c_void_p, c_void_p, c_int64, c_int, c_int, c_int,
                                     c_int, c_int, c_void_p, c_void_p, c_size_t, c_void_p]),
    "planmoe_lz_blocks": (c_int64, [c_int64]),
    "planmoe_lz_workspace_bytes": (c_size_t, [c_int64]),
    "planmoe_lz_compress": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                    c_size_t, c_void_p]),
    "planmoe_lz_decompress": (c_int, [c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]),
}


class PlanMoEError(RuntimeError):
    """Raised when a libplanmoe_hip entry point reports an error (mirrors the c10::Error ->
    RuntimeError path of the reference's AT_ASSERTM checks)."""


def _load():
    if not os.path.exists(LIB_PATH):
        raise ImportError(
            "planmoe_amd: %s is missing. This package has no CPU fall-back; build the HIP "
            "library first (make -C planmoe_amd/csrc, or __graft_entry__.build())." % LIB_PATH)
    lib = ctypes.CDLL(LIB_PATH)
    for name, (restype, argtypes) in SIGNATURES.items():
        fn = getattr(lib, name)          # AttributeError if the build lacks a declared symbol
        fn.restype = restype
        fn.argtypes = argtypes
    got = lib.planmoe_abi_version()
    if got != ABI_VERSION:
        raise ImportError("planmoe_amd: ABI version mismatch (library %d, binding %d)" % (got, ABI_VERSION))
    return lib


lib = _load()


def check(rc):
    if rc != 0:
        raise PlanMoEError(lib.planmoe_last_error().decode("utf-8", "replace"))
