"""ctypes binding of libw4a16hip.so (include/w4a16_hip.h).  No fallback: if the library or its gfx950 code objects
are missing, loading fails with an error that says how to build them."""
import ctypes as C
import os

PKG = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(PKG, "libw4a16hip.so")

ERR_SHAPE, ERR_SYMBOL, ERR_UNSUPPORTED, ERR_NOT_FOUND, ERR_ARG, ERR_ASSET, ERR_STALE_GRAPH = (
    10001, 10002, 10003, 10004, 10005, 10006, 10007)
PATH_AUTO, PATH_LANE, PATH_DECODE, PATH_PREFILL, PATH_STREAM = 0, 1, 2, 3, 4
ACT_SILU, ACT_GELU_TANH = 0, 1


class W4a16Error(RuntimeError):
    def __init__(self, code, message):
        super().__init__("%s [code %d]" % (message, code))
        self.code = code
        self.message = message


_SIGS = {
    "w4a16_last_error": (C.c_char_p, []),
    "w4a16_ctx_create": (C.c_int, [C.c_int, C.c_char_p, C.POINTER(C.c_void_p)]),
    "w4a16_ctx_destroy": (None, [C.c_void_p]),
    "w4a16_module_load": (C.c_int, [C.c_void_p, C.c_char_p, C.c_void_p, C.c_size_t, C.POINTER(C.c_char_p), C.c_size_t]),
    "w4a16_has_symbol": (C.c_int, [C.c_void_p, C.c_char_p]),
    "w4a16_launch": (C.c_int, [C.c_void_p, C.c_char_p, C.c_uint, C.c_uint, C.c_uint, C.c_uint, C.POINTER(C.c_void_p)]),
    "w4a16_last_launch_symbol": (C.c_char_p, [C.c_void_p]),
    "w4a16_alloc": (C.c_int, [C.c_void_p, C.c_size_t, C.POINTER(C.c_uint64)]),
    "w4a16_free": (C.c_int, [C.c_void_p, C.c_uint64]),
    "w4a16_h2d": (C.c_int, [C.c_void_p, C.c_uint64, C.c_void_p, C.c_size_t]),
    "w4a16_d2h": (C.c_int, [C.c_void_p, C.c_void_p, C.c_uint64, C.c_size_t]),
    "w4a16_d2d": (C.c_int, [C.c_void_p, C.c_uint64, C.c_uint64, C.c_size_t]),
    "w4a16_memset0": (C.c_int, [C.c_void_p, C.c_uint64, C.c_size_t]),
    "w4a16_sync": (C.c_int, [C.c_void_p]),
    "w4a16_allocated_bytes": (C.c_size_t, [C.c_void_p]),
    "w4a16_event_create": (C.c_int, [C.c_void_p, C.POINTER(C.c_void_p)]),
    "w4a16_event_record": (C.c_int, [C.c_void_p, C.c_void_p]),
    "w4a16_event_elapsed_ms": (C.c_int, [C.c_void_p, C.c_void_p, C.c_void_p, C.POINTER(C.c_float)]),
    "w4a16_event_destroy": (None, [C.c_void_p, C.c_void_p]),
    "w4a16_capture_begin": (C.c_int, [C.c_void_p]),
    "w4a16_capture_end": (C.c_int, [C.c_void_p, C.POINTER(C.c_void_p)]),
    "w4a16_graph_launch": (C.c_int, [C.c_void_p, C.c_void_p]),
    "w4a16_graph_nodes": (C.c_size_t, [C.c_void_p]),
    "w4a16_graph_destroy": (None, [C.c_void_p, C.c_void_p]),
    "w4a16_manifest": (C.c_size_t, [C.c_size_t, C.POINTER(C.c_char_p), C.POINTER(C.POINTER(C.c_char_p))]),
    "w4a16_check_shapes": (C.c_int, [C.c_size_t] * 7),
    "w4a16_kernel_sym": (C.c_char_p, [C.c_int, C.c_int]),
    "w4a16_gemm_host": (C.c_int, [C.c_void_p, C.c_void_p, C.c_size_t, C.c_void_p, C.c_void_p, C.c_size_t, C.c_size_t,
                                  C.c_size_t, C.c_int, C.c_void_p]),
    "w4a16_upload_lin": (C.c_int, [C.c_void_p, C.c_char_p, C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t, C.c_size_t,
                                   C.c_size_t, C.c_size_t, C.c_int]),
    "w4a16_lin_drop_raw": (C.c_int, [C.c_void_p, C.c_char_p]),
    "w4a16_lin_info": (C.c_int, [C.c_void_p, C.c_char_p, C.POINTER(C.c_size_t), C.POINTER(C.c_size_t),
                                 C.POINTER(C.c_size_t), C.POINTER(C.c_int), C.POINTER(C.c_int), C.POINTER(C.c_int)]),
    "w4a16_lin_forward": (C.c_int, [C.c_void_p, C.c_char_p, C.c_uint64, C.c_uint64, C.c_size_t, C.c_int, C.c_int]),
    "w4a16_lin_forward_noalloc": (C.c_int, [C.c_void_p, C.c_char_p, C.c_uint64, C.c_uint64, C.c_size_t, C.c_int]),
    "w4a16_noalloc_workspace_bytes": (C.c_size_t, []),
    "w4a16_plan_decode": (C.c_int, [C.c_size_t, C.c_size_t, C.c_size_t, C.c_size_t, C.c_int, C.c_int, C.POINTER(C.c_int),
                                    C.POINTER(C.c_int), C.POINTER(C.c_int), C.POINTER(C.c_size_t)]),
    "w4a16_plan_prefill": (C.c_int, [C.c_size_t, C.c_size_t, C.c_size_t, C.c_size_t, C.c_int, C.c_int, C.c_int,
                                     C.POINTER(C.c_size_t), C.POINTER(C.c_double)]),
    "w4a16_lin_forward_glu": (C.c_int, [C.c_void_p, C.c_char_p, C.c_uint64, C.c_uint64, C.c_size_t]),
    "w4a16_lin_forward_glu_act": (C.c_int, [C.c_void_p, C.c_char_p, C.c_uint64, C.c_uint64, C.c_size_t, C.c_int]),
    "w4a16_lin_forward_deferred_norm": (C.c_int, [C.c_void_p, C.c_char_p, C.c_uint64, C.c_size_t, C.c_size_t, C.c_uint64,
                                                  C.c_size_t, C.c_size_t, C.c_uint64, C.c_int, C.c_uint64, C.c_size_t,
                                                  C.POINTER(C.c_size_t), C.c_uint64, C.c_uint64]),
    "w4a16_lin_forward_glu_deferred_norm": (C.c_int, [C.c_void_p, C.c_char_p, C.c_uint64, C.c_size_t, C.c_size_t,
                                                      C.c_uint64, C.c_size_t, C.c_size_t, C.c_uint64, C.c_int]),
    "w4a16_lin_forward_deferred_norm_scaled": (C.c_int, [C.c_void_p, C.c_char_p, C.c_uint64, C.c_size_t, C.c_size_t,
                                                         C.c_uint64, C.c_size_t, C.c_size_t, C.c_int, C.c_uint64, C.c_int,
                                                         C.c_int, C.c_uint64, C.c_size_t, C.POINTER(C.c_size_t),
                                                         C.c_uint64, C.c_uint64]),
    "w4a16_lin_forward_glu_deferred_norm_scaled": (C.c_int, [C.c_void_p, C.c_char_p, C.c_uint64, C.c_size_t, C.c_size_t,
                                                             C.c_uint64, C.c_size_t, C.c_size_t, C.c_int, C.c_uint64,
                                                             C.c_int, C.c_int]),
    "w4a16_lin_row_norm_max": (C.c_int, [C.c_void_p, C.c_char_p, C.POINTER(C.c_float)]),
    "w4a16_lin_forward_host": (C.c_int, [C.c_void_p, C.c_char_p, C.c_void_p, C.c_void_p, C.c_size_t, C.c_int, C.c_int]),
    "w4a16_dequant_dump": (C.c_int, [C.c_void_p, C.c_char_p, C.c_int, C.c_uint64]),
    "w4a16_lin_untile": (C.c_int, [C.c_void_p, C.c_char_p, C.c_uint64, C.c_uint64]),
    "w4a16_lin_fuse": (C.c_int, [C.c_void_p, C.c_char_p, C.POINTER(C.c_char_p), C.c_size_t, C.c_int]),
    "w4a16_lin_forward_multi": (C.c_int, [C.c_void_p, C.c_char_p, C.c_uint64, C.POINTER(C.c_uint64), C.c_size_t, C.c_size_t,
                                          C.c_int]),
    "w4a16_set_decode_shape": (C.c_int, [C.c_void_p, C.c_int, C.c_int]),
    "w4a16_set_decode_ksplit": (C.c_int, [C.c_void_p, C.c_int]),
    "w4a16_set_prefill_tile": (C.c_int, [C.c_void_p, C.c_int]),
    "w4a16_set_prefill_ksplit": (C.c_int, [C.c_void_p, C.c_int]),
    "w4a16_bench_forward": (C.c_int, [C.c_void_p, C.POINTER(C.c_char_p), C.c_size_t, C.c_uint64, C.c_uint64, C.c_size_t,
                                      C.c_int, C.c_int, C.c_size_t, C.c_size_t, C.POINTER(C.c_float),
                                      C.POINTER(C.c_double)]),
    "w4a16_upload_experts": (C.c_int, [C.c_void_p, C.c_char_p, C.c_size_t, C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t,
                                       C.c_void_p, C.c_size_t, C.c_void_p, C.c_size_t, C.c_size_t, C.c_size_t, C.c_size_t,
                                       C.c_int]),
    "w4a16_experts_info": (C.c_int, [C.c_void_p, C.c_char_p, C.POINTER(C.c_size_t), C.POINTER(C.c_size_t),
                                     C.POINTER(C.c_size_t), C.POINTER(C.c_size_t), C.POINTER(C.c_int)]),
    "w4a16_experts_dequant_dump": (C.c_int, [C.c_void_p, C.c_char_p, C.c_int, C.c_size_t, C.c_uint64]),
    "w4a16_moe_topk_host": (C.c_int, [C.c_void_p, C.c_size_t, C.c_size_t, C.c_size_t, C.c_void_p, C.c_void_p]),
    "w4a16_moe_route": (C.c_int, [C.c_void_p, C.c_uint64, C.c_size_t, C.c_size_t, C.c_size_t, C.c_uint64, C.c_uint64]),
    "w4a16_moe_align": (C.c_int, [C.c_void_p, C.c_uint64, C.c_size_t, C.c_size_t, C.c_size_t, C.c_uint64, C.c_uint64,
                                  C.c_uint64]),
    "w4a16_moe_ffn": (C.c_int, [C.c_void_p, C.c_char_p, C.c_uint64, C.c_uint64, C.c_uint64, C.c_size_t, C.c_size_t,
                                C.c_uint64]),
    "w4a16_moe_ffn_act": (C.c_int, [C.c_void_p, C.c_char_p, C.c_uint64, C.c_uint64, C.c_uint64, C.c_size_t, C.c_size_t,
                                    C.c_uint64, C.c_int]),
    "w4a16_moe_scratch": (C.c_int, [C.c_void_p, C.c_int, C.POINTER(C.c_uint64), C.POINTER(C.c_size_t),
                                    C.POINTER(C.c_size_t)]),
    "w4a16_set_moe_shape": (C.c_int, [C.c_void_p, C.c_int, C.c_int]),
    "w4a16_set_moe_tiled": (C.c_int, [C.c_void_p, C.c_int]),
    "w4a16_upload_lin_synth": (C.c_int, [C.c_void_p, C.c_char_p, C.c_size_t, C.c_size_t, C.c_size_t, C.c_uint64, C.c_uint64,
                                         C.c_float, C.c_float]),
    "w4a16_rms_rescale_f16": (C.c_int, [C.c_void_p, C.c_uint64, C.c_size_t, C.c_size_t, C.c_size_t, C.c_uint64]),
    "w4a16_norm_resid": (C.c_int, [C.c_void_p, C.c_uint64, C.c_uint64, C.c_uint64, C.c_uint64, C.c_uint64, C.c_uint64,
                                   C.c_size_t, C.c_size_t, C.c_size_t]),
    "w4a16_silu_mul_f16": (C.c_int, [C.c_void_p, C.c_uint64, C.c_size_t, C.c_size_t, C.c_uint64]),
    "w4a16_act_mul_f16": (C.c_int, [C.c_void_p, C.c_uint64, C.c_size_t, C.c_size_t, C.c_uint64, C.c_int]),
    "w4a16_chain_forward": (C.c_int, [C.c_void_p, C.c_char_p, C.c_size_t, C.c_size_t, C.c_uint64, C.c_size_t, C.c_uint64]),
    "w4a16_chain_forward_fused": (C.c_int, [C.c_void_p, C.c_char_p, C.c_size_t, C.c_size_t, C.c_uint64, C.c_size_t, C.c_uint64]),
    "w4a16_chain_graph_create": (C.c_int, [C.c_void_p, C.c_char_p, C.c_size_t, C.c_size_t, C.c_uint64, C.c_size_t,
                                           C.c_uint64, C.c_int, C.POINTER(C.c_void_p)]),
    "w4a16_bench_chain": (C.c_int, [C.c_void_p, C.c_char_p, C.c_size_t, C.c_uint64, C.c_size_t, C.c_uint64, C.c_size_t,
                                    C.c_size_t, C.c_int, C.c_int, C.POINTER(C.c_float), C.POINTER(C.c_double)]),
    "w4a16_bench_moe": (C.c_int, [C.c_void_p, C.POINTER(C.c_char_p), C.c_size_t, C.c_uint64, C.c_uint64, C.c_uint64,
                                  C.c_size_t, C.c_size_t, C.c_uint64, C.c_size_t, C.c_size_t, C.POINTER(C.c_float),
                                  C.POINTER(C.c_double)]),
}

_lib = None


def load():
    """Load the in-tree shared library; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("libw4a16hip.so is not built: run `python -m llm170_amd.build` (needs hipcc)")
        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in _SIGS.items():
            fn = getattr(lib, name)  # AttributeError if the library lacks a declared entry point
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def declared_symbols():
    return sorted(_SIGS)


def check(rc):
    if rc != 0:
        raise W4a16Error(rc, load().w4a16_last_error().decode("utf-8", "replace"))


def manifest():
    lib = load()
    out = {}
    count = lib.w4a16_manifest(1 << 30, None, None)
    for a in range(count):
        name = C.c_char_p()
        syms = C.POINTER(C.c_char_p)()
        lib.w4a16_manifest(a, C.byref(name), C.byref(syms))
        lst = []
        i = 0
        while syms[i]:
            lst.append(syms[i].decode())
            i += 1
        out[name.value.decode()] = lst
    return out
