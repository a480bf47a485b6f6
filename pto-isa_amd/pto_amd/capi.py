"""ctypes binding of libpto_amd.so (the C ABI declared in include/pto_amd.h).

Device pointers are passed as integers (e.g. torch.Tensor.data_ptr()); streams as integers
(torch.cuda.current_stream().cuda_stream) or 0 for the default stream.  The library must have been
built (python pto-isa_amd/build.py): loading fails loudly otherwise, there is no fallback path.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LIB_PATH = os.path.join(_HERE, "libpto_amd.so")

OK, ERR_BAD_ARG, ERR_UNSUPPORTED, ERR_HIP, ERR_WORKSPACE = 0, -1, -2, -3, -4
CAST_RINT, CAST_ROUND, CAST_FLOOR, CAST_CEIL, CAST_TRUNC, CAST_ODD = 1, 2, 3, 4, 5, 6

SYMBOLS = {
    "pto_init": (C.c_int, []),
    "pto_version": (C.c_char_p, []),
    "pto_last_hip_error": (C.c_int, []),
    "pto_gemm_f16f32": (C.c_int, [C.c_void_p] * 4 + [C.c_int] * 3),
    "pto_gemm_mxfp8": (C.c_int, [C.c_void_p] * 6 + [C.c_int] * 5),
    "pto_gemm_mxfp4": (C.c_int, [C.c_void_p] * 6 + [C.c_int] * 4),
    "pto_topk_f32": (C.c_int, [C.c_void_p] * 5 + [C.c_int] * 4),
    "pto_quant_mxfp8_f32": (C.c_int, [C.c_void_p] * 4 + [C.c_size_t] * 2),
    "pto_attention_auto_f32": (C.c_int, [C.c_void_p] * 5 + [C.c_int] * 4),
    "pto_mla_attention_f32_s64_d32_r16": (C.c_int, [C.c_void_p] * 9 + [C.c_int] * 2),
    "pto_fa_fwd_f16": (C.c_int, [C.c_void_p] * 6 + [C.c_int] * 7),
    "pto_tcvt_f32_f16": (C.c_int, [C.c_void_p] * 3 + [C.c_size_t, C.c_int]),
    "pto_tcvt_f32_bf16": (C.c_int, [C.c_void_p] * 3 + [C.c_size_t, C.c_int]),
    "pto_gather_rows": (C.c_int, [C.c_void_p] * 4 + [C.c_size_t] * 3 + [C.c_int]),
    "pto_tgather_index_f16_16x1024_16x128": (C.c_int, [C.c_void_p] * 4),
}

# Test-only library (include/pto_amd_st.h): single-tile programs and tuning hooks, on top of every product symbol.
ST_LIB_PATH = os.path.join(_HERE, "libpto_st.so")
_V = [C.c_void_p] * 4 + [C.c_int] * 4
ST_SYMBOLS = {
    "pto_gemm_f16f32_variant": (C.c_int, _V),
    "pto_gemm_f16f32_w4_variant": (C.c_int, _V),
    "pto_gemm_mxfp8_variant": (C.c_int, [C.c_void_p] * 6 + [C.c_int] * 6),
    "pto_fa_fwd_f16_variant": (C.c_int, [C.c_void_p] * 6 + [C.c_int] * 7),
    "pto_st_softmax_step_f32_64x256": (C.c_int, [C.c_void_p] * 8 + [C.c_float, C.c_int, C.c_int]),
    "pto_st_gu_step_f32_64x128": (C.c_int, [C.c_void_p] * 6 + [C.c_int]),
    "pto_st_tri_mask_f32_64x128": (C.c_int, [C.c_void_p] * 3 + [C.c_int, C.c_float, C.c_int]),
    "pto_st_tgather_mask_b16_16x64": (C.c_int, [C.c_void_p] * 3 + [C.c_int]),
    "pto_st_mgather_b16_8x128": (C.c_int, [C.c_void_p] * 4 + [C.c_int]),
    "pto_st_tload_pad_f32_16x32": (C.c_int, [C.c_void_p] * 3),
    "pto_st_tload_5d_f32": (C.c_int, [C.c_void_p] * 4),
    "pto_st_mat_view_walk": (C.c_int, [C.c_void_p, C.c_void_p, C.c_int]),
    "pto_st_textract_windows_f16": (C.c_int, [C.c_void_p] * 7 + [C.c_int] * 2),
    "pto_st_matmul_bias_128x64x256": (C.c_int, [C.c_void_p] * 5 + [C.c_int]),
    "pto_st_matmul_ragged": (C.c_int, [C.c_void_p] * 5 + [C.c_int]),
    "pto_st_matmul_s8_128x128x256": (C.c_int, [C.c_void_p] * 4 + [C.c_int]),
    "pto_st_matmul_f32_128x32x256": (C.c_int, [C.c_void_p] * 4 + [C.c_int]),
    "pto_st_matmul_mx_128x256x128": (C.c_int, [C.c_void_p] * 6 + [C.c_int] * 3),
    "pto_st_tquant_mxfp8": (C.c_int, [C.c_void_p] * 6 + [C.c_int] * 3),
    "pto_st_matmul_mx_bias_128x256x128": (C.c_int, [C.c_void_p] * 7 + [C.c_int] * 2),
    "pto_st_vec_op_typed_64x128": (C.c_int, [C.c_void_p] * 5 + [C.c_float, C.c_int, C.c_int]),
    "pto_st_matmul_vec_operands_f16_64x64x128": (C.c_int, [C.c_void_p] * 5),
    "pto_st_tpart_f32_64x128": (C.c_int, [C.c_void_p] * 4 + [C.c_int] * 7),
    "pto_st_scatter_f32_64x128": (C.c_int, [C.c_void_p] * 4 + [C.c_int] * 3),
    "pto_st_tgatherb_f32_16x128": (C.c_int, [C.c_void_p] * 4 + [C.c_int] * 2),
    "pto_st_tci_s32_1x1024": (C.c_int, [C.c_void_p] * 2 + [C.c_int] * 3),
    "pto_st_tsort32_8x128": (C.c_int, [C.c_void_p] * 4 + [C.c_int] * 3),
    "pto_st_tmrgsort_blocks_f32_1x1024": (C.c_int, [C.c_void_p] * 3 + [C.c_int] * 2),
    "pto_st_tmrgsort_lists_f32": (C.c_int, [C.c_void_p] * 7 + [C.c_int] * 7),
    "pto_st_tmrgsort_blocks_16_1x2048": (C.c_int, [C.c_void_p] * 3 + [C.c_int] * 3),
    "pto_st_tmrgsort_lists_16": (C.c_int, [C.c_void_p] * 7 + [C.c_int] * 8),
    "pto_st_ttrans_f32_64x128": (C.c_int, [C.c_void_p] * 3),
    "pto_st_prefetch_pack_print_s32_16x64": (C.c_int, [C.c_void_p] * 4 + [C.c_int]),
    "pto_st_vec_bitop_64x128": (C.c_int, [C.c_void_p] * 5 + [C.c_float, C.c_int, C.c_int, C.c_int]),
    "pto_st_vec_op_f32_64x128": (C.c_int, [C.c_void_p] * 5 + [C.c_float, C.c_int]),
    "pto_st_reduce_f32_64x128": (C.c_int, [C.c_void_p] * 3 + [C.c_int] * 3),
    "pto_st_cmps_sel_f32_64x128": (C.c_int, [C.c_void_p] * 5 + [C.c_float, C.c_int]),
    "pto_st_fillpad_f32_64x128": (C.c_int, [C.c_void_p] * 3 + [C.c_int] * 3),
    "pto_st_matmul_tmov_f16_64x64x128": (C.c_int, [C.c_void_p] * 4 + [C.c_int, C.c_float]),
    "pto_st_pushpop_f16_64x64x128": (C.c_int, [C.c_void_p] * 7 + [C.c_int]),
}

_lib = None
_st_lib = None


def load():
    """Load the shared library and declare every symbol of include/pto_amd.h."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError("libpto_amd.so is not built: run `python pto-isa_amd/build.py`")
        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in SYMBOLS.items():
            fn = getattr(lib, name)          # AttributeError if the library lacks a declared symbol
            fn.restype = res
            fn.argtypes = args
        _lib = lib
    return _lib


def load_st():
    """Load the test-only library and declare every symbol of include/pto_amd_st.h (and of pto_amd.h: it holds the
    product's entry points too, so a test can drive both through one handle)."""
    global _st_lib
    if _st_lib is None:
        if not os.path.exists(ST_LIB_PATH):
            raise RuntimeError("libpto_st.so is not built: run `python pto-isa_amd/build.py`")
        lib = C.CDLL(ST_LIB_PATH)
        for name, (res, args) in list(SYMBOLS.items()) + list(ST_SYMBOLS.items()):
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
        _st_lib = lib
    return _st_lib


class PtoError(RuntimeError):
    pass


def check(rc, what):
    if rc != OK:
        names = {ERR_BAD_ARG: "bad argument", ERR_UNSUPPORTED: "unsupported shape", ERR_HIP: "HIP error",
                 ERR_WORKSPACE: "workspace too small"}
        raise PtoError("%s failed: %s (%d), hip=%d" % (what, names.get(rc, "?"), rc, load().pto_last_hip_error()))
