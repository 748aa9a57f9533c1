"""ctypes binding of libalpha_hip.so -- the same symbols, argument for argument, that a Bun-FFI shim binds
(include/alpha_hip.h).  Loading fails loudly when the library is missing: there is no CPU fallback."""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libalpha_hip.so")

F32, BF16, I32, F16 = 0, 1, 2, 3
DTYPE_CODE = {"f32": F32, "bf16": BF16, "i32": I32, "f16": F16}
DTYPE_BYTES = {"f32": 4, "bf16": 2, "i32": 4, "f16": 2}

ADD, SUB, MUL, DIV = 0, 1, 2, 3
NEG, EXP, LOG, SQRT, POW, SCALE, CLAMP, GELU, RELU, SILU, SOFTCAP = range(11)
GELU_BWD, RELU_BWD, SILU_BWD, CLAMP_BWD, SOFTCAP_BWD = range(5)
GEMM_NN, GEMM_NT, GEMM_TN = 0, 1, 2
EPI_NONE, EPI_ACCUM, EPI_GELU, EPI_RESIDUAL, EPI_GELU_BWD, EPI_GELU_GRAD, EPI_MUL_AUX = range(7)

u64, i64, i32, f32 = C.c_uint64, C.c_int64, C.c_int32, C.c_float
p_i64 = C.POINTER(C.c_int64)


class AhDeviceInfo(C.Structure):
    _fields_ = [("name", C.c_char * 128), ("arch", C.c_char * 32), ("compute_units", i32), ("wavefront", i32),
                ("clock_khz", i32), ("lds_bytes_per_block", i32), ("hbm_bytes", u64)]


class AhStats(C.Structure):
    _fields_ = [("live_allocs", u64), ("live_bytes", u64), ("pool_blocks", u64), ("pool_bytes", u64),
                ("device_mallocs", u64), ("ops_launched", u64), ("graphs_live", u64),
                ("steps_recorded", u64), ("steps_replayed", u64), ("steps_fallback", u64), ("step_node_updates", u64)]


class AhGemm(C.Structure):
    _fields_ = [("layout", i32), ("in_dtype", i32), ("out_dtype", i32), ("epilogue", i32),
                ("m", i64), ("n", i64), ("k", i64), ("lda", i64), ("ldb", i64), ("ldc", i64),
                ("batch", i64), ("stride_a", i64), ("stride_b", i64), ("stride_c", i64),
                ("a", u64), ("b", u64), ("c", u64), ("aux", u64)]


class AhFlash(C.Structure):
    _fields_ = [("dtype", i32), ("batch", i32), ("heads", i32), ("seq", i32), ("head_dim", i32),
                ("q_sb", i64), ("q_sh", i64), ("q_st", i64), ("k_sb", i64), ("k_sh", i64), ("k_st", i64),
                ("v_sb", i64), ("v_sh", i64), ("v_st", i64), ("o_sb", i64), ("o_sh", i64), ("o_st", i64),
                ("scale", f32), ("soft_cap", f32),
                ("q", u64), ("k", u64), ("v", u64), ("o", u64), ("lse", u64),
                ("d_o", u64), ("dq", u64), ("dk", u64), ("dv", u64), ("bwd_variant", i32), ("reserved", i32)]


class AhRng(C.Structure):
    _fields_ = [("s0", i32), ("s1", i32), ("has_spare", i32), ("_pad", i32), ("spare", C.c_double)]


class AhColsumJob(C.Structure):
    _fields_ = [("partials", C.c_uint64), ("dw", C.c_uint64), ("db", C.c_uint64), ("rows", C.c_int64), ("dim", C.c_int64),
                ("accumulate", C.c_int32), ("reserved", C.c_int32)]


class AhAdamW(C.Structure):
    _fields_ = [("lr", f32), ("beta1", f32), ("beta2", f32), ("eps", f32), ("weight_decay", f32),
                ("bc1", f32), ("bc2", f32), ("grad_scale", f32)]


class AhAdamWItem(C.Structure):
    _fields_ = [("p", u64), ("g", u64), ("m", u64), ("v", u64), ("shadow", u64), ("n", u64), ("weight_decay", f32), ("reserved", i32)]


class AhLion(C.Structure):
    _fields_ = [("lr", C.c_double), ("beta1", C.c_double), ("beta2", C.c_double), ("weight_decay", C.c_double), ("grad_scale", C.c_double)]


class AhAdafactor(C.Structure):
    _fields_ = [("lr", C.c_double), ("beta2", C.c_double), ("eps", C.c_double), ("clip_threshold", C.c_double),
                ("weight_decay", C.c_double), ("grad_scale", C.c_double)]


# name -> argtypes (every function returns int32 except ah_last_error)
SIGNATURES = {
    "ah_init": [i32], "ah_shutdown": [], "ah_device_info": [C.POINTER(AhDeviceInfo)], "ah_sync": [],
    "ah_alloc": [u64, C.POINTER(u64)], "ah_free": [u64], "ah_upload": [u64, C.c_void_p, u64],
    "ah_download": [C.c_void_p, u64, u64], "ah_download_begin": [u64, u64, C.POINTER(u64)], "ah_download_end": [u64, C.c_void_p, u64],
    "ah_copy": [u64, u64, u64], "ah_fill_f32": [u64, f32, u64],
    "ah_fill_i32": [u64, i32, u64], "ah_stats": [C.POINTER(AhStats)], "ah_reset_op_count": [], "ah_trim_pool": [],
    "ah_graph_begin": [], "ah_graph_end": [C.POINTER(u64)], "ah_graph_launch": [u64], "ah_graph_destroy": [u64],
    "ah_event_create": [C.POINTER(u64)], "ah_event_record": [u64], "ah_event_elapsed_ms": [u64, u64, C.POINTER(f32)],
    "ah_event_destroy": [u64],
    "ah_binary": [i32, u64, u64, u64, u64],
    "ah_binary_broadcast": [i32, u64, u64, u64, i32, p_i64, p_i64, p_i64],
    "ah_unary": [i32, u64, u64, u64, f32, f32],
    "ah_add_inplace": [u64, u64, u64], "ah_scale_inplace": [u64, f32, u64], "ah_axpy_inplace": [u64, u64, f32, u64],
    "ah_unary_bwd": [i32, u64, u64, u64, u64, f32, f32],
    "ah_channel_act": [i32, u64, C.c_void_p, i32, u64, i64, i64], "ah_channel_act_bwd": [i32, u64, C.c_void_p, i32, u64, u64, C.c_void_p, i32, i64, i64],
    "ah_add_bf16": [u64, u64, u64, u64],
    "ah_sum_sq_list": [C.c_void_p, C.c_void_p, i32, u64],
    "ah_adamw_list": [C.c_void_p, i32, C.c_void_p, u64, u64],
    "ah_swiglu": [i32, u64, u64, i64, i64], "ah_swiglu_bwd": [i32, u64, u64, u64, i64, i64],
    "ah_silu_mul": [u64, u64, u64, u64], "ah_silu_mul_bwd": [u64, u64, u64, u64, u64, u64],
    "ah_residual_dropout_add": [u64, u64, u64, u64, u64],
    "ah_dropout_mask": [u64, u64, i32, i32, C.c_double],
    "ah_dropout_apply": [u64, i32, u64, u64, i32, u64, u64, i32, C.c_double],
    "ah_masked_fill": [u64, u64, u64, u64, u64, f32], "ah_causal_mask": [u64, i64],
    "ah_cast": [u64, i32, u64, i32, u64], "ah_check_finite": [u64, u64, u64],
    "ah_transpose": [u64, u64, i32, p_i64, i32, i32],
    "ah_slice": [u64, u64, i32, p_i64, p_i64, p_i64],
    "ah_scatter_slice": [u64, u64, i32, p_i64, p_i64, p_i64],
    "ah_cat_part": [u64, u64, i32, p_i64, p_i64, i32, i64],
    "ah_slice_qkv": [u64, u64, u64, u64, i64, i64],
    "ah_broadcast": [u64, u64, i32, p_i64, p_i64],
    "ah_sum_axis": [u64, u64, i64, i64, i64, i32], "ah_sum_all": [u64, u64, u64, i32],
    "ah_softmax": [u64, u64, i64, i64, i64, i32], "ah_argmax": [u64, u64, i64, i64, i64],
    "ah_sum_sq": [u64, u64, u64], "ah_sum_sq_static": [u64, u64, u64], "ah_softmax_bwd": [u64, u64, u64, i64, i64],
    "ah_embedding": [u64, u64, u64, i64, i64, i64, i32],
    "ah_embedding_tok_pos": [u64, u64, u64, u64, i64, i64, i64, i64, i32],
    "ah_embedding_bwd": [u64, u64, u64, i64, i64, i64, i32],
    "ah_embedding_index_bytes": [i64, i64], "ah_embedding_index": [u64, i64, i64, u64],
    "ah_embedding_bwd_indexed": [u64, u64, u64, i64, i64, i64, i32],
    "ah_token_windows": [u64, i64, u64, i64, i64, u64, u64],
    "ah_pos_embedding_bwd": [u64, u64, i64, i64, i64, i32],
    "ah_layernorm": [u64, u64, u64, u64, i64, i64, f32, i32, i32],
    "ah_layernorm_bwd": [u64, u64, u64, i32, u64, u64, u64, u64, u64, i64, i64, f32, i32, i32],
    "ah_layernorm_bwd_partials_bytes": [i64, i64],
    "ah_layernorm_bwd_deferred": [u64, u64, u64, i32, u64, u64, u64, u64, i64, i64, f32, i32],
    "ah_layernorm_colsums": [C.POINTER(AhColsumJob), i32],
    "ah_cross_entropy": [u64, i32, u64, u64, u64, i64, i64],
    "ah_cross_entropy_bwd": [u64, i32, u64, u64, u64, f32, u64, i64, i64],
    "ah_cross_entropy_fwd_bwd": [u64, i32, u64, u64, u64, u64, f32, u64, i64, i64],
    "ah_gemm": [C.POINTER(AhGemm)],
    "ah_gemm_planes": [C.POINTER(AhGemm), i64, i64, i64, i64, i32],
    "ah_gemm_grouped_plan": [C.POINTER(AhGemm), C.c_int32, C.POINTER(C.c_uint64)],
    "ah_gemm_grouped_run": [u64, i32],
    "ah_gemm_grouped_run_sumsq": [u64, i32, u64],
    "ah_gemm_grouped_update": [u64, C.POINTER(AhGemm), C.c_int32],
    "ah_gemm_grouped_destroy": [u64],
    "ah_gemm_last_kernel": [C.c_char_p, C.c_int32, C.POINTER(C.c_int32)],
    "ah_probe_mfma_bf16": [i32, i32, i32, C.POINTER(C.c_double)],
    "ah_probe_issue": [i32, i32, i32, C.POINTER(C.c_double)],
    "ah_flash_fwd": [C.POINTER(AhFlash)], "ah_flash_bwd": [C.POINTER(AhFlash)],
    "ah_adamw": [u64, u64, u64, u64, u64, C.POINTER(AhAdamW), u64, u64, u64],
    "ah_clip_coef": [u64, f32, f32, u64],
    "ah_side_begin": [], "ah_side_end": [], "ah_side_join": [],
    "ah_step_begin": [u64], "ah_step_end": [C.POINTER(C.c_int32)], "ah_step_reset": [u64], "ah_step_kick": [],
    "ah_step_guard": [u64, u64, f32, f32, C.c_double, C.c_double, u64, u64, u64],
    "ah_lion": [u64, u64, u64, u64, C.POINTER(AhLion)], "ah_sgd": [u64, u64, u64, C.c_double, C.c_double],
    "ah_adafactor_2d": [u64, u64, u64, u64, i64, i64, C.POINTER(AhAdafactor)],
    "ah_adafactor_flat": [u64, u64, u64, u64, C.POINTER(AhAdafactor)],
    "ah_rng_seed": [C.POINTER(AhRng), i32], "ah_rng_next": [C.POINTER(AhRng), C.POINTER(C.c_double)],
    "ah_rng_next_gauss": [C.POINTER(AhRng), C.POINTER(C.c_double)],
    "ah_rng_fill_gauss_f32": [C.POINTER(AhRng), C.c_void_p, u64, C.c_double],
    "ah_rng_fill_uniform_f64": [C.POINTER(AhRng), C.c_void_p, u64],
}


class AlphaHipError(RuntimeError):
    def __init__(self, code: int, msg: str):
        super().__init__(f"alpha_hip error {code}: {msg}")
        self.code = code


_lib = None


def load():
    """dlopen the library and type every export.  Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise ImportError(f"{LIB_PATH} is missing: build it with `python -m alpha2_amd.build` "
                          "(there is no CPU fallback for the HIP backend)")
    lib = C.CDLL(LIB_PATH)
    for name, args in SIGNATURES.items():
        fn = getattr(lib, name)
        fn.argtypes = args
        fn.restype = i32
    lib.ah_layernorm_bwd_partials_bytes.restype = i64       # a size, not a status
    lib.ah_embedding_index_bytes.restype = i64
    lib.ah_last_error.argtypes = []
    lib.ah_last_error.restype = C.c_char_p
    lib.ah_step_note.argtypes = []
    lib.ah_step_note.restype = C.c_char_p
    _lib = lib
    return lib


def check(rc: int):
    if rc != 0:
        raise AlphaHipError(rc, load().ah_last_error().decode("utf-8", "replace"))


def shape_arr(seq):
    return (C.c_int64 * max(1, len(seq)))(*[int(x) for x in seq])
