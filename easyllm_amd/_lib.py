"""ctypes binding of libezl.so (the C ABI declared in include/ezl.h).

There is no fallback: if the library is missing, or a call fails, a RuntimeError is raised.
"""
import ctypes
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libezl.so")

_vp, _i64, _i32, _f32 = ctypes.c_void_p, ctypes.c_int64, ctypes.c_int, ctypes.c_float
_i64p = ctypes.POINTER(ctypes.c_int64)
_vpp = ctypes.POINTER(ctypes.c_void_p)

# name -> argtypes; the single source of truth for the symbol table on the Python side
SIGNATURES = {
    "ezl_rmsnorm_fwd": [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _f32, _vp],
    "ezl_rmsnorm_bwd": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _vp, _i64, _i64, _i64, _vp],
    "ezl_rmsnorm_bwd_noalloc": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i32, _i64, _i64, _vp],
    "ezl_swiglu_fwd": [_vp, _vp, _vp, _i64, _vp],
    "ezl_swiglu_bwd": [_vp, _vp, _vp, _vp, _vp, _i64, _vp],
    "ezl_rope_table": [_vp, _vp, _vp, _i64, _i64, _f32, _vp],
    "ezl_rope_apply": [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i32, _vp],
    "ezl_rope_apply_pair": [_vp, _vp, _i64, _i64, _i64, _vp, _vp, _i64, _i64, _i64, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i32, _vp],
    "ezl_ids_in_range": [_vp, _i64, _i64, _vp, _vp],
    "ezl_embed_gather": [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _vp],
    "ezl_embed_scatter_add": [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i32, _vp],
    "ezl_transpose01": [_vp, _vp, _i64, _i64, _i64, _vp],
    "ezl_add": [_vp, _vp, _vp, _i64, _vp],
    "ezl_cast_bf16_to_f32": [_vp, _vp, _i64, _vp],
    "ezl_cast_f32_to_bf16": [_vp, _vp, _i64, _vp],
    "ezl_bias_add": [_vp, _vp, _vp, _i64, _i64, _vp],
    "ezl_bias_grad": [_vp, _vp, _vp, _i32, _vp, _i64, _i64, _i64, _vp],
    "ezl_gemm_bf16": [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i32, _i32, _i32, _i32, _vp, _i64, _vp],
    "ezl_gemm_bf16_ksplit": [_i32, _vpp, _vpp, _vp, _i64, _i64, _i64p, _i64, _i64, _i64, _i32, _i32, _i32, _i32, _vp, _i64, _vp],
    "ezl_attn_fwd": [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _f32, _i64p, _vp],
    "ezl_attn_bwd": [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _f32,
                     _i64p, _vp, _i64, _vp],
    "ezl_mask_compact": [_vp, _i64, _i64, _vp, _vp, _vp, _vp],
    "ezl_rows_gather": [_vp, _vp, _vp, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _i64, _vp],
    "ezl_ce_prepare": [_vp, _vp, _i32, _i64, _vp, _vp, _i64, _vp],
    "ezl_ce_fwd": [_vp, _vp, _vp, _vp, _i64, _i64, _i64, _i32, _vp],
    "ezl_ce_bwd": [_vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i32, _vp],
    "ezl_ce_fused": [_vp, _vp, _vp, _vp, _vp, _vp, _i64, _i64, _i64, _i32, _vp],
    "ezl_ce_reduce": [_vp, _vp, _vp, _vp, _i64, _vp],
    "ezl_scale_by_scalar": [_vp, _vp, _i64, _i32, _vp],
    "ezl_sumsq_f32": [_vp, _i64, _vp, _vp],
    "ezl_clip_coef": [_vp, _i64, _f32, _vp, _vp],
    "ezl_build_location_idx": [_vp, _i64, _vp, _i64, _i64, _i64, _i64, _vp, _i64],
    "ezl_adamw_step": [_vp, _vp, _vp, _vp, _vp, _i64, _f32, _f32, _f32, _f32, _f32, _i64, _i32, _vp, _vp],
}
_SPECIAL = {
    "ezl_version": ([], ctypes.c_int),
    "ezl_last_error": ([], ctypes.c_char_p),
    "ezl_rmsnorm_bwd_workspace_bytes": ([_i64, _i64], _i64),
    "ezl_rmsnorm_bwd_noalloc_max_h": ([], _i64),
    "ezl_bias_grad_workspace_bytes": ([_i64, _i64], _i64),
    "ezl_embed_scatter_add_workspace_bytes": ([_i64, _i64], _i64),
    "ezl_attn_bwd_workspace_bytes": ([_i64, _i64, _i64, _i64, _i64], _i64),
    "ezl_gemm_workspace_bytes": ([_i64, _i64, _i64], _i64),
    "ezl_sumsq_partials": ([], _i64),
    "ezl_location_idx_rows": ([_i64, _i64, _i64], _i64),
}

_lib = None


def exported_symbols():
    return sorted(list(SIGNATURES) + list(_SPECIAL))


def load():
    """Loads the shared library once; raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "libezl.so not found at %s -- build it with `python -m easyllm_amd.csrc.build` "
                "(there is no fallback path)" % LIB_PATH)
        lib = ctypes.CDLL(LIB_PATH)
        for name, argtypes in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.argtypes = argtypes
            fn.restype = ctypes.c_int
        for name, (argtypes, restype) in _SPECIAL.items():
            fn = getattr(lib, name)
            fn.argtypes = argtypes
            fn.restype = restype
        _lib = lib
    return _lib


def call(name, *args):
    """Calls an int-returning entry point and raises RuntimeError with the library's message on failure."""
    lib = load()
    rc = getattr(lib, name)(*args)
    if rc != 0:
        msg = lib.ezl_last_error()
        raise RuntimeError("%s failed (%d): %s" % (name, rc, msg.decode() if msg else "?"))


def rmsnorm_bwd_workspace_bytes(rows, h):
    return load().ezl_rmsnorm_bwd_workspace_bytes(rows, h)


def bias_grad_workspace_bytes(rows, n):
    return load().ezl_bias_grad_workspace_bytes(rows, n)


def embed_scatter_add_workspace_bytes(rows, vocab):
    return load().ezl_embed_scatter_add_workspace_bytes(rows, vocab)


def attn_bwd_workspace_bytes(total_tokens, ndocs, nq, nk, d):
    return load().ezl_attn_bwd_workspace_bytes(total_tokens, ndocs, nq, nk, d)


def gemm_workspace_bytes(M, N, K):
    return load().ezl_gemm_workspace_bytes(M, N, K)


def sumsq_partials():
    return load().ezl_sumsq_partials()


def location_idx_rows(seq_length, num_epochs, tokens_per_epoch):
    return load().ezl_location_idx_rows(seq_length, num_epochs, tokens_per_epoch)
