"""ctypes binding of libggufhip.so (C ABI: include/ggufhip.h).

There is no fallback: if the shared library is missing or a symbol is absent, importing this
module raises. Every entry point returns 0 on success; `check` turns anything else into a
RuntimeError carrying gt_last_error().
"""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libggufhip.so")

if not os.path.exists(LIB_PATH):
    raise ImportError(
        f"{LIB_PATH} is not built. Run `make -C {os.path.join(_HERE, 'csrc')}` (hipcc, gfx950). "
        "This backend has no CPU path.")

lib = C.CDLL(LIB_PATH)

buf = C.c_uint64
ctxp = C.c_void_p
i32, i64, f32, f64, sz = C.c_int, C.c_int64, C.c_float, C.c_double, C.c_size_t


class ProfRec(C.Structure):
    _fields_ = [("label", C.c_char * 32), ("ms", C.c_double), ("count", C.c_int64), ("work", C.c_double)]


_SIG = {
    "gt_ctx_create": [i32, C.POINTER(ctxp)],
    "gt_ctx_destroy": [ctxp],
    "gt_alloc": [ctxp, sz, i32, C.POINTER(buf)],
    "gt_free": [ctxp, buf],
    "gt_memset0": [ctxp, buf, sz],
    "gt_h2d": [ctxp, buf, C.c_void_p, sz],
    "gt_d2h": [ctxp, C.c_void_p, buf, sz],
    "gt_d2d": [ctxp, buf, buf, sz],
    "gt_sync": [ctxp],
    "gt_stream_mark": [ctxp],
    "gt_stream_wait": [ctxp, ctxp],
    "gt_resident_bytes": [ctxp, C.POINTER(C.c_uint64)],
    "gt_set_option": [ctxp, C.c_char_p, i32],
    "gt_gemm": [ctxp, i32, i32, i32, i32, i32, buf, buf, buf],
    "gt_gemm_pair": [ctxp, i32, i32, i32, i32, i32, buf, buf, i32, buf, buf, buf],
    "gt_gemm_group": [ctxp, i32, i32, C.POINTER(i32), C.POINTER(i32), i32, C.POINTER(buf), C.POINTER(buf), C.POINTER(buf), C.POINTER(i32)],
    "gt_gemm_batched": [ctxp, i32, i32, i32, i32, i32, buf, i64, buf, i64, buf, i64, i32],
    "gt_rank_down": [ctxp, i32, i32, i32, buf, buf, i32, f32, buf],
    "gt_rank_grad": [ctxp, i32, i32, i32, buf, buf, i32, i32, buf],
    "gt_rank_grad_slices": [ctxp, i32, i32, i32, buf, C.POINTER(i32)],
    "gt_rank_grad_parts": [ctxp, i32, i32, i32, buf, buf, i32, buf],
    "gt_rank_slices_group": [ctxp, i32, C.POINTER(buf), C.POINTER(i32), C.POINTER(i32), C.POINTER(buf), C.POINTER(i32)],
    "gt_add_fwd": [ctxp, i64, buf, buf, buf],
    "gt_mul_fwd": [ctxp, i64, buf, buf, buf],
    "gt_silu_fwd": [ctxp, i64, buf, buf],
    "gt_gelu_fwd": [ctxp, i64, buf, buf],
    "gt_scale_fwd": [ctxp, i64, buf, f32, buf],
    "gt_add_bwd": [ctxp, i64, buf, buf, i32, buf, i32],
    "gt_mul_bwd": [ctxp, i64, buf, buf, buf, buf, i32, buf, i32],
    "gt_silu_bwd": [ctxp, i64, buf, buf, buf, i32],
    "gt_gelu_bwd": [ctxp, i64, buf, buf, buf, i32],
    "gt_scale_bwd": [ctxp, i64, buf, f32, buf, i32],
    "gt_glu_fwd": [ctxp, i32, i64, buf, buf, buf],
    "gt_glu_bwd": [ctxp, i32, i64, buf, buf, buf, buf, i32, buf, i32],
    "gt_rmsnorm_fwd": [ctxp, i32, i32, f32, buf, buf, buf, buf],
    "gt_rmsnorm_bwd": [ctxp, i32, i32, buf, buf, buf, buf, buf, i32, buf, i32],
    "gt_rmsnorm_bwd_static": [ctxp, i32, i32, buf, buf, buf, buf, buf, i32, buf, i32],
    "gt_rmsnorm_bwd_from": [ctxp, i32, i32, buf, buf, buf, buf, buf, buf, buf, i32],
    "gt_rmsnorm_parts_rows": [ctxp, i32, i32, C.POINTER(i32)],
    "gt_rmsnorm_bwd_parts": [ctxp, i32, i32, buf, buf, buf, buf, buf, buf, i32, buf],
    "gt_colsum_group": [ctxp, i32, C.POINTER(buf), C.POINTER(i32), C.POINTER(i32), C.POINTER(buf), C.POINTER(i32)],
    "gt_embedding_fwd": [ctxp, i32, i32, i32, buf, buf, buf],
    "gt_embedding_bwd": [ctxp, i32, i32, i32, buf, buf, buf, i32],
    "gt_rope": [ctxp, i32, i32, i32, i32, f64, i32, i32, buf, buf, i32],
    "gt_rope_pair": [ctxp, i32, i32, i32, f64, i32, i32, i32, buf, buf, i32, i32, buf, buf, i32],
    "gt_attn_fwd": [ctxp, i32, i32, i32, i32, i32, i32, buf, buf, buf, buf, buf],
    "gt_attn_bwd": [ctxp, i32, i32, i32, i32, i32, i32, buf, buf, buf, buf, buf, buf, buf, i32, buf, i32, buf, i32],
    "gt_gemm_add": [ctxp, i32, i32, i32, i32, buf, buf, buf, buf],
    "gt_gemm_sum": [ctxp, i32, i32, i32, i32, i32, C.POINTER(i32), C.POINTER(buf), C.POINTER(buf), buf],
    "gt_attn_scores_bytes": [ctxp, i32, i32, i32, i32, i32, i32, C.POINTER(C.c_uint64)],
    "gt_attn_fwd_scores": [ctxp, i32, i32, i32, i32, i32, i32, buf, buf, buf, buf, buf, buf],
    "gt_attn_bwd_scores": [ctxp, i32, i32, i32, i32, i32, i32, buf, buf, buf, buf, buf, buf, buf, buf, i32, buf, i32, buf, i32],
    "gt_attn_bwd_scores_rope": [ctxp, i32, i32, i32, i32, i32, i32, buf, buf, buf, buf, buf, buf, buf, f64, i32, i32, i32, buf, i32, buf, i32, buf, i32],
    "gt_ce_fwd": [ctxp, i32, i32, i32, buf, buf, buf, buf, buf],
    "gt_ce_bwd": [ctxp, i32, i32, i32, buf, buf, buf, buf, f32, buf, i32],
    "gt_ce_chunk_stats": [ctxp, i32, i32, i32, i32, i32, buf, buf, buf, buf, buf],
    "gt_ce_loss_from_stats": [ctxp, i32, i32, i32, buf, buf, buf, buf, buf, buf],
    "gt_ce_chunk_grad": [ctxp, i32, i32, i32, i32, i32, buf, buf, buf, buf, buf, f32],
    "gt_soft_ce_fwd": [ctxp, i32, i32, i32, buf, buf, buf, f32, buf, buf, buf],
    "gt_soft_ce_bwd": [ctxp, i32, i32, i32, buf, buf, buf, f32, buf, buf, f32, buf, i32],
    "gt_adamw_create": [ctxp, i32, C.POINTER(buf), C.POINTER(buf), C.POINTER(buf), C.POINTER(buf), C.POINTER(i64),
                        f64, f64, f64, f64, f64, C.POINTER(C.c_void_p)],
    "gt_grad_fold": [ctxp, i32, C.POINTER(buf), C.POINTER(i32), i32, C.POINTER(buf), C.POINTER(i64)],
    "gt_adamw_step": [ctxp, C.c_void_p, f64, f64, f64],
    "gt_adamw_grad_norm": [ctxp, C.c_void_p, C.POINTER(f32)],
    "gt_adamw_destroy": [ctxp, C.c_void_p],
    "gt_muon_create": [ctxp, i32, C.POINTER(buf), C.POINTER(buf), C.POINTER(buf), C.POINTER(i32), C.POINTER(i32),
                       f64, i32, i32, C.POINTER(C.c_void_p)],
    "gt_muon_step": [ctxp, C.c_void_p, f64],
    "gt_muon_destroy": [ctxp, C.c_void_p],
    "gt_newton_schulz": [ctxp, i32, i32, i32, buf, buf],
    "gt_prof_begin": [ctxp, C.c_char_p],
    "gt_prof_end": [ctxp, C.POINTER(ProfRec), i32, C.POINTER(i32)],
    "gt_timer_start": [ctxp],
    "gt_timer_stop": [ctxp, C.POINTER(f64)],
}

for _name, _args in _SIG.items():
    _fn = getattr(lib, _name)          # AttributeError here = the library does not export what the header declares
    _fn.argtypes = _args
    _fn.restype = C.c_int
lib.gt_last_error.argtypes = [ctxp]
lib.gt_last_error.restype = C.c_char_p
lib.gt_device_name.argtypes = [ctxp]
lib.gt_device_name.restype = C.c_char_p

EXPORTS = sorted(list(_SIG) + ["gt_last_error", "gt_device_name"])
NT, NN, TN = 0, 1, 2


class HipError(RuntimeError):
    pass


def check(ctx, rc: int, what: str = ""):
    if rc != 0:
        msg = lib.gt_last_error(ctx)
        raise HipError(f"{what}: {msg.decode() if msg else 'unknown error'}")
