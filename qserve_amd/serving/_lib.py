"""ctypes binding of libqserve_serve.so (include/qserve_serve.h): the kernels of the paged serving engine.

The library is loaded on first use.  If it has not been built yet it is built then (hipcc, a few seconds); a build or load
failure raises - on a GPU there is no other compute path.
"""
import ctypes as C
import os
import threading

_vp, _i, _i64, _f = C.c_void_p, C.c_int, C.c_int64, C.c_float
SIGNATURES = {
    "qsv_version": (_i, []),
    "qsv_arch": (C.c_char_p, []),
    "qsv_last_error": (C.c_char_p, []),
    "qsv_embed": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _vp]),
    "qsv_add_layer_norm": (_i, [_vp, _vp, _vp, _vp, _f, _i, _i, _i, _vp]),
    "qsv_layer_norm_rows": (_i, [_vp, _vp, _vp, _vp, _f, _i, _i, _i, _vp]),
    "qsv_latent_prep": (_i, [_vp, _i64, _i, _i, _vp, _vp, _i, _i, _vp, _i, _i, _vp, _vp, _vp, _vp, _f, _i, _i, _vp]),
    "qsv_latent_query": (_i, [_vp, _vp, _vp, _vp, _vp, _f, _i, _i, _i, _i, _i, _i, _i, _vp]),
    "qsv_latent_attention": (_i, [_vp, _vp, _vp, _vp, _i, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i64, _i, _vp, _i, _i, _vp, _vp, _i64, _i, _i,
                                  _i, _i, _vp]),
    "qsv_pool_blocks": (_i, [_vp, _i64, _vp, _i64, _vp, _i, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp]),
    "qsv_latent_attention_tile_tokens": (_i, [_i]),
    "qsv_latent_attention_mfma_ok": (_i, [_i, _i, _i]),
    "qsv_latent_attention_mfma": (_i, [_vp, _vp, _vp, _vp, _i, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _vp, _vp, _i, _i, _i, _i64, _i, _vp,
                                       _i, _i, _vp, _vp, _i64, _i, _i, _vp]),
    "qsv_sigmoid_gate": (_i, [_vp, _vp, _i64, _i, _i, _i, _vp]),
    "qsv_moe_route": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _i, _i, _i, _vp, _i, _f, _i, _vp]),
    "qsv_moe_up": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _f, _i, _i, _vp]),
    "qsv_expert_rows": (_i, [_vp, _vp, _vp, _i, _vp, _vp, _i, _i, _i, _i, _f, _vp]),
    "qsv_grouped_gemm_tile_slots": (_i, []),
    "qsv_grouped_gemm_k_step": (_i, []),
    "qsv_grouped_gemm": (_i, [_vp, _vp, _vp, _i, _vp, _vp, _i, _i, _i, _i, _f, _vp]),
    "qsv_gather_rows": (_i, [_vp, _vp, _vp, _i, _i, _i, _i, _vp]),
    "qsv_relu_sq": (_i, [_vp, _i64, _i, _vp]),
    "qsv_moe_combine": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _vp, _vp, _i, _i, _vp]),
    "qsv_moe_down": (_i, [_vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp, _i, _i, _vp]),
    "qsv_embed_streams": (_i, [_vp, _vp, _vp, _f, _i, _i, _i, _i, _vp]),
    "qsv_hc_read": (_i, [_vp, _vp, _vp, _vp, _vp, _f, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp]),
    "qsv_hc_write": (_i, [_vp, _vp, _vp, _vp, _i, _i, _i, _vp, _vp, _vp, _vp, _f, _i, _vp]),
    "qsv_dyt_sum_rows": (_i, [_vp, _vp, _vp, _vp, _vp, _f, _i, _i, _i, _i, _vp]),
    "qsv_rms_pair_mean": (_i, [_vp, _vp, _vp, _vp, _vp, _f, _i, _i, _i, _vp]),
    "qsv_glu": (_i, [_vp, _vp, _i, _i, _i, _f, _i, _vp]),
    "qsv_decay": (_i, [_vp, _vp, _i64, _vp, _vp, _f, _i, _i, _i, _i, _vp]),
    "qsv_conv_silu_unit": (_i, [_vp, _vp, _i64, _i, _i, _i, _vp, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _i, _vp]),
    "qsv_min_gru_scan": (_i, [_vp, _vp, _i64, _i, _i, _i, _vp, _vp, _vp, _vp, _i, _i, _i, _i, _vp]),
    "qsv_add_normed_rms_norm": (_i, [_vp, _vp, _vp, _vp, _i, _vp, _i, _f, _i, _i, _i, _vp]),
    "qsv_qk_norm_rope_prep": (_i, [_vp, _vp, _i64, _vp, _i64, _vp, _i64, _i, _i, _i, _i, _i, _vp, _vp, _i, _f, _vp, _i, _f, _vp, _i64,
                                   _vp, _vp, _i, _i, _vp]),
    "qsv_recurrent_scan": (_i, [_vp, _vp, _i64, _vp, _i64, _vp, _i64, _i, _vp, _vp, _i64, _i, _vp, _vp, _i, _i, _i, _i, _i, _i, _f, _vp,
                                _i, _i, _vp]),
    "qsv_head_rms_gate": (_i, [_vp, _vp, _vp, _vp, _i64, _i, _f, _i, _i, _i, _i, _i, _vp, _i, _vp]),
    "qsv_max_gates": (_i, [_vp, _vp, _vp, _vp, _vp, _i64, _vp, _vp, _f, _vp, _vp, _i, _i, _i, _vp]),
    "qsv_embed_sinusoid": (_i, [_vp, _vp, _vp, _vp, _vp, _f, _i, _i, _i, _vp]),
    "qsv_add_rms_norm": (_i, [_vp, _vp, _vp, _vp, _vp, _vp, _f, _i, _i, _i, _vp]),
    "qsv_rms_norm_rows": (_i, [_vp, _vp, _vp, _vp, _f, _i, _i, _i, _vp]),
    "qsv_normed_attention_prep": (_i, [_vp, _vp, _i64, _vp, _i64, _i, _i, _i, _i, _i, _i, _i, _vp, _vp, _f, _f, _vp, _i64, _f, _vp, _i,
                                       _i, _vp]),
    "qsv_attention_prep": (_i, [_vp, _vp, _i64, _vp, _i64, _i, _i, _i, _i, _i, _i, _i, _i, _vp, _vp, _f, _vp, _vp, _i, _i, _vp]),
    "qsv_rotate_heads": (_i, [_vp, _vp, _vp, _f, _i, _i, _i, _i, _vp]),
}

_lock = threading.Lock()
_lib = None


def lib():
    global _lib
    if _lib is not None:
        return _lib
    with _lock:
        if _lib is None:
            from .. import build as b
            path = os.environ.get("QS_SERVE_LIBRARY") or b.SERVE_LIB
            if not os.path.exists(path):
                b.build_serve(verbose=True)
            L = C.CDLL(path)
            for name, (res, args) in SIGNATURES.items():
                fn = getattr(L, name)              # AttributeError if the built library is older than this binding: loud by design
                fn.restype, fn.argtypes = res, args
            _lib = L
    return _lib


def check(rc, what):
    if rc != 0:
        msg = lib().qsv_last_error()
        raise RuntimeError(f"{what}: {msg.decode() if msg else 'error'} (code {rc})")
