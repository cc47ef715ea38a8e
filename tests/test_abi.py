"""The C-ABI library builds for gfx950, loads, and exports every symbol include/qserve_amd.h declares.
No kernel is launched here (argument validation happens before any HIP call)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def header_symbols():
    txt = open(os.path.join(ROOT, "include", "qserve_amd.h")).read()
    txt = re.sub(r"/\*.*?\*/", "", txt, flags=re.S)
    return sorted(set(re.findall(r"\b(qs_[a-z0-9_]+)\s*\(", txt)))


def test_header_declares_expected_entry_points():
    syms = header_symbols()
    for s in ["qs_w4a8_per_chn_gemm", "qs_w4a8_per_group_gemm", "qs_single_query_attention",
              "qs_apply_bias_rope_update_kv_cache", "qs_compute_padding_offsets", "qs_w8a8_gemm"]:
        assert s in syms


def test_library_exports_every_declared_symbol(built_lib):
    lib = ctypes.CDLL(built_lib)
    for s in header_symbols():
        assert hasattr(lib, s), f"{s} declared in include/qserve_amd.h but not exported"


def test_ctypes_binding_covers_header(built_lib):
    from qserve_amd import _lib
    assert sorted(_lib.SIGNATURES) == header_symbols()
    assert _lib.lib.qs_arch() == b"gfx950" and _lib.lib.qs_version() >= 1


def test_argument_validation_without_gpu(built_lib):
    from qserve_amd._lib import check, lib
    rc = lib.qs_w4a8_per_chn_gemm(1, 1, 1, 1, 1, 1, 1, 4, 100, 128, None)     # N % 64 != 0
    assert rc == -1 and b"multiple of 64" in lib.qs_last_error()
    rc = lib.qs_w4a8_per_group_gemm(1, 1, 1, 1, 1, 1, 1, 4, 64, 96, None)     # K % 128 != 0
    assert rc == -1
    rc = lib.qs_w4a8_per_chn_gemm(0, 1, 1, 1, 1, 1, 1, 4, 64, 128, None)      # null pointer
    assert rc == -1
    rc = lib.qs_single_query_attention(1, 1, 1, 1, 1, 1, 2, 32, 8, 64, 6144, 6144, 4, 8192, 64, 512, 10, 64, 1e4, 1, 1, 1, None)
    assert rc == -2                                                           # head_dim 64 never instantiated
    with pytest.raises(RuntimeError):
        check(rc, "x")


def test_backend_modules_mirror_reference_names(built_lib):
    import qserve_backend
    import qserve_backend.fused_attention as fa
    import qserve_backend.qgemm_w4a8_per_chn as pc
    import qserve_backend.qgemm_w4a8_per_group as pg
    assert callable(pc.gemm_forward_cuda) and callable(pg.gemm_forward_cuda)
    for name in ("single_query_attention", "apply_bias_rope_update_kv_cache", "compute_padding_offsets"):
        assert callable(getattr(fa, name))
    for mod, fn in (("fused_kernels", "invoke_quant_fuse_sum"), ("layernorm_ops", "rms_norm_general_fuse_sum"),
                    ("activation_ops", "silu_and_mul"), ("qgemm_w8a8", "w8a8_gemm_forward_cuda")):
        assert callable(getattr(getattr(qserve_backend, mod), fn))


def test_product_does_not_import_oracle():
    bad = []
    for base in ("qserve_amd", "qserve_backend"):
        for dp, _, fs in os.walk(os.path.join(ROOT, base)):
            for f in fs:
                if f.endswith((".py", ".hip", ".h")):
                    if re.search(r"^\s*(from|import)\s+oracle\b", open(os.path.join(dp, f)).read(), flags=re.M):
                        bad.append(os.path.join(dp, f))
    assert not bad, f"product code imports the oracle: {bad}"


# ---- libqserve_serve.so (include/qserve_serve.h): the paged serving engine's kernels ----------------------------------------------

def serve_header_symbols():
    txt = open(os.path.join(ROOT, "include", "qserve_serve.h")).read()
    txt = re.sub(r"/\*.*?\*/", "", txt, flags=re.S)
    return sorted(set(re.findall(r"\b(qsv_[a-z0-9_]+)\s*\(", txt)))


def test_serve_library_builds_and_matches_its_header():
    from qserve_amd import build
    from qserve_amd.serving import _lib
    lib = ctypes.CDLL(build.build_serve(verbose=False))
    for s in serve_header_symbols():
        assert hasattr(lib, s), f"{s} declared in include/qserve_serve.h but not exported"
    assert sorted(_lib.SIGNATURES) == serve_header_symbols()
    assert _lib.lib().qsv_arch() == b"gfx950"


def test_serve_argument_validation_without_gpu():
    from qserve_amd.serving._lib import check, lib
    L = lib()
    assert L.qsv_moe_route(1, 1, 1, 1, None, 0, 4, 64, 8, 3, 4, 1, 0, None, 1, 1.0, 0, None) == 1  # top 3 of one kept group of 2
    assert b"experts" in L.qsv_last_error()
    assert L.qsv_moe_route(1, 1, 1, 1, None, 0, 4, 64, 8, 2, 4, 1, 2, None, 1, 1.0, 0, None) == 1  # unknown score function
    assert L.qsv_latent_attention(1, 1, 1, 1, 4, 1, 1, 0, 4, 2, 1000, 1032, 64, 2, 0, 0, None, 0, 0, None, None, 0, 0, 0, 0, 1, None) == 1   # rows wider than 1024
    assert L.qsv_latent_attention(1, 1, 1, 1, 4, 1, 1, 0, 4, 2, 64, 96, 64, 2, 0, -3, None, 0, 0, None, None, 0, 0, 0, 0, 1, None) == 1      # negative chunk
    assert L.qsv_latent_attention(1, 1, 1, 1, 4, 1, 1, 0, 4, 2, 64, 96, 64, 2, 0, 0, 1, 0, 0, None, None, 0, 0, 0, 0, 1, None) == 1          # bias table without entries
    assert L.qsv_latent_attention(1, 1, 1, 1, 4, 1, 1, 0, 4, 2, 64, 96, 64, 2, 0, 0, None, 0, 5, None, None, 0, 0, 0, 0, 1, None) == 1      # kept first positions without a window
    assert L.qsv_latent_attention(1, 1, 1, 1, 4, 1, 1, 32, 4, 2, 64, 96, 64, 2, 0, 0, None, 0, 0, None, 1, 0, 12, 5, 0, 1, None) == 1       # five block rows of 12 positions do not cover a page of 64
    assert b"pooled" in L.qsv_last_error()
    assert L.qsv_latent_attention_mfma_ok(64, 80, 0) == 1 and L.qsv_latent_attention_mfma_ok(64, 80, 1) == 0
    assert L.qsv_latent_attention_mfma_ok(70, 70, 0) == 0
    assert [L.qsv_latent_attention_tile_tokens(h) for h in (1, 3, 6, 16, 32, 40)] == [64, 16, 8, 4, 4, 4]
    assert L.qsv_recurrent_scan(1, 1, 8, 1, 8, 1, 8, 1, 1, None, 0, 0, 1, 1, 1, 5, 3, 2, 8, 8, 1.0, None, 0, 0, None) == 1   # 3 heads over 2
    assert b"heads" in L.qsv_last_error()
    assert L.qsv_recurrent_scan(1, 1, 8, 1, 8, 1, 8, 1, 1, None, 0, 0, 1, 1, 1, 5, 2, 2, 8, 8, 1.0, None, 1, 12, None) == 1  # more value columns than the state has
    assert L.qsv_head_rms_gate(1, 1, 1, 1, 16, 1, 1e-5, 2, 2, 8, 8, 1, 1, 0, None) == 1                       # a normaliser without its column
    assert L.qsv_max_gates(1, 1, 1, 1, 1, 4, 1, 1, 0.0, 1, 1, 1, 4, 0, None) == 1                             # gate cap 0
    assert L.qsv_glu(1, 1, 2, 8, 7, 0.0, 0, None) == 1                                                        # unknown activation
    assert L.qsv_glu(1, 1, 2, 8, 2, 0.0, 0, None) == 1                                                        # clamped units without a limit
    assert L.qsv_add_rms_norm(1, 1, None, None, None, None, 1e-5, 2, 8, 0, None) == 1                         # a norm without its weight
    assert L.qsv_hc_write(1, 1, 1, 1, 2, 17, 8, None, None, None, None, 0.0, 0, None) == 1                    # 17 streams
    assert L.qsv_moe_up(1, 1, 1, 1, 1, 1, 8, 7, 2, 0.0, 4, 0, None) == 1                                      # gated units, odd rows
    assert L.qsv_moe_up(1, 1, 1, 1, 1, 1, 8, 8, 3, 0.0, 4, 0, None) == 1                                      # clamped units without a limit
    assert L.qsv_add_normed_rms_norm(1, 1, 1, None, 0, 1, 0, 1e-5, 2, 8, 0, None) == 1                        # an added sublayer output without its gain
    assert L.qsv_qk_norm_rope_prep(1, 1, 64, None, 0, None, 0, 0, 2, 1, 32, 32, 1, None, 1, 1e-5, 1, 40, 1.0, None, 0, None, 1, 2, 0, None) == 1   # 40 rotated dimensions of 32
    assert L.qsv_min_gru_scan(1, 1, 16, 0, 8, 16, 1, 1, 1, 1, 1, 1, 8, 0, None) == 1                            # the gate's columns lie outside the rows
    with pytest.raises(RuntimeError):
        check(L.qsv_embed(0, 1, 1, 1, 1, 8, 0, None), "embed")


def test_serving_package_does_not_need_the_w4a8_library():
    """Importing the serving engine (and replaying a trace) must not load libqserve_amd.so: a fresh checkout builds only
    the serving kernels."""
    import subprocess
    import sys
    code = ("import sys; import qserve_amd.serving, qserve_amd.models.vekalorn, qserve_amd.models.mumelix, qserve_amd.models.vepolix, qserve_amd.models.pemolorn, qserve_amd.serving.trace; "
            "bad = [m for m in sys.modules if m in ('qserve_amd._lib', 'qserve_amd.decode', 'qserve_backend')]; sys.exit(1 if bad else 0)")
    assert subprocess.run([sys.executable, "-c", code], cwd=ROOT).returncode == 0
