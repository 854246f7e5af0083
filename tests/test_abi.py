"""CPU-only checks of the drop-in boundary: the shared library loads, exports
every symbol the public header declares, and the Python mirror refuses to run
without device memory (no silent fallback)."""
import ctypes
import importlib
import os
import re

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
g2 = importlib.import_module("cuda-gpt2-inference_amd")


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "gpt2_mi355x.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = re.findall(r"\b([a-z][a-z0-9_]*)\s*\(", text)
    return sorted({n for n in names if n not in ("defined",)})


def test_header_and_python_export_lists_agree():
    assert declared_symbols() == sorted(g2.EXPORTS)


def test_library_exports_every_declared_symbol():
    assert os.path.exists(g2.LIB_PATH), "build with __graft_entry__.build() first"
    L = ctypes.CDLL(g2.LIB_PATH)
    missing = [s for s in declared_symbols() if not hasattr(L, s)]
    assert not missing, missing


def test_last_error_is_a_string():
    assert isinstance(g2.lib().gpt2hip_last_error(), bytes)


def test_launchers_reject_host_memory():
    a = np.zeros(8, np.float32)
    with pytest.raises(TypeError):
        g2.residual_forward(a, a, a, 8)


def test_shape_errors_are_reported_not_aborted():
    # Argument validation happens before any HIP call, so it runs without a GPU.
    L = g2.lib()
    fake = ctypes.c_void_p(4096)
    assert L.matmul_forward_status(fake, fake, fake, None, 1, 1, 0, 8) == 1
    assert b"bad shape" in L.gpt2hip_last_error()
    assert L.matmul_forward_status(None, fake, fake, None, 1, 1, 8, 8) == 1
    assert L.attention_forward_status(fake, None, None, fake, 1, 8, 30, 4) == 1  # C % NH != 0
    assert L.layernorm_forward_status(fake, None, None, fake, fake, None, 1, 1, 8) == 1
    assert L.residual_forward_status(fake, fake, None, 8) == 1
    assert L.argmax_forward_status(fake, fake, 1, 0) == 1
    assert L.encoder_forward_status(fake, fake, fake, fake, 1, 1, 0) == 1
    # empty work is a no-op, not an error
    assert L.residual_forward_status(fake, fake, fake, 0) == 0
    assert L.matmul_forward_status(fake, fake, fake, None, 0, 5, 8, 8) == 0


def test_synthetic_params_match_oracle_layout():
    import oracle
    syn = importlib.import_module("cuda-gpt2-inference_amd.synthetic")
    cfg = dict(max_seq_len=16, vocab_size=97, num_layers=2, num_heads=2, channels=32)
    p = syn.make_params(0, **cfg)
    assert p.size == oracle.num_parameters(16, 97, 2, 32)
    sizes = oracle.param_sizes(16, 97, 2, 32)
    shapes = syn.param_shapes(**cfg)
    assert list(sizes) == list(syn.PARAM_NAMES)
    for k in sizes:
        assert sizes[k] == int(np.prod(shapes[k]))


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU; asked for more it says so and exits (before touching a GPU)."""
    import subprocess, sys
    bench = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "bench.py")
    proc = subprocess.run([sys.executable, bench, "--gpus", "2"], capture_output=True, text=True, timeout=300)
    assert proc.returncode != 0
    assert "--gpus 1" in (proc.stdout + proc.stderr)


def test_tile_choice_needs_no_gpu_and_avoids_partial_rounds():
    """The GEMM's tile choice: 124M at B*T = 8192 keeps the largest tile (3, 1, 4, 1 whole
    rounds of 256 tiles), the same layer shapes at B*T = 4096 take the tile that divides
    evenly (128x96: 768 and 256 tiles instead of 384 and 128 tiles of 128x192)."""
    import importlib
    g2 = importlib.import_module("cuda-gpt2-inference_amd")
    for C, OC in ((768, 2304), (768, 768), (3072, 768)):
        assert g2.matmul_forward_tile_shape(8, 1024, C, OC) == (128, 192)
    assert g2.matmul_forward_tile_shape(8, 1024, 768, 3072) == (256, 192)       # 512 tiles: two exact rounds
    assert g2.matmul_forward_tile_shape(4, 1024, 1024, 4096) == (256, 128)      # 350M fc: 512 tiles
    assert g2.matmul_forward_tile_shape(4, 1024, 1024, 3072) == (256, 192)      # 350M qkv: 256 tiles
    assert g2.matmul_forward_tile_shape(4, 1024, 768, 2304) == (128, 96)
    assert g2.matmul_forward_tile_shape(4, 1024, 768, 768) == (128, 96)
    assert g2.matmul_forward_tile_shape(4, 1024, 1024, 1024) == (128, 128)      # 350M
    assert g2.matmul_forward_tile_shape(8, 1024, 768, 50257) == (128, 192)      # lm-head
    assert g2.matmul_forward_tile_shape(4, 64, 768, 768) == (32, 32)            # short prompt
    assert g2.matmul_forward_tile_shape(1, 100, 36, 200) == (0, 0)              # K % 32 != 0
    assert g2.matmul_forward_tile_shape(1, 16, 768, 768) == (0, 0)              # <= 16 rows
    # whatever is chosen never needs more rounds of work than the largest tile would
    for M in range(64, 8193, 448):
        for C, OC in ((768, 2304), (768, 768), (1024, 4096), (4096, 1024)):
            bm, bn = g2.matmul_forward_tile_shape(1, M, C, OC)
            rounds = -(-(-(-M // bm) * -(-OC // bn)) // 256)
            big = -(-(-(-M // 128) * -(-OC // 192)) // 256)
            assert rounds * bm * bn <= big * 128 * 192 * 1.45, (M, C, OC, bm, bn)
    with pytest.raises(g2.GPT2HipError):
        g2.matmul_forward_tile_shape(0, 5, 32, 32)


def test_splitk_plan_without_a_gpu():
    """The K-split planner is host arithmetic: no workspace means no split; the BASELINE
    shapes (exact rounds of the largest tile) never split; fcproj (K = 3072) at short and
    middling B*T does; every plan fits the workspace it was given."""
    import importlib
    g2 = importlib.import_module("cuda-gpt2-inference_amd")
    ws = g2.lib().matmul_forward_splitk_workspace()
    assert ws > g2.SPLITK_COUNTER_BYTES
    for M in (64, 256, 2048, 8192):
        for C, OC in ((768, 2304), (768, 768), (768, 3072), (3072, 768)):
            bm, bn, sp = g2.matmul_forward_splitk_plan(1, M, C, OC, 0)
            assert sp == 1 and (bm, bn) == g2.matmul_forward_tile_shape(1, M, C, OC)
            bm, bn, sp = g2.matmul_forward_splitk_plan(1, M, C, OC, ws)
            tiles = -(-M // bm) * -(-OC // bn)
            assert 1 <= sp <= C // 32
            assert sp == 1 or tiles * sp * bm * bn * 4 <= ws - g2.SPLITK_COUNTER_BYTES
            if M == 8192:
                assert (bm, bn, sp) == ((256, 192, 1) if OC == 3072 else (128, 192, 1))
    for M in (64, 128, 512, 1024, 3072):
        assert g2.matmul_forward_splitk_plan(1, M, 3072, 768, ws)[2] > 1, M
    # a workspace that only holds the counters cannot split
    assert g2.matmul_forward_splitk_plan(1, 1024, 3072, 768, g2.SPLITK_COUNTER_BYTES)[2] == 1
    assert g2.matmul_forward_splitk_plan(1, 100, 36, 200, ws) == (0, 0, 1)      # K % 32 != 0


def test_thread_workspace_setting_is_validated_without_a_gpu():
    """gpt2hip_set_workspace only records a pointer: alignment and size are checked up front."""
    L = g2.lib()
    assert L.gpt2hip_set_workspace(ctypes.c_void_p(4096 + 64), 1 << 20) == 1
    assert b"aligned" in L.gpt2hip_last_error()
    assert L.gpt2hip_set_workspace(ctypes.c_void_p(4096), 1024) == 1
    assert b"counters" in L.gpt2hip_last_error()
    assert L.gpt2hip_set_workspace(ctypes.c_void_p(4096), 1 << 20) == 0
    assert L.gpt2hip_set_workspace(None, 0) == 0


def test_library_links_no_blas():
    """The product is hand-written HIP: the shared library must not depend on a vendor BLAS
    (rocBLAS / hipBLAS / hipBLASLt), not even indirectly through its own link line."""
    import subprocess
    out = subprocess.run(["readelf", "-d", g2.LIB_PATH], capture_output=True, text=True, check=True).stdout
    needed = re.findall(r"\(NEEDED\)\s+Shared library: \[(.*?)\]", out)
    assert needed, out
    assert not [n for n in needed if re.search(r"blas|miopen|rccl|torch", n, re.I)], needed
    syms = subprocess.run(["nm", "-D", "--undefined-only", g2.LIB_PATH], capture_output=True, text=True,
                          check=True).stdout
    assert not re.search(r"rocblas_|hipblas|hipblaslt", syms, re.I)


def test_where_the_driver_forms_the_residual_sums_is_a_pure_function_of_the_size():
    """gpt2_forward adds the residual stream in the projections' epilogues from B*T*channels =
    3e6 on (the headline size and GPT-2 350M at B=4) and keeps the reference's fused
    residual+layernorm below; the answer needs no GPU."""
    assert g2.forward_sums_in_matmul(g2.GPT2_124M, 8, 1024)
    assert g2.forward_sums_in_matmul(g2.GPT2_124M, 4, 1024)
    assert g2.forward_sums_in_matmul(g2.GPT2_350M, 4, 1024)
    assert not g2.forward_sums_in_matmul(g2.GPT2_124M, 2, 1024)
    assert not g2.forward_sums_in_matmul(g2.GPT2_124M, 4, 64)
    assert g2.lib().gpt2_forward_sums_in_matmul(None, 8, 1024) == 0


def test_wide_products_are_planned_as_whole_rounds_plus_the_columns_left():
    """The lm-head at a few hundred to a few thousand rows: the first launch covers a whole
    number of rounds of its tile over the 256 compute units; tall or narrow products are one launch."""
    for M in (256, 512, 1024, 2048):
        first = g2.matmul_forward_first_columns(1, M, 768, 50257)
        bm, bn = g2.matmul_forward_tile_shape(1, M, 768, 50257)
        assert 0 < first < 50257 and first % bn == 0 and (first // bn) * -(-M // bm) % 256 == 0, (M, first, bm, bn)
    assert g2.matmul_forward_first_columns(1, 1024, 768, 2304) == 2048      # 16 x 16 tiles of 64x128, then 256 columns
    assert g2.matmul_forward_first_columns(1, 8192, 768, 50257) == 50257
    assert g2.matmul_forward_first_columns(1, 2048, 768, 3072) == 3072
    assert g2.matmul_forward_first_columns(1, 8, 768, 50257) == 50257
    assert g2.matmul_forward_first_columns(0, 8, 768, 50257) == 0
