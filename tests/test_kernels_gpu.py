"""GPU parity: every launcher, called through the C ABI, against the CPU oracle
on the same seeded inputs.

Bar: bit-exact for the embedding gather, the residual add and argmax;
|gpu - cpu| <= 1e-5 + 1e-4*|cpu| for every floating-point kernel.
"""
import importlib
import sys

import numpy as np
import pytest
import torch

import oracle

g2 = importlib.import_module("cuda-gpt2-inference_amd")

pytestmark = pytest.mark.gpu

RTOL, ATOL = 1e-4, 1e-5


def say(msg):
    print(msg, flush=True)
    sys.stdout.flush()


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def assert_close(gpu, cpu, what, rtol=RTOL, atol=ATOL):
    gpu = gpu.detach().cpu().numpy() if isinstance(gpu, torch.Tensor) else gpu
    assert gpu.shape == cpu.shape, (what, gpu.shape, cpu.shape)
    err = np.abs(gpu.astype(np.float64) - cpu.astype(np.float64))
    tol = atol + rtol * np.abs(cpu.astype(np.float64))
    bad = err > tol
    if bad.any() or not np.isfinite(gpu).all():
        i = np.unravel_index(np.argmax(err - tol), err.shape)
        raise AssertionError(f"{what}: {bad.sum()} of {bad.size} outside tolerance; worst at {i}: "
                             f"gpu={gpu[i]!r} cpu={cpu[i]!r} err={err[i]:.3e} tol={tol[i]:.3e}")
    return float(err.max())


def guard(shape, dtype=torch.float32):
    """Output buffer with NaN guard bands on both sides to catch stray writes."""
    n = int(np.prod(shape))
    pad = 1024
    full = torch.full((n + 2 * pad,), float("nan") if dtype == torch.float32 else -7,
                      dtype=dtype, device="cuda")
    return full, full[pad:pad + n].view(*shape), pad


def check_guard(full, pad):
    head, tail = full[:pad], full[-pad:]
    if full.dtype == torch.float32:
        assert torch.isnan(head).all() and torch.isnan(tail).all(), "write outside the output"
    else:
        assert (head == -7).all() and (tail == -7).all(), "write outside the output"


# ------------------------------------------------------------------ encoder
@pytest.mark.parametrize("B,T,C,V", [(4, 64, 768, 50257), (2, 5, 12, 11), (3, 7, 10, 13),
                                     (8, 1024, 768, 50257)])
def test_encoder_bit_exact(B, T, C, V):
    say(f"encoder B={B} T={T} C={C} V={V}")
    r = np.random.default_rng(100)
    wte = r.standard_normal((V, C), dtype=np.float32) * np.float32(0.02)
    wpe = r.standard_normal((max(T, 8), C), dtype=np.float32) * np.float32(0.01)
    ids = r.integers(0, V, (B, T), dtype=np.int32)
    full, out, pad = guard((B, T, C))
    g2.encoder_forward(out, dev(ids), dev(wte), dev(wpe), B, T, C)
    torch.cuda.synchronize()
    check_guard(full, pad)
    assert np.array_equal(out.cpu().numpy(), oracle.encoder_forward(ids, wte, wpe))


# ------------------------------------------------------------------ residual / gelu
@pytest.mark.parametrize("N", [0, 1, 3, 4, 1023, 4096 + 5, 8192 * 768])
def test_residual_bit_exact(N):
    say(f"residual N={N}")
    r = np.random.default_rng(101)
    a = r.standard_normal(N, dtype=np.float32)
    b = r.standard_normal(N, dtype=np.float32)
    full, out, pad = guard((N,))
    g2.residual_forward(out, dev(a), dev(b), N)
    torch.cuda.synchronize()
    check_guard(full, pad)
    assert np.array_equal(out.cpu().numpy(), oracle.residual_forward(a, b))


def test_residual_unaligned_pointers():
    N = 1001
    r = np.random.default_rng(102)
    a = r.standard_normal(N + 1, dtype=np.float32)
    b = r.standard_normal(N + 1, dtype=np.float32)
    da, db = dev(a), dev(b)
    out = torch.zeros(N + 1, device="cuda")
    g2.residual_forward(out[1:], da[1:], db[1:], N)  # 4-byte aligned only
    assert np.array_equal(out[1:].cpu().numpy(), a[1:] + b[1:])
    assert out[0].item() == 0.0


@pytest.mark.parametrize("N", [1, 7, 4096 + 3, 8192 * 3072])
def test_gelu(N):
    say(f"gelu N={N}")
    r = np.random.default_rng(103)
    x = r.standard_normal(N, dtype=np.float32) * np.float32(3.0)
    full, out, pad = guard((N,))
    g2.gelu_forward(out, dev(x), N)
    torch.cuda.synchronize()
    check_guard(full, pad)
    assert_close(out, oracle.gelu_forward(x), "gelu")


def test_gelu_special_values():
    x = np.array([0.0, -0.0, 30.0, -30.0, 1e-20, 88.0, -88.0], np.float32)
    out = torch.empty(x.size, device="cuda")
    g2.gelu_forward(out, dev(x), x.size)
    assert_close(out, oracle.gelu_forward(x), "gelu special")


# ------------------------------------------------------------------ layernorm
def ln_inputs(N, C, seed):
    r = np.random.default_rng(seed)
    x = r.standard_normal((N, C), dtype=np.float32)
    res = r.standard_normal((N, C), dtype=np.float32)
    w = (1 + 0.1 * r.standard_normal(C)).astype(np.float32)
    b = (0.1 * r.standard_normal(C)).astype(np.float32)
    return x, res, w, b


@pytest.mark.parametrize("N,C", [(8192, 768), (8192, 1024), (256, 768), (5, 64), (7, 260),
                                 (3, 2048), (2, 4096), (9, 4100), (6, 50), (1, 1)])
def test_layernorm(N, C):
    say(f"layernorm N={N} C={C}")
    x, _, w, b = ln_inputs(N, C, 110)
    fo, out, po = guard((N, C))
    fm, mean, pm = guard((N,))
    fr, rstd, pr = guard((N,))
    g2.layernorm_forward(out, mean, rstd, dev(x), dev(w), dev(b), 1, N, C)
    torch.cuda.synchronize()
    for f, p in ((fo, po), (fm, pm), (fr, pr)):
        check_guard(f, p)
    eo, em, er = oracle.layernorm_forward(x, w, b)
    assert_close(out, eo, "layernorm out")
    assert_close(mean, em, "layernorm mean")
    assert_close(rstd, er, "layernorm rstd")


def test_layernorm_null_stats_and_constant_row():
    N, C = 4, 768
    x = np.full((N, C), 3.25, np.float32)
    _, _, w, b = ln_inputs(N, C, 111)
    out = torch.empty((N, C), device="cuda")
    g2.layernorm_forward(out, None, None, dev(x), dev(w), dev(b), 2, 2, C)
    assert np.array_equal(out.cpu().numpy(), np.broadcast_to(b, (N, C)))


# every form the launcher chooses between by row count: one, two, four and eight rows per wave
# (N < 2048, < 8192, >= 8192), at 768 and 1024 channels, and the forms with bounds checks
@pytest.mark.parametrize("N,C", [(8192, 768), (8192, 1024), (256, 768), (5, 64), (7, 260),
                                 (3, 2048), (9, 4100), (6, 50),
                                 (4096, 768), (4096, 1024), (2048, 1024), (2040, 768), (1000, 1024),
                                 (1001, 768), (512, 256), (4100, 768), (2048, 2048), (16, 512),
                                 (4096, 1280), (2048, 1600), (300, 1280), (8192, 1600)])
def test_fused_residual_layernorm(N, C):
    say(f"fused_residual_layernorm N={N} C={C}")
    x, res, w, b = ln_inputs(N, C, 112)
    fo, out, po = guard((N, C))
    fs, rsum, ps = guard((N, C))
    fm, mean, pm = guard((N,))
    fr, rstd, pr = guard((N,))
    g2.fused_residual_layernorm_forward(rsum, out, mean, rstd, dev(x), dev(res), dev(w), dev(b), 1,
                                        N, C)
    torch.cuda.synchronize()
    for f, p in ((fo, po), (fs, ps), (fm, pm), (fr, pr)):
        check_guard(f, p)
    es, eo, em, er = oracle.fused_residual_layernorm_forward(x, res, w, b)
    assert np.array_equal(rsum.cpu().numpy(), es), "residual sum must be bit-exact"
    assert_close(out, eo, "fused ln out")
    assert_close(mean, em, "fused mean")
    assert_close(rstd, er, "fused rstd")


def test_fused_residual_layernorm_in_place_residual():
    N, C = 300, 768
    x, res, w, b = ln_inputs(N, C, 113)
    dx = dev(x)
    out = torch.empty((N, C), device="cuda")
    g2.fused_residual_layernorm_forward(dx, out, None, None, dx, dev(res), dev(w), dev(b), 1, N, C)
    es, eo, _, _ = oracle.fused_residual_layernorm_forward(x, res, w, b)
    assert np.array_equal(dx.cpu().numpy(), es)
    assert_close(out, eo, "fused ln out (in place)")


# ------------------------------------------------------------------ matmul
def mm_inputs(M, C, OC, seed, bias=True):
    r = np.random.default_rng(seed)
    x = r.standard_normal((M, C), dtype=np.float32)
    w = r.standard_normal((OC, C), dtype=np.float32) * np.float32(0.02)
    b = (r.standard_normal(OC, dtype=np.float32) * np.float32(0.02)) if bias else None
    return x, w, b


def run_matmul(x, w, b, gelu=None):
    M, C = x.shape
    OC = w.shape[0]
    full, out, pad = guard((M, OC))
    db = dev(b) if b is not None else None
    if gelu is None:
        g2.matmul_forward(out, dev(x), dev(w), db, 1, M, C, OC)
    else:
        g2.matmul_forward_gelu(out, dev(x), dev(w), db, 1, M, C, OC, gelu)
    torch.cuda.synchronize()
    check_guard(full, pad)
    return out


@pytest.mark.parametrize("M,C,OC", [
    (8192, 768, 2304), (8192, 768, 768), (8192, 768, 3072), (8192, 3072, 768),   # GPT-2 124M
    (256, 768, 2304), (256, 3072, 768),                                          # B=4, T=64
    (4096, 1024, 3072), (4096, 4096, 1024),                                      # GPT-2 350M
    (4096, 768, 768), (1024, 1024, 1024), (1000, 96, 1000), (64, 768, 3072),     # 64x64 / 32x32 tiles
    (1, 768, 2304), (8, 3072, 768), (16, 768, 50257), (5, 48, 37), (3, 1040, 100),  # <= 16 rows
    (128, 32, 192), (1, 4, 1), (130, 36, 200), (77, 100, 81), (300, 768, 50),    # edges
])
def test_matmul_bias(M, C, OC):
    say(f"matmul M={M} C={C} OC={OC}")
    x, w, b = mm_inputs(M, C, OC, 120)
    out = run_matmul(x, w, b)
    assert_close(out, oracle.matmul_forward(x, w, b), "matmul")


# Problems whose tile count does not come out in whole rounds of 256 with the largest tile
# (GPT-2 124M at B*T = 4096, 2048, 6144, ...), each with ragged edges in both dimensions, one
# or more per tile shape of the dispatcher; the expected shape is asserted so that the list
# keeps covering all of them.
@pytest.mark.parametrize("M,C,OC,tile", [
    (4096, 768, 2304, (128, 96)), (4093, 768, 2301, (128, 96)), (4096, 3072, 768, (128, 96)),
    (2048, 768, 768, (64, 96)), (6140, 768, 2300, (64, 96)), (500, 768, 2304, (64, 96)),
    (2045, 768, 771, (64, 128)), (2048, 1024, 1000, (64, 128)),
    (3072, 768, 2304, (64, 64)), (3070, 1024, 1000, (64, 64)),
    (1536, 768, 2304, (128, 128)), (4090, 1024, 1020, (128, 128)),
    (2048, 768, 3072, (128, 192)), (500, 768, 768, (32, 32)),
    (4096, 768, 3072, (256, 192)), (4090, 1024, 3070, (256, 192)),
    (8190, 768, 3070, (256, 192)), (2040, 1024, 4090, (256, 128)),
    # widths that are multiples of 160 (GPT-2 large: 1280 channels): 128x160, with ragged rows
    (4096, 1280, 1280, (128, 160)), (4090, 1280, 3840, (128, 160)), (2045, 1600, 4800, (128, 160)),
])
def test_matmul_every_tile_shape_with_edges(M, C, OC, tile):
    say(f"matmul M={M} C={C} OC={OC} tile={tile}")
    assert g2.matmul_forward_tile_shape(1, M, C, OC) == tile
    x, w, b = mm_inputs(M, C, OC, 123)
    out = run_matmul(x, w, b)
    assert_close(out, oracle.matmul_forward(x, w, b), "matmul")


# K split between the workgroups of a tile, every kernel form (tile shape x LDS-DMA / ring),
# ragged edges in both dimensions, split counts that do and do not divide the K slabs.  The
# same workspace serves all calls: every call must leave its counters at zero.  Two calls
# give bitwise equal results (the parts are summed in part order whoever arrives last).
SPLITK_CASES = [
    (2048, 768, 768, (128, 192), 4), (2045, 3072, 771, (128, 192), 3), (1000, 768, 2300, (128, 128), 2),
    (1530, 3072, 760, (128, 96), 5), (1024, 768, 768, (64, 128), 8), (1021, 3072, 700, (64, 128), 7),
    (2048, 768, 2304, (64, 64), 2), (256, 3072, 768, (64, 64), 5), (250, 768, 2300, (64, 64), 3),
    (256, 3072, 768, (32, 32), 2), (130, 1024, 1000, (32, 32), 4), (64, 96, 50, (32, 32), 3),
    (2048, 768, 2304, (128, 192), 2),
    (2048, 768, 768, (64, 96), 1), (2045, 768, 771, (64, 96), 2), (700, 3072, 2300, (64, 96), 5),
    (1000, 768, 1000, (256, 192), 1), (500, 1024, 380, (256, 192), 3), (700, 768, 250, (256, 128), 2),
    (1000, 768, 1270, (128, 160), 1), (500, 1280, 1280, (128, 160), 3), (129, 96, 161, (128, 160), 2),
]


@pytest.fixture(scope="module")
def splitk_workspace():
    return g2.matmul_forward_splitk_workspace()


@pytest.mark.parametrize("M,C,OC,tile,splits", SPLITK_CASES)
@pytest.mark.parametrize("gelu", [False, True])
def test_matmul_splitk_forced(M, C, OC, tile, splits, gelu, splitk_workspace):
    say(f"matmul split-K M={M} C={C} OC={OC} tile={tile} splits={splits} gelu={gelu}")
    x, w, b = mm_inputs(M, C, OC, 131)
    dx, dw, db = dev(x), dev(w), dev(b)
    outs = []
    for _ in range(2):
        full, out, pad = guard((M, OC))
        g2.matmul_forward_splitk(out, dx, dw, db, 1, M, C, OC, splitk_workspace, is_gelu=gelu,
                                 plan=(*tile, splits))
        torch.cuda.synchronize()
        check_guard(full, pad)
        outs.append(out)
    assert torch.equal(outs[0], outs[1]), "two runs of a K split differ"
    assert int(splitk_workspace[:g2.SPLITK_COUNTER_BYTES].max()) == 0, "counters not left at zero"
    exp = oracle.matmul_forward(x, w, b)
    if gelu:
        exp = oracle.gelu_forward(exp)
    assert_close(outs[0], exp, "matmul split-K")


# The plans the cost model picks at the GPT-2 124M shapes over M (with a workspace), against
# the oracle; at least some of them must split.
@pytest.mark.parametrize("M", [64, 256, 1024, 3072])
def test_matmul_splitk_chosen_plan(M, splitk_workspace):
    nsplit = 0
    for C, OC in [(768, 2304), (768, 768), (768, 3072), (3072, 768)]:
        plan = g2.matmul_forward_splitk_plan(1, M, C, OC, splitk_workspace.numel())
        say(f"matmul split-K chosen M={M} C={C} OC={OC} plan={plan}")
        nsplit += plan[2] > 1
        x, w, b = mm_inputs(M, C, OC, 132)
        full, out, pad = guard((M, OC))
        g2.matmul_forward_splitk(out, dev(x), dev(w), dev(b), 1, M, C, OC, splitk_workspace)
        torch.cuda.synchronize()
        check_guard(full, pad)
        assert_close(out, oracle.matmul_forward(x, w, b), "matmul split-K (chosen)")
    assert int(splitk_workspace[:g2.SPLITK_COUNTER_BYTES].max()) == 0
    assert nsplit > 0


@pytest.mark.parametrize("M", [256, 1024, 3072])
def test_matmul_llmc_signature_splits_k_through_the_thread_workspace(M, splitk_workspace):
    """matmul_forward / matmul_forward_gelu carry no workspace argument; with one lent through
    gpt2hip_set_workspace they give matmul_forward_splitk's result bit for bit (the same plan),
    and with none they are as before."""
    C, OC = 3072, 768
    plan = g2.matmul_forward_splitk_plan(1, M, C, OC, splitk_workspace.numel())
    say(f"matmul_forward with a thread workspace M={M} C={C} OC={OC} plan={plan}")
    assert plan[2] > 1
    x, w, b = mm_inputs(M, C, OC, 134)
    dx, dw, db = dev(x), dev(w), dev(b)
    want = torch.empty((M, OC), device="cuda")
    g2.matmul_forward_splitk(want, dx, dw, db, 1, M, C, OC, splitk_workspace)
    want_gelu = torch.empty((M, OC), device="cuda")
    g2.matmul_forward_splitk(want_gelu, dx, dw, db, 1, M, C, OC, splitk_workspace, is_gelu=True)
    plain = torch.empty((M, OC), device="cuda")
    g2.matmul_forward(plain, dx, dw, db, 1, M, C, OC)
    g2.set_workspace(splitk_workspace)
    try:
        full, out, pad = guard((M, OC))
        g2.matmul_forward(out, dx, dw, db, 1, M, C, OC)
        out_gelu = torch.empty((M, OC), device="cuda")
        g2.matmul_forward_gelu(out_gelu, dx, dw, db, 1, M, C, OC, True)
        torch.cuda.synchronize()
        check_guard(full, pad)
        assert torch.equal(out, want) and torch.equal(out_gelu, want_gelu)
        assert_close(out, oracle.matmul_forward(x, w, b), "matmul_forward (thread workspace)")
        assert int(splitk_workspace[:g2.SPLITK_COUNTER_BYTES].max()) == 0
    finally:
        g2.set_workspace(None)
    again = torch.empty((M, OC), device="cuda")
    g2.matmul_forward(again, dx, dw, db, 1, M, C, OC)
    assert torch.equal(again, plain)


# out = resid + (x . w^T + b), the residual add in the product's epilogue: every kernel family
# (the LDS-DMA kernel with the tile of resid fetched during the slab loop at 128x192 / 128x128 /
# 128x96, the same kernel reading it in the epilogue at 256x192, the ring kernel, K split between
# workgroups, edge tiles, the <= 16-row kernel, the generic one).  The sum must equal the plain
# product plus resid bit for bit (one fp32 addition per entry, the product's bits unchanged).
@pytest.mark.parametrize("M,C,OC", [
    (8192, 768, 768), (8192, 3072, 768), (4096, 1024, 1024), (4090, 768, 770), (8192, 768, 3072),
    (6000, 768, 1536), (4096, 1280, 1280), (2048, 768, 768), (2045, 3072, 771), (256, 3072, 768),
    (100, 96, 50), (33, 30, 17), (8, 768, 768),
    # one, two, three and five K slabs of 128x192 tiles: fewer pairs of slabs than the eight waves
    # that take turns fetching the residual during them
    (8192, 32, 768), (8192, 64, 768), (8192, 96, 768), (8192, 160, 768)])
@pytest.mark.parametrize("lend", [False, True])
def test_matmul_residual_epilogue(M, C, OC, lend, splitk_workspace):
    ws = splitk_workspace if lend else None
    plan = g2.matmul_forward_splitk_plan(1, M, C, OC, ws.numel() if lend else 0)
    say(f"matmul + residual M={M} C={C} OC={OC} workspace={lend} plan={plan}")
    x, w, b = mm_inputs(M, C, OC, 135)
    r = np.random.default_rng(136).standard_normal((M, OC), dtype=np.float32)
    dx, dw, db, dr = dev(x), dev(w), dev(b), dev(r)
    plain = torch.empty((M, OC), device="cuda")
    g2.matmul_forward_splitk(plain, dx, dw, db, 1, M, C, OC, ws)
    full, out, pad = guard((M, OC))
    g2.matmul_forward_residual(out, dx, dw, db, dr, 1, M, C, OC, ws)
    torch.cuda.synchronize()
    check_guard(full, pad)
    assert torch.equal(dr, dev(r)), "resid was modified"
    assert torch.equal(out, plain + dr), "not the plain product plus resid"
    if lend:
        assert int(ws[:g2.SPLITK_COUNTER_BYTES].max()) == 0, "counters not left at zero"
    elif M * C * OC <= 8192 * 768 * 768:
        assert_close(out, oracle.matmul_forward(x, w, b) + r, "matmul + residual")


# A wide product whose tiles come out just above whole rounds (the lm-head's 50257 columns at a
# few hundred to a few thousand rows) runs as two launches over ranges of its columns, rows of
# out staying OC floats apart: with bias, GELU, a residual, ragged rows, with and without a
# workspace for the second launch to split K through.
@pytest.mark.parametrize("M,C,OC,mode", [
    (256, 256, 50257, "bias"), (1000, 256, 50257, "gelu"), (1000, 128, 50257, "resid"),
    (2048, 128, 50257, "none"), (256, 768, 50257, "bias"), (1024, 768, 2304, "bias"), (1000, 1600, 6400, "gelu"),
    (2048, 1600, 1600, "resid")])
@pytest.mark.parametrize("lend", [False, True])
def test_matmul_wide_product_in_two_column_ranges(M, C, OC, mode, lend, splitk_workspace):
    ws = splitk_workspace if lend else None
    plan = g2.matmul_forward_splitk_plan(1, M, C, OC, ws.numel() if lend else 0)
    say(f"matmul in two column ranges M={M} C={C} OC={OC} {mode} workspace={lend} first launch {plan}")
    first = g2.matmul_forward_first_columns(1, M, C, OC, ws.numel() if lend else 0)
    assert 0 < first < OC and first % plan[1] == 0 and (first // plan[1]) * -(-M // plan[0]) % 256 == 0, first
    x, w, b = mm_inputs(M, C, OC, 138, bias=mode != "none")
    exp = oracle.matmul_forward(x, w, b)
    full, out, pad = guard((M, OC))
    if mode == "resid":
        r = np.random.default_rng(139).standard_normal((M, OC), dtype=np.float32)
        g2.matmul_forward_residual(out, dev(x), dev(w), dev(b), dev(r), 1, M, C, OC, ws)
        exp = exp + r
    else:
        g2.matmul_forward_splitk(out, dev(x), dev(w), None if b is None else dev(b), 1, M, C, OC, ws,
                                 is_gelu=mode == "gelu")
        if mode == "gelu":
            exp = oracle.gelu_forward(exp)
    torch.cuda.synchronize()
    check_guard(full, pad)
    assert_close(out, exp, "matmul in two column ranges")
    if lend:
        assert int(ws[:g2.SPLITK_COUNTER_BYTES].max()) == 0, "counters not left at zero"


def test_matmul_residual_rejects_overlap_and_null():
    M, C, OC = 64, 64, 64
    x, w, b = mm_inputs(M, C, OC, 137)
    buf = torch.zeros(2 * M * OC, device="cuda")
    out = buf[:M * OC].view(M, OC)
    with pytest.raises(RuntimeError, match="overlap"):
        g2.matmul_forward_residual(out, dev(x), dev(w), dev(b), out, 1, M, C, OC)
    with pytest.raises(RuntimeError, match="overlap"):
        g2.matmul_forward_residual(out, dev(x), dev(w), dev(b), buf[OC:OC + M * OC].view(M, OC), 1, M, C, OC)
    with pytest.raises(RuntimeError, match="null residual"):
        g2.matmul_forward_residual(out, dev(x), dev(w), dev(b), None, 1, M, C, OC)
    g2.matmul_forward_residual(out, dev(x), dev(w), dev(b), buf[M * OC:].view(M, OC), 1, M, C, OC)
    torch.cuda.synchronize()


def test_matmul_splitk_rejects_what_does_not_fit(splitk_workspace):
    x, w, b = mm_inputs(64, 64, 64, 133)
    out = torch.empty((64, 64), device="cuda")
    with pytest.raises(g2.GPT2HipError):  # 2 K slabs cannot be split three ways
        g2.matmul_forward_splitk(out, dev(x), dev(w), dev(b), 1, 64, 64, 64, splitk_workspace,
                                 plan=(32, 32, 3))
    with pytest.raises(g2.GPT2HipError):  # no such tile
        g2.matmul_forward_splitk(out, dev(x), dev(w), dev(b), 1, 64, 64, 64, splitk_workspace,
                                 plan=(48, 48, 2))
    small = torch.zeros(g2.SPLITK_COUNTER_BYTES + 1024, dtype=torch.uint8, device="cuda")
    with pytest.raises(g2.GPT2HipError):  # partial tiles do not fit
        g2.matmul_forward_splitk(out, dev(x), dev(w), dev(b), 1, 64, 64, 64, small, plan=(32, 32, 2))
    # without a workspace the call is matmul_forward_gelu
    g2.matmul_forward_splitk(out, dev(x), dev(w), dev(b), 1, 64, 64, 64, None)
    torch.cuda.synchronize()
    assert_close(out, oracle.matmul_forward(x, w, b), "matmul split-K without workspace")


def test_matmul_lm_head_no_bias():
    # 768 -> 50257 without bias; the oracle runs on a row subset to stay in seconds,
    # which is exact because rows are independent.
    M, C, OC = 8192, 768, 50257
    say(f"matmul lm-head M={M} C={C} OC={OC}")
    x, w, _ = mm_inputs(M, C, OC, 121, bias=False)
    out = run_matmul(x, w, None)
    rows = np.r_[0:64, 4000:4064, 8128:8192]
    exp = oracle.matmul_forward(x[rows], w, None)
    assert_close(out[torch.from_numpy(rows).cuda()], exp, "lm-head rows")
    # size-independent property over the full output: linearity in the input rows
    # (row i + row j through the same weights) checked on a column subset in float64
    got = out[:, ::997].cpu().numpy().astype(np.float64)
    ref = x.astype(np.float64) @ w[::997].astype(np.float64).T
    assert np.abs(got - ref).max() < 3e-5


def test_matmul_scaling_the_input_by_two_scales_the_output_exactly():
    """A property that holds at any size with no oracle: multiplying by a power of two is
    exact in fp32, so out(2 x) must equal 2 out(x) bit for bit -- at the full lm-head size."""
    M, C, OC = 8192, 768, 50257
    say(f"matmul scaling property M={M} C={C} OC={OC}")
    x, w, _ = mm_inputs(M, C, OC, 122, bias=False)
    out1 = run_matmul(x, w, None)
    out2 = run_matmul(2.0 * x, w, None)
    assert torch.equal(out2, 2.0 * out1)
    del out1, out2


def test_matmul_generic_path_unaligned_k():
    x, w, b = mm_inputs(33, 30, 17, 122)  # C % 4 != 0
    assert_close(run_matmul(x, w, b), oracle.matmul_forward(x, w, b), "matmul generic")
    assert_close(run_matmul(x, w, None), oracle.matmul_forward(x, w, None), "matmul generic nobias")


@pytest.mark.parametrize("M,C,OC", [(8192, 768, 3072), (256, 768, 3072), (70, 64, 100), (8, 768, 3072)])
def test_matmul_gelu_epilogue(M, C, OC):
    say(f"matmul+gelu M={M} C={C} OC={OC}")
    x, w, b = mm_inputs(M, C, OC, 123)
    exp = oracle.matmul_forward(x, w, b)
    assert_close(run_matmul(x, w, b, gelu=0), exp, "matmul is_gelu=0")
    out = run_matmul(x, w, b, gelu=1)
    # gelu has slope <= 1.13, so the matmul tolerance carries over to the composition
    assert_close(out, oracle.gelu_forward(exp), "matmul is_gelu=1")


def test_matmul_identity_weight():
    M, C = 200, 192
    r = np.random.default_rng(124)
    x = r.standard_normal((M, C), dtype=np.float32)
    b = r.standard_normal(C, dtype=np.float32)
    out = run_matmul(x, np.eye(C, dtype=np.float32), b)
    assert np.array_equal(out.cpu().numpy(), b[None, :] + x)


def test_matmul_probe_form_same_result_and_sane_clocks():
    M, C, OC = 2048, 768, 3072                         # 16 x 16 tiles of 128x192: one per CU
    x, w, b = mm_inputs(M, C, OC, 125)
    ref = run_matmul(x, w, b)
    out = torch.empty((M, OC), device="cuda")
    p = g2.matmul_forward_probe(out, dev(x), dev(w), dev(b), 1, M, C, OC)
    assert torch.equal(out, ref), "the probe instantiation must compute the same bits"
    assert p.shape == (16 * 16, 4)
    wall = (p[:, 1] - p[:, 0]) * 10e-9                 # seconds
    clk = p[:, 3] - p[:, 2]
    assert (wall > 0).all() and (clk > 0).all()
    per_slab = clk / (C // 32)
    # a slab of a 128x192 tile is 384 MFMAs = 6144 cycles on each of the CU's four SIMDs,
    # so anything below that is impossible; far above means a broken pipeline
    assert (per_slab >= 6144).all() and per_slab.mean() < 2 * 6144, per_slab.mean()
    mhz = clk.sum() / wall.sum() / 1e6
    assert 500 < mhz < 3000, mhz


def test_matmul_probe_rejects_small_buffer_and_odd_k():
    x, w, _ = mm_inputs(256, 64, 192, 126)
    out = torch.empty((256, 192), device="cuda")
    L = g2.lib()
    import ctypes
    probe = torch.zeros(4 * 47, dtype=torch.int64, device="cuda")
    n = ctypes.c_int(0)
    rc = L.matmul_forward_probe_status(out.data_ptr(), dev(x).data_ptr(), dev(w).data_ptr(), None,
                                       1, 256, 64, 192, probe.data_ptr(), 47, ctypes.byref(n))
    assert rc == 1 and b"probe buffer" in L.gpt2hip_last_error()
    x2, w2, _ = mm_inputs(256, 36, 192, 127)             # K % 32 != 0: register-staged kernel
    probe = torch.zeros(4 * 48, dtype=torch.int64, device="cuda")
    rc = L.matmul_forward_probe_status(out.data_ptr(), dev(x2).data_ptr(), dev(w2).data_ptr(), None,
                                       1, 256, 36, 192, probe.data_ptr(), 48, ctypes.byref(n))
    assert rc == 1 and b"C % 32" in L.gpt2hip_last_error()


# ------------------------------------------------------------------ attention
@pytest.mark.parametrize("B,T,NH", [(8, 1024, 12), (8, 256, 12), (8, 1024, 16), (8, 256, 16),
                                    (2, 1024, 16), (4, 256, 16), (4, 64, 12), (1, 1, 2), (2, 33, 3),
                                    (1, 130, 2), (1, 200, 1), (3, 512, 5), (1, 448, 12),
                                    # all workgroups resident at once, dealt to the compute units in
                                    # alternating direction: three full rows of 256, a partial second row
                                    (2, 1024, 12), (1, 1024, 12), (5, 160, 13)])
def test_attention_hs64(B, T, NH):
    say(f"attention B={B} T={T} NH={NH} HS=64")
    C = NH * 64
    qkv = np.random.default_rng(130).standard_normal((B, T, 3 * C), dtype=np.float32)
    dq = dev(qkv)
    full, out, pad = guard((B, T, C))
    g2.attention_forward(out, None, None, dq, B, T, C, NH)
    torch.cuda.synchronize()
    check_guard(full, pad)
    assert np.array_equal(dq.cpu().numpy(), qkv), "attention must not write its input"
    assert_close(out, oracle.attention_forward(qkv, NH), "attention")


@pytest.mark.parametrize("B,T,NH", [(2, 33, 3), (1, 130, 2), (3, 95, 1), (2, 1, 2)])
def test_attention_ragged_length_never_reads_past_its_rows(B, T, NH):
    """T is not a multiple of the 32-key sub-tile: the rows behind the last sequence must not
    reach the result.  qkv is a view into a larger tensor whose other elements are NaN (so
    nothing is read outside an allocation); a value row past T that met a zero softmax weight
    would still turn the whole query group into NaN."""
    say(f"attention ragged B={B} T={T} NH={NH} inside NaN")
    C = NH * 64
    qkv = np.random.default_rng(134).standard_normal((B, T, 3 * C), dtype=np.float32)
    n = qkv.size
    pad = 64 * 3 * C  # two sub-tiles' worth of rows on either side
    big = torch.full((n + 2 * pad,), float("nan"), device="cuda")
    big[pad:pad + n] = dev(qkv).view(-1)
    dq = big[pad:pad + n].view(B, T, 3 * C)
    full, out, opad = guard((B, T, C))
    g2.attention_forward(out, None, None, dq, B, T, C, NH)
    torch.cuda.synchronize()
    check_guard(full, opad)
    assert torch.isfinite(out).all()
    assert_close(out, oracle.attention_forward(qkv, NH), "attention ragged")


@pytest.mark.parametrize("B,T,NH,hs", [(2, 40, 4, 32), (1, 70, 2, 16), (1, 9, 3, 128), (2, 65, 2, 20)])
def test_attention_other_head_sizes(B, T, NH, hs):
    say(f"attention generic B={B} T={T} NH={NH} HS={hs}")
    C = NH * hs
    qkv = np.random.default_rng(131).standard_normal((B, T, 3 * C), dtype=np.float32)
    out = torch.empty((B, T, C), device="cuda")
    g2.attention_forward(out, None, None, dev(qkv), B, T, C, NH)
    assert_close(out, oracle.attention_forward(qkv, NH), "attention generic")


def test_attention_scaling_the_values_by_two_scales_the_output_exactly():
    """Size-independent property at the benchmark shape: the output is linear in v, and
    doubling is exact in fp32, so doubling v must double the output bit for bit."""
    B, T, NH = 8, 1024, 12
    C = NH * 64
    say(f"attention scaling property B={B} T={T} NH={NH}")
    qkv = np.random.default_rng(131).standard_normal((B, T, 3 * C), dtype=np.float32)
    qkv2 = qkv.copy()
    qkv2[:, :, 2 * C:] *= 2.0
    outs = []
    for a in (qkv, qkv2):
        out = torch.empty(B, T, C, device="cuda")
        g2.attention_forward(out, None, None, dev(a), B, T, C, NH)
        outs.append(out)
    torch.cuda.synchronize()
    assert torch.equal(outs[1], 2.0 * outs[0])


def test_attention_large_scores_stay_finite():
    B, T, NH = 1, 160, 2
    C = NH * 64
    qkv = np.random.default_rng(132).standard_normal((B, T, 3 * C), dtype=np.float32)
    qkv[..., :2 * C] *= 6.0  # scores of a few hundred: softmax is nearly one-hot
    out = torch.empty((B, T, C), device="cuda")
    g2.attention_forward(out, None, None, dev(qkv), B, T, C, NH)
    # Far outside the N(0,1) inputs the 1e-4/1e-5 bar is stated for: with score
    # differences in the hundreds, one fp32 rounding of the exponent's argument is
    # already ~2e-5 relative in the probability, in the oracle as much as on the GPU.
    # This case checks range handling (no overflow, no NaN), at a 5x wider tolerance.
    assert_close(out, oracle.attention_forward(qkv, NH), "attention large scores",
                 rtol=5e-4, atol=5e-5)


def test_attention_causality():
    """Perturbing tokens >= 100 must not change earlier outputs.

    Queries are processed in groups of 32 that share one decision about when the
    softmax shift moves (a shift never changes the value, only its rounding), so
    groups wholly before the perturbation (t < 96) must be bit-identical and the
    four unperturbed queries that share a group with perturbed ones must agree to
    fp32 rounding.
    """
    B, T, NH = 1, 192, 2
    C = NH * 64
    qkv = np.random.default_rng(133).standard_normal((B, T, 3 * C), dtype=np.float32)
    out1 = torch.empty((B, T, C), device="cuda")
    out2 = torch.empty((B, T, C), device="cuda")
    g2.attention_forward(out1, None, None, dev(qkv), B, T, C, NH)
    qkv2 = qkv.copy()
    qkv2[0, 100:] += 3.0
    g2.attention_forward(out2, None, None, dev(qkv2), B, T, C, NH)
    assert torch.equal(out1[0, :96], out2[0, :96])
    assert torch.allclose(out1[0, 96:100], out2[0, 96:100], rtol=2e-6, atol=2e-7)
    assert not torch.allclose(out1[0, 100:], out2[0, 100:], rtol=1e-3, atol=1e-3)


# ------------------------------------------------------------------ argmax
@pytest.mark.parametrize("N,V", [(256, 50257), (3, 5), (17, 257), (4, 1)])
def test_argmax_bit_exact(N, V):
    say(f"argmax N={N} V={V}")
    r = np.random.default_rng(140)
    x = r.standard_normal((N, V), dtype=np.float32)
    if V > 4:
        x[0, 3] = x[0, V - 1] = 9.0   # tie: lowest index must win
        x[1, :] = 1.5                 # all equal
    full, ids, pad = guard((N,), torch.int32)
    g2.argmax_forward(ids, dev(x), N, V)
    torch.cuda.synchronize()
    check_guard(full, pad)
    assert np.array_equal(ids.cpu().numpy(), oracle.argmax_forward(x))


# ------------------------------------------------------------------ fused matmul + argmax
@pytest.mark.parametrize("M,C,OC,bias", [
    (8192, 768, 50257, False),      # the lm-head: 4-wave tiles, ragged last column tile
    (256, 768, 50257, False),       # 8-wave tiles
    (300, 64, 1000, True),          # ragged rows and columns, bias
    (128, 32, 192, True),           # a single K slab, exactly one column tile
    (70, 36, 81, True),             # K % 32 != 0: one-block-per-row kernel
    (33, 30, 17, False),            # K % 4 != 0
])
def test_matmul_argmax_equals_unfused(M, C, OC, bias):
    say(f"matmul+argmax M={M} C={C} OC={OC}")
    x, w, b = mm_inputs(M, C, OC, 141, bias=bias)
    db = dev(b) if bias else None
    full, ids, pad = guard((M,), torch.int32)
    g2.matmul_forward_argmax(ids, dev(x), dev(w), db, 1, M, C, OC)
    torch.cuda.synchronize()
    check_guard(full, pad)
    got = ids.cpu().numpy()
    logits = torch.empty((M, OC), device="cuda")
    g2.matmul_forward(logits, dev(x), dev(w), db, 1, M, C, OC)
    if C % 32 == 0:
        # same accumulators as matmul_forward: exactly the argmax of its output
        unfused = torch.empty(M, dtype=torch.int32, device="cuda")
        g2.argmax_forward(unfused, logits, M, OC)
        assert np.array_equal(got, unfused.cpu().numpy())
    # against the oracle on a row subset: the chosen column's oracle value is the oracle's
    # maximum up to the matmul tolerance (an exact tie-break is only defined per backend)
    rows = np.unique(np.linspace(0, M - 1, 96).astype(np.int64))
    exp = oracle.matmul_forward(x[rows], w, b)
    chosen = exp[np.arange(len(rows)), got[rows]]
    assert (exp.max(-1) - chosen <= 1e-5 + 1e-4 * np.abs(exp.max(-1))).all()


def test_matmul_argmax_ties_nan_and_workspace_check():
    M, C, OC = 64, 32, 400
    x = np.zeros((M, C), np.float32)
    w = np.zeros((OC, C), np.float32)
    b = np.zeros(OC, np.float32)
    b[[7, 200, 399]] = 2.0          # three equal maxima in different tiles and waves: lowest wins
    x[1, 0] = np.nan                # a row of NaN products: nothing beats the start, index 0
    ids = torch.full((M,), -1, dtype=torch.int32, device="cuda")
    g2.matmul_forward_argmax(ids, dev(x), dev(w), dev(b), 1, M, C, OC)
    got = ids.cpu().numpy()
    assert got[0] == 7 and got[1] == 0 and (got[2:] == 7).all()
    need = g2.lib().matmul_forward_argmax_workspace(1, M, OC)
    assert need == M * 3 * 2 * 8     # 3 column tiles x 2 waves along N x (value, index)
    small = torch.empty(need - 1, dtype=torch.uint8, device="cuda")
    with pytest.raises(g2.GPT2HipError, match="workspace"):
        g2.matmul_forward_argmax(ids, dev(x), dev(w), dev(b), 1, M, C, OC, workspace=small)


# ------------------------------------------------------------------ error paths
def test_bad_shapes_raise_and_leave_the_device_usable():
    a = torch.zeros(64, device="cuda")
    with pytest.raises(g2.GPT2HipError):
        g2.matmul_forward(a, a, a, None, 1, 1, 0, 8)
    with pytest.raises(g2.GPT2HipError):
        g2.attention_forward(a, None, None, a, 1, 4, 30, 4)
    g2.residual_forward(a, a, a, 64)
    torch.cuda.synchronize()
