"""End-to-end parity of the gpt2_forward driver against the CPU oracle.

Bar: logits max-abs difference <= 2e-3; argmax ids bit-exact.  Argmax of two
different fp32 summation orders can only differ where the oracle's top-2 gap is
itself at rounding level, so a mismatch is reported together with that gap.
"""
import importlib
import os
import sys

import numpy as np
import pytest
import torch

import oracle

g2 = importlib.import_module("cuda-gpt2-inference_amd")
syn = importlib.import_module("cuda-gpt2-inference_amd.synthetic")

pytestmark = pytest.mark.gpu

LOGIT_TOL = 2e-3


def run_both(cfg, B, T, seed, perturb=False, host_ids=True):
    print(f"gpt2 e2e cfg={cfg} B={B} T={T} seed={seed}", flush=True)
    sys.stdout.flush()
    params = syn.make_params(seed, perturb_affine=perturb, **cfg)
    ids = syn.make_tokens(seed + 1, B, T, cfg["vocab_size"])
    model = g2.GPT2(**cfg)
    try:
        model.load_params(params)
        model.forward(ids if host_ids else torch.from_numpy(ids).cuda())
        torch.cuda.synchronize()
        logits = model.logits().cpu().numpy()
        lnf = model.lnf().cpu().numpy()
        am = model.argmax().cpu().numpy()
    finally:
        model.close()
    exp_logits, exp_ids, exp_lnf = oracle.gpt2_forward(
        params, ids, maxT=cfg["max_seq_len"], V=cfg["vocab_size"], L=cfg["num_layers"],
        NH=cfg["num_heads"], C=cfg["channels"], want_lnf=True)
    return logits, lnf, am, exp_logits, exp_lnf, exp_ids


def check(logits, lnf, am, exp_logits, exp_lnf, exp_ids):
    assert np.isfinite(logits).all()
    d = np.abs(logits.astype(np.float64) - exp_logits.astype(np.float64)).max()
    dl = np.abs(lnf.astype(np.float64) - exp_lnf.astype(np.float64)).max()
    print(f"  max|dlogits|={d:.3e} max|dlnf|={dl:.3e}", flush=True)
    assert d <= LOGIT_TOL, f"logits differ by {d}"
    # the GPU argmax kernel on the GPU's own logits must be the exact argmax of them
    assert np.array_equal(am, logits.argmax(-1).astype(np.int32))
    if not np.array_equal(am, exp_ids):
        bad = np.argwhere(am != exp_ids)
        top2 = np.sort(exp_logits[tuple(bad.T)], axis=-1)[:, -2:]
        gaps = top2[:, 1] - top2[:, 0]
        raise AssertionError(f"argmax differs at {len(bad)} positions {bad[:5].tolist()}; oracle "
                             f"top-2 gaps there: {gaps[:5]}")


def test_gpt2_124M_B4_T64():
    check(*run_both(dict(g2.GPT2_124M), 4, 64, seed=1337))


def test_gpt2_124M_device_ids_and_perturbed_affine():
    check(*run_both(dict(g2.GPT2_124M), 2, 128, seed=7, perturb=True, host_ids=False))


def test_gpt2_small_config_odd_sizes():
    # head size 64 (MFMA attention), T not a multiple of any tile, odd vocabulary
    cfg = dict(max_seq_len=80, vocab_size=331, num_layers=3, num_heads=2, channels=128)
    check(*run_both(cfg, 3, 77, seed=11, perturb=True))


def test_gpt2_small_config_generic_attention():
    cfg = dict(max_seq_len=32, vocab_size=97, num_layers=2, num_heads=2, channels=64)  # hs=32
    check(*run_both(cfg, 2, 19, seed=12, perturb=True))


def test_gpt2_350M_B1_T128():
    check(*run_both(dict(g2.GPT2_350M), 1, 128, seed=21))


@pytest.mark.parametrize("C,NH", [(1280, 20), (1600, 25)])
def test_gpt2_wider_models_one_layer(C, NH):
    # the widths of GPT-2 large and XL (one block of each): K and N the 124M / 350M shapes do
    # not exercise (1280, 3840, 5120, 1600, 4800, 6400), 20 and 25 heads
    cfg = dict(max_seq_len=1024, vocab_size=50257, num_layers=1, num_heads=NH, channels=C)
    check(*run_both(cfg, 2, 200, seed=51, perturb=True))


@pytest.mark.parametrize("name,B,T", [("124M", 8, 1024), ("350M", 4, 1024)])
def test_gpt2_full_size_against_the_oracle(name, B, T):
    """The benchmark's own workloads, whole: every logit of the (B*T, V) result against the
    CPU oracle's.  With 8192 / 4096 positions a few argmax near-ties are expected between two
    fp32 summation orders, so ids must agree wherever the oracle's top-2 gap exceeds twice the
    largest logit difference (which is every position where the order cannot matter)."""
    cfg = dict(g2.GPT2_124M if name == "124M" else g2.GPT2_350M)
    logits, lnf, am, exp_logits, exp_lnf, exp_ids = run_both(cfg, B, T, seed=4242)
    V = cfg["vocab_size"]
    logits = logits.reshape(-1, V)
    exp_logits = exp_logits.reshape(-1, V)
    am = am.reshape(-1)
    exp_ids = exp_ids.reshape(-1)
    d = 0.0
    for r in range(0, logits.shape[0], 512):
        a, e = logits[r:r + 512], exp_logits[r:r + 512]
        assert np.isfinite(a).all()
        d = max(d, float(np.abs(a - e).max()))
        assert np.array_equal(am[r:r + 512], a.argmax(-1).astype(np.int32))
    dl = float(np.abs(lnf - exp_lnf).max())
    print(f"  full size {name}: max|dlogits|={d:.3e} max|dlnf|={dl:.3e} "
          f"argmax mismatches={int((am != exp_ids).sum())} of {am.size}", flush=True)
    assert d <= LOGIT_TOL
    bad = np.flatnonzero(am != exp_ids)
    if bad.size:
        top2 = np.sort(exp_logits[bad], axis=-1)[:, -2:]
        gaps = top2[:, 1] - top2[:, 0]
        print(f"  oracle top-2 gaps at the mismatches: {gaps[:8]}", flush=True)
        assert (gaps <= 2 * d).all(), f"argmax differs where the oracle's gap is {gaps.max()}"


def test_gpt2_against_committed_float64_fixture():
    from golden import load_gpt2_tiny
    cfg, params, ids, exp_logits, exp_lnf = load_gpt2_tiny()
    model = g2.GPT2(**cfg)
    try:
        model.load_params(params)
        model.forward(ids)
        torch.cuda.synchronize()
        logits = model.logits().cpu().numpy()
        lnf = model.lnf().cpu().numpy()
        am = model.argmax().cpu().numpy()
    finally:
        model.close()
    print(f"  fixture: max|dlogits|={np.abs(logits - exp_logits).max():.3e}", flush=True)
    assert np.abs(lnf - exp_lnf).max() < 2e-5
    assert np.abs(logits - exp_logits).max() < 2e-5
    top2 = np.sort(exp_logits, -1)[..., -2:]
    clear = (top2[..., 1] - top2[..., 0]) > 1e-4
    assert np.array_equal(am[clear], exp_logits.argmax(-1)[clear])


def test_gpt2_forward_argmax_matches_forward_then_argmax():
    for cfg, B, T in ((dict(g2.GPT2_124M), 2, 128),
                      (dict(max_seq_len=80, vocab_size=331, num_layers=2, num_heads=2, channels=128),
                       3, 77)):
        print(f"gpt2 forward_argmax cfg={cfg} B={B} T={T}", flush=True)
        params = syn.make_params(31, perturb_affine=True, **cfg)
        ids = torch.from_numpy(syn.make_tokens(32, B, T, cfg["vocab_size"])).cuda()
        model = g2.GPT2(**cfg)
        try:
            model.load_params(params)
            model.forward(ids)
            want = model.argmax().clone()
            model.logits().fill_(float("nan"))          # the fused pass must not need them
            got = model.forward_argmax(ids)
            torch.cuda.synchronize()
            assert torch.equal(got, want)
            assert torch.isnan(model.logits()).all(), "forward_argmax must not write logits"
            with pytest.raises(g2.GPT2HipError):
                model.argmax()                          # no logits were left by that pass
        finally:
            model.close()


def test_gpt2_device_ids_outside_vocabulary_give_nan_rows_not_faults():
    cfg = dict(max_seq_len=16, vocab_size=50, num_layers=1, num_heads=1, channels=64)
    model = g2.GPT2(**cfg)
    try:
        model.load_params(syn.make_params(41, **cfg))
        ids = syn.make_tokens(42, 3, 8, 50)
        ids[1, 3] = 50
        ids[0, 5] = -1
        model.forward(torch.from_numpy(ids).cuda())
        torch.cuda.synchronize()
        bad = torch.isnan(model.logits()).all(-1).cpu().numpy()
        # a NaN row shows at its own and every later position of its sequence (earlier
        # positions of that sequence are unspecified); other sequences are untouched
        assert bad[0, 5:].all() and bad[1, 3:].all() and not bad[2].any()
    finally:
        model.close()


def test_gpt2_graph_replays_match_eager_with_eager_work_between():
    cfg = dict(max_seq_len=64, vocab_size=211, num_layers=2, num_heads=2, channels=128)
    model = g2.GPT2(**cfg)
    try:
        model.load_params(syn.make_params(51, perturb_affine=True, **cfg))
        batches = [torch.from_numpy(syn.make_tokens(60 + i, 2, 48, 211)).cuda() for i in range(4)]
        other = torch.from_numpy(syn.make_tokens(70, 1, 9, 211)).cuda()
        eager = []
        for ids in batches:
            model.forward(ids)
            eager.append(model.logits().clone())
        for rep in range(3):                             # first call captures, the rest replay
            for ids, want in zip(batches, eager):
                model.forward_graph(ids)
                torch.cuda.synchronize()
                assert torch.equal(model.logits(), want), f"replay {rep}"
                model.forward(other)                     # eager work between replays
                scratch = torch.randn(1 << 16, device="cuda").sum().item()
                assert np.isfinite(scratch)
        model.forward_graph(other)                       # a second graph, smaller shape
        model.forward(other)
        want_other = model.logits().clone()
        model.forward_graph(other)
        torch.cuda.synchronize()
        assert torch.equal(model.logits(), want_other)
        big = torch.from_numpy(syn.make_tokens(71, 3, 64, 211)).cuda()
        model.forward_graph(big)                         # reallocation drops the old graphs
        model.forward_graph(batches[0])                  # and a dropped shape is re-captured
        torch.cuda.synchronize()
        assert torch.equal(model.logits(), eager[0])
    finally:
        model.close()


def test_gpt2_graph_replays_with_k_split_gemms():
    """A model whose 4C -> C projection splits K between workgroups (C = 256 at B*T = 96): the
    split's counters are reset by the kernels themselves, so a captured forward must replay to
    the eager result every time, with eager forwards of another shape in between."""
    cfg = dict(max_seq_len=64, vocab_size=211, num_layers=2, num_heads=4, channels=256)
    assert g2.matmul_forward_splitk_plan(2, 48, 1024, 256, g2.lib().matmul_forward_splitk_workspace())[2] > 1
    model = g2.GPT2(**cfg)
    try:
        model.load_params(syn.make_params(54, perturb_affine=True, **cfg))
        ids = torch.from_numpy(syn.make_tokens(55, 2, 48, 211)).cuda()
        other = torch.from_numpy(syn.make_tokens(56, 1, 33, 211)).cuda()
        model.forward(ids)
        want = model.logits().clone()
        exp_logits, _ = oracle.gpt2_forward(syn.make_params(54, perturb_affine=True, **cfg),
                                            ids.cpu().numpy(), maxT=64, V=211, L=2, NH=4, C=256)
        assert np.abs(want.cpu().numpy().reshape(exp_logits.shape).astype(np.float64) - exp_logits).max() <= 2e-3
        for rep in range(4):
            model.forward_graph(ids)
            torch.cuda.synchronize()
            assert torch.equal(model.logits(), want), f"replay {rep}"
            model.forward(other)
            torch.cuda.synchronize()
    finally:
        model.close()


def test_gpt2_graph_capture_and_replay_after_every_gemm_form_has_been_used():
    """The launchers raise a kernel's dynamic-LDS limit the first time a thread uses it and
    remember the kernels they have done it for (a table that used to hold 64 of them and now
    grows).  Every tiled GEMM form the library has is touched first -- each tile shape, with and
    without GELU, with and without a K split, the probed and the argmax forms -- then a forward
    pass is captured and replayed: the capture must not contain (or trip over) an attribute call,
    and the replays must give the eager result."""
    import oracle as _oracle
    ws = g2.matmul_forward_splitk_workspace()
    M, C, OC = 320, 128, 448
    r = np.random.default_rng(77)
    x = torch.from_numpy(r.standard_normal((M, C), dtype=np.float32)).cuda()
    w = torch.from_numpy((r.standard_normal((OC, C)) * 0.05).astype(np.float32)).cuda()
    b = torch.from_numpy((r.standard_normal(OC) * 0.05).astype(np.float32)).cuda()
    want = _oracle.matmul_forward(x.cpu().numpy(), w.cpu().numpy(), b.cpu().numpy())
    out = torch.empty((M, OC), device="cuda")
    forms = 0
    for tile in ((256, 192), (256, 128), (128, 192), (128, 128), (128, 96), (64, 128), (64, 96), (64, 64), (32, 32)):
        for splits in (1, 2):
            for gelu in (False, True):
                g2.matmul_forward_splitk(out, x, w, b, 1, M, C, OC, ws, is_gelu=gelu, plan=(*tile, splits))
                forms += 1
            torch.cuda.synchronize()
        g2.matmul_forward_splitk(out, x, w, b, 1, M, C, OC, ws, plan=(*tile, 1))
        torch.cuda.synchronize()
        assert np.abs(out.cpu().numpy() - want).max() <= 1e-4, tile
    # many 64x64 tiles take the two-buffer kernel instead of the ring (two more forms), many
    # 128x192 tiles the four-wave form, K % 32 != 0 the register-staged kernel
    big = torch.empty((2048, 1024), device="cuda")
    xb = torch.randn(2048, 128, device="cuda")
    wb = torch.randn(1024, 128, device="cuda") * 0.05
    for gelu in (False, True):
        g2.matmul_forward_splitk(big, xb, wb, None, 1, 2048, 128, 1024, ws, is_gelu=gelu, plan=(64, 64, 1))
        g2.matmul_forward_gelu(out, x[:, :100].contiguous(), w[:, :100].contiguous(), b, 1, M, 100, OC, gelu)
        forms += 2
    g2.matmul_forward_probe(out, x, w, b, 1, M, C, OC)
    ids_out = torch.empty(M, dtype=torch.int32, device="cuda")
    g2.matmul_forward_argmax(ids_out, x, w, b, 1, M, C, OC)
    forms += 2
    torch.cuda.synchronize()
    print(f"  {forms} GEMM forms used before the capture", flush=True)
    assert int(ws[:g2.SPLITK_COUNTER_BYTES].max()) == 0

    cfg = dict(max_seq_len=64, vocab_size=211, num_layers=2, num_heads=4, channels=256)
    model = g2.GPT2(**cfg)
    try:
        model.load_params(syn.make_params(57, perturb_affine=True, **cfg))
        ids = torch.from_numpy(syn.make_tokens(58, 2, 48, 211)).cuda()
        model.forward(ids)
        eager = model.logits().clone()
        for rep in range(3):
            model.forward_graph(ids)
            torch.cuda.synchronize()
            assert torch.equal(model.logits(), eager), f"replay {rep}"
            g2.matmul_forward_splitk(out, x, w, b, 1, M, C, OC, ws, plan=(64, 96, 2))   # eager work between
            torch.cuda.synchronize()
    finally:
        model.close()


def test_launchers_follow_the_selected_stream():
    cfg = dict(max_seq_len=64, vocab_size=211, num_layers=2, num_heads=2, channels=128)
    model = g2.GPT2(**cfg)
    side = torch.cuda.Stream()
    try:
        model.load_params(syn.make_params(52, **cfg))
        ids = torch.from_numpy(syn.make_tokens(53, 2, 40, 211)).cuda()
        model.forward(ids)
        want = model.logits().clone()
        torch.cuda.synchronize()
        g2.set_stream(side)
        assert g2.lib().gpt2hip_get_stream() == side.cuda_stream
        model.logits().zero_()
        torch.cuda.synchronize()
        model.forward(ids)
        side.synchronize()                               # waits for the forward only if it ran there
        assert torch.equal(model.logits(), want)
    finally:
        g2.set_stream(None)
        model.close()
    assert not g2.lib().gpt2hip_get_stream()


@pytest.mark.parametrize("cfg,B,T0,steps", [
    (dict(max_seq_len=80, vocab_size=331, num_layers=3, num_heads=2, channels=128), 3, 37, 6),
    (dict(max_seq_len=32, vocab_size=97, num_layers=2, num_heads=2, channels=64), 2, 1, 5),   # hs=32
    (dict(g2.GPT2_124M), 2, 100, 4),
    (dict(max_seq_len=48, vocab_size=211, num_layers=2, num_heads=2, channels=128), 17, 20, 3),  # > 16 rows
    (dict(max_seq_len=40, vocab_size=97, num_layers=2, num_heads=3, channels=60), 2, 9, 3),      # C % 16 != 0
])
def test_gpt2_prefill_and_decode_match_the_full_forward(cfg, B, T0, steps):
    """Teacher-forced: after a prompt of T0 tokens, every decode step's logits must be the
    oracle's full-sequence logits at that position."""
    print(f"gpt2 decode cfg={cfg} B={B} T0={T0} steps={steps}", flush=True)
    params = syn.make_params(81, perturb_affine=True, **cfg)
    ids = syn.make_tokens(82, B, T0 + steps, cfg["vocab_size"])
    exp_logits, _, _ = oracle.gpt2_forward(params, ids, maxT=cfg["max_seq_len"], V=cfg["vocab_size"],
                                           L=cfg["num_layers"], NH=cfg["num_heads"],
                                           C=cfg["channels"], want_lnf=True)
    dids = torch.from_numpy(ids).cuda()
    model = g2.GPT2(**cfg)
    try:
        model.load_params(params)
        got = model.prefill(dids[:, :T0].contiguous()).cpu().numpy()
        assert model.cache_length() == T0
        d = np.abs(got - exp_logits[:, T0 - 1]).max()
        print(f"  prefill: max|dlogits|={d:.3e}", flush=True)
        assert d <= LOGIT_TOL
        for s in range(steps):
            got = model.decode(dids[:, T0 + s].contiguous()).cpu().numpy()
            d = np.abs(got - exp_logits[:, T0 + s]).max()
            print(f"  step {s}: max|dlogits|={d:.3e}", flush=True)
            assert d <= LOGIT_TOL
            assert np.array_equal(got.argmax(-1), exp_logits[:, T0 + s].argmax(-1))
        assert model.cache_length() == T0 + steps
        # a new prompt with another batch size restarts the cache
        got = model.prefill(dids[:1, :T0].contiguous()).cpu().numpy()
        assert np.abs(got - exp_logits[:1, T0 - 1]).max() <= LOGIT_TOL
    finally:
        model.close()


@pytest.mark.parametrize("cfg,B,T0,steps", [
    (dict(max_seq_len=48, vocab_size=211, num_layers=2, num_heads=4, channels=256), 3, 5, 6),
    (dict(max_seq_len=300, vocab_size=1031, num_layers=2, num_heads=8, channels=512), 5, 7, 3),
    (dict(max_seq_len=64, vocab_size=331, num_layers=2, num_heads=4, channels=256), 13, 37, 3),
    (dict(max_seq_len=128, vocab_size=3001, num_layers=2, num_heads=16, channels=1024), 4, 100, 3),
    (dict(max_seq_len=300, vocab_size=1031, num_layers=3, num_heads=8, channels=512), 16, 250, 5),
    (dict(max_seq_len=64, vocab_size=50257, num_layers=2, num_heads=12, channels=768), 1, 1, 4),
    (dict(g2.GPT2_124M), 8, 120, 10),
    # the cache attention's sweeps of 256 positions: steps across the first and second boundary
    (dict(max_seq_len=600, vocab_size=211, num_layers=2, num_heads=4, channels=256), 2, 252, 8),
    (dict(max_seq_len=600, vocab_size=211, num_layers=2, num_heads=4, channels=256), 3, 508, 8),
    # long contexts cut every (sequence, head) into ranges of positions: 4, 3 and 2 of them
    (dict(max_seq_len=400, vocab_size=211, num_layers=2, num_heads=4, channels=256), 1, 380, 8),
    (dict(max_seq_len=400, vocab_size=331, num_layers=2, num_heads=16, channels=1024), 3, 390, 3),
    (dict(max_seq_len=400, vocab_size=331, num_layers=2, num_heads=8, channels=512), 7, 391, 3),
    (dict(max_seq_len=700, vocab_size=331, num_layers=2, num_heads=8, channels=512), 7, 637, 6),
    (dict(max_seq_len=400, vocab_size=331, num_layers=2, num_heads=8, channels=512), 13, 391, 3),
    # up to the last position the cache holds
    (dict(max_seq_len=1024, vocab_size=211, num_layers=2, num_heads=4, channels=256), 2, 1012, 12),
    # five and nine sequences (two and three groups of four per phase) at the widest model, and
    # batches beyond the persistent kernel's sixteen, which take one launch per operation
    (dict(max_seq_len=64, vocab_size=331, num_layers=2, num_heads=4, channels=256), 5, 21, 3),
    (dict(max_seq_len=64, vocab_size=331, num_layers=2, num_heads=16, channels=1024), 9, 30, 3),
    (dict(max_seq_len=48, vocab_size=1031, num_layers=2, num_heads=12, channels=768), 17, 20, 3),
    (dict(max_seq_len=48, vocab_size=331, num_layers=2, num_heads=12, channels=768), 64, 30, 3),
    # GPT-2 large's width (1280 channels, 20 heads): one to four groups of four sequences, ranges of
    # positions at a long context
    (dict(max_seq_len=64, vocab_size=331, num_layers=2, num_heads=20, channels=1280), 3, 20, 3),
    (dict(max_seq_len=64, vocab_size=1031, num_layers=3, num_heads=20, channels=1280), 8, 30, 4),
    (dict(max_seq_len=400, vocab_size=331, num_layers=2, num_heads=20, channels=1280), 2, 390, 3),
    (dict(max_seq_len=64, vocab_size=331, num_layers=2, num_heads=20, channels=1280), 9, 20, 2),
    (dict(max_seq_len=64, vocab_size=331, num_layers=2, num_heads=20, channels=1280), 12, 25, 3),
    # (13 sequences of 20 heads are more (sequence, head) pairs than the kernel has workgroups)
    (dict(max_seq_len=64, vocab_size=331, num_layers=2, num_heads=20, channels=1280), 13, 25, 2),
])
def test_gpt2_persistent_decode_matches_the_oracle_and_the_launch_per_operation_path(cfg, B, T0, steps):
    print(f"persistent decode cfg={cfg} B={B} T0={T0} steps={steps}", flush=True)
    params = syn.make_params(91, perturb_affine=True, **cfg)
    ids = syn.make_tokens(92, B, T0 + steps, cfg["vocab_size"])
    exp_logits, _, _ = oracle.gpt2_forward(params, ids, maxT=cfg["max_seq_len"], V=cfg["vocab_size"],
                                           L=cfg["num_layers"], NH=cfg["num_heads"],
                                           C=cfg["channels"], want_lnf=True)
    dids = torch.from_numpy(ids).cuda()
    model = g2.GPT2(**cfg)
    try:
        model.load_params(params)
        runs = {}
        for persistent in (False, True):
            model.decode_options(persistent=persistent)
            model.prefill(dids[:, :T0].contiguous())
            # the path that is meant runs: the persistent kernel takes up to 16 sequences
            assert (model.decode_probe_size() > 0) == (persistent and B <= 16 and B * cfg["num_heads"] <= 256)
            out = []
            for s in range(steps):
                print(f"  persistent={persistent} step {s}", flush=True)
                out.append(model.decode(dids[:, T0 + s].contiguous()).cpu().numpy())
            runs[persistent] = np.stack(out)
            assert model.cache_length() == T0 + steps
        for s in range(steps):
            d = np.abs(runs[True][s] - exp_logits[:, T0 + s]).max()
            dd = np.abs(runs[True][s] - runs[False][s]).max()
            print(f"  step {s}: max|dlogits| vs oracle {d:.3e}, vs per-launch path {dd:.3e}", flush=True)
            assert np.isfinite(runs[True][s]).all()
            assert d <= LOGIT_TOL
            assert np.array_equal(runs[True][s].argmax(-1), exp_logits[:, T0 + s].argmax(-1))
    finally:
        model.close()

@pytest.mark.parametrize("persistent", [True, False])
def test_gpt2_greedy_generation_equals_greedy_decoding_by_full_forward_passes(persistent):
    """Prefill + argmax + decode steps, chained on the device, against the same continuation
    produced the slow way: a full forward pass over the growing sequences for every token."""
    cfg = dict(max_seq_len=64, vocab_size=331, num_layers=2, num_heads=4, channels=256)
    B, T0, steps = 3, 9, 12
    print(f"greedy generation persistent={persistent}", flush=True)
    params = syn.make_params(95, perturb_affine=True, **cfg)
    prompt = torch.from_numpy(syn.make_tokens(96, B, T0, cfg["vocab_size"])).cuda()
    model = g2.GPT2(**cfg)
    try:
        model.load_params(params)
        model.decode_options(persistent=persistent)
        got = model.generate_greedy(prompt, steps)
        seq = prompt.clone()
        for s in range(steps):
            nxt = model.forward_argmax(seq)[:, -1:].contiguous()
            seq = torch.cat([seq, nxt], dim=1).contiguous()
        want = seq[:, T0:]
        assert torch.equal(got, want), (got.cpu(), want.cpu())
    finally:
        model.close()


def test_gpt2_persistent_decode_gives_up_a_barrier_wait_cleanly():
    """Failure handling of the persistent kernel's grid barrier, forced from the host: with a
    spin limit of 0 the first workgroup that has to wait gives up and every workgroup leaves the
    kernel.  Steps are queued WITHOUT synchronisation, as generate_greedy queues them: none of
    them may pass stale logits off as its own (they are NaN), the failure is reported by the
    first call that can know of it, the cache is rolled back to the failed position, and the
    model carries on from there with one launch per operation."""
    cfg = dict(max_seq_len=32, vocab_size=211, num_layers=2, num_heads=4, channels=256)
    params = syn.make_params(93, perturb_affine=True, **cfg)
    ids = torch.from_numpy(syn.make_tokens(94, 2, 12, cfg["vocab_size"])).cuda()
    model = g2.GPT2(**cfg)
    try:
        model.load_params(params)
        model.decode_options(persistent=False)
        model.prefill(ids[:, :7].contiguous())
        want7 = model.decode(ids[:, 7].contiguous()).clone()
        want8 = model.decode(ids[:, 8].contiguous()).clone()
        model.decode_options(persistent=True, spin_limit=0)
        stale = model.prefill(ids[:, :7].contiguous()).clone()   # finite logits of position 6
        print("  three steps with spin limit 0, queued without synchronisation", flush=True)
        seen = []
        try:
            for t in (7, 8, 9):                                   # the first one gives up on the device
                seen.append(model.decode(ids[:, t].contiguous()).clone())
        except g2.GPT2HipError as e:                              # allowed: the host already knew
            assert "grid barrier" in str(e)
        with_error = False
        try:
            model.decode_sync()
        except g2.GPT2HipError as e:
            assert "grid barrier" in str(e) and "position 7" in str(e)
            with_error = True
        torch.cuda.synchronize()
        assert with_error or len(seen) < 3, "the failure was never reported"
        for lg in seen:                                           # never finite stale values
            assert torch.isnan(lg).any() and not torch.equal(lg, stale)
        assert model.cache_length() == 7                          # rolled back to the failed step
        print("  resumed from the rolled-back cache, one launch per operation", flush=True)
        got7 = model.decode(ids[:, 7].contiguous()).clone()
        got8 = model.decode(ids[:, 8].contiguous()).clone()
        model.decode_sync()
        assert (got7 - want7).abs().max().item() <= 1e-4
        assert (got8 - want8).abs().max().item() <= 1e-4
        # asking for the persistent kernel again brings it back, after a new prompt or not
        model.decode_options(persistent=True)
        model.prefill(ids[:, :7].contiguous())
        got = model.decode(ids[:, 7].contiguous())
        model.decode_sync()
        assert (got - want7).abs().max().item() <= 1e-4
        assert g2.lib().gpt2_decode_probe_size(model._h) > 0      # ... and it is the persistent kernel
        # a failure nobody asked about does not outlive the next prompt, and the prompt's own
        # call succeeds without a stale message
        model.decode_options(persistent=True, spin_limit=0)
        model.decode(ids[:, 8].contiguous())
        model.prefill(ids[:, :7].contiguous())
        assert g2.lib().gpt2hip_last_error() == b""
        model.decode_options(persistent=True)
        assert g2.lib().gpt2_decode_probe_size(model._h) > 0
        got = model.decode(ids[:, 7].contiguous())
        model.decode_sync()
        assert (got - want7).abs().max().item() <= 1e-4
        # gpt2_decode_options settles a failure that is still pending (and reports it) before it
        # re-enables the persistent kernel, so that the request is not undone behind its back
        model.decode_options(persistent=True, spin_limit=0)
        model.decode(ids[:, 8].contiguous())
        with pytest.raises(g2.GPT2HipError, match="grid barrier"):
            model.decode_options(persistent=True)
        assert model.cache_length() == 8
        assert g2.lib().gpt2_decode_probe_size(model._h) > 0      # the options were applied all the same
        got8b = model.decode(ids[:, 8].contiguous())
        model.decode_sync()
        assert (got8b - want8).abs().max().item() <= 1e-4
    finally:
        model.close()


def test_gpt2_decode_probe_clocks_are_ordered():
    cfg = dict(max_seq_len=32, vocab_size=211, num_layers=2, num_heads=4, channels=256)
    model = g2.GPT2(**cfg)
    try:
        model.load_params(syn.make_params(95, **cfg))
        ids = torch.from_numpy(syn.make_tokens(96, 3, 6, cfg["vocab_size"])).cuda()
        model.prefill(ids[:, :5].contiguous())
        ref = model.decode(ids[:, 5].contiguous()).clone()
        model.prefill(ids[:, :5].contiguous())
        clk = model.decode_probe(ids[:, 5].contiguous()).cpu().numpy()
        torch.cuda.synchronize()
        assert torch.equal(model.step_logits(), ref)           # the probe changes no result
        phases = 5 * cfg["num_layers"] + 1
        assert clk.shape[:2] == (phases, 2)
        done, passed = clk[:, 0, :], clk[:-1, 1, :]
        assert (done > 0).all() and (passed > 0).all()
        assert (passed >= done[:-1]).all()                      # a barrier is passed after arriving
        assert (passed.min(axis=1) >= done[:-1].max(axis=1)).all()   # ... and after EVERYBODY arrived
        assert (done[1:] >= passed).all()
        # a model the persistent kernel does not take
        small = g2.GPT2(max_seq_len=16, vocab_size=50, num_layers=1, num_heads=1, channels=64)
        try:
            small.load_params(syn.make_params(97, max_seq_len=16, vocab_size=50, num_layers=1, num_heads=1,
                                              channels=64))
            small.prefill(torch.zeros(1, 3, dtype=torch.int32, device="cuda"))
            with pytest.raises(g2.GPT2HipError):
                small.decode_probe(torch.zeros(1, dtype=torch.int32, device="cuda"))
        finally:
            small.close()
    finally:
        model.close()


def test_cpp_driver_calling_the_launchers_equals_gpt2_forward():
    """The plain-C++ llm.c-style driver (examples/llmc_style_driver.cpp, built by build()): its
    layer-by-layer launcher calls must give the logits of the library's own gpt2_forward bit
    for bit, and the _status forms must report errors instead of aborting."""
    import subprocess
    assert os.path.exists(g2.EXAMPLE_BIN), "build() compiles the example driver"
    # second run: prompts long enough for gpt2_forward to add the residual stream in the
    # projections' epilogues, while the example keeps fused_residual_layernorm_forward
    for extra in ([], ["long"]):
        print("running", g2.EXAMPLE_BIN, *extra, flush=True)
        proc = subprocess.run([g2.EXAMPLE_BIN, *extra], capture_output=True, text=True, timeout=100)
        print(proc.stdout, proc.stderr, flush=True)
        assert proc.returncode == 0
        assert "max|launchers - gpt2_forward|=0 " in proc.stdout
        assert f"sums_in_matmul={len(extra)}" in proc.stdout


def test_gpt2_decode_error_paths():
    cfg = dict(max_seq_len=8, vocab_size=50, num_layers=1, num_heads=1, channels=64)
    model = g2.GPT2(**cfg)
    try:
        model.load_params(syn.make_params(83, **cfg))
        tok = torch.zeros(2, dtype=torch.int32, device="cuda")
        assert g2.lib().gpt2_decode_status(model._h, tok.data_ptr()) == 1      # nothing prefilled
        model.prefill(torch.from_numpy(syn.make_tokens(84, 2, 7, 50)).cuda())
        model.decode(tok)                                                       # position 7: the last
        assert model.cache_length() == 8
        with pytest.raises(g2.GPT2HipError, match="full"):
            model.decode(tok)
    finally:
        model.close()


def test_gpt2_rejects_bad_inputs():
    model = g2.GPT2(max_seq_len=16, vocab_size=50, num_layers=1, num_heads=1, channels=64)
    try:
        with pytest.raises(g2.GPT2HipError):
            model.forward(np.zeros((1, 17), np.int32))          # T > max_seq_len
        with pytest.raises(g2.GPT2HipError):
            model.forward(np.full((1, 4), 50, np.int32))        # token id out of range
        with pytest.raises(g2.GPT2HipError):
            model.load_params(np.zeros(3, np.float32))          # wrong parameter count
    finally:
        model.close()


def test_gpt2_forward_is_deterministic_and_reusable():
    cfg = dict(max_seq_len=64, vocab_size=211, num_layers=2, num_heads=2, channels=128)
    params = syn.make_params(3, **cfg)
    model = g2.GPT2(**cfg)
    try:
        model.load_params(params)
        ids = syn.make_tokens(4, 2, 64, 211)
        model.forward(ids)
        a = model.logits().clone()
        model.forward(syn.make_tokens(5, 1, 10, 211))   # smaller shape in between
        model.forward(ids)
        assert torch.equal(a, model.logits())
    finally:
        model.close()
