"""Persistent decode-step kernel against the CPU oracle and against one launch per operation."""
import importlib

import numpy as np
import pytest
import torch

import oracle

g2 = importlib.import_module("cuda-gpt2-inference_amd")
syn = importlib.import_module("cuda-gpt2-inference_amd.synthetic")

pytestmark = pytest.mark.gpu
LOGIT_TOL = 2e-3


@pytest.mark.parametrize("cfg,B,T0,steps", [
    (dict(max_seq_len=48, vocab_size=211, num_layers=2, num_heads=4, channels=256), 3, 5, 6),
    (dict(max_seq_len=300, vocab_size=1031, num_layers=2, num_heads=8, channels=512), 5, 7, 3),
    (dict(max_seq_len=64, vocab_size=331, num_layers=2, num_heads=4, channels=256), 13, 37, 3),
    (dict(max_seq_len=128, vocab_size=3001, num_layers=2, num_heads=16, channels=1024), 4, 100, 3),
    (dict(max_seq_len=300, vocab_size=1031, num_layers=3, num_heads=8, channels=512), 16, 250, 5),
    (dict(max_seq_len=64, vocab_size=50257, num_layers=2, num_heads=12, channels=768), 1, 1, 4),
    (dict(g2.GPT2_124M), 8, 120, 10),
])
def test_persistent_decode_matches_the_oracle_and_the_launch_per_operation_path(cfg, B, T0, steps):
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
