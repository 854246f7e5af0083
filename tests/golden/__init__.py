"""Loader for the committed golden fixtures (data only; see make_golden.py)."""
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))


def load_gpt2_tiny():
    """Returns (config dict, fp32 params, int32 ids (B,T), float64 logits, float64 lnf)."""
    z = np.load(os.path.join(_HERE, "gpt2_tiny_f64.npz"))
    maxT, V, L, NH, C = (int(v) for v in z["config"])
    cfg = dict(max_seq_len=maxT, vocab_size=V, num_layers=L, num_heads=NH, channels=C)
    sizes = [V * C, maxT * C, L * C, L * C, L * 3 * C * C, L * 3 * C, L * C * C, L * C, L * C, L * C,
             L * 4 * C * C, L * 4 * C, L * 4 * C * C, L * C, C, C]
    off = np.concatenate([[0], np.cumsum(sizes)])
    p = z["params_q"].astype(np.float32) / np.float32(256)
    for gain in (2, 8, 14):                       # layernorm gains are stored as (gain - 1)
        p[off[gain]:off[gain + 1]] += np.float32(1)
    return cfg, p, z["ids"], z["logits"], z["lnf"]
