"""Writes tests/golden/gpt2_tiny_f64.npz: a small GPT-2 forward evaluated in float64.

The reference holds no golden vectors and cannot be built or run offline, so this
fixture comes from an independent float64 numpy evaluation of the same network
(pre-layernorm blocks, tanh GELU, causal softmax attention, tied lm-head, llm.c
parameter order: reference README.md and llm.c's train_gpt2.c gpt2_forward).  It shares
no code with the C oracle or with the HIP kernels; both are tested against it.

Parameters are stored as int8 and mean int8 / 256 (layernorm gains: 1 + int8 / 256),
exactly representable in fp32.  Run from the repository root:
    python tests/golden/make_golden.py
"""
import math
import os

import numpy as np

CFG = dict(max_seq_len=32, vocab_size=97, num_layers=2, num_heads=1, channels=64)
B, T = 2, 24


def sizes(maxT, V, L, C):
    return [V * C, maxT * C, L * C, L * C, L * 3 * C * C, L * 3 * C, L * C * C, L * C, L * C, L * C,
            L * 4 * C * C, L * 4 * C, L * 4 * C * C, L * C, C, C]


def decode_params(q: np.ndarray) -> np.ndarray:
    """int8 fixture -> fp32 parameter buffer (gains of the three layernorms are 1 + q/256)."""
    maxT, V, L, C = CFG["max_seq_len"], CFG["vocab_size"], CFG["num_layers"], CFG["channels"]
    off = np.concatenate([[0], np.cumsum(sizes(maxT, V, L, C))])
    p = q.astype(np.float32) / np.float32(256)
    for gain in (2, 8, 14):
        p[off[gain]:off[gain + 1]] += np.float32(1)
    return p


def forward_f64(params, ids):
    maxT, V, L, C = CFG["max_seq_len"], CFG["vocab_size"], CFG["num_layers"], CFG["channels"]
    NH = CFG["num_heads"]
    hs = C // NH
    off = np.concatenate([[0], np.cumsum(sizes(maxT, V, L, C))])
    p = [params[off[i]:off[i + 1]].astype(np.float64) for i in range(16)]
    wte, wpe = p[0].reshape(V, C), p[1].reshape(maxT, C)
    nb, nt = ids.shape

    def ln(x, w, b):
        m = x.mean(-1, keepdims=True)
        v = ((x - m) ** 2).mean(-1, keepdims=True)
        return (x - m) / np.sqrt(v + 1e-5) * w + b

    x = wte[ids] + wpe[:nt]
    mask = np.tril(np.ones((nt, nt), bool))
    for l in range(L):
        h = ln(x, p[2].reshape(L, C)[l], p[3].reshape(L, C)[l])
        qkv = h @ p[4].reshape(L, 3 * C, C)[l].T + p[5].reshape(L, 3 * C)[l]
        q, k, v = (qkv[..., i * C:(i + 1) * C].reshape(nb, nt, NH, hs).transpose(0, 2, 1, 3)
                   for i in range(3))
        s = q @ k.transpose(0, 1, 3, 2) / math.sqrt(hs)
        s = np.where(mask, s, -np.inf)
        s = np.exp(s - s.max(-1, keepdims=True))
        a = (s / s.sum(-1, keepdims=True)) @ v
        a = a.transpose(0, 2, 1, 3).reshape(nb, nt, C)
        x = x + a @ p[6].reshape(L, C, C)[l].T + p[7].reshape(L, C)[l]
        h = ln(x, p[8].reshape(L, C)[l], p[9].reshape(L, C)[l])
        f = h @ p[10].reshape(L, 4 * C, C)[l].T + p[11].reshape(L, 4 * C)[l]
        f = 0.5 * f * (1 + np.tanh(math.sqrt(2 / math.pi) * (f + 0.044715 * f ** 3)))
        x = x + f @ p[12].reshape(L, C, 4 * C)[l].T + p[13].reshape(L, C)[l]
    x = ln(x, p[14], p[15])
    return x @ wte.T, x


def main():
    maxT, V, L, C = CFG["max_seq_len"], CFG["vocab_size"], CFG["num_layers"], CFG["channels"]
    rng = np.random.default_rng(20240326)
    n = sum(sizes(maxT, V, L, C))
    q = np.clip(np.rint(rng.standard_normal(n) * 20), -127, 127).astype(np.int8)
    ids = rng.integers(0, V, (B, T)).astype(np.int32)
    logits, lnf = forward_f64(decode_params(q), ids)
    path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "gpt2_tiny_f64.npz")
    np.savez_compressed(path, params_q=q, ids=ids, logits=logits, lnf=lnf,
                        config=np.array([maxT, V, L, CFG["num_heads"], C], np.int32))
    print(path, os.path.getsize(path), "bytes; |logits| max", np.abs(logits).max())


if __name__ == "__main__":
    main()
