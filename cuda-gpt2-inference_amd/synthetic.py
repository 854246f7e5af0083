"""Seeded synthetic GPT-2 parameters and token ids (host side, numpy).

There are no checkpoints offline, so weights follow GPT-2's initialisation:
N(0, 0.02) for wte / qkvw / fcw, the two residual projections scaled by
1/sqrt(2L), wpe N(0, 0.01), layernorm gamma 1 / beta 0, biases 0.  The flat
buffer is in llm.c checkpoint order (the order gpt2_params_device() documents).
"""
from __future__ import annotations

import math

import numpy as np

PARAM_NAMES = ("wte", "wpe", "ln1w", "ln1b", "qkvw", "qkvb", "attprojw", "attprojb", "ln2w",
               "ln2b", "fcw", "fcb", "fcprojw", "fcprojb", "lnfw", "lnfb")


def param_shapes(*, max_seq_len, vocab_size, num_layers, num_heads, channels):
    V, maxT, L, C = vocab_size, max_seq_len, num_layers, channels
    return {
        "wte": (V, C), "wpe": (maxT, C), "ln1w": (L, C), "ln1b": (L, C),
        "qkvw": (L, 3 * C, C), "qkvb": (L, 3 * C), "attprojw": (L, C, C), "attprojb": (L, C),
        "ln2w": (L, C), "ln2b": (L, C), "fcw": (L, 4 * C, C), "fcb": (L, 4 * C),
        "fcprojw": (L, C, 4 * C), "fcprojb": (L, C), "lnfw": (C,), "lnfb": (C,),
    }


def make_params(seed: int, *, perturb_affine: bool = False, **config) -> np.ndarray:
    """Flat float32 parameter buffer.  perturb_affine also randomises the
    layernorm affine terms and the biases (so tests exercise them)."""
    shapes = param_shapes(**config)
    L = config["num_layers"]
    rng = np.random.default_rng(seed)
    total = sum(int(np.prod(s)) for s in shapes.values())
    flat = np.empty(total, np.float32)
    off = 0
    for name in PARAM_NAMES:
        n = int(np.prod(shapes[name]))
        dst = flat[off:off + n]
        if name in ("wte", "qkvw", "fcw"):
            dst[:] = rng.standard_normal(n, dtype=np.float32) * np.float32(0.02)
        elif name in ("attprojw", "fcprojw"):
            dst[:] = rng.standard_normal(n, dtype=np.float32) * np.float32(0.02 / math.sqrt(2 * L))
        elif name == "wpe":
            dst[:] = rng.standard_normal(n, dtype=np.float32) * np.float32(0.01)
        elif name in ("ln1w", "ln2w", "lnfw"):
            dst[:] = 1.0
            if perturb_affine:
                dst += rng.standard_normal(n, dtype=np.float32) * np.float32(0.1)
        else:  # layernorm betas and linear biases
            dst[:] = 0.0
            if perturb_affine:
                dst += rng.standard_normal(n, dtype=np.float32) * np.float32(0.02)
        off += n
    return flat


def make_tokens(seed: int, B: int, T: int, vocab_size: int) -> np.ndarray:
    rng = np.random.default_rng(seed)
    return rng.integers(0, vocab_size, (B, T), dtype=np.int32)


def write_llmc_checkpoint(path, flat_params: np.ndarray, *, version: int = 3, pad_to: int = 128,
                          pad_value: float = 7.5, **config) -> None:
    """Write parameters as an llm.c checkpoint file: 256 int32 header words, then the
    tensors.  Versions 3 (fp32) and 5 (bf16: the upper 16 bits of each fp32, so pass
    parameters that are bf16-representable) pad wte's rows to a multiple of pad_to (filled
    with pad_value, which a correct loader must never let through); version 1 (fp32) does
    not pad."""
    V, C = config["vocab_size"], config["channels"]
    Vp = -(-V // pad_to) * pad_to if version in (3, 5) else V
    header = np.zeros(256, np.int32)
    header[:7] = [20240326, version, config["max_seq_len"], V, config["num_layers"],
                  config["num_heads"], C]
    if version in (3, 5):
        header[7] = Vp

    def stored(a):
        a = np.ascontiguousarray(a, np.float32)
        if version == 5:
            return (a.view(np.uint32) >> 16).astype(np.uint16).tobytes()
        return a.tobytes()

    with open(path, "wb") as f:
        f.write(header.tobytes())
        f.write(stored(flat_params[:V * C]))
        if Vp > V:
            f.write(stored(np.full((Vp - V) * C, pad_value, np.float32)))
        f.write(stored(flat_params[V * C:]))


def round_to_bf16(a: np.ndarray) -> np.ndarray:
    """fp32 values rounded to the nearest bf16 (ties to even), returned as fp32."""
    bits = np.ascontiguousarray(a, np.float32).view(np.uint32).astype(np.uint64)
    bits = (bits + 0x7FFF + ((bits >> 16) & 1)) & 0xFFFF0000
    return bits.astype(np.uint32).view(np.float32)
