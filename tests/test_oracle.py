"""Pins the CPU oracle (oracle/gpt2_cpu.c) without the reference.

The reference holds no golden vectors for this path, so each oracle function is
checked against what the mathematics fixes: float64 brute force written
independently in numpy, closed forms, invariants and torch's CPU library
routines.  Every check is chosen so that a plausible slip (transposed weight,
dropped bias, off-by-one in the causal mask, wrong scale, population vs sample
variance, missing eps) fails at least one of them.
"""
import math

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import oracle


def rng(seed):
    return np.random.default_rng(seed)


# ---------------------------------------------------------------- encoder
def test_encoder_bruteforce_exact():
    r = rng(0)
    B, T, C, V = 2, 3, 4, 7
    wte = r.standard_normal((V, C)).astype(np.float32)
    wpe = r.standard_normal((T + 2, C)).astype(np.float32)
    ids = r.integers(0, V, (B, T)).astype(np.int32)
    out = oracle.encoder_forward(ids, wte, wpe)
    for b in range(B):
        for t in range(T):
            exp = wte[ids[b, t]] + wpe[t]
            assert np.array_equal(out[b, t], exp)


def test_encoder_position_only_depends_on_t():
    r = rng(1)
    wte = np.zeros((5, 8), np.float32)
    wpe = r.standard_normal((6, 8)).astype(np.float32)
    ids = r.integers(0, 5, (3, 6)).astype(np.int32)
    out = oracle.encoder_forward(ids, wte, wpe)
    assert np.array_equal(out, np.broadcast_to(wpe, (3, 6, 8)))


# ---------------------------------------------------------------- residual
def test_residual_exact():
    r = rng(2)
    a = r.standard_normal(1000).astype(np.float32)
    b = r.standard_normal(1000).astype(np.float32)
    assert np.array_equal(oracle.residual_forward(a, b), a + b)


# ---------------------------------------------------------------- layernorm
@pytest.mark.parametrize("C", [4, 768, 1024])
def test_layernorm_vs_float64_and_torch(C):
    r = rng(3)
    N = 17
    x = (r.standard_normal((N, C)) * 2 + 0.5).astype(np.float32)
    w = (1 + 0.1 * r.standard_normal(C)).astype(np.float32)
    b = (0.1 * r.standard_normal(C)).astype(np.float32)
    out, mean, rstd = oracle.layernorm_forward(x, w, b)
    x64 = x.astype(np.float64)
    m = x64.mean(1)
    v = x64.var(1)  # population variance: ddof=0
    s = 1.0 / np.sqrt(v + 1e-5)
    exp = (x64 - m[:, None]) * s[:, None] * w + b
    assert np.allclose(mean, m, rtol=1e-6, atol=1e-6)
    assert np.allclose(rstd, s, rtol=2e-6)
    assert np.allclose(out, exp, rtol=1e-5, atol=1e-5)
    tout = F.layer_norm(torch.from_numpy(x), (C,), torch.from_numpy(w), torch.from_numpy(b), 1e-5)
    assert np.allclose(out, tout.numpy(), rtol=1e-5, atol=1e-5)


def test_layernorm_constant_row_gives_beta_and_eps_rstd():
    C = 64
    x = np.full((3, C), 2.5, np.float32)
    w = rng(4).standard_normal(C).astype(np.float32)
    b = rng(5).standard_normal(C).astype(np.float32)
    out, mean, rstd = oracle.layernorm_forward(x, w, b)
    assert np.array_equal(mean, np.full(3, 2.5, np.float32))
    assert np.allclose(rstd, 1.0 / math.sqrt(1e-5), rtol=1e-6)
    assert np.array_equal(out, np.broadcast_to(b, (3, C)))


def test_layernorm_unit_affine_moments():
    C = 768
    x = (rng(6).standard_normal((9, C)) * 3 + 1).astype(np.float32)
    out, _, _ = oracle.layernorm_forward(x, np.ones(C, np.float32), np.zeros(C, np.float32))
    assert np.all(np.abs(out.mean(1)) < 1e-5)
    assert np.allclose(out.astype(np.float64).var(1), 1.0, atol=1e-4)


def test_fused_is_residual_then_layernorm_bitwise():
    r = rng(7)
    N, C = 33, 768
    a = r.standard_normal((N, C)).astype(np.float32)
    b = r.standard_normal((N, C)).astype(np.float32)
    w = (1 + 0.1 * r.standard_normal(C)).astype(np.float32)
    bb = (0.1 * r.standard_normal(C)).astype(np.float32)
    res, ln, mean, rstd = oracle.fused_residual_layernorm_forward(a, b, w, bb)
    assert np.array_equal(res, a + b)
    ln2, mean2, rstd2 = oracle.layernorm_forward(a + b, w, bb)
    assert np.array_equal(ln, ln2) and np.array_equal(mean, mean2) and np.array_equal(rstd, rstd2)


# ---------------------------------------------------------------- gelu
def test_gelu_known_answers():
    x = np.array([0.0, 1.0, -1.0, 3.0, -3.0, 20.0, -20.0], np.float32)
    y = oracle.gelu_forward(x)
    assert y[0] == 0.0
    # textbook values of the tanh approximation
    assert abs(y[1] - 0.8411919906082768) < 1e-6
    assert abs(y[2] + 0.15880800939172324) < 1e-6
    assert abs(y[3] - 2.99636) < 1e-4
    assert y[5] == 20.0 and y[6] == 0.0
    # gelu(x) - gelu(-x) = x  (the tanh term is odd)
    xs = rng(8).standard_normal(1000).astype(np.float32) * 3
    d = oracle.gelu_forward(xs) - oracle.gelu_forward(-xs)
    assert np.allclose(d, xs, rtol=1e-6, atol=1e-6)


def test_gelu_vs_torch_tanh():
    xs = (rng(9).standard_normal(4096) * 3).astype(np.float32)
    t = F.gelu(torch.from_numpy(xs), approximate="tanh").numpy()
    assert np.allclose(oracle.gelu_forward(xs), t, rtol=1e-5, atol=1e-6)


# ---------------------------------------------------------------- matmul
@pytest.mark.parametrize("N,C,OC", [(5, 7, 3), (16, 64, 81), (9, 48, 33), (1030, 32, 40)])
def test_matmul_float64_bruteforce(N, C, OC):
    r = rng(10)
    x = r.standard_normal((N, C)).astype(np.float32)
    w = (0.02 * r.standard_normal((OC, C))).astype(np.float32)
    b = (0.02 * r.standard_normal(OC)).astype(np.float32)
    exp = x.astype(np.float64) @ w.astype(np.float64).T + b
    for naive in (True, False):
        out = oracle.matmul_forward(x, w, b, naive=naive)
        assert np.allclose(out, exp, rtol=1e-5, atol=1e-6)
        out_nb = oracle.matmul_forward(x, w, None, naive=naive)
        assert np.allclose(out_nb, exp - b, rtol=1e-5, atol=1e-6)


def test_matmul_identity_weight_returns_input_plus_bias():
    r = rng(11)
    C = 40
    x = r.standard_normal((12, C)).astype(np.float32)
    b = r.standard_normal(C).astype(np.float32)
    out = oracle.matmul_forward(x, np.eye(C, dtype=np.float32), b)
    # bias first, then +0 ... + x*1 + 0 ...: exactly b + x in fp32
    assert np.array_equal(out, b[None, :] + x)


def test_matmul_is_not_transposed():
    # weight is (OC, C): a one-hot weight row o picks input column c
    x = np.arange(12, dtype=np.float32).reshape(3, 4)
    w = np.zeros((2, 4), np.float32)
    w[0, 3] = 1.0
    w[1, 1] = 2.0
    out = oracle.matmul_forward(x, w, None)
    assert np.array_equal(out[:, 0], x[:, 3]) and np.array_equal(out[:, 1], 2 * x[:, 1])


@pytest.mark.parametrize("N,C,OC", [(37, 768, 100), (520, 96, 67)])
def test_matmul_blocked_equals_naive_bitwise(N, C, OC):
    r = rng(12)
    x = r.standard_normal((N, C)).astype(np.float32)
    w = (0.02 * r.standard_normal((OC, C))).astype(np.float32)
    b = (0.02 * r.standard_normal(OC)).astype(np.float32)
    assert np.array_equal(oracle.matmul_forward(x, w, b), oracle.matmul_forward(x, w, b, naive=True))
    assert np.array_equal(oracle.matmul_forward(x, w), oracle.matmul_forward(x, w, naive=True))


def test_matmul_vs_torch_linear():
    r = rng(13)
    x = r.standard_normal((64, 768)).astype(np.float32)
    w = (0.02 * r.standard_normal((96, 768))).astype(np.float32)
    b = (0.02 * r.standard_normal(96)).astype(np.float32)
    t = F.linear(torch.from_numpy(x), torch.from_numpy(w), torch.from_numpy(b)).numpy()
    assert np.allclose(oracle.matmul_forward(x, w, b), t, rtol=1e-4, atol=1e-5)


# ---------------------------------------------------------------- attention
def attention_f64(qkv, NH):
    B, T, C3 = qkv.shape
    C = C3 // 3
    hs = C // NH
    x = qkv.astype(np.float64)
    out = np.zeros((B, T, C))
    for b in range(B):
        for h in range(NH):
            q = x[b, :, h * hs:(h + 1) * hs]
            k = x[b, :, C + h * hs:C + (h + 1) * hs]
            v = x[b, :, 2 * C + h * hs:2 * C + (h + 1) * hs]
            s = q @ k.T / math.sqrt(hs)
            s = np.where(np.tril(np.ones((T, T), bool)), s, -np.inf)
            p = np.exp(s - s.max(1, keepdims=True))
            p /= p.sum(1, keepdims=True)
            out[b, :, h * hs:(h + 1) * hs] = p @ v
    return out


@pytest.mark.parametrize("B,T,NH,hs", [(1, 8, 2, 4), (2, 33, 3, 16), (1, 70, 2, 64)])
def test_attention_float64_bruteforce(B, T, NH, hs):
    qkv = rng(14).standard_normal((B, T, 3 * NH * hs)).astype(np.float32)
    out = oracle.attention_forward(qkv, NH)
    assert np.allclose(out, attention_f64(qkv, NH), rtol=1e-5, atol=1e-6)


def test_attention_T1_returns_v():
    NH, hs = 3, 8
    C = NH * hs
    qkv = rng(15).standard_normal((4, 1, 3 * C)).astype(np.float32)
    out = oracle.attention_forward(qkv, NH)
    assert np.array_equal(out[:, 0], qkv[:, 0, 2 * C:])


def test_attention_zero_query_gives_running_mean_of_v():
    NH, hs, T = 2, 8, 16
    C = NH * hs
    qkv = rng(16).standard_normal((1, T, 3 * C)).astype(np.float32)
    qkv[:, :, :C] = 0.0
    out = oracle.attention_forward(qkv, NH)
    v = qkv[0, :, 2 * C:].astype(np.float64)
    exp = np.cumsum(v, 0) / np.arange(1, T + 1)[:, None]
    assert np.allclose(out[0], exp, rtol=1e-5, atol=1e-6)


def test_attention_is_causal_bitwise():
    NH, hs, T = 2, 8, 12
    C = NH * hs
    qkv = rng(17).standard_normal((1, T, 3 * C)).astype(np.float32)
    out = oracle.attention_forward(qkv, NH)
    qkv2 = qkv.copy()
    qkv2[0, 7:] += 5.0
    out2 = oracle.attention_forward(qkv2, NH)
    assert np.array_equal(out[0, :7], out2[0, :7])
    assert not np.array_equal(out[0, 7:], out2[0, 7:])


def test_attention_heads_are_independent():
    NH, hs, T = 3, 4, 6
    C = NH * hs
    qkv = rng(18).standard_normal((1, T, 3 * C)).astype(np.float32)
    out = oracle.attention_forward(qkv, NH)
    qkv2 = qkv.copy()
    qkv2[..., C + hs:C + 2 * hs] *= -2.0  # keys of head 1 only
    out2 = oracle.attention_forward(qkv2, NH)
    assert np.array_equal(out[..., :hs], out2[..., :hs])
    assert np.array_equal(out[..., 2 * hs:], out2[..., 2 * hs:])
    assert not np.array_equal(out[..., hs:2 * hs], out2[..., hs:2 * hs])


def test_attention_vs_torch_sdpa():
    B, T, NH, hs = 2, 40, 4, 64
    C = NH * hs
    qkv = rng(19).standard_normal((B, T, 3 * C)).astype(np.float32)
    t = torch.from_numpy(qkv)
    q, k, v = (t[..., i * C:(i + 1) * C].view(B, T, NH, hs).transpose(1, 2) for i in range(3))
    ref = F.scaled_dot_product_attention(q, k, v, is_causal=True).transpose(1, 2).reshape(B, T, C)
    assert np.allclose(oracle.attention_forward(qkv, NH), ref.numpy(), rtol=1e-4, atol=1e-5)


# ---------------------------------------------------------------- argmax
def test_argmax_lowest_index_wins_ties():
    x = np.array([[1, 5, 5, 2], [7, 7, 7, 7], [-3, -1, -2, -1]], np.float32)
    assert oracle.argmax_forward(x).tolist() == [1, 0, 1]
    r = rng(20).standard_normal((50, 997)).astype(np.float32)
    assert np.array_equal(oracle.argmax_forward(r), r.argmax(1).astype(np.int32))


# ---------------------------------------------------------------- gpt2
def gpt2_f64(params, ids, maxT, V, L, NH, C):
    """Independent float64 GPT-2 forward in numpy (pre-LN, tied lm-head)."""
    sizes = [V * C, maxT * C, L * C, L * C, L * 3 * C * C, L * 3 * C, L * C * C, L * C, L * C, L * C,
             L * 4 * C * C, L * 4 * C, L * 4 * C * C, L * C, C, C]
    off = np.concatenate([[0], np.cumsum(sizes)])
    p = [params[off[i]:off[i + 1]].astype(np.float64) for i in range(16)]
    wte, wpe = p[0].reshape(V, C), p[1].reshape(maxT, C)
    B, T = ids.shape

    def ln(x, w, b):
        m = x.mean(-1, keepdims=True)
        v = x.var(-1, keepdims=True)
        return (x - m) / np.sqrt(v + 1e-5) * w + b

    x = wte[ids] + wpe[:T]
    for l in range(L):
        h = ln(x, p[2].reshape(L, C)[l], p[3].reshape(L, C)[l])
        qkv = h @ p[4].reshape(L, 3 * C, C)[l].T + p[5].reshape(L, 3 * C)[l]
        a = attention_f64(qkv, NH)
        x = x + a @ p[6].reshape(L, C, C)[l].T + p[7].reshape(L, C)[l]
        h = ln(x, p[8].reshape(L, C)[l], p[9].reshape(L, C)[l])
        f = h @ p[10].reshape(L, 4 * C, C)[l].T + p[11].reshape(L, 4 * C)[l]
        f = 0.5 * f * (1 + np.tanh(math.sqrt(2 / math.pi) * (f + 0.044715 * f ** 3)))
        x = x + f @ p[12].reshape(L, C, 4 * C)[l].T + p[13].reshape(L, C)[l]
    x = ln(x, p[14], p[15])
    return x @ wte.T, x


def test_gpt2_forward_tiny_float64():
    maxT, V, L, NH, C = 16, 97, 2, 2, 32
    n = oracle.num_parameters(maxT, V, L, C)
    r = rng(21)
    params = (0.2 * r.standard_normal(n)).astype(np.float32)
    ids = r.integers(0, V, (2, 8)).astype(np.int32)
    logits, am, lnf = oracle.gpt2_forward(params, ids, maxT=maxT, V=V, L=L, NH=NH, C=C,
                                          want_lnf=True)
    exp, exp_lnf = gpt2_f64(params, ids, maxT, V, L, NH, C)
    assert np.allclose(lnf, exp_lnf, rtol=1e-4, atol=1e-4)
    assert np.allclose(logits, exp, rtol=1e-4, atol=1e-4)
    assert np.array_equal(am, logits.argmax(-1))


def test_gpt2_forward_against_committed_float64_fixture():
    from golden import load_gpt2_tiny
    cfg, params, ids, exp_logits, exp_lnf = load_gpt2_tiny()
    logits, am, lnf = oracle.gpt2_forward(params, ids, maxT=cfg["max_seq_len"], V=cfg["vocab_size"],
                                          L=cfg["num_layers"], NH=cfg["num_heads"],
                                          C=cfg["channels"], want_lnf=True)
    assert np.abs(lnf - exp_lnf).max() < 2e-5
    assert np.abs(logits - exp_logits).max() < 2e-5
    top2 = np.sort(exp_logits, -1)[..., -2:]
    clear = (top2[..., 1] - top2[..., 0]) > 1e-4
    assert np.array_equal(am[clear], exp_logits.argmax(-1)[clear])


def test_param_count_124M():
    assert oracle.num_parameters(1024, 50257, 12, 768) == 124_439_808
    assert oracle.num_parameters(1024, 50257, 24, 1024) == 354_823_168
