"""matmul_forward_argmax_noalloc_status: the lm-head + argmax entry point that allocates
nothing (its pairs live in a static device array inside the library), called through the C
ABI and checked bit for bit against matmul_forward_argmax_status, which takes a caller's
workspace.  Collected last on purpose (file name): a failure here hides no other test."""
import importlib

import numpy as np
import pytest

torch = pytest.importorskip("torch")
g2 = importlib.import_module("cuda-gpt2-inference_amd")

pytestmark = pytest.mark.gpu


def _inputs(M, C, OC, seed, bias=True):
    rng = np.random.default_rng(seed)
    x = torch.from_numpy(rng.standard_normal((M, C), dtype=np.float32)).cuda()
    w = torch.from_numpy(rng.standard_normal((OC, C), dtype=np.float32) * np.float32(0.02)).cuda()
    b = torch.from_numpy(rng.standard_normal(OC, dtype=np.float32) * np.float32(0.02)).cuda() \
        if bias else None
    return x, w, b


def _with_workspace(x, w, b, M, C, OC):
    L = g2.lib()
    need = L.matmul_forward_argmax_workspace(1, M, OC)
    ws = torch.empty(max(need, 1), dtype=torch.uint8, device="cuda")
    ids = torch.full((M,), -1, dtype=torch.int32, device="cuda")
    rc = L.matmul_forward_argmax_status(ids.data_ptr(), ws.data_ptr(), ws.numel(), x.data_ptr(),
                                        w.data_ptr(), b.data_ptr() if b is not None else None,
                                        1, M, C, OC)
    assert rc == 0, L.gpt2hip_last_error()
    return ids


def _noalloc(x, w, b, M, C, OC):
    L = g2.lib()
    ids = torch.full((M + 64,), -7, dtype=torch.int32, device="cuda")  # guard band behind the ids
    rc = L.matmul_forward_argmax_noalloc_status(ids.data_ptr(), x.data_ptr(), w.data_ptr(),
                                                b.data_ptr() if b is not None else None,
                                                1, M, C, OC)
    assert rc == 0, L.gpt2hip_last_error()
    torch.cuda.synchronize()
    assert (ids[M:] == -7).all()
    return ids[:M]


def test_two_calls_in_a_row_the_second_smaller():
    # first call: many pairs per row (the scratch array is left full of them);
    # second call: fewer rows and fewer pairs per row, which must not see the leftovers
    print("no-alloc argmax: M=1000 C=256 OC=5000, then M=130 C=64 OC=700", flush=True)
    big = _inputs(1000, 256, 5000, 201)
    small = _inputs(130, 64, 700, 202, bias=False)
    want_big = _with_workspace(*big, 1000, 256, 5000)
    want_small = _with_workspace(*small, 130, 64, 700)
    got_big = _noalloc(*big, 1000, 256, 5000)
    got_small = _noalloc(*small, 130, 64, 700)
    assert torch.equal(got_big, want_big)
    assert torch.equal(got_small, want_small)
    # and the oracle's maximum is where the ids point (tolerance of the matmul test)
    import oracle
    x, w, _ = small
    exp = oracle.matmul_forward(x.cpu().numpy(), w.cpu().numpy(), None)
    chosen = exp[np.arange(130), got_small.cpu().numpy()]
    assert (exp.max(-1) - chosen <= 1e-5 + 1e-4 * np.abs(exp.max(-1))).all()


def test_lm_head_shape_at_the_limit_and_beyond():
    print("no-alloc argmax: M=8192 C=768 OC=50257 (the limit), then M=8320 (rejected)", flush=True)
    L = g2.lib()
    M, C, OC = 8192, 768, 50257
    assert L.matmul_forward_argmax_workspace(1, M, OC) <= g2.ARGMAX_NOALLOC_BYTES
    x, w, _ = _inputs(M, C, OC, 203, bias=False)
    want = _with_workspace(x, w, None, M, C, OC)
    got = _noalloc(x, w, None, M, C, OC)
    assert torch.equal(got, want)
    # a smaller call right after the largest one
    got2 = _noalloc(x[:300], w[:1000], None, 300, C, 1000)
    assert torch.equal(got2, _with_workspace(x[:300], w[:1000], None, 300, C, 1000))
    ids = torch.zeros(8320, dtype=torch.int32, device="cuda")
    xx = torch.zeros((8320, C), device="cuda")
    rc = L.matmul_forward_argmax_noalloc_status(ids.data_ptr(), xx.data_ptr(), w.data_ptr(), None,
                                                1, 8320, C, OC)
    assert rc == 1 and b"static scratch array holds" in L.gpt2hip_last_error()


def test_generic_path_and_empty_input_need_no_scratch():
    print("no-alloc argmax: C=36 (generic kernel), M=0", flush=True)
    x, w, b = _inputs(50, 36, 90, 204)
    assert torch.equal(_noalloc(x, w, b, 50, 36, 90), _with_workspace(x, w, b, 50, 36, 90))
    L = g2.lib()
    assert L.matmul_forward_argmax_noalloc_status(None, None, None, None, 0, 5, 32, 64) == 0
