"""llm.c checkpoint files: header parsing (CPU) and loading (GPU).

Most files are written by the package's own synthetic.write_llmc_checkpoint (256 int32
header words, tensors in checkpoint order, wte rows padded in versions 3 and 5); the
"literal layout" tests at the end build a file byte by byte from offsets written in this
file, so that the loader is also checked against a layout it shares no code with.  No file
produced by llm.c itself is available offline: agreement with one is not pinned.
"""
import importlib

import numpy as np
import pytest

g2 = importlib.import_module("cuda-gpt2-inference_amd")
syn = importlib.import_module("cuda-gpt2-inference_amd.synthetic")

CFG = dict(max_seq_len=32, vocab_size=331, num_layers=2, num_heads=2, channels=128)


@pytest.mark.parametrize("version", [1, 3, 5])
def test_header_roundtrip(tmp_path, version):
    params = syn.make_params(5, **CFG)
    path = tmp_path / f"v{version}.bin"
    syn.write_llmc_checkpoint(path, params, version=version, **CFG)
    assert g2.read_checkpoint_config(path) == CFG
    pad_rows = (-CFG["vocab_size"]) % 128 if version != 1 else 0
    elem = 2 if version == 5 else 4
    assert path.stat().st_size == 1024 + elem * (params.size + pad_rows * CFG["channels"])


def test_header_rejections(tmp_path):
    params = syn.make_params(5, **CFG)
    good = tmp_path / "good.bin"
    syn.write_llmc_checkpoint(good, params, **CFG)
    raw = bytearray(good.read_bytes())

    def variant(name, word, value):
        b = bytearray(raw)
        b[4 * word:4 * word + 4] = np.int32(value).tobytes()
        p = tmp_path / name
        p.write_bytes(bytes(b))
        return p

    with pytest.raises(g2.GPT2HipError, match="bad magic"):
        g2.read_checkpoint_config(variant("magic.bin", 0, 1234))
    with pytest.raises(g2.GPT2HipError, match="version 4"):
        g2.read_checkpoint_config(variant("v4.bin", 1, 4))
    with pytest.raises(g2.GPT2HipError, match="implausible"):
        g2.read_checkpoint_config(variant("heads.bin", 5, 3))      # C % NH != 0
    with pytest.raises(g2.GPT2HipError, match="implausible"):
        g2.read_checkpoint_config(variant("vp.bin", 7, 10))        # padded V < V
    short = tmp_path / "short.bin"
    short.write_bytes(bytes(raw[:100]))
    with pytest.raises(g2.GPT2HipError, match="shorter than"):
        g2.read_checkpoint_config(short)
    with pytest.raises(g2.GPT2HipError, match="cannot open"):
        g2.read_checkpoint_config(tmp_path / "missing.bin")


@pytest.mark.gpu
@pytest.mark.parametrize("version", [1, 3, 5])
def test_checkpoint_model_equals_directly_loaded_model(tmp_path, version):
    import torch
    params = syn.make_params(6, perturb_affine=True, **CFG)
    if version == 5:  # a bf16 file: its parameters widen to fp32 exactly
        params = syn.round_to_bf16(params)
    path = tmp_path / "model.bin"
    syn.write_llmc_checkpoint(path, params, version=version, **CFG)
    ids = syn.make_tokens(7, 2, 32, CFG["vocab_size"])
    a = g2.GPT2.from_checkpoint(path)
    b = g2.GPT2(**CFG)
    try:
        assert a.num_parameters == params.size
        # the pad rows of wte (7.5 everywhere) must not have reached the device
        assert np.array_equal(a.params_tensor().cpu().numpy(), params)
        b.load_params(params)
        a.forward(ids)
        b.forward(ids)
        torch.cuda.synchronize()
        assert torch.equal(a.logits(), b.logits())
    finally:
        a.close()
        b.close()


@pytest.mark.gpu
def test_truncated_checkpoint_is_an_error(tmp_path):
    params = syn.make_params(6, **CFG)
    path = tmp_path / "model.bin"
    syn.write_llmc_checkpoint(path, params, **CFG)
    data = path.read_bytes()
    path.write_bytes(data[:len(data) // 2])
    with pytest.raises(g2.GPT2HipError, match="truncated"):
        g2.GPT2.from_checkpoint(path)


# ---------------------------------------------------------------------------------------
# A file laid out from literal byte offsets, sharing nothing with synthetic.write_llmc_checkpoint
# (so that the loader and the package's own writer cannot agree on a common mistake).
# llm.c's train_gpt2.c documents the layout: a 1024-byte header of little-endian int32 words,
# word 0 magic 20240326, 1 version, 2 max_seq_len, 3 vocab_size, 4 num_layers, 5 num_heads,
# 6 channels, 7 padded_vocab_size; then the sixteen tensors, wte with padded_vocab_size rows.
# No llm.c-produced file exists offline, so the format itself stays unpinned by upstream data.
LIT = dict(max_seq_len=8, vocab_size=130, num_layers=2, num_heads=2, channels=64)
LIT_VP = 256


def _literal_tensors():
    """(name, shape, values) in file order; tensor k holds ((13 k + flat index) mod 251) - 125."""
    maxT, V, L, C = LIT["max_seq_len"], LIT["vocab_size"], LIT["num_layers"], LIT["channels"]
    shapes = [("wte", (V, C)), ("wpe", (maxT, C)), ("ln1w", (L, C)), ("ln1b", (L, C)),
              ("qkvw", (L, 3 * C, C)), ("qkvb", (L, 3 * C)), ("attprojw", (L, C, C)),
              ("attprojb", (L, C)), ("ln2w", (L, C)), ("ln2b", (L, C)), ("fcw", (L, 4 * C, C)),
              ("fcb", (L, 4 * C)), ("fcprojw", (L, C, 4 * C)), ("fcprojb", (L, C)),
              ("lnfw", (C,)), ("lnfb", (C,))]
    out = []
    for k, (name, shape) in enumerate(shapes):
        n = int(np.prod(shape))
        # integers of at most 8 significant bits: exact in bf16 as well as in fp32; the phase
        # 13 k makes a tensor read from a neighbour's offset differ at every element
        vals = ((13 * k + np.arange(n)) % 251) - 125.0
        out.append((name, shape, vals.astype(np.float32).reshape(shape)))
    return out


def _literal_file(path, version):
    import struct
    import torch
    words = [20240326, version, LIT["max_seq_len"], LIT["vocab_size"], LIT["num_layers"],
             LIT["num_heads"], LIT["channels"], LIT_VP if version != 1 else 0]
    blob = bytearray(1024)
    for i, w in enumerate(words):
        struct.pack_into("<i", blob, 4 * i, w)

    def raw(a):
        if version == 5:  # bf16 by torch's conversion, not by the package's bit shifting
            return torch.from_numpy(np.ascontiguousarray(a)).to(torch.bfloat16).view(torch.int16) \
                .numpy().astype("<i2").tobytes()
        return np.ascontiguousarray(a).astype("<f4").tobytes()

    for name, shape, vals in _literal_tensors():
        blob += raw(vals)
        if name == "wte" and version != 1:
            pad = np.full((LIT_VP - LIT["vocab_size"], LIT["channels"]), -777.0, np.float32)
            blob += raw(pad)
    path.write_bytes(bytes(blob))


@pytest.mark.parametrize("version", [1, 3, 5])
def test_literal_layout_header(tmp_path, version):
    p = tmp_path / "lit.bin"
    _literal_file(p, version)
    assert g2.read_checkpoint_config(p) == LIT
    n = sum(v.size for _, _, v in _literal_tensors())
    pad = (LIT_VP - LIT["vocab_size"]) * LIT["channels"] if version != 1 else 0
    assert p.stat().st_size == 1024 + (2 if version == 5 else 4) * (n + pad)


@pytest.mark.gpu
@pytest.mark.parametrize("version", [1, 3, 5])
def test_literal_layout_loads_every_tensor_in_place(tmp_path, version):
    p = tmp_path / "lit.bin"
    _literal_file(p, version)
    m = g2.GPT2.from_checkpoint(p)
    try:
        flat = m.params_tensor().cpu().numpy()
        off = 0
        for name, shape, vals in _literal_tensors():
            got = flat[off:off + vals.size].reshape(shape)
            assert np.array_equal(got, vals), f"{name} (version {version})"
            off += vals.size
        assert off == flat.size == m.num_parameters
    finally:
        m.close()
