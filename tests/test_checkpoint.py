"""llm.c checkpoint files: header parsing (CPU) and loading (GPU).

The files are written here with numpy in llm.c's on-disk layout (256 int32 header
words, fp32 tensors in checkpoint order, wte rows padded in version 3), independently
of the loader under test.
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
