"""Python host-side mirror of the llm.c-style launcher surface, bound over the
C ABI of ``libgpt2_mi355x.so`` (declared in ``include/gpt2_mi355x.h``).

The launchers keep the reference's names and argument order
(``matmul_forward(out, inp, weight, bias, B, T, C, OC)`` and so on: reference
``kernels/matmul/2_matmul_cublas.cuh:34-42``,
``kernels/attention/3_flash_attention_permute.cuh:346-351``,
``kernels/fused_residual_layernorm/fused_residual_layernorm.cuh:88-90``).
Arguments are torch CUDA tensors, used only as owners of device memory: the
library receives raw pointers.  There is no CPU fallback: if the shared library
is missing or no GPU is present, calls raise.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from typing import Optional

_HERE = os.path.dirname(os.path.abspath(__file__))
_ROOT = os.path.dirname(_HERE)
LIB_PATH = os.path.join(_HERE, "libgpt2_mi355x.so")
SOURCES = ("layernorm.hip", "elementwise.hip", "matmul.hip", "attention.hip", "decode.hip",
           "gpt2.hip")
HIPCC_FLAGS = (
    "-O3", "--offload-arch=gfx950", "-std=c++17", "-fPIC", "-shared",
    # packed-fp32 VALU forms are switched off for every HIP translation unit
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    # keep MFMA accumulators in ordinary VGPRs: the softmax reads them with VALU
    # instructions, and copies out of the accumulation registers would cost issue slots
    "-mllvm", "-amdgpu-mfma-vgpr-form",
)

EXPORTS = (
    "gpt2hip_last_error", "gpt2hip_set_stream", "gpt2hip_get_stream", "gpt2hip_set_workspace",
    "encoder_forward", "encoder_forward_status",
    "layernorm_forward", "layernorm_forward_status",
    "fused_residual_layernorm_forward", "fused_residual_layernorm_forward_status",
    "residual_forward", "residual_forward_status",
    "gelu_forward", "gelu_forward_status",
    "matmul_forward", "matmul_forward_status",
    "matmul_forward_gelu", "matmul_forward_gelu_status", "matmul_forward_probe_status",
    "matmul_forward_tile_shape",
    "matmul_forward_splitk_workspace", "matmul_forward_splitk_status",
    "matmul_forward_splitk_plan", "matmul_forward_splitk_forced_status",
    "matmul_forward_residual_status", "matmul_forward_first_columns",
    "attention_forward", "attention_forward_status",
    "argmax_forward", "argmax_forward_status",
    "matmul_forward_argmax_workspace", "matmul_forward_argmax_status",
    "matmul_forward_argmax_noalloc_status",
    "gpt2_checkpoint_read_config", "gpt2_build_from_checkpoint",
    "gpt2_create", "gpt2_destroy", "gpt2_num_parameters", "gpt2_params_device",
    "gpt2_load_params_host", "gpt2_reserve", "gpt2_forward", "gpt2_forward_status",
    "gpt2_forward_device_status", "gpt2_forward_graph_status",
    "gpt2_prefill_status", "gpt2_decode_status", "gpt2_decode_sync_status", "gpt2_decode_options", "gpt2_decode_probe_status", "gpt2_decode_probe_size",
    "gpt2_step_logits", "gpt2_cache_length",
    "gpt2_forward_argmax_status", "gpt2_forward_sums_in_matmul",
    "gpt2_forward_profiled_status", "gpt2hip_profile_marker_overhead_us", "gpt2_logits", "gpt2_lnf", "gpt2_argmax_status",
    "gpt2hip_timer_create", "gpt2hip_timer_destroy", "gpt2hip_timer_start",
    "gpt2hip_timer_stop_ms",
)


def build(verbose: bool = False) -> str:
    """Compile every HIP source for gfx950 into ``libgpt2_mi355x.so`` (in-tree)."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc, *HIPCC_FLAGS, "-I", os.path.join(_ROOT, "include"), "-o", LIB_PATH]
    cmd += [os.path.join(_HERE, "csrc", s) for s in SOURCES]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in proc.stderr.splitlines() if noise not in l)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed ({proc.returncode}):\n{err}")
    if verbose and err.strip():
        print(err)
    build_example()
    return LIB_PATH


EXAMPLE_SRC = os.path.join(_HERE, "examples", "llmc_style_driver.cpp")
EXAMPLE_BIN = os.path.join(_HERE, "examples", "llmc_style_driver")


def build_example() -> str:
    """Compile the plain-C++ llm.c-style driver against the library's C ABI (host code only)."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc, "-O2", "-std=c++17", EXAMPLE_SRC, "-I", os.path.join(_ROOT, "include"),
           "-L", _HERE, "-lgpt2_mi355x", "-Wl,-rpath,$ORIGIN/..", "-o", EXAMPLE_BIN]
    proc = subprocess.run(cmd, capture_output=True, text=True)
    if proc.returncode != 0:
        raise RuntimeError(f"hipcc failed on the example driver ({proc.returncode}):\n{proc.stderr}")
    return EXAMPLE_BIN


class GPT2Config(ctypes.Structure):
    _fields_ = [("max_seq_len", ctypes.c_int), ("vocab_size", ctypes.c_int),
                ("num_layers", ctypes.c_int), ("num_heads", ctypes.c_int),
                ("channels", ctypes.c_int)]


# order of the GPT2_PROF_* enum in the header
PROF_CATEGORIES = ("encoder", "layernorm", "matmul_qkv", "attention", "matmul_attproj",
                   "fused_residual_layernorm", "matmul_fc_gelu", "matmul_fcproj", "matmul_lmhead")

GPT2_124M = dict(max_seq_len=1024, vocab_size=50257, num_layers=12, num_heads=12, channels=768)
GPT2_350M = dict(max_seq_len=1024, vocab_size=50257, num_layers=24, num_heads=16, channels=1024)
GPT2_774M = dict(max_seq_len=1024, vocab_size=50257, num_layers=36, num_heads=20, channels=1280)    # "large"
GPT2_1558M = dict(max_seq_len=1024, vocab_size=50257, num_layers=48, num_heads=25, channels=1600)   # "XL"

_lib: Optional[ctypes.CDLL] = None


def lib() -> ctypes.CDLL:
    """The loaded C-ABI library.  Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} is missing: build it with __graft_entry__.build() "
                "(there is no CPU or PyTorch fallback for these kernels)")
        L = ctypes.CDLL(LIB_PATH)
        vp, ci, cz = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t
        L.gpt2hip_last_error.restype = ctypes.c_char_p
        sig = {
            "encoder_forward": [vp] * 4 + [ci] * 3,
            "layernorm_forward": [vp] * 6 + [ci] * 3,
            "fused_residual_layernorm_forward": [vp] * 8 + [ci] * 3,
            "residual_forward": [vp] * 3 + [ci],
            "gelu_forward": [vp] * 2 + [ci],
            "matmul_forward": [vp] * 4 + [ci] * 4,
            "matmul_forward_gelu": [vp] * 4 + [ci] * 5,
            "attention_forward": [vp] * 4 + [ci] * 4,
            "argmax_forward": [vp] * 2 + [ci] * 2,
        }
        for name, args in sig.items():
            f = getattr(L, name)
            f.argtypes, f.restype = args, None
            f = getattr(L, name + "_status")
            f.argtypes, f.restype = args, ci
        L.matmul_forward_probe_status.argtypes = [vp] * 4 + [ci] * 4 + [vp, ci, ctypes.POINTER(ci)]
        L.matmul_forward_probe_status.restype = ci
        L.matmul_forward_tile_shape.argtypes = [ci] * 4 + [ctypes.POINTER(ci)] * 2
        L.matmul_forward_tile_shape.restype = ci
        L.matmul_forward_splitk_workspace.argtypes = []
        L.matmul_forward_splitk_workspace.restype = cz
        L.matmul_forward_splitk_status.argtypes = [vp] * 4 + [ci] * 5 + [vp, cz]
        L.matmul_forward_splitk_status.restype = ci
        L.matmul_forward_splitk_forced_status.argtypes = [vp] * 4 + [ci] * 5 + [vp, cz] + [ci] * 3
        L.matmul_forward_splitk_forced_status.restype = ci
        L.matmul_forward_first_columns.argtypes = [ci] * 4 + [cz]
        L.matmul_forward_first_columns.restype = ci
        L.matmul_forward_residual_status.argtypes = [vp] * 5 + [ci] * 4 + [vp, cz]
        L.matmul_forward_residual_status.restype = ci
        L.matmul_forward_splitk_plan.argtypes = [ci] * 4 + [cz] + [ctypes.POINTER(ci)] * 3
        L.matmul_forward_splitk_plan.restype = ci
        L.gpt2_create.argtypes, L.gpt2_create.restype = [ctypes.POINTER(GPT2Config)], vp
        L.gpt2_destroy.argtypes, L.gpt2_destroy.restype = [vp], None
        L.gpt2_checkpoint_read_config.argtypes = [ctypes.c_char_p, ctypes.POINTER(GPT2Config)]
        L.gpt2_checkpoint_read_config.restype = ci
        L.gpt2_build_from_checkpoint.argtypes = [ctypes.c_char_p]
        L.gpt2_build_from_checkpoint.restype = vp
        L.gpt2_num_parameters.argtypes, L.gpt2_num_parameters.restype = [vp], cz
        L.gpt2_params_device.argtypes, L.gpt2_params_device.restype = [vp], vp
        L.gpt2_load_params_host.argtypes, L.gpt2_load_params_host.restype = [vp, vp, cz], ci
        L.gpt2_reserve.argtypes, L.gpt2_reserve.restype = [vp, ci, ci], ci
        L.gpt2_forward.argtypes, L.gpt2_forward.restype = [vp, vp, ci, ci], None
        L.gpt2_forward_status.argtypes, L.gpt2_forward_status.restype = [vp, vp, ci, ci], ci
        L.gpt2_forward_device_status.argtypes = [vp, vp, ci, ci]
        L.gpt2_forward_device_status.restype = ci
        L.gpt2_prefill_status.argtypes, L.gpt2_prefill_status.restype = [vp, vp, ci, ci], ci
        L.gpt2_decode_status.argtypes, L.gpt2_decode_status.restype = [vp, vp], ci
        L.gpt2_decode_options.argtypes, L.gpt2_decode_options.restype = [vp, ci, ctypes.c_uint], ci
        L.gpt2_decode_sync_status.argtypes, L.gpt2_decode_sync_status.restype = [vp], ci
        L.gpt2_decode_probe_status.argtypes, L.gpt2_decode_probe_status.restype = [vp, vp, vp, cz], ci
        L.gpt2_decode_probe_size.argtypes, L.gpt2_decode_probe_size.restype = [vp], cz
        L.gpt2_step_logits.argtypes, L.gpt2_step_logits.restype = [vp], vp
        L.gpt2_cache_length.argtypes, L.gpt2_cache_length.restype = [vp], ci
        L.gpt2_forward_graph_status.argtypes = [vp, vp, ci, ci]
        L.gpt2_forward_graph_status.restype = ci
        L.gpt2hip_set_stream.argtypes, L.gpt2hip_set_stream.restype = [vp], None
        L.gpt2hip_get_stream.argtypes, L.gpt2hip_get_stream.restype = [], vp
        L.gpt2hip_set_workspace.argtypes, L.gpt2hip_set_workspace.restype = [vp, cz], ci
        L.gpt2_forward_sums_in_matmul.argtypes = [ctypes.POINTER(GPT2Config), ci, ci]
        L.gpt2_forward_sums_in_matmul.restype = ci
        L.gpt2_forward_argmax_status.argtypes = [vp, vp, ci, ci, vp]
        L.gpt2_forward_argmax_status.restype = ci
        L.matmul_forward_argmax_workspace.argtypes = [ci, ci, ci]
        L.matmul_forward_argmax_workspace.restype = cz
        L.matmul_forward_argmax_status.argtypes = [vp, vp, cz, vp, vp, vp, ci, ci, ci, ci]
        L.matmul_forward_argmax_status.restype = ci
        L.matmul_forward_argmax_noalloc_status.argtypes = [vp, vp, vp, vp, ci, ci, ci, ci]
        L.matmul_forward_argmax_noalloc_status.restype = ci
        L.gpt2_forward_profiled_status.argtypes = [vp, vp, ci, ci, ctypes.POINTER(ctypes.c_float)]
        L.gpt2_forward_profiled_status.restype = ci
        L.gpt2hip_profile_marker_overhead_us.argtypes = [ci]
        L.gpt2hip_profile_marker_overhead_us.restype = ctypes.c_float
        L.gpt2_logits.argtypes, L.gpt2_logits.restype = [vp], vp
        L.gpt2_lnf.argtypes, L.gpt2_lnf.restype = [vp], vp
        L.gpt2_argmax_status.argtypes, L.gpt2_argmax_status.restype = [vp, vp], ci
        L.gpt2hip_timer_create.argtypes, L.gpt2hip_timer_create.restype = [], vp
        L.gpt2hip_timer_destroy.argtypes, L.gpt2hip_timer_destroy.restype = [vp], None
        L.gpt2hip_timer_start.argtypes, L.gpt2hip_timer_start.restype = [vp], ci
        L.gpt2hip_timer_stop_ms.argtypes, L.gpt2hip_timer_stop_ms.restype = [vp], ctypes.c_float
        _lib = L
    return _lib


class GPT2HipError(RuntimeError):
    pass


def _check(rc: int, what: str) -> None:
    if rc != 0:
        msg = lib().gpt2hip_last_error().decode(errors="replace")
        raise GPT2HipError(f"{what} failed (code {rc}): {msg}")


def _ptr(t, dtype=None) -> Optional[int]:
    """Device pointer of a contiguous CUDA tensor (None passes NULL)."""
    if t is None:
        return None
    import torch
    if not isinstance(t, torch.Tensor) or not t.is_cuda:
        raise TypeError("expected a CUDA tensor: these launchers take device memory only")
    if not t.is_contiguous():
        raise ValueError("tensor must be contiguous")
    if dtype is not None and t.dtype != dtype:
        raise TypeError(f"expected {dtype}, got {t.dtype}")
    return t.data_ptr()


def _f32(t):
    import torch
    return _ptr(t, torch.float32)


def _i32(t):
    import torch
    return _ptr(t, torch.int32)


# ---- launchers: same names, argument order and meaning as the reference's ----

def encoder_forward(out, inp, wte, wpe, B, T, C):
    _check(lib().encoder_forward_status(_f32(out), _i32(inp), _f32(wte), _f32(wpe), B, T, C),
           "encoder_forward")


def layernorm_forward(out, mean, rstd, inp, weight, bias, B, T, C):
    _check(lib().layernorm_forward_status(_f32(out), _f32(mean), _f32(rstd), _f32(inp),
                                          _f32(weight), _f32(bias), B, T, C), "layernorm_forward")


def fused_residual_layernorm_forward(res_out, layernorm_out, mean, rstd, inp1, inp2, weight, bias,
                                     B, T, C):
    _check(lib().fused_residual_layernorm_forward_status(
        _f32(res_out), _f32(layernorm_out), _f32(mean), _f32(rstd), _f32(inp1), _f32(inp2),
        _f32(weight), _f32(bias), B, T, C), "fused_residual_layernorm_forward")


def residual_forward(out, inp1, inp2, N):
    _check(lib().residual_forward_status(_f32(out), _f32(inp1), _f32(inp2), N), "residual_forward")


def gelu_forward(out, inp, N):
    _check(lib().gelu_forward_status(_f32(out), _f32(inp), N), "gelu_forward")


def matmul_forward(out, inp, weight, bias, B, T, C, OC):
    _check(lib().matmul_forward_status(_f32(out), _f32(inp), _f32(weight), _f32(bias), B, T, C,
                                       OC), "matmul_forward")


def matmul_forward_gelu(out, inp, weight, bias, B, T, C, OC, is_gelu):
    _check(lib().matmul_forward_gelu_status(_f32(out), _f32(inp), _f32(weight), _f32(bias), B, T,
                                            C, OC, int(bool(is_gelu))), "matmul_forward_gelu")


def matmul_forward_probe(out, inp, weight, bias, B, T, C, OC):
    """matmul_forward with the in-kernel clock probe.  Returns a (workgroups, 4) int64
    array: wall clock (10 ns ticks) at K-loop start / end, shader clock at the same."""
    import torch
    cap = ((B * T + 31) // 32) * ((OC + 31) // 32)
    probe = torch.zeros((cap, 4), dtype=torch.int64, device="cuda")
    n = ctypes.c_int(0)
    _check(lib().matmul_forward_probe_status(_f32(out), _f32(inp), _f32(weight), _f32(bias), B, T,
                                             C, OC, probe.data_ptr(), cap, ctypes.byref(n)),
           "matmul_forward_probe")
    torch.cuda.synchronize()
    return probe[:n.value].cpu().numpy()


def matmul_forward_tile_shape(B, T, C, OC):
    """(rows, columns) of the workgroup tile matmul_forward gives this problem; (0, 0) if it
    takes a kernel that is not tiled this way.  No GPU needed."""
    bm, bn = ctypes.c_int(0), ctypes.c_int(0)
    _check(lib().matmul_forward_tile_shape(B, T, C, OC, ctypes.byref(bm), ctypes.byref(bn)),
           "matmul_forward_tile_shape")
    return bm.value, bn.value


SPLITK_COUNTER_BYTES = 16384


def matmul_forward_splitk_workspace():
    """A zero-filled workspace (uint8 CUDA tensor) of the size the library recommends."""
    import torch
    return torch.zeros(lib().matmul_forward_splitk_workspace(), dtype=torch.uint8, device="cuda")


def matmul_forward_splitk(out, inp, weight, bias, B, T, C, OC, workspace, is_gelu=False, plan=None):
    """matmul_forward_gelu with a workspace that lets K be split between workgroups.
    workspace: uint8 CUDA tensor whose first SPLITK_COUNTER_BYTES were zero before its first
    use.  plan: optional (tile_rows, tile_cols, splits) to force instead of the cost model's."""
    ws, nbytes = (None, 0) if workspace is None else (workspace.data_ptr(), workspace.numel())
    if plan is None:
        _check(lib().matmul_forward_splitk_status(_f32(out), _f32(inp), _f32(weight), _f32(bias), B,
                                                  T, C, OC, int(bool(is_gelu)), ws, nbytes),
               "matmul_forward_splitk")
    else:
        _check(lib().matmul_forward_splitk_forced_status(_f32(out), _f32(inp), _f32(weight),
                                                         _f32(bias), B, T, C, OC, int(bool(is_gelu)),
                                                         ws, nbytes, *map(int, plan)),
               "matmul_forward_splitk_forced")


def matmul_forward_residual(out, inp, weight, bias, resid, B, T, C, OC, workspace=None):
    """out = resid + (inp . weight^T + bias), the residual add in the product's epilogue.
    workspace: as for matmul_forward_splitk (None: K is not split between workgroups)."""
    ws, nbytes = (None, 0) if workspace is None else (workspace.data_ptr(), workspace.numel())
    _check(lib().matmul_forward_residual_status(_f32(out), _f32(inp), _f32(weight), _f32(bias),
                                                _f32(resid), B, T, C, OC, ws, nbytes),
           "matmul_forward_residual")


def matmul_forward_first_columns(B, T, C, OC, workspace_bytes=0):
    """Columns computed by the first launch of a product (OC: the product is one launch)."""
    return lib().matmul_forward_first_columns(B, T, C, OC, workspace_bytes)


def forward_sums_in_matmul(config, B, T):
    """Whether gpt2_forward at this size adds the residual stream in the projections' epilogues
    (config: a dict with the GPT2Config fields, e.g. GPT2_124M).  No GPU needed."""
    cfg = GPT2Config(**config)
    return bool(lib().gpt2_forward_sums_in_matmul(ctypes.byref(cfg), B, T))


def matmul_forward_splitk_plan(B, T, C, OC, workspace_bytes):
    """(tile_rows, tile_cols, splits) that matmul_forward_splitk would use.  No GPU needed."""
    bm, bn, sp = ctypes.c_int(0), ctypes.c_int(0), ctypes.c_int(0)
    _check(lib().matmul_forward_splitk_plan(B, T, C, OC, workspace_bytes, ctypes.byref(bm),
                                            ctypes.byref(bn), ctypes.byref(sp)),
           "matmul_forward_splitk_plan")
    return bm.value, bn.value, sp.value


def attention_forward(out, qkvr, att, inp, B, T, C, NH):
    _check(lib().attention_forward_status(_f32(out), _f32(qkvr), _f32(att), _f32(inp), B, T, C,
                                          NH), "attention_forward")


def argmax_forward(ids, logits, N, V):
    _check(lib().argmax_forward_status(_i32(ids), _f32(logits), N, V), "argmax_forward")


def matmul_forward_argmax(ids, inp, weight, bias, B, T, C, OC, workspace=None):
    """ids (B*T int32) = per-row argmax of inp . weight^T + bias, without storing the product.
    workspace: optional uint8 CUDA tensor of matmul_forward_argmax_workspace(B, T, OC) bytes."""
    import torch
    need = lib().matmul_forward_argmax_workspace(B, T, OC)
    if workspace is None:
        workspace = torch.empty(max(need, 1), dtype=torch.uint8, device="cuda")
    _check(lib().matmul_forward_argmax_status(_i32(ids), workspace.data_ptr(), workspace.numel(),
                                              _f32(inp), _f32(weight), _f32(bias), B, T, C, OC),
           "matmul_forward_argmax")


ARGMAX_NOALLOC_BYTES = 33 << 20  # GPT2HIP_ARGMAX_NOALLOC_BYTES


def matmul_forward_argmax_noalloc(ids, inp, weight, bias, B, T, C, OC):
    """matmul_forward_argmax with the pairs in the library's static device array: no
    allocation, no workspace argument; shapes beyond ARGMAX_NOALLOC_BYTES of pairs raise."""
    _check(lib().matmul_forward_argmax_noalloc_status(_i32(ids), _f32(inp), _f32(weight),
                                                      _f32(bias), B, T, C, OC),
           "matmul_forward_argmax_noalloc")


def set_stream(stream) -> None:
    """Make every launcher of this thread use `stream` (a torch.cuda.Stream, a raw
    hipStream_t value, or None for the null stream)."""
    raw = getattr(stream, "cuda_stream", stream)
    lib().gpt2hip_set_stream(raw or None)


def set_workspace(workspace) -> None:
    """Lend matmul_forward / matmul_forward_gelu of this thread a K-split workspace (a uint8
    CUDA tensor whose first SPLITK_COUNTER_BYTES were zero before its first use, e.g. from
    matmul_forward_splitk_workspace(); the caller keeps it alive), or None to take it back."""
    if workspace is None:
        _check(lib().gpt2hip_set_workspace(None, 0), "gpt2hip_set_workspace")
    else:
        _check(lib().gpt2hip_set_workspace(workspace.data_ptr(), workspace.numel()),
               "gpt2hip_set_workspace")


def read_checkpoint_config(path) -> dict:
    """Header of an llm.c checkpoint file as GPT2(**config) keywords (no GPU needed)."""
    cfg = GPT2Config()
    _check(lib().gpt2_checkpoint_read_config(os.fsencode(path), ctypes.byref(cfg)),
           "gpt2_checkpoint_read_config")
    return {name: getattr(cfg, name) for name, _ in GPT2Config._fields_}


class Timer:
    """HIP-event timer on the null stream, the stream every launcher uses."""

    def __init__(self):
        self._h = lib().gpt2hip_timer_create()
        if not self._h:
            raise GPT2HipError("gpt2hip_timer_create failed")

    def start(self):
        _check(lib().gpt2hip_timer_start(self._h), "gpt2hip_timer_start")

    def stop_ms(self) -> float:
        ms = lib().gpt2hip_timer_stop_ms(self._h)
        if ms < 0:
            raise GPT2HipError("gpt2hip_timer_stop_ms failed")
        return float(ms)

    def __del__(self):
        if getattr(self, "_h", None) and _lib is not None:  # at interpreter exit the module may be gone
            _lib.gpt2hip_timer_destroy(self._h)
            self._h = None


class GPT2:
    """The gpt2_forward driver (C++ side owns parameters and activations)."""

    def __init__(self, *, max_seq_len, vocab_size, num_layers, num_heads, channels, _handle=None):
        self.config = GPT2Config(max_seq_len, vocab_size, num_layers, num_heads, channels)
        self._h = _handle or lib().gpt2_create(ctypes.byref(self.config))
        if not self._h:
            raise GPT2HipError("gpt2_create failed: " + lib().gpt2hip_last_error().decode())
        self.num_parameters = int(lib().gpt2_num_parameters(self._h))
        self._shape = None

    @classmethod
    def from_checkpoint(cls, path):
        """Build from an llm.c fp32 checkpoint file (gpt2_124M.bin format)."""
        cfg = read_checkpoint_config(path)
        h = lib().gpt2_build_from_checkpoint(os.fsencode(path))
        if not h:
            raise GPT2HipError("gpt2_build_from_checkpoint failed: "
                               + lib().gpt2hip_last_error().decode())
        return cls(_handle=h, **cfg)

    def close(self):
        if getattr(self, "_h", None) and _lib is not None:  # at interpreter exit the module may be gone
            _lib.gpt2_destroy(self._h)
            self._h = None

    __del__ = close

    def load_params(self, host_params):
        """host_params: contiguous float32 numpy array in checkpoint order."""
        import numpy as np
        a = np.ascontiguousarray(host_params, dtype=np.float32)
        _check(lib().gpt2_load_params_host(self._h, a.ctypes.data, a.size), "gpt2_load_params_host")

    def params_tensor(self):
        """A torch view of the flat device parameter buffer (no copy)."""
        return _device_view(lib().gpt2_params_device(self._h), (self.num_parameters,), "float32")

    def reserve(self, B, T):
        _check(lib().gpt2_reserve(self._h, B, T), "gpt2_reserve")

    def forward(self, inputs):
        """inputs: (B,T) int32, numpy (host, llm.c style) or CUDA tensor (device)."""
        import numpy as np
        B, T = inputs.shape
        if isinstance(inputs, np.ndarray):
            a = np.ascontiguousarray(inputs, dtype=np.int32)
            _check(lib().gpt2_forward_status(self._h, a.ctypes.data, B, T), "gpt2_forward")
        else:
            _check(lib().gpt2_forward_device_status(self._h, _i32(inputs), B, T), "gpt2_forward")
        self._shape = (B, T)

    def prefill(self, inputs_device):
        """Run a prompt (B,T) of device ids, filling the key/value cache; returns the (B,V)
        logits of the last position (library-owned memory, overwritten by the next step)."""
        B, T = inputs_device.shape
        _check(lib().gpt2_prefill_status(self._h, _i32(inputs_device), B, T), "gpt2_prefill")
        self._step_batch = B
        return self.step_logits()

    def decode(self, next_ids_device):
        """Append one token per sequence ((B,) device ids); returns that position's (B,V) logits."""
        if next_ids_device.numel() != getattr(self, "_step_batch", -1):
            raise GPT2HipError("decode: expected one token id per prefilled sequence")
        _check(lib().gpt2_decode_status(self._h, _i32(next_ids_device)), "gpt2_decode")
        return self.step_logits()

    def generate_greedy(self, prompt_device, steps: int):
        """Greedy continuation of a (B,T) prompt of device ids by `steps` tokens: prefill, then
        argmax_forward over the step logits and one decode step per token, all queued on the
        stream with no host synchronisation in between.  Returns (B, steps) int32 device ids."""
        import torch
        B, T = prompt_device.shape
        V = self.config.vocab_size
        out = torch.empty((steps, B), dtype=torch.int32, device="cuda")
        logits = self.prefill(prompt_device)
        for s in range(steps):
            argmax_forward(out[s], logits, B, V)
            if s + 1 < steps:
                logits = self.decode(out[s])
        self.decode_sync()  # a step that failed on the device would have left NaN logits behind
        return out.t().contiguous()

    def decode_sync(self) -> None:
        """Wait for the decode steps queued so far; raises if one of them gave up on the device
        (the cache is then rolled back to the positions before it, see cache_length())."""
        _check(lib().gpt2_decode_sync_status(self._h), "gpt2_decode_sync")

    def decode_probe(self, next_ids_device):
        """One decode step of the persistent kernel with its clock probe: returns a
        (phases, 2, workgroups) int64 tensor of 100 MHz wall-clock readings (work done / barrier
        passed) -- see gpt2_decode_probe_status in the header."""
        import torch
        n = lib().gpt2_decode_probe_size(self._h)
        if n == 0:
            raise GPT2HipError("decode_probe: the persistent kernel does not take this model")
        clocks = torch.zeros(n, dtype=torch.int64, device="cuda")
        _check(lib().gpt2_decode_probe_status(self._h, _i32(next_ids_device), clocks.data_ptr(), n),
               "gpt2_decode_probe")
        phases = 5 * self.config.num_layers + 1
        return clocks.view(phases, 2, -1)

    def decode_probe_size(self) -> int:
        """Clock slots decode_probe needs; 0 if the next step would not be the persistent kernel."""
        return int(lib().gpt2_decode_probe_size(self._h))

    def decode_options(self, persistent: bool = True, spin_limit: int = 1 << 21):
        """Choose between the persistent decode-step kernel and one launch per operation."""
        _check(lib().gpt2_decode_options(self._h, int(persistent), spin_limit), "gpt2_decode_options")

    def step_logits(self):
        return _device_view(lib().gpt2_step_logits(self._h),
                            (self._step_batch, self.config.vocab_size), "float32")

    def cache_length(self) -> int:
        return lib().gpt2_cache_length(self._h)

    def forward_graph(self, inputs_device):
        """forward() of device ids, replayed from a HIP graph captured on first use per (B,T)."""
        B, T = inputs_device.shape
        _check(lib().gpt2_forward_graph_status(self._h, _i32(inputs_device), B, T),
               "gpt2_forward_graph")
        self._shape = (B, T)

    def forward_argmax(self, inputs_device):
        """Forward that keeps only each position's argmax token id; returns (B,T) int32."""
        import torch
        B, T = inputs_device.shape
        ids = torch.empty((B, T), dtype=torch.int32, device="cuda")
        _check(lib().gpt2_forward_argmax_status(self._h, _i32(inputs_device), B, T,
                                                ids.data_ptr()), "gpt2_forward_argmax")
        self._shape = (B, T)
        return ids

    def forward_profiled(self, inputs_device):
        """Forward with per-launch HIP events; returns {category: ms} for this pass."""
        B, T = inputs_device.shape
        ms = (ctypes.c_float * len(PROF_CATEGORIES))()
        _check(lib().gpt2_forward_profiled_status(self._h, _i32(inputs_device), B, T, ms),
               "gpt2_forward_profiled")
        self._shape = (B, T)
        return dict(zip(PROF_CATEGORIES, (float(x) for x in ms)))

    def logits(self):
        B, T = self._shape
        return _device_view(lib().gpt2_logits(self._h), (B, T, self.config.vocab_size), "float32")

    def lnf(self):
        B, T = self._shape
        return _device_view(lib().gpt2_lnf(self._h), (B, T, self.config.channels), "float32")

    def argmax(self):
        import torch
        B, T = self._shape
        ids = torch.empty((B, T), dtype=torch.int32, device="cuda")
        _check(lib().gpt2_argmax_status(self._h, ids.data_ptr()), "gpt2_argmax")
        return ids


def _device_view(ptr: int, shape, dtype: str):
    """Wrap library-owned device memory as a torch tensor without copying."""
    import numpy as np
    import torch

    class _Holder:
        pass

    h = _Holder()
    n = int(np.prod(shape))
    h.__cuda_array_interface__ = {
        "shape": (n,), "typestr": {"float32": "<f4", "int32": "<i4"}[dtype],
        "data": (int(ptr), False), "version": 3, "strides": None,
    }
    return torch.as_tensor(h, device="cuda").view(*shape)
