"""Glue between torch tensors and the numpy oracle (raw-bit views)."""
import numpy as np
import torch

NAME = {torch.float32: "f32", torch.bfloat16: "bf16", torch.float16: "f16", torch.float8_e4m3fn: "fp8"}


def raw(t: torch.Tensor) -> np.ndarray:
    """Tensor -> numpy array of its storage codes (f32 / uint16 for bf16 and fp16 / uint8)."""
    t = t.detach().cpu().contiguous()
    if t.dtype == torch.float32:
        return t.numpy()
    if t.dtype in (torch.bfloat16, torch.float16):
        return t.view(torch.int16).numpy().view(np.uint16)
    if t.dtype == torch.float8_e4m3fn:
        return t.view(torch.uint8).numpy()
    if t.dtype in (torch.int32, torch.int64):
        return t.numpy()
    raise TypeError(t.dtype)


def to_f64(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().to(torch.float64).numpy()


def assert_close_attn(got: np.ndarray, want: np.ndarray, atol: float, rtol: float, what=""):
    """Pass if every element is within atol OR within rtol relative."""
    err = np.abs(got - want)
    ok = (err <= atol) | (err <= rtol * np.abs(want))
    if not ok.all():
        i = np.unravel_index(np.argmax(np.where(ok, 0, err)), err.shape)
        raise AssertionError(f"{what}: {(~ok).sum()} of {ok.size} elements out of tolerance; "
                             f"worst at {i}: got {got[i]}, want {want[i]}, max abs err {err.max():.3e}")
    assert np.isfinite(got).all(), f"{what}: non-finite output"
