"""Shared parity helpers for the GPU tests (tolerances of the attention path)."""

import numpy as np
import torch

# Attention outputs must be within max-abs 2e-3 and max-rel 1e-2 of an fp32-accumulated
# reference. max-rel is the largest absolute error divided by the largest reference magnitude of
# the tensor (the normalised max error); element-wise ratios are meaningless for outputs that
# pass through zero.
MAX_ABS = 2e-3
MAX_REL = 1e-2


def to_np16(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().contiguous().numpy()


def assert_attention_close(got: torch.Tensor, ref, what: str = "") -> None:
    g = got.detach().float().cpu().numpy()
    r = np.asarray(ref, dtype=np.float32)
    assert g.shape == r.shape, (g.shape, r.shape)
    assert np.isfinite(g).all(), f"{what}: non-finite output"
    diff = np.abs(g - r)
    max_abs = float(diff.max(initial=0.0))
    max_rel = max_abs / max(float(np.abs(r).max(initial=0.0)), 1e-12)
    assert max_abs <= MAX_ABS, f"{what}: max-abs {max_abs:.3e} > {MAX_ABS}"
    assert max_rel <= MAX_REL, f"{what}: max-rel {max_rel:.3e} > {MAX_REL}"


def assert_bit_exact(got: torch.Tensor, ref, what: str = "") -> None:
    g = got.detach().cpu().contiguous().view(torch.int16).numpy()
    r = ref.detach().cpu().contiguous().view(torch.int16).numpy() if isinstance(ref, torch.Tensor) \
        else np.ascontiguousarray(ref).view(np.int16)
    assert g.shape == r.shape, (g.shape, r.shape)
    bad = int((g != r).sum())
    assert bad == 0, f"{what}: {bad} of {g.size} fp16 words differ"
