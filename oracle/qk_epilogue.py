"""TEST INFRASTRUCTURE ONLY -- CPU restatement (numpy) of the step before the KV append on the
reference's attention path: per-head RMSNorm of q and k, rotary embedding of both, concatenation
of k and v and the scatter into the slot rows. Nothing under llama_lite_npu_amd/ may import this.

Reference lines followed:
  rms_norm        lite_llama/kernels/skip_rmsnorm.py:117-146 (`rms_norm_kernel`: fp32 x,
                  var = sum(x*x/N), rrms = 1/sqrt(var+eps), y = (x*rrms).to(fp16) * w) and the torch
                  form `python_rmsnorm` :231-235
  rope            lite_llama/kernels/rope_emb.py:40-87 (first half / second half pairing with the
                  first D/2 entries of the token's cos / sin row):
                      new1 = x1*cos - x2*sin,  new2 = x2*cos + x1*sin
  append          lite_llama/models/qwen3.py:29, 62 (`torch.cat([xk, xv], dim=-2)`) and
                  lite_llama/kernels/update_kv_buffer.py:47-56, 104-105 (buf[slots] = values)

Pinned in tests/test_oracle.py by: the fp64 closed form x / sqrt(mean(x^2) + eps) * w; rotation as
multiplication of the complex number x1 + i*x2 by exp(i*theta) (an independent formulation: a
swapped sign or half fails it); position 0 is the identity; rotating by theta1 then theta2 equals
rotating by theta1 + theta2; the pair norms are preserved; append equals index assignment.
The reference's own test of this kernel (tests/kernels/test_rope_forward.py) compares against an
inline torch rotate_half on the device and holds no stored vectors: numeric parity with the
Triton-Ascend kernel's fp16 intermediate rounding is parity unpinned; the rotation here is
evaluated in fp32 from fp16 inputs and rounded once.
"""

from __future__ import annotations

from typing import Optional

import numpy as np


def rms_norm(x: np.ndarray, w: np.ndarray, eps: float) -> np.ndarray:
    """x [..., D] fp16, w [D] fp16 -> fp16, rounding where the reference kernel rounds."""
    xf = x.astype(np.float32)
    var = (xf * xf).sum(axis=-1, keepdims=True, dtype=np.float32) / np.float32(x.shape[-1])
    rrms = np.float32(1.0) / np.sqrt(var + np.float32(eps), dtype=np.float32)
    y = (xf * rrms).astype(np.float16)
    return (y.astype(np.float32) * w.astype(np.float32)).astype(np.float16)


def rope(x: np.ndarray, cos: np.ndarray, sin: np.ndarray) -> np.ndarray:
    """x [T, H, D] fp16; cos, sin [T, >= D/2] fp16 (the rows of each token's position) -> fp16."""
    d = x.shape[-1]
    h = d // 2
    x1, x2 = x[..., :h].astype(np.float32), x[..., h:].astype(np.float32)
    c = cos[:, None, :h].astype(np.float32)
    s = sin[:, None, :h].astype(np.float32)
    return np.concatenate([x1 * c - x2 * s, x2 * c + x1 * s], axis=-1).astype(np.float16)


def qk_norm_rope_append(q: np.ndarray, k: np.ndarray, v: np.ndarray, slot_mapping: np.ndarray,
                        kv_pool: np.ndarray, q_norm_weight: Optional[np.ndarray] = None,
                        k_norm_weight: Optional[np.ndarray] = None, cos: Optional[np.ndarray] = None,
                        sin: Optional[np.ndarray] = None, eps: float = 1e-6):
    """Returns (q_out fp16 [T, Hq, D], pool fp16 copy with the k / v rows of valid slots written)."""
    q, k = q.astype(np.float16), k.astype(np.float16)
    if q_norm_weight is not None:
        q, k = rms_norm(q, q_norm_weight, eps), rms_norm(k, k_norm_weight, eps)
    if cos is not None:
        q, k = rope(q, cos, sin), rope(k, cos, sin)
    pool = kv_pool.copy()
    hkv = k.shape[1]
    slots = np.asarray(slot_mapping).astype(np.int64)
    ok = (slots >= 0) & (slots < pool.shape[0])
    pool[slots[ok], :hkv] = k[ok]
    pool[slots[ok], hkv:] = v[ok]
    return q, pool
