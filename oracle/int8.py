"""TEST INFRASTRUCTURE ONLY -- CPU restatement (numpy) of the int8 KV storage: signed 8-bit codes with
one fp32 scale per kv head. Nothing under llama_lite_npu_amd/ may import this.

The reference's int8 cache kernel (lite_llama/kernels/others/context_flashattention_nopad.py:374-553)
reads int8 K/V as they are, without scales, and has no quantising append to follow, so this file
states the scheme in closed form -- the one the fp8 pools use, with integer codes:
    encode(x, scale) = clamp(round_half_to_even(x * (1 / scale)), -127, 127)      (x * (1/scale) in fp32)
    decode(code, scale) = code * scale
Inputs that are not finite: +-Inf saturate like any large value; the clamp is maxNum(x, -127) then
minNum(., 127) (IEEE 754-2008: a quiet NaN operand is dropped), so NaN is stored as -127. An int8
pool cannot hold a NaN; the rule only makes what is stored a function of the input.
Numeric parity with the reference is **parity unpinned** (nothing to compare with).

Pinned in tests/test_oracle.py by: halves going to the even integer, saturation at +-127 (-128 is
never produced), decode(encode(v)) == v for every integer in range, monotonicity, PyTorch's
independent round + clamp on every fp16 input in range, hand-computed examples with scales, and
the codes of NaN and +-Inf.
Attention over an int8 pool is the fp16 oracle applied to the decoded pool (codes are exact in
fp16; the scale is applied in fp32).
"""

from __future__ import annotations

import numpy as np

INT8_MAX = 127.0


def encode(x: np.ndarray) -> np.ndarray:
    """float32 (already divided by the scale) -> int8 codes: round half to even, clamp to +-127."""
    x = np.asarray(x, dtype=np.float32)
    r = np.rint(x)                                   # numpy rounds halves to even
    r = np.fmin(np.fmax(r, -INT8_MAX), INT8_MAX)     # maxNum / minNum: NaN -> -127, +-Inf -> +-127
    return r.astype(np.int8)


def decode(codes: np.ndarray) -> np.ndarray:
    return np.asarray(codes).view(np.int8).astype(np.float32)


def quantize_rows(rows: np.ndarray, scales: np.ndarray) -> np.ndarray:
    """rows [T, H, D] fp16, scales [H] fp32 -> codes [T, H, D] int8 (x * (1/scale) in fp32, then encode)."""
    inv = (np.float32(1.0) / np.asarray(scales, dtype=np.float32)).astype(np.float32)
    y = rows.astype(np.float32) * inv[None, :, None]
    return encode(y.astype(np.float32))


def kv_append(k: np.ndarray, v: np.ndarray, slot_mapping: np.ndarray, pool: np.ndarray, scales: np.ndarray) -> None:
    """pool [slots, 2H, D] int8, in place; slots outside the pool are skipped."""
    h = k.shape[1]
    codes = np.concatenate([quantize_rows(k, scales[:h]), quantize_rows(v, scales[h:])], axis=1)
    for t, slot in enumerate(np.asarray(slot_mapping)):
        if 0 <= slot < pool.shape[0]:
            pool[slot] = codes[t]


def dequantize_pool(pool: np.ndarray, scales: np.ndarray) -> np.ndarray:
    """codes [slots, 2H, D] -> float32 values (code * scale in fp32)."""
    return decode(pool) * np.asarray(scales, dtype=np.float32)[None, :, None]
