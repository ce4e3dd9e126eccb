"""TEST INFRASTRUCTURE ONLY -- CPU restatement (numpy) of the FP8 KV storage: OCP E4M3FN codes with one
fp32 scale per kv head. Nothing under llama_lite_npu_amd/ may import this.

The reference has no fp8 path to follow (README.md:89 lists FP8 as not yet stabilized; its unused
int8 prefill kernel, lite_llama/kernels/others/context_flashattention_nopad.py:374-553, reads the
cache without scales), so this file restates the published format instead -- OCP 8-bit Floating
Point Specification (OFP8) v1.0, E4M3: 1 sign bit, 4 exponent bits with bias 7, 3 mantissa bits,
subnormals at exponent 0, largest finite value 448 (S.1111.110), S.1111.111 = NaN, no infinities;
conversion rounds to nearest even and saturates:
    encode(x, scale) = e4m3(clamp(x * (1 / scale), -448, 448))
    decode(code, scale) = value(code) * scale
Inputs that are not finite: +-Inf saturate to +-448; the clamp is maxNum(x, -448) then
minNum(., 448) (IEEE 754-2008: a quiet NaN operand is dropped), so NaN is stored as -448 (0xFE),
never as one of the format's NaN codes.
Numeric parity with the reference is **parity unpinned** (nothing to compare with).

Pinned in tests/test_oracle.py by: the closed form of all 256 code values; PyTorch's independent
float8_e4m3fn conversion on the CPU for every fp16 input in range (both directions); ties going to
the even code; saturation at +-448; decode(encode(v)) == v for every representable v; monotonicity;
the codes of NaN and +-Inf.
Attention over an fp8 pool is the fp16 oracle applied to the decoded pool (decoding is exact in
fp16 before the scale; the scale is applied in fp32).
"""

from __future__ import annotations

import numpy as np

FP8_MAX = 448.0


def code_values() -> np.ndarray:
    """float32 value of each of the 256 codes (NaN for 0x7f and 0xff)."""
    codes = np.arange(256)
    sign = np.where(codes & 0x80, -1.0, 1.0)
    e = (codes >> 3) & 0xF
    m = codes & 0x7
    normal = (1.0 + m / 8.0) * np.exp2(e - 7.0)
    sub = (m / 8.0) * np.exp2(-6.0)
    val = np.where(e == 0, sub, normal)
    val = np.where((e == 15) & (m == 7), np.nan, val)
    return (sign * val).astype(np.float32)


def encode(x: np.ndarray) -> np.ndarray:
    """float32 (already divided by the scale) -> uint8 codes: clamp to +-448, round to nearest even."""
    x = np.asarray(x, dtype=np.float32)
    x = np.fmin(np.fmax(x, np.float32(-FP8_MAX)), np.float32(FP8_MAX))   # maxNum / minNum: NaN -> -448
    a = np.abs(x.astype(np.float64))
    # spacing of the representable numbers around a: 2^(floor(log2 a) - 3), at least 2^-9
    with np.errstate(divide="ignore"):
        exp = np.floor(np.log2(np.where(a > 0, a, 1.0)))
    exp = np.clip(exp, -6, 8)
    quantum = np.exp2(exp - 3)
    steps = np.round(a / quantum)              # numpy rounds halves to even
    a_q = steps * quantum                      # may land on the next binade's first value: still exact
    a_q = np.minimum(a_q, FP8_MAX)
    # back to a code
    with np.errstate(divide="ignore"):
        e_q = np.floor(np.log2(np.where(a_q > 0, a_q, 1.0)))
    is_sub = a_q < np.exp2(-6.0)
    e_field = np.where(is_sub, 0, e_q + 7).astype(np.int64)
    m_field = np.where(is_sub, np.round(a_q / np.exp2(-9.0)), np.round((a_q / np.exp2(e_q) - 1.0) * 8.0)).astype(np.int64)
    code = (e_field << 3) | m_field
    code = np.where(np.signbit(x), code | 0x80, code)
    return code.astype(np.uint8)


def decode(codes: np.ndarray) -> np.ndarray:
    return code_values()[np.asarray(codes, dtype=np.uint8)]


def quantize_rows(rows: np.ndarray, scales: np.ndarray) -> np.ndarray:
    """rows [T, H, D] fp16, scales [H] fp32 -> codes [T, H, D] uint8 (x * (1/scale) in fp32, then encode)."""
    inv = (np.float32(1.0) / np.asarray(scales, dtype=np.float32)).astype(np.float32)
    y = rows.astype(np.float32) * inv[None, :, None]
    return encode(y.astype(np.float32))


def kv_append(k: np.ndarray, v: np.ndarray, slot_mapping: np.ndarray, pool: np.ndarray, scales: np.ndarray) -> None:
    """pool [slots, 2H, D] uint8, in place; slots outside the pool are skipped."""
    h = k.shape[1]
    codes = np.concatenate([quantize_rows(k, scales[:h]), quantize_rows(v, scales[h:])], axis=1)
    for t, slot in enumerate(np.asarray(slot_mapping)):
        if 0 <= slot < pool.shape[0]:
            pool[slot] = codes[t]


def dequantize_pool(pool: np.ndarray, scales: np.ndarray) -> np.ndarray:
    """codes [slots, 2H, D] -> float32 values (decode * scale in fp32)."""
    return decode(pool) * np.asarray(scales, dtype=np.float32)[None, :, None]
