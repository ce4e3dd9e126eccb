"""GPU parity of the fused QK-norm + RoPE + KV append against the numpy oracle, through the C ABI."""

import numpy as np
import pytest
import torch

from llama_lite_npu_amd import ops
from oracle import qk_epilogue
from tests.parity import to_np16

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
D = 128
# The kernel and the oracle round at the same points; what may differ is the last bit of the
# reciprocal square root. One fp16 ulp of the largest values seen here (|x| < 8) is 3.9e-3.
MAX_ABS = 4e-3
MIN_EXACT = 0.995


def _inputs(seed, t, hq, hkv, D=D):
    slots_in_pool = max(256, 2 * t)
    g = torch.Generator(device=DEV).manual_seed(seed)
    qkv = torch.randn((t, hq + 2 * hkv, D), generator=g, device=DEV, dtype=torch.float16) * 1.7
    q, k, v = qkv[:, :hq], qkv[:, hq:hq + hkv], qkv[:, hq + hkv:]        # strided views, as after a fused projection
    wq = (1.0 + 0.2 * torch.randn(D, generator=g, device=DEV)).half()
    wk = (1.0 + 0.2 * torch.randn(D, generator=g, device=DEV)).half()
    pos = torch.randint(0, 8192, (t,), generator=g, device=DEV).double()
    inv = 10000.0 ** (-torch.arange(0, D, 2, device=DEV, dtype=torch.float64) / D)
    emb = torch.cat([pos[:, None] * inv[None, :]] * 2, dim=1)
    cos, sin = emb.cos().half(), emb.sin().half()
    pool = torch.randn((slots_in_pool, 2 * hkv, D), generator=g, device=DEV, dtype=torch.float16)
    slots = torch.randperm(slots_in_pool, generator=g, device=DEV)[:t].to(torch.int32)
    return q, k, v, wq, wk, cos, sin, pool, slots


def _check(got16, want16, what):
    got, want = got16.astype(np.float32), want16.astype(np.float32)
    assert np.isfinite(got).all(), what
    diff = np.abs(got - want)
    exact = float((got16 == want16).mean())
    assert diff.max() <= MAX_ABS and exact >= MIN_EXACT, f"{what}: max abs {diff.max():.3e}, exact {exact:.4f}"


@pytest.mark.parametrize("t,hq,hkv,norm,rope", [
    (33, 64, 8, True, True),        # Qwen3-32B decode-sized batch
    (1, 16, 8, True, True),
    (300, 32, 4, True, True),
    (17, 28, 4, False, True),       # models without QK norm
    (9, 16, 1, True, False),
    (5, 8, 8, False, False),        # degenerates to the plain append
])
def test_fused_epilogue_matches_oracle(t, hq, hkv, norm, rope):
    _epilogue_case(t, hq, hkv, norm, rope, D)


@pytest.mark.parametrize("head_dim", [64, 32, 256])
@pytest.mark.parametrize("t,hq,hkv,norm,rope", [(33, 14, 2, True, True), (7, 16, 8, False, True), (9, 8, 1, True, False)])
def test_fused_epilogue_other_head_dims(head_dim, t, hq, hkv, norm, rope):
    _epilogue_case(t, hq, hkv, norm, rope, head_dim)


@pytest.mark.parametrize("head_dim,t,hq,hkv", [(128, 3301, 64, 8), (256, 4101, 16, 8), (64, 5465, 64, 8), (32, 8197, 64, 8)])
def test_fused_epilogue_prefill_sized(head_dim, t, hq, hkv):
    """Launches large enough for the kernel's other shape (four tokens per lane instead of one),
    with a token count that leaves the last group partly filled."""
    _epilogue_case(t, hq, hkv, True, True, head_dim)


def _epilogue_case(t, hq, hkv, norm, rope, head_dim):
    print(f"qk epilogue T={t} {hq}/{hkv} norm={norm} rope={rope} head_dim={head_dim}", flush=True)
    q, k, v, wq, wk, cos, sin, pool, slots = _inputs(900 + t, t, hq, hkv, head_dim)
    slots[t // 2] = -1                              # a padding row: q still processed, nothing stored
    if t > 3:
        slots[3] = pool.shape[0] + 5
    q_in, pool_in = to_np16(q), to_np16(pool)
    want_q, want_pool = qk_epilogue.qk_norm_rope_append(
        q_in, to_np16(k), to_np16(v), slots.cpu().numpy(), pool_in,
        to_np16(wq) if norm else None, to_np16(wk) if norm else None,
        to_np16(cos) if rope else None, to_np16(sin) if rope else None, 1e-6)
    k_before, v_before = k.clone(), v.clone()
    out = ops.qk_norm_rope_append(q, k, v, slots, pool, wq if norm else None, wk if norm else None,
                                  cos if rope else None, sin if rope else None, 1e-6)
    torch.cuda.synchronize()
    assert out.data_ptr() == q.data_ptr()
    assert torch.equal(k, k_before) and torch.equal(v, v_before)      # inputs of the append are not touched
    _check(to_np16(q), want_q, "q")
    got_pool = to_np16(pool)
    _check(got_pool[:, :hkv], want_pool[:, :hkv], "k rows in the pool")
    assert np.array_equal(got_pool[:, hkv:], want_pool[:, hkv:]), "v rows and untouched slots are bit exact"
    valid = slots.cpu().numpy()
    valid = valid[(valid >= 0) & (valid < pool.shape[0])]
    untouched = np.setdiff1d(np.arange(pool.shape[0]), valid)
    assert np.array_equal(got_pool[untouched], pool_in[untouched])
    if not norm and not rope:
        assert np.array_equal(got_pool, want_pool) and np.array_equal(to_np16(q), q_in)


def test_fused_epilogue_feeds_decode_like_separate_append():
    """k written by the fused launch == rope'd k appended with kv_append (same bits)."""
    print("qk epilogue vs separate append", flush=True)
    q, k, v, wq, wk, cos, sin, pool, slots = _inputs(950, 40, 16, 8)
    pool2 = pool.clone()
    k_ref = torch.from_numpy(qk_epilogue.rope(qk_epilogue.rms_norm(to_np16(k), to_np16(wk), 1e-6),
                                             to_np16(cos), to_np16(sin))).to(DEV)
    ops.kv_append(k_ref, v.contiguous(), slots, pool2)
    ops.qk_norm_rope_append(q, k, v, slots, pool, wq, wk, cos, sin, 1e-6)
    torch.cuda.synchronize()
    same = float((pool == pool2).float().mean())
    assert same >= MIN_EXACT and float((pool.float() - pool2.float()).abs().max()) <= MAX_ABS
