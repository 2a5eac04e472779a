"""Pins the CPU oracle (oracle/oracle.c) before anything is compared with it.

Each oracle function is checked against (1) the known-answer vectors held by the reference's
own tests (tests/golden/reference_kats.json) and (2) independent mathematics chosen so that a
plausible mistake (dropped term, wrong sign/index, transposed operand) fails: float64 brute
force, closed forms, invariants, numpy/torch library routines.
"""
import json
import os

import numpy as np
import pytest

import oracle

GOLDEN = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_kats.json")))


def ulp_close(a, b, ulps=4):
    """gtest's EXPECT_FLOAT_EQ: within 4 units in the last place."""
    a = np.asarray(a, np.float32)
    b = np.asarray(b, np.float32)
    ai = a.view(np.int32).astype(np.int64)
    bi = b.view(np.int32).astype(np.int64)
    ai = np.where(ai < 0, -(ai & 0x7FFFFFFF), ai)
    bi = np.where(bi < 0, -(bi & 0x7FFFFFFF), bi)
    return np.all(np.abs(ai - bi) <= ulps)


# ------------------------------------------------------------------ RmsNormalization

def test_rms_kat_iota():
    x = np.arange(24, dtype=np.float32).reshape(2, 3, 4)
    w = np.array([1, 2, 3, 4], dtype=np.float32)
    y = oracle.rms_norm(x, w, 0.0)
    # the reference test's inline formula, evaluated in float64
    ref = np.zeros_like(x, dtype=np.float64)
    for i in range(6):
        row = x.reshape(6, 4)[i].astype(np.float64)
        rms = 1.0 / np.sqrt((row * row).sum() / 4) if (row * row).sum() else np.inf
        ref.reshape(6, 4)[i] = row * rms * w
    assert ulp_close(y.reshape(-1)[4:], ref.astype(np.float32).reshape(-1)[4:])


def test_rms_kat_constant_row():
    x = np.full((2, 3, 4096), 2.0, np.float32)
    w = np.full((4096,), 3.0, np.float32)
    y = oracle.rms_norm(x, w, 0.0)
    assert np.all(y == 3.0)


def test_rms_recorded_vector():
    rec = [c for c in GOLDEN["rms_normalization"] if c["kind"] == "recorded"][0]
    y = oracle.rms_norm(np.array(rec["x"], np.float32).reshape(rec["shape"]),
                        np.array(rec["w"], np.float32), rec["eps"])
    assert ulp_close(y.reshape(-1), np.array(rec["expect"], np.float32), ulps=1)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
def test_rms_against_float64_brute_force_and_invariants(dtype):
    rng = np.random.default_rng(1)
    x = rng.standard_normal((7, 5, 333)).astype(dtype)
    w = rng.uniform(0.5, 1.5, 333).astype(dtype)
    eps = 1e-5
    y = oracle.rms_norm(x, w, eps)
    x64, w64 = x.astype(np.float64), w.astype(np.float64)
    ms = (x64 * x64).mean(-1, keepdims=True)
    ref = x64 / np.sqrt(ms + np.float64(np.float32(eps))) * w64
    tol = 1e-5 if dtype == np.float32 else 1e-12
    assert np.all(np.abs(y - ref) <= tol * np.abs(ref) + 1e-30)
    # invariant: sum_j (y_j / w_j)^2 == D * ms / (ms + eps)
    lhs = ((y.astype(np.float64) / w64) ** 2).sum(-1)
    rhs = 333 * ms[..., 0] / (ms[..., 0] + eps)
    assert np.allclose(lhs, rhs, rtol=1e-4 if dtype == np.float32 else 1e-10)
    # threads do not change a bit
    assert np.array_equal(y, oracle.rms_norm(x, w, eps, threads=3))


def test_rms_serial_float_accumulation_is_followed():
    # 2^24 + 1 is not representable: a serial float sum of ones saturates, a pairwise one does not
    # (cols chosen so the per-row serial sum of squares hits the float spacing).
    x = np.ones((1, 1 << 12), np.float32) * np.float32(4096.0)  # x^2 = 2^24
    x[0, 1:] = 1.0  # every later addend (1.0) is below half the spacing of 2^24 -> absorbed
    y = oracle.rms_norm(x, np.ones(1 << 12, np.float32), 0.0)
    expect_first = np.float32(4096.0) * np.float32(1.0 / np.sqrt(np.float64(np.float32(2.0 ** 24) / np.float32(4096))))
    assert y[0, 0] == expect_first


# ------------------------------------------------------------------ Softmax

def test_softmax_kat_zeros_axis1_f64():
    c = GOLDEN["softmax"][0]
    x = np.zeros(c["shape"], np.float64)
    y = oracle.softmax(x, axis=c["axis"])
    assert np.all(y == 1.0 / 3)


def test_softmax_literal_defect_vectors():
    for case in GOLDEN["softmax"][1]["cases"]:
        y = oracle.softmax_literal(np.array(case["x"], np.float32))
        assert np.allclose(y, case["expect"], atol=5e-5)
        # and the corrected oracle deliberately differs (it is a true softmax)
        z = oracle.softmax(np.array(case["x"], np.float32))
        assert abs(z.sum() - 1) < 1e-6 and not np.allclose(y, z, atol=1e-3)


@pytest.mark.parametrize("dtype", [np.float32, np.float64])
@pytest.mark.parametrize("axis", [0, 1, 2, 3])
def test_softmax_against_float64_textbook_all_axes(dtype, axis):
    rng = np.random.default_rng(3)
    x = (3 * rng.standard_normal((3, 4, 5, 6))).astype(dtype)
    y = oracle.softmax(x, axis=axis)
    x64 = x.astype(np.float64)
    e = np.exp(x64 - x64.max(axis=axis, keepdims=True))
    ref = e / e.sum(axis=axis, keepdims=True)
    assert np.allclose(y, ref, rtol=2e-6 if dtype == np.float32 else 1e-14, atol=0)
    assert np.allclose(y.sum(axis=axis), 1.0, atol=1e-6)
    # shift invariance and thread independence
    assert np.allclose(oracle.softmax((x + dtype(7)).astype(dtype), axis=axis), y, rtol=1e-5)
    assert np.array_equal(y, oracle.softmax(x, axis=axis, threads=4))


def test_softmax_matches_torch_library():
    import torch
    rng = np.random.default_rng(4)
    x = (3 * rng.standard_normal((2, 3, 64, 257))).astype(np.float32)
    ref = torch.softmax(torch.from_numpy(x).double(), dim=-1).numpy()
    assert np.allclose(oracle.softmax(x), ref, rtol=3e-6, atol=1e-12)


def test_softmax_causal_equals_data_masked_and_structure():
    rng = np.random.default_rng(5)
    for rows, cols in [(6, 6), (4, 9), (1, 5)]:
        x = (3 * rng.standard_normal((2, 3, rows, cols))).astype(np.float32)
        y = oracle.softmax_causal(x)
        masked = x.copy()
        r = np.arange(rows)[:, None]
        c = np.arange(cols)[None, :]
        masked[..., c > r + (cols - rows)] = -np.inf
        assert np.array_equal(y, oracle.softmax(masked))  # exp(-inf) = 0 exactly, sums identical
        assert np.all(y[..., c > r + (cols - rows)] == 0)
        if rows == cols:
            assert np.all(y[..., 0, 0] == 1.0)  # row 0 is one-hot
        assert np.allclose(y.sum(-1), 1.0, atol=1e-6)


# ------------------------------------------------------------------ MatMulInteger

def _i8(a, zp, signed):
    """mathematical restatement: difference modulo 256 read as int8."""
    if signed:
        d = a.astype(np.int8).astype(np.int64) - np.asarray(zp).astype(np.int8).astype(np.int64)
    else:
        d = a.astype(np.uint8).astype(np.int64) - np.asarray(zp).astype(np.uint8).astype(np.int64)
    return ((d + 128) % 256) - 128


def test_matmul_integer_kats():
    k0, k1, k2, k3 = GOLDEN["mat_mul_integer"]
    y = oracle.matmul_integer(np.array(k0["a"], np.uint8).reshape(k0["a_shape"]),
                              np.array(k0["b"], np.uint8).reshape(k0["b_shape"]))
    assert y.reshape(-1).tolist() == k0["expect"]
    a = np.arange(1, 5, dtype=np.uint8).reshape(1, 4)
    b = np.tile(np.arange(1, 13, dtype=np.uint8), (4, 1))
    assert oracle.matmul_integer(a, b).reshape(-1).tolist() == [10 * i for i in range(1, 13)]
    for rec in (k2, k3):
        a = np.array(rec["a"], np.uint8).reshape(rec["a_shape"])
        b = np.array(rec["b"], np.int8).reshape(rec["b_shape"])
        az = np.array([rec["a_zp"]], np.uint8) if "a_zp" in rec else None
        bz = np.array([rec["b_zp"]], np.int8) if "b_zp" in rec else None
        assert oracle.matmul_integer(a, b, az, bz).reshape(-1).tolist() == rec["expect"]


def test_matmul_integer_against_int64_brute_force():
    rng = np.random.default_rng(5)
    a = rng.integers(0, 256, (37, 53), dtype=np.uint8)
    b = rng.integers(-128, 128, (53, 29), dtype=np.int8)
    az = np.array([128], np.uint8)
    bz = np.array([0], np.int8)
    y = oracle.matmul_integer(a, b, az, bz, threads=3)
    ref = (a.astype(np.int64) - 128) @ b.astype(np.int64)
    assert np.array_equal(y, ref)
    # a - 128 == int8(a ^ 0x80): the identity the HIP kernel's fused zero point relies on
    assert np.array_equal((a ^ 0x80).view(np.int8).astype(np.int64), a.astype(np.int64) - 128)
    # non-square, transposition-sensitive: A @ B != (B.T @ A.T) unless transposed back
    assert not np.array_equal(y, ref.T.copy().reshape(ref.shape)) or ref.shape[0] == ref.shape[1]


def test_matmul_integer_extremes_and_wrap():
    a = np.full((2, 4096), 0, np.uint8)      # a - 128 = -128
    b = np.full((4096, 3), -128, np.int8)
    y = oracle.matmul_integer(a, b, np.array([128], np.uint8), None)
    assert np.all(y == 2 ** 26)
    # outside the representable range the reference WRAPS (255 - 1 = 254 -> -2), it does not saturate
    a = np.array([[255, 0]], np.uint8)
    b = np.array([[1], [1]], np.int8)
    y = oracle.matmul_integer(a, b, np.array([1], np.uint8), None)
    assert y.item() == (-2) + (-1)


def test_matmul_integer_zero_point_variants_and_broadcast():
    rng = np.random.default_rng(6)
    a = rng.integers(0, 256, (2, 1, 5, 7), dtype=np.uint8)
    b = rng.integers(0, 256, (1, 3, 7, 4), dtype=np.uint8)
    # per-row zero point for A: one per (batch, row); for B as written: one per (batch, row of B)
    az = rng.integers(0, 256, (2 * 5,), dtype=np.uint8)
    bz = rng.integers(-128, 128, (3 * 7,), dtype=np.int8)  # I8 zero point => B bytes read signed
    y = oracle.matmul_integer(a, b, az, bz)
    A = _i8(a, az.reshape(2, 1, 5, 1), signed=False)
    B = _i8(b, bz.reshape(1, 3, 7, 1), signed=True)
    ref = np.einsum("abik,abkj->abij", np.broadcast_to(A, (2, 3, 5, 7)), np.broadcast_to(B, (2, 3, 7, 4)))
    assert y.shape == (2, 3, 5, 4) and np.array_equal(y, ref)


# ------------------------------------------------------------------ DequantizeLinear

def test_dequantize_kat():
    c = GOLDEN["dequantize_linear"][0]
    y = oracle.dequantize_linear(np.array(c["x"], np.uint8), np.float32(c["scale"]), np.array([c["zp"]], np.uint8))
    assert y.tolist() == c["expect"]


@pytest.mark.parametrize("dt", [np.uint8, np.int8, np.uint16, np.int16, np.int32])
def test_dequantize_scalar_and_per_axis_closed_form(dt):
    rng = np.random.default_rng(7)
    info = np.iinfo(dt)
    lo, hi = max(info.min, -(1 << 20)), min(info.max, 1 << 20)
    x = rng.integers(lo, hi + 1, (3, 5, 4), dtype=dt)
    zp1 = rng.integers(lo, hi + 1, (1,), dtype=dt)
    s1 = np.float32(0.0123)
    y = oracle.dequantize_linear(x, s1, zp1)
    ref = (x.astype(np.int64) - int(zp1[0])).astype(np.float32) * s1
    assert np.array_equal(y, ref)
    for axis in (0, 1, 2):
        n = x.shape[axis]
        s = rng.uniform(1e-3, 1e-2, n).astype(np.float32)
        zp = rng.integers(lo, hi + 1, (n,), dtype=dt)
        shape = [1, 1, 1]
        shape[axis] = n
        ref = (x.astype(np.int64) - zp.astype(np.int64).reshape(shape)).astype(np.float32) * s.reshape(shape)
        assert np.array_equal(oracle.dequantize_linear(x, s, zp, axis=axis, threads=2), ref)
        assert np.array_equal(oracle.dequantize_linear(x, s, None, axis=axis),
                              x.astype(np.float32) * s.reshape(shape))


# ------------------------------------------------------------------ DynamicQuantizeLinear

def test_dynamic_quantize_kats():
    c = GOLDEN["dynamic_quantize_linear"][0]
    y, scale, zp = oracle.dynamic_quantize_linear(np.array(c["x"], np.float32))
    assert scale == np.float32(c["scale_num"]) / np.float32(c["scale_den"])
    assert zp == c["zp"] and y.tolist() == c["expect_y"]
    c = GOLDEN["dynamic_quantize_linear"][1]
    x = (3 * np.arange(20) + 15).astype(np.float32)
    y, scale, zp = oracle.dynamic_quantize_linear(x)
    assert scale == np.float32(c["scale_num"]) / np.float32(c["scale_den"]) and zp == c["zp"]
    q = x / scale
    assert np.all(np.abs(q - np.round(q)) != 0.5)  # no ties: numpy's rounding rule does not matter here
    assert np.array_equal(y, np.round(q).astype(np.uint8)) and y[-1] == 255


def test_dynamic_quantize_properties():
    rng = np.random.default_rng(31)
    for lo, hi in [(-3.0, 5.0), (0.5, 9.0), (-7.0, -0.25), (-1e-3, 2e-3)]:
        x = rng.uniform(lo, hi, 4097).astype(np.float32)
        x[17] = 0.0
        y, scale, zp = oracle.dynamic_quantize_linear(x)
        mn, mx = min(float(x.min()), 0.0), max(float(x.max()), 0.0)
        assert scale == np.float32(np.float32(mx) - np.float32(mn)) / np.float32(255)
        # the zero point is where 0 lands, and the ends of the covered range land on 0 and 255
        assert y[17] == zp
        assert zp == int(np.clip(np.floor(-mn / float(scale) + 0.5), 0, 255))
        assert y.min() == (0 if lo < 0 else y.min()) and y.max() == (255 if hi > 0 else y.max())
        # float64 recomputation: equal except for values within rounding noise of a tie
        q64 = np.clip(np.floor(np.abs(x.astype(np.float64) / float(scale)) + 0.5) * np.sign(x) + int(zp), 0, 255)
        assert np.max(np.abs(y.astype(np.int64) - q64.astype(np.int64))) <= 1
        assert np.mean(y == q64.astype(np.uint8)) > 0.999
        # dequantising recovers x to half a step
        back = (y.astype(np.float64) - int(zp)) * float(scale)
        inside = (x >= mn) & (x <= mx)
        assert np.max(np.abs(back - x)[inside]) <= 0.5 * float(scale) * (1 + 1e-5)


def test_dynamic_quantize_rounds_half_away_and_saturates():
    # scale exactly 1, zero point 0: ties must go away from zero (2.5 -> 3, 0.5 -> 1), not to even
    x = np.array([0.0, 255.0, 2.5, 0.5, 1.5, 254.5], np.float32)
    y, scale, zp = oracle.dynamic_quantize_linear(x)
    assert scale == 1.0 and zp == 0 and y.tolist() == [0, 255, 3, 1, 2, 255]
    # zero point saturates at 255 for an all-negative input; an all-zero input stays all zero
    y, scale, zp = oracle.dynamic_quantize_linear(np.array([-4.0, -2.0, -1.0], np.float32))
    assert zp == 255 and y.tolist() == [0, 128, 191] and scale == np.float32(4) / np.float32(255)
    y, scale, zp = oracle.dynamic_quantize_linear(np.zeros(9, np.float32))
    # the running maximum starts at the smallest normal float, which keeps the range positive
    assert scale == np.float32(np.finfo(np.float32).tiny) / np.float32(255) and zp == 0 and not y.any()


# ------------------------------------------------------------------ MatMul / Mul (oracle blocks)

def test_matmul_f32_exact_on_integer_operands_and_transb():
    rng = np.random.default_rng(8)
    a = rng.integers(-8, 9, (5, 11)).astype(np.float32)
    b = rng.integers(-8, 9, (11, 7)).astype(np.float32)
    assert np.array_equal(oracle.matmul_f32(a, b), (a.astype(np.float64) @ b.astype(np.float64)).astype(np.float32))
    bt = np.ascontiguousarray(b.T)
    assert np.array_equal(oracle.matmul_f32(a, bt, trans_b=True), oracle.matmul_f32(a, b))
    assert np.array_equal(oracle.matmul_f32(a, b, alpha=0.5), 0.5 * oracle.matmul_f32(a, b))
    assert np.array_equal(oracle.mul_f32(a, np.float32(0.25)), a * np.float32(0.25))


# ------------------------------------------------------------------ Attention (parity unpinned by the reference)

def _attention_f64(q, kc, vc, past, scale):
    seq = q.shape[0]
    s = (q.astype(np.float64) @ kc.astype(np.float64).T) * scale
    cols = np.arange(past + seq)[None, :]
    rows = np.arange(seq)[:, None]
    s[cols > past + rows] = -np.inf
    p = np.exp(s - s.max(-1, keepdims=True))
    p /= p.sum(-1, keepdims=True)
    return p @ vc.astype(np.float64)


def test_attention_head_vs_float64_brute_force_tiny():
    rng = np.random.default_rng(9)
    for seq, past, D in [(1, 0, 8), (1, 5, 8), (4, 3, 8), (7, 0, 16)]:
        q = rng.standard_normal((seq, D)).astype(np.float32)
        kc = rng.standard_normal((past + seq, D)).astype(np.float32)
        vc = rng.standard_normal((past + seq, D)).astype(np.float32)
        o = oracle.attention_head(q, kc, vc, past, 1 / np.sqrt(D))
        assert np.allclose(o, _attention_f64(q, kc, vc, past, 1 / np.sqrt(D)), rtol=1e-5, atol=1e-6)


def test_attention_invariants():
    rng = np.random.default_rng(10)
    D = 16
    # seq=1, past=0 => O = V
    q = rng.standard_normal((1, D)).astype(np.float32)
    k = rng.standard_normal((1, D)).astype(np.float32)
    v = rng.standard_normal((1, D)).astype(np.float32)
    assert np.array_equal(oracle.attention_head(q, k, v, 0, 0.25), v)
    # uniform K => O = mean(V)
    L = 9
    kc = np.tile(k, (L, 1))
    vc = rng.standard_normal((L, D)).astype(np.float32)
    o = oracle.attention_head(q, kc, vc, L - 1, 0.25)
    assert np.allclose(o[0], vc.mean(0), rtol=1e-5, atol=1e-6)
    # permuting past positions leaves a decode output unchanged (up to summation order)
    kc = rng.standard_normal((L, D)).astype(np.float32)
    perm = np.concatenate([rng.permutation(L - 1), [L - 1]])
    o1 = oracle.attention_head(q, kc, vc, L - 1, 0.25)
    o2 = oracle.attention_head(q, kc[perm], vc[perm], L - 1, 0.25)
    assert np.allclose(o1, o2, rtol=1e-5, atol=1e-6)


def test_attention_kvcache_vs_torch_sdpa_gqa():
    import torch
    rng = np.random.default_rng(11)
    N, H, Hkv, seq, D, S = 2, 4, 2, 3, 8, 10
    q = rng.standard_normal((N, H, seq, D)).astype(np.float32)
    k = rng.standard_normal((N, Hkv, seq, D)).astype(np.float32)
    v = rng.standard_normal((N, Hkv, seq, D)).astype(np.float32)
    kc = rng.standard_normal((N, Hkv, S, D)).astype(np.float32)
    vc = rng.standard_normal((N, Hkv, S, D)).astype(np.float32)
    past = np.array([4, 6])
    o, kco, vco = oracle.attention_kvcache(q, k, v, kc, vc, past, 1 / np.sqrt(D))
    for b in range(N):
        p = past[b]
        assert np.array_equal(kco[b, :, p:p + seq], k[b]) and np.array_equal(vco[b, :, p:p + seq], v[b])
        assert np.array_equal(kco[b, :, :p], kc[b, :, :p]) and np.array_equal(kco[b, :, p + seq:], kc[b, :, p + seq:])
        L = p + seq
        mask = torch.ones(seq, L, dtype=torch.bool).tril(diagonal=int(p))
        kk = torch.from_numpy(kco[b, :, :L]).repeat_interleave(H // Hkv, dim=0)
        vv = torch.from_numpy(vco[b, :, :L]).repeat_interleave(H // Hkv, dim=0)
        ref = torch.nn.functional.scaled_dot_product_attention(
            torch.from_numpy(q[b]).double(), kk.double(), vv.double(), attn_mask=mask)
        assert np.allclose(o[b], ref.numpy(), rtol=1e-5, atol=1e-6)


# ------------------------------------------------------------------ RoPE (parity unpinned by the reference)

def _rope_hf_f64(x, pos, theta):
    """Independent HF-style rotate_half formulation in float64."""
    D = x.shape[-1]
    inv = 1.0 / (theta ** (np.arange(0, D, 2, dtype=np.float64) / D))
    ang = pos[..., None].astype(np.float64) * inv           # [B, S, D/2]
    emb = np.concatenate([ang, ang], -1)[:, :, None, :]      # [B, S, 1, D]
    x64 = x.astype(np.float64)
    rot = np.concatenate([-x64[..., D // 2:], x64[..., :D // 2]], -1)
    return x64 * np.cos(emb) + rot * np.sin(emb)


def test_rope_vs_independent_float64_and_invariants():
    rng = np.random.default_rng(12)
    B, S, H, D = 2, 50, 3, 16
    x = rng.standard_normal((B, S, H, D)).astype(np.float32)
    pos = np.tile(np.arange(S, dtype=np.int64), (B, 1))
    y = oracle.rope(x, pos, 10000.0)
    assert np.allclose(y, _rope_hf_f64(x, pos, 10000.0), atol=2e-5)
    # [seq] positions broadcast over batch
    assert np.array_equal(y, oracle.rope(x, pos[0], 10000.0))
    # pos 0 => identity
    assert np.array_equal(oracle.rope(x, np.zeros((B, S), np.int64)), x)
    # pairwise norm preserved
    n_in = x[..., :D // 2] ** 2 + x[..., D // 2:] ** 2
    n_out = y[..., :D // 2] ** 2 + y[..., D // 2:] ** 2
    assert np.allclose(n_in, n_out, rtol=1e-5, atol=1e-6)
    # R(p1) R(p2) = R(p1 + p2); inverse by negated position
    p1 = rng.integers(0, 100, (B, S)).astype(np.int64)
    p2 = rng.integers(0, 100, (B, S)).astype(np.int64)
    assert np.allclose(oracle.rope(oracle.rope(x, p1), p2), oracle.rope(x, p1 + p2), atol=1e-4)
    assert np.allclose(oracle.rope(oracle.rope(x, p1), -p1), x, atol=1e-5)
    # large positions (the config's range) still within 1e-3 of float64 angles
    big = np.full((B, S), 2047, np.int64)
    assert np.allclose(oracle.rope(x, big), _rope_hf_f64(x, big, 10000.0), atol=1e-3)
    assert np.array_equal(oracle.rope(x, p1, threads=4), oracle.rope(x, p1))


# ------------------------------------------------------------------ Cast
def test_cast_reference_kat():
    # src/04kernel/test/kernels/cast/test_cpu.cpp: F64 iota [2,3,4,5] -> I8, y[i] == i
    c = GOLDEN["cast"][0]
    x = np.arange(120, dtype=np.float64).reshape(c["shape"])
    y = oracle.cast(x, c["from"], c["to"])
    assert y.dtype == np.int8 and np.array_equal(y.reshape(-1), np.arange(120))


def test_cast_integer_and_bool_rules_against_python_arithmetic():
    rng = np.random.default_rng(3)
    v = rng.integers(-2 ** 63, 2 ** 63, 500, dtype=np.int64)
    for name, bits, signed in (("u8", 8, False), ("i8", 8, True), ("u16", 16, False), ("i16", 16, True),
                               ("u32", 32, False), ("i32", 32, True), ("u64", 64, False)):
        want = [(int(t) % (1 << bits)) - ((1 << bits) if signed and (int(t) % (1 << bits)) >= (1 << (bits - 1)) else 0)
                for t in v]
        assert oracle.cast(v, "i64", name).tolist() == want                      # narrowing wraps modulo 2^bits
    f = np.array([-2.9, -0.5, 0.0, 0.5, 2.9, 126.99], np.float64)
    assert oracle.cast(f, "f64", "i8").tolist() == [int(t) for t in f]           # truncation toward zero
    assert oracle.cast(f, "f64", "bool").tolist() == [t != 0 for t in f]
    assert oracle.cast(np.array([0, 1, 1, 0], np.bool_), "bool", "f32").tolist() == [0.0, 1.0, 1.0, 0.0]
    big = np.array([2 ** 24 + 1, 2 ** 24 + 3, -(2 ** 24 + 1), 2 ** 53 + 1], np.int64)
    import struct
    want = [struct.unpack("f", struct.pack("f", float(int(t))))[0] for t in big[:3]]   # struct rounds to nearest even
    assert oracle.cast(big[:3], "i64", "f32").tolist() == want
    assert oracle.cast(big[3:], "i64", "f64").tolist() == [float(2 ** 53)]


def _nearest_narrow(value, mant_bits, emin, emax):
    """value (Fraction) rounded to nearest-even in a binary format with `mant_bits` explicit
    mantissa bits and exponent range [emin, emax]; returns a Fraction or inf."""
    from fractions import Fraction
    if value == 0:
        return Fraction(0)
    sign = -1 if value < 0 else 1
    a = abs(value)
    e = 0
    while Fraction(2) ** (e + 1) <= a:
        e += 1
    while Fraction(2) ** e > a:
        e -= 1
    e = max(e, emin)
    ulp = Fraction(2) ** (e - mant_bits)
    q, r = divmod(a, ulp)
    if r * 2 > ulp or (r * 2 == ulp and q % 2 == 1):
        q += 1
    out = q * ulp
    if out >= Fraction(2) ** (emax + 1):
        return sign * float("inf")
    return sign * out


def test_cast_to_fp16_and_bf16_round_to_nearest_even_against_exact_arithmetic():
    from fractions import Fraction
    rng = np.random.default_rng(4)
    x = np.concatenate([rng.standard_normal(300).astype(np.float32) * 100,
                        np.array([2049., 2051., 65519.9, 65520., 1e-7, 6e-8, -3e-8, 0.0], np.float32),
                        np.array([0x3F808000, 0x3F818000, 0x3F808001], np.uint32).view(np.float32)])
    h = oracle.cast(x, "f32", "fp16")
    b = oracle.cast(x, "f32", "bf16")
    for i, t in enumerate(x):
        want_h = _nearest_narrow(Fraction(float(t)), 10, -14, 15)
        assert float(h[i]) == float(want_h), (t, h[i], want_h)
        want_b = _nearest_narrow(Fraction(float(t)), 7, -126, 127)
        got_b = float((np.uint32(b[i]) << 16).view(np.float32))
        assert got_b == float(want_b), (t, got_b, want_b)
    # a double goes through float first (reference: __float2half(double argument)): 1 + 2^-11 + 2^-26
    # rounds to the tie 1 + 2^-11 in float and then to 1.0, where a single rounding would give 1 + 2^-10
    assert oracle.cast(np.array([1 + 2.0 ** -11 + 2.0 ** -26]), "f64", "fp16").view(np.uint16).tolist() == [0x3C00]


def test_cast_integers_to_fp16_bf16_go_through_int_and_round_toward_zero():
    assert oracle.cast(np.array([2049, 2051, -2049, 70000, -70000, 16777217], np.int32), "i32", "fp16").tolist() == \
        [2048.0, 2050.0, -2048.0, 65504.0, -65504.0, 65504.0]
    assert oracle.cast(np.array([257, -257, 16777217, 2 ** 31 - 1], np.int32), "i32", "bf16").tolist() == \
        [0x4380, 0xC380, 0x4B80, 0x4EFF]
    # the value is taken as `int`: 3e9 as uint32 is negative as int
    assert oracle.cast(np.array([3000000000], np.uint32), "u32", "fp16").tolist() == [-65504.0]
    # and back: truncated as int, then converted to the target like any int (wraps)
    assert oracle.cast(np.array([-1.5, 2.9, 300.7], np.float16), "fp16", "u8").tolist() == [255, 2, 44]
    assert oracle.cast(np.array([0x4380, 0xC3A0], np.uint16), "bf16", "i16").tolist() == [256, -320]


def test_cast_bool_from_floating_sources_reference_defect_fixture():
    x = np.array([0.0, 1.5, -0.0], np.float32)
    assert oracle.cast(x, "f32", "bool").tolist() == [False, True, False]
    assert oracle.cast_bool_reference_literal(x, "f32").tolist() == [True, False, True]   # not reproduced


# ------------------------------------------------------------------ MatMul (with bias, transposes, broadcast)
def test_matmul_reference_vectors():
    for c in GOLDEN["mat_mul"]:
        if "y" not in c:
            continue
        a = np.array(c["a"], np.float32).reshape(c["a_shape"])
        b = np.array(c["b"], np.float32).reshape(c["b_shape"])
        bias = np.array(c["c"], np.float32).reshape(c["c_shape"])
        y = oracle.matmul(a, b, bias, alpha=c["alpha"], beta=c["beta"])
        assert y.reshape(-1).tolist() == c["y"]


def test_matmul_against_exact_integer_arithmetic():
    # integer-valued operands: every product and partial sum is exact in float32, so numpy's int64
    # product is the exact answer for any transposition, alpha, beta and bias broadcast
    rng = np.random.default_rng(12)
    for ta in (False, True):
        for tb in (False, True):
            m, k, n = 5, 7, 3
            a = rng.integers(-8, 9, (2, 1) + ((k, m) if ta else (m, k))).astype(np.float32)
            b = rng.integers(-8, 9, (1, 3) + ((n, k) if tb else (k, n))).astype(np.float32)
            bias = rng.integers(-8, 9, (m, 1)).astype(np.float32)
            A = np.swapaxes(a, -1, -2) if ta else a
            B = np.swapaxes(b, -1, -2) if tb else b
            want = 2 * (A.astype(np.int64) @ B.astype(np.int64)) + 3 * bias.astype(np.int64)
            got = oracle.matmul(a, b, bias, ta, tb, alpha=2.0, beta=3.0)
            assert got.shape == (2, 3, m, n) and np.array_equal(got, want.astype(np.float32))
            got64 = oracle.matmul(a.astype(np.float64), b.astype(np.float64), bias.astype(np.float64), ta, tb, 2.0, 3.0, "f64")
            assert np.array_equal(got64, want.astype(np.float64))
    # without bias beta does not enter
    a, b = np.eye(4, dtype=np.float32), np.arange(16, dtype=np.float32).reshape(4, 4)
    assert np.array_equal(oracle.matmul(a, b, None, beta=5.0), b)


def test_matmul_fp16_rounds_alpha_and_the_result_once():
    a = np.array([[1.0, 2.0 ** -11]], np.float16)
    b = np.array([[1.0], [1.0]], np.float16)
    # the sum 1 + 2^-11 is exact in float and a tie in fp16: one rounding to even gives 1.0
    assert oracle.matmul(a, b, dtype="fp16").view(np.uint16).tolist() == [[0x3C00]]
    # alpha = 1 + 2^-12 is not an fp16 number: it is 1.0 after the conversion the reference applies
    assert oracle.matmul(np.array([[3.0]], np.float16), np.array([[1.0]], np.float16), alpha=1 + 2.0 ** -12,
                         dtype="fp16").tolist() == [[3.0]]


# ------------------------------------------------------------------ Transpose

def test_transpose_digest_reference_vectors():
    for c in GOLDEN["transpose_info"]["cases"]:
        dims, block, count = oracle.transpose_info(c["shape"], c["perm"], 4)
        assert (block, count, len(dims)) == (c["block_size"], c["block_count"], c["dims"])
        if "strides" in c:
            assert dims == [tuple(v) for v in c["strides"]]


def test_transpose_against_numpy_and_its_invariants():
    # numpy.transpose is the library routine; identity, involution and composition are what the mathematics fixes
    rng = np.random.default_rng(3)
    for t in range(300):
        rank = int(rng.integers(1, 7))
        shape = tuple(int(v) for v in rng.integers(1, 6, rank))
        perm = tuple(int(v) for v in rng.permutation(rank))
        x = rng.integers(0, 1 << 15, shape).astype([np.uint8, np.int16, np.float32, np.float64][t % 4])
        y = oracle.transpose(x, perm)
        assert y.shape == tuple(shape[p] for p in perm) and np.array_equal(y, np.transpose(x, perm))
        inverse = tuple(int(v) for v in np.argsort(perm))
        assert np.array_equal(oracle.transpose(y, inverse), x)
        second = tuple(int(v) for v in rng.permutation(rank))
        assert np.array_equal(oracle.transpose(y, second), np.transpose(x, [perm[i] for i in second]))
    x = np.arange(30, dtype=np.float32).reshape(1, 3, 2, 5)          # src/04kernel/test/kernels/transpose/test_cpu.cpp:9-15
    assert np.array_equal(oracle.transpose(x, (2, 3, 0, 1)), np.transpose(x, (2, 3, 0, 1)))
    assert np.array_equal(oracle.transpose(x, (0, 1, 2, 3)), x)



# ------------------------------------------------------------------ Split / Concat / Expand / Where
def test_split_concat_reference_vectors_and_numpy():
    c = GOLDEN["split_info"]
    assert oracle.split_info(c["parts"], c["axis"], 8) == (c["block_count"], c["sum"], c["segments"])
    k = GOLDEN["split_concat"]
    x = np.arange(np.prod(k["joined_shape"]), dtype=np.float32).reshape(k["joined_shape"])
    parts = oracle.split(x, k["sizes"], k["axis"])
    offsets = np.concatenate([[0], np.cumsum(k["sizes"])])
    for j, part in enumerate(parts):              # the reference's own check, split/test_cpu.cpp:60-68
        flat = part.reshape(6, -1)
        for i in range(6):
            assert np.array_equal(flat[i], i * 20 * 49 + offsets[j] * 49 + np.arange(k["sizes"][j] * 49))
    iotas = [np.arange(p.size, dtype=np.float32).reshape(p.shape) for p in parts]
    joined = oracle.concat(iotas, k["axis"]).reshape(6, -1)
    for i in range(6):                            # concat/test_cpu.cpp:61-69
        for j, n in enumerate(k["sizes"]):
            assert np.array_equal(joined[i, offsets[j] * 49:offsets[j + 1] * 49], i * n * 49 + np.arange(n * 49))
    # numpy.split / numpy.concatenate are the library routines; the two are inverse to each other
    rng = np.random.default_rng(5)
    for t in range(200):
        rank = int(rng.integers(1, 6))
        shape = [int(v) for v in rng.integers(1, 6, rank)]
        axis = int(rng.integers(0, rank))
        sizes = [int(v) for v in rng.integers(0, 5, int(rng.integers(1, 6)))]
        shape[axis] = sum(sizes)
        x = rng.integers(0, 1 << 15, shape).astype([np.uint8, np.int16, np.float32, np.float64][t % 4])
        parts = oracle.split(x, sizes, axis)
        ref = np.split(x, np.cumsum(sizes)[:-1], axis=axis)
        assert all(np.array_equal(a, b) for a, b in zip(parts, ref))
        assert np.array_equal(oracle.concat(ref, axis), x)


def test_expand_reference_vectors_and_numpy():
    c = GOLDEN["expand_info"]
    pairs, block, count = oracle.expand_info(c["input"], c["output"], 4)
    assert (pairs, block, count) == ([tuple(v) for v in c["strides"]], c["block_size"], c["block_count"])
    d = np.arange(72, dtype=np.float32).reshape(c["input"])
    y = oracle.expand(d, c["output"]).reshape(2, 12, 5, 6)
    for j in range(12):                            # expand/test_cpu.cpp:27-38
        assert np.array_equal(y[:, j], np.broadcast_to(6 * j + np.arange(6, dtype=np.float32), (2, 5, 6)))
    rng = np.random.default_rng(6)
    for t in range(300):
        rank = int(rng.integers(1, 7))
        out = [int(rng.choice([1, 1, 2, 3, 4, 5])) for _ in range(rank)]
        keep = int(rng.integers(0, rank + 1))
        inp = [o if rng.random() < 0.5 else 1 for o in out[rank - keep:]]
        x = rng.integers(0, 1 << 15, inp).astype([np.uint8, np.int16, np.float32, np.float64][t % 4])
        assert np.array_equal(oracle.expand(x, out), np.broadcast_to(x, out))


def test_broadcaster_and_where_reference_vectors_and_numpy():
    c = GOLDEN["broadcaster"]
    rows, count = oracle.broadcaster(c["shapes"])
    assert rows == c["strides"] and count == c["outputs_count"]
    for k, want in c["locate"].items():             # broadcaster.cc:87-100
        rem, at = int(k), [0] * 4
        for row in rows:
            q, rem = divmod(rem, row[4])
            at = [a + s * q for a, s in zip(at, row[:4])]
        assert at == want
    w = GOLDEN["where"]
    out = oracle.where(np.ones(w["c_shape"], bool), np.full(w["x_shape"], w["x"], np.float32), np.full(w["y_shape"], w["y"], np.float32))
    assert out.shape == tuple(w["x_shape"]) and np.all(out == w["expected"])
    rng = np.random.default_rng(7)
    for t in range(300):
        rank = int(rng.integers(0, 5))
        out_shape = [int(rng.choice([1, 2, 3, 4])) for _ in range(rank)]
        shapes = []
        for _ in range(3):
            keep = int(rng.integers(0, rank + 1))
            shapes.append([o if rng.random() < 0.6 else 1 for o in out_shape[rank - keep:]])
        dt = [np.uint8, np.int16, np.float32, np.float64][t % 4]
        cnd = rng.integers(0, 2, shapes[0]).astype(bool)
        x, y = rng.integers(0, 100, shapes[1]).astype(dt), rng.integers(100, 200, shapes[2]).astype(dt)
        assert np.array_equal(oracle.where(cnd, x, y), np.where(cnd, x, y))
