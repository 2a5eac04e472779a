"""Parity of the HIP kernels (called through the C ABI) against the CPU oracle.

Bars: bit-exact for MatMulInteger / DequantizeLinear; <= 1e-5 relative for fp32 RmsNormalization
and fp32 Softmax; <= 2e-3 absolute for fp16 paths (oracle in fp32 on up-cast inputs).
"""
import ctypes as C
import json
import math
import os

import numpy as np
import pytest
import torch

import oracle
from refactorgraph_amd import abi, ops

pytestmark = pytest.mark.gpu

REL_F32 = 1e-5
ABS_F16 = 2e-3
DEV = "cuda"
GOLDEN = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "reference_kats.json")))


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).to(DEV)


def host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


def assert_rel(y, ref, rel):
    y = y.astype(np.float64)
    ref = ref.astype(np.float64)
    err = np.abs(y - ref)
    bad = err > rel * np.abs(ref) + 1e-30
    assert not bad.any(), f"max rel err {np.max(err / (np.abs(ref) + 1e-30)):.3e}"


# ------------------------------------------------------------------ RmsNormalization

@pytest.mark.parametrize("shape", [(2, 3, 4), (2, 3, 4096), (5, 7, 100), (3, 8192), (2, 10000), (4, 4097),
                                   (64, 128, 512)])
def test_rms_norm_f32(shape):
    rng = np.random.default_rng(1)
    x = rng.standard_normal(shape).astype(np.float32)
    w = np.random.default_rng(2).uniform(0.5, 1.5, shape[-1]).astype(np.float32)
    y = host(ops.rms_norm(dev(x), dev(w), 1e-5))
    assert_rel(y, oracle.rms_norm(x, w, 1e-5, threads=8), REL_F32)


@pytest.mark.parametrize("rows,cols", [(300, 128), (101, 16), (50, 64), (17, 256), (1000, 8), (7, 32)])
def test_rms_norm_short_rows_several_to_a_wavefront(rows, cols):
    # a head's 128 elements (normalisation of queries and keys per head) and shorter rows: 4 to 32 lanes per row
    rng = np.random.default_rng(rows)
    x = rng.standard_normal((rows, cols)).astype(np.float32)
    w = rng.uniform(0.5, 1.5, cols).astype(np.float32)
    assert_rel(host(ops.rms_norm(dev(x), dev(w), 1e-5)), oracle.rms_norm(x, w, 1e-5, threads=8), REL_F32)
    xt, wt = dev(x).half(), dev(w).half()
    ref = oracle.rms_norm(host(xt.float()), host(wt.float()), 1e-5)
    assert np.max(np.abs(host(ops.rms_norm(xt, wt, 1e-5).float()) - ref)) <= ABS_F16 * max(1.0, np.abs(ref).max() / 2)
    xd = x.astype(np.float64)
    assert_rel(host(ops.rms_norm(dev(xd), dev(w.astype(np.float64)), 1e-5)), oracle.rms_norm(xd, w.astype(np.float64), 1e-5), 1e-12)


def test_rms_norm_reference_kats():
    # reference tests: iota [2,3,4] with eps 0; x=2, w=3 on [2,3,4096] -> exactly 3
    x = np.arange(24, dtype=np.float32).reshape(2, 3, 4)
    w = np.arange(1, 5, dtype=np.float32)
    y = host(ops.rms_norm(dev(x), dev(w), 0.0))
    assert_rel(y[0, 1:], oracle.rms_norm(x, w, 0.0)[0, 1:], 4 * 1.2e-7)
    x = np.full((2, 3, 4096), 2.0, np.float32)
    w = np.full(4096, 3.0, np.float32)
    assert np.all(host(ops.rms_norm(dev(x), dev(w), 0.0)) == 3.0)


@pytest.mark.parametrize("rows,cols", [(8, 4096), (3, 8192), (5, 2048), (1100, 5120), (1030, 8192), (1024, 4104), (1, 16384)])
def test_rms_norm_long_rows_a_wavefront_or_a_workgroup_each(rows, cols):
    # few rows, and many 16-bit rows of more than 4096 elements, take a workgroup per row; the others a wavefront
    rng = np.random.default_rng(rows + cols)
    x = rng.standard_normal((rows, cols)).astype(np.float32)
    w = rng.uniform(0.5, 1.5, cols).astype(np.float32)
    assert_rel(host(ops.rms_norm(dev(x), dev(w), 1e-5)), oracle.rms_norm(x, w, 1e-5, threads=8), REL_F32)
    for dt in (torch.float16, torch.bfloat16):
        xt, wt = dev(x).to(dt), dev(w).to(dt)
        ref = oracle.rms_norm(host(xt.float()), host(wt.float()), 1e-5, threads=8)
        tol = ABS_F16 if dt == torch.float16 else 4e-2
        assert np.max(np.abs(host(ops.rms_norm(xt, wt, 1e-5).float()) - ref)) <= tol * max(1.0, np.abs(ref).max() / 2)


def test_rms_norm_f64_and_halves():
    rng = np.random.default_rng(3)
    x = rng.standard_normal((33, 1024))
    w = rng.uniform(0.5, 1.5, 1024)
    y = host(ops.rms_norm(dev(x), dev(w), 1e-5))
    assert_rel(y, oracle.rms_norm(x, w, 1e-5), 1e-12)
    for dt in (torch.float16, torch.bfloat16):
        xt = dev(x.astype(np.float32)).to(dt)
        wt = dev(w.astype(np.float32)).to(dt)
        y = ops.rms_norm(xt, wt, 1e-5).float()
        ref = oracle.rms_norm(host(xt.float()), host(wt.float()), 1e-5)
        tol = ABS_F16 if dt == torch.float16 else 4e-2
        assert np.max(np.abs(host(y) - ref)) <= tol * max(1.0, np.abs(ref).max() / 2)


def test_rms_norm_full_config_in_place():
    # the full configuration [32,128,4096] fp32, checked on a row sample against the oracle and fully
    # through the invariant sum_j (y_j/w_j)^2 = D*ms/(ms+eps)
    rng = np.random.default_rng(1)
    x = rng.standard_normal((32, 128, 4096), dtype=np.float32)
    w = np.random.default_rng(2).uniform(0.5, 1.5, 4096).astype(np.float32)
    xd = dev(x)
    y = host(ops.rms_norm(xd, dev(w), 1e-5, out=xd))  # y aliases x
    rows = np.random.default_rng(0).choice(32 * 128, 256, replace=False)
    assert_rel(y.reshape(-1, 4096)[rows], oracle.rms_norm(x.reshape(-1, 4096)[rows], w, 1e-5), REL_F32)
    ms = (x.astype(np.float64) ** 2).mean(-1)
    lhs = ((y.astype(np.float64) / w) ** 2).sum(-1)
    assert np.allclose(lhs, 4096 * ms / (ms + 1e-5), rtol=1e-5)


# ------------------------------------------------------------------ Softmax

@pytest.mark.parametrize("shape,axis", [((2, 3, 2, 4), 1), ((4, 5, 2048), 2), ((3, 1000), 1), ((6, 7, 33), 2),
                                        ((2, 64, 5), 1), ((8, 4096), 1), ((2, 3, 9000), 2), ((5, 6), 0)])
def test_softmax_f32(shape, axis):
    rng = np.random.default_rng(3)
    x = (3 * rng.standard_normal(shape)).astype(np.float32)
    y = host(ops.softmax(dev(x), axis))
    assert_rel(y, oracle.softmax(x, axis, threads=8), REL_F32)


@pytest.mark.parametrize("shape,axis", [((300, 70), 0), ((3, 1100, 40), 1), ((2, 64, 3, 5), 1), ((1500, 2), 0), ((4, 33, 33), 1)])
def test_softmax_along_an_axis_that_is_not_the_innermost(shape, axis):
    # 32 slices and 8 or 32 threads per slice to a workgroup; running maximum and sum, -inf among the inputs, a slice
    # count that is no multiple of 32; float, double and fp16
    rng = np.random.default_rng(7)
    x = (3 * rng.standard_normal(shape)).astype(np.float32)
    x[rng.random(shape) < 0.05] = -np.inf
    assert_rel(host(ops.softmax(dev(x), axis)), oracle.softmax(x, axis, threads=8), 2 * REL_F32)
    xd = x.astype(np.float64)
    assert_rel(host(ops.softmax(dev(xd), axis)), oracle.softmax(xd, axis), 1e-12)
    x16 = dev(x).half()
    got = host(ops.softmax(x16, axis).float())
    assert np.max(np.abs(got - oracle.softmax(host(x16.float()), axis, threads=8))) <= ABS_F16


@pytest.mark.parametrize("rows,mid", [(1000, 8), (513, 2), (300, 7), (64, 24), (70, 128), (33, 1), (257, 31), (90, 32), (41, 12)])
def test_softmax_short_rows(rows, mid):
    # scores over a handful of experts or classes: 1 to 16 lanes per row where the row is whole vectors, one thread per
    # row where it is not; plain and causal, float, double and fp16
    rng = np.random.default_rng(rows + mid)
    x = (3 * rng.standard_normal((rows, mid))).astype(np.float32)
    assert_rel(host(ops.softmax(dev(x))), oracle.softmax(x, threads=8), REL_F32)
    xd = x.astype(np.float64)
    assert_rel(host(ops.softmax(dev(xd))), oracle.softmax(xd), 1e-12)
    x16 = dev(x).half()
    x32 = host(x16.float())
    assert np.max(np.abs(host(ops.softmax(x16).float()) - oracle.softmax(x32, threads=8))) <= ABS_F16
    if mid > 1 and rows % mid == 0:
        sq = x32[:rows // mid * mid].reshape(-1, mid, mid)
        got = host(ops.softmax(dev(sq).half(), causal=True).float())
        assert np.max(np.abs(got - oracle.softmax_causal(sq, threads=8))) <= ABS_F16


@pytest.mark.parametrize("heads, seq, mid", [(3, 37, 300), (2, 45, 301), (5, 33, 33), (1, 99, 700), (2, 150, 150), (3, 7, 390)])
def test_softmax_rows_that_start_anywhere_within_a_vector(heads, seq, mid):
    # rows of a length that is no whole number of 16-byte vectors, 16, 32 or 64 lanes each (several rows to a
    # wavefront, a last workgroup with rows to spare): plain and causal, fp16, bf16 and float
    rng = np.random.default_rng(seq * 1000 + mid)
    x = (3 * rng.standard_normal((heads, seq, mid))).astype(np.float32)
    x[0, -1, :5] = -np.inf  # (the last row keeps every column under the causal mask too)
    for dt, tol in ((torch.float16, ABS_F16), (torch.bfloat16, 8 * ABS_F16)):
        xh = dev(x).to(dt)
        x32 = host(xh.float())
        assert np.max(np.abs(host(ops.softmax(xh).float()) - oracle.softmax(x32, threads=8))) <= tol
        if mid >= seq:
            assert np.max(np.abs(host(ops.softmax(xh, causal=True).float()) - oracle.softmax_causal(x32, threads=8))) <= tol
    if mid % 4:
        assert_rel(host(ops.softmax(dev(x))), oracle.softmax(x, threads=8), REL_F32)
        if mid >= seq:
            assert_rel(host(ops.softmax(dev(x), causal=True)), oracle.softmax_causal(x, threads=8), REL_F32)


@pytest.mark.parametrize("shape", [(1, 70001), (3, 32768), (2, 1, 40001), (16, 50257)])
def test_softmax_few_very_long_rows_in_chunks(shape):
    # logits over a vocabulary: the rows are cut into chunks, a workgroup each, whose maxima and sums travel through the
    # first bytes of the chunks' places in the output (three launches); in place the one-workgroup kernel stays
    rng = np.random.default_rng(shape[-1])
    x = (3 * rng.standard_normal(shape)).astype(np.float32)
    x.reshape(-1)[7] = -np.inf
    ref = oracle.softmax(x.astype(np.float64), threads=8)
    y = host(ops.softmax(dev(x)))
    assert not np.isnan(y).any()
    assert_rel(y, ref, 2 * REL_F32)
    z = dev(x)
    assert_rel(host(ops.softmax(z, out=z)), ref, 2 * REL_F32)
    for dt, tol in ((torch.float16, ABS_F16), (torch.bfloat16, 2e-2)):
        xt = dev(x).to(dt)
        got = host(ops.softmax(xt).float())
        assert np.max(np.abs(got - oracle.softmax(host(xt.float()), threads=8))) <= tol


def test_softmax_reference_kat_and_f64():
    x = np.zeros((2, 3, 2, 4), np.float64)
    assert np.all(host(ops.softmax(dev(x), 1)) == 1.0 / 3)
    x = 3 * np.random.default_rng(3).standard_normal((17, 513))
    assert_rel(host(ops.softmax(dev(x), 1)), oracle.softmax(x, 1), 1e-13)


@pytest.mark.parametrize("dt,tol", [(torch.float16, ABS_F16), (torch.bfloat16, 8e-3)])
def test_softmax_16bit_plain_and_causal(dt, tol):
    rng = np.random.default_rng(3)
    for shape in [(2, 3, 256, 256), (1, 2, 64, 2048), (3, 130, 136), (2, 2048, 2048)]:
        x16 = dev((3 * rng.standard_normal(shape)).astype(np.float32)).to(dt)
        x32 = host(x16.float())
        y = host(ops.softmax(x16).float())
        assert np.max(np.abs(y - oracle.softmax(x32, threads=8))) <= tol
        # causal flag == data-masked input, bit for bit, and both match the oracle
        yc = ops.softmax(x16, causal=True)
        R, Cc = shape[-2], shape[-1]
        mask = torch.arange(Cc, device=DEV)[None, :] > torch.arange(R, device=DEV)[:, None] + (Cc - R)
        ym = ops.softmax(x16.masked_fill(mask, float("-inf")))
        assert torch.equal(yc, ym)
        assert np.max(np.abs(host(yc.float()) - oracle.softmax_causal(x32, threads=8))) <= tol
        assert torch.all(yc[..., mask] == 0)


def test_softmax_long_rows():
    # rows beyond what the register kernel holds (1024 16-byte vectors): the looped kernel, with the row cached in
    # 64 KiB or 128 KiB of LDS or, beyond that, read twice
    rng = np.random.default_rng(31)
    for shape, dt in [((5, 16384), torch.float16), ((3, 32768), torch.float16), ((2, 40000), torch.bfloat16),
                      ((2, 2, 70000), torch.float16), ((3, 8192), torch.float32), ((2, 50000), torch.float32),
                      ((2, 4104), torch.float64)]:
        x = dev(3 * rng.standard_normal(shape)).to(dt)
        x[0, ..., 5:9000:7] = float("-inf")        # masked entries inside the row
        x[-1, ..., 100] = 40.0                     # a late maximum far above what came before it
        ref = oracle.softmax(host(x.double() if dt == torch.float64 else x.float()), threads=8)
        y = ops.softmax(x)
        if dt == torch.float32:
            # the oracle adds the 50000 terms of a row one after the other in float, as the reference does, which
            # alone costs up to n * 2^-24 of the sum: the float64 softmax is the tighter check at this length
            assert_rel(host(y), ref, 1e-4)
            assert_rel(host(y), oracle.softmax(host(x.double()), threads=8), REL_F32)
        elif dt == torch.float64:
            assert_rel(host(y), ref, 1e-13)
        else:
            assert np.max(np.abs(host(y.float()) - ref)) <= (ABS_F16 if dt == torch.float16 else 8e-3)
        assert float((y.double().sum(-1) - 1).abs().max()) < 2e-2
        assert torch.all(y[0, ..., 5:9000:7] == 0)
    # causal over a long row: 24 query rows against 16408 keys, flag == data-masked input bit for bit
    x16 = dev(3 * rng.standard_normal((2, 24, 16408)).astype(np.float32)).half()
    yc = ops.softmax(x16, causal=True)
    mask = torch.arange(16408, device=DEV)[None, :] > torch.arange(24, device=DEV)[:, None] + (16408 - 24)
    assert torch.equal(yc, ops.softmax(x16.masked_fill(mask, float("-inf"))))
    assert np.max(np.abs(host(yc.float()) - oracle.softmax_causal(host(x16.float()), threads=8))) <= ABS_F16
    assert torch.all(yc[..., mask] == 0)


def test_softmax_rows_that_fit_no_vectors():
    # row lengths that are no multiple of a 128-bit vector (scores over 1025 positions, a vocabulary of 50257) and rows
    # that start off a 16-byte boundary: aligned vectors in the middle of a row, single elements at its ends
    rng = np.random.default_rng(41)
    for shape, dt in [((5, 1025), torch.float16), ((3, 7, 33), torch.float32), ((4, 2047), torch.bfloat16),
                      ((3, 50257), torch.float16), ((2, 3, 4097), torch.float32), ((6, 5), torch.float64),
                      ((2, 40001), torch.float32), ((9, 1), torch.float16), ((3, 2049), torch.float64)]:
        x = dev(3 * rng.standard_normal(shape)).to(dt)
        if shape[-1] > 40:
            x[0, ..., 5:40:7] = float("-inf")
        ref = oracle.softmax(host(x.double() if dt == torch.float64 else x.float()), threads=8)
        y = ops.softmax(x)
        if dt == torch.float32:
            assert_rel(host(y), oracle.softmax(host(x.double()), threads=8), REL_F32)
        elif dt == torch.float64:
            assert_rel(host(y), ref, 1e-13)
        else:
            assert np.max(np.abs(host(y.float()) - ref)) <= (ABS_F16 if dt == torch.float16 else 8e-3)
    # rows of a multiple of the vector length that start two bytes off a boundary; output aligned alike, then differently
    base = dev(3 * rng.standard_normal(4 * 1024 + 1).astype(np.float32)).half()
    x = base[1:].view(4, 1024)
    ref = oracle.softmax(host(x.float()), threads=8)
    out_alike = torch.empty(4 * 1024 + 1, dtype=torch.float16, device=DEV)[1:].view(4, 1024)
    out_other = torch.empty((4, 1024), dtype=torch.float16, device=DEV)
    for out in (out_alike, out_other):
        assert np.max(np.abs(host(ops.softmax(x, out=out).float()) - ref)) <= ABS_F16
    # causal flag on ragged rows: equal to the data-masked input bit for bit
    x16 = dev(3 * rng.standard_normal((2, 130, 135)).astype(np.float32)).half()
    yc = ops.softmax(x16, causal=True)
    mask = torch.arange(135, device=DEV)[None, :] > torch.arange(130, device=DEV)[:, None] + 5
    assert torch.equal(yc, ops.softmax(x16.masked_fill(mask, float("-inf"))))
    assert np.max(np.abs(host(yc.float()) - oracle.softmax_causal(host(x16.float()), threads=8))) <= ABS_F16
    assert torch.all(yc[..., mask] == 0)


def test_softmax_full_config_properties():
    # [8,32,2048,2048] fp16: a slab against the oracle, the whole tensor through row sums
    g = torch.Generator(device=DEV).manual_seed(3)
    x = (3 * torch.randn((8, 32, 2048, 2048), generator=g, device=DEV, dtype=torch.float32)).half()
    y = ops.softmax(x)
    yc = ops.softmax(x, causal=True)
    sums = y.float().sum(-1)
    assert float((sums - 1).abs().max()) < 2e-2  # 2048 roundings of fp16 outputs
    assert float((yc.float().sum(-1) - 1).abs().max()) < 2e-2
    assert torch.all(yc[0, 0].triu(1) == 0) and torch.all(yc[7, 31].triu(1) == 0)
    slab = host(x[5, 17, 1000:1064].float())
    assert np.max(np.abs(host(y[5, 17, 1000:1064].float()) - oracle.softmax(slab))) <= ABS_F16
    ref_c = oracle.softmax_causal(host(x[2, 9].float()), threads=8)
    assert np.max(np.abs(host(yc[2, 9].float()) - ref_c)) <= ABS_F16


# ------------------------------------------------------------------ RotaryEmbedding

@pytest.mark.parametrize("B,S,H,D", [(2, 50, 3, 16), (1, 33, 32, 128), (3, 17, 8, 64), (2, 9, 40, 256),
                                     (2, 7, 5, 6), (1, 2048, 4, 128)])
def test_rope_f16(B, S, H, D):
    rng = np.random.default_rng(4)
    x16 = dev(rng.standard_normal((B, S, H, D)).astype(np.float32)).half()
    pos = np.tile(np.arange(S, dtype=np.int64), (B, 1))
    ref = oracle.rope(host(x16.float()), pos, 10000.0, threads=8)
    y = host(ops.rope(x16, dev(pos), 10000.0).float())
    assert np.max(np.abs(y - ref)) <= ABS_F16
    # [seq] positions broadcast; in place
    y2 = ops.rope(x16.clone(), dev(pos[0]), 10000.0)
    assert np.array_equal(host(y2.float()), y)
    xin = x16.clone()
    ops.rope(xin, dev(pos), 10000.0, out=xin)
    assert np.array_equal(host(xin.float()), y)


def test_rope_f32_random_positions_and_bf16():
    rng = np.random.default_rng(4)
    x = rng.standard_normal((2, 40, 6, 128)).astype(np.float32)
    pos = rng.integers(0, 4096, (2, 40)).astype(np.int64)
    ref = oracle.rope(x, pos, 10000.0)
    y = host(ops.rope(dev(x), dev(pos), 10000.0))
    assert np.max(np.abs(y - ref)) <= 2e-5
    xb = dev(x).bfloat16()
    yb = host(ops.rope(xb, dev(pos), 500000.0).float())
    assert np.max(np.abs(yb - oracle.rope(host(xb.float()), pos, 500000.0))) <= 2e-2


def test_rope_full_config_properties():
    # [16,2048,32,128] fp16: pos 0 rows are the identity, pair norms are preserved, a token slab
    # matches the oracle
    g = torch.Generator(device=DEV).manual_seed(4)
    x = torch.randn((16, 2048, 32, 128), generator=g, device=DEV, dtype=torch.float32).half()
    pos = torch.arange(2048, device=DEV, dtype=torch.int64).repeat(16, 1)
    y = ops.rope(x, pos)
    assert torch.equal(y[:, 0], x[:, 0])
    n_in = x[3].float()[..., :64] ** 2 + x[3].float()[..., 64:] ** 2
    n_out = y[3].float()[..., :64] ** 2 + y[3].float()[..., 64:] ** 2
    assert float((n_in - n_out).abs().max()) < 4e-2
    sl = slice(1990, 2048)
    ref = oracle.rope(host(x[11:12, sl].float()), host(pos[11:12, sl]), 10000.0, threads=8)
    assert np.max(np.abs(host(y[11:12, sl].float()) - ref)) <= ABS_F16


# ------------------------------------------------------------------ DynamicQuantizeLinear (bit-exact)

def _dql_check(x):
    y, scale, zp = ops.dynamic_quantize_linear(dev(x))
    ry, rs, rz = oracle.dynamic_quantize_linear(x)
    assert host(scale)[0] == rs and host(zp)[0] == rz
    assert np.array_equal(host(y), ry)
    return host(y), host(scale)[0], host(zp)[0]


def test_rms_norm_quantize_fused_pair():
    # the fused pair against its two operators: the normalised tensor bit for bit what rg_hip_rms_norm writes, the
    # quantised tensor, scale and zero point bit for bit what the CPU kernel computes from that tensor
    rng = np.random.default_rng(31)
    for rows, cols in ((4096, 4096), (7, 4096), (1024, 132), (300, 8192), (3, 1024), (2048, 512)):
        x = torch.from_numpy(rng.standard_normal((rows, cols)).astype(np.float32) * 2 + 0.25).to(DEV)
        w = torch.from_numpy(rng.uniform(0.5, 1.5, cols).astype(np.float32)).to(DEV)
        y, yq, scale, zp = ops.rms_norm_quantize(x, w, 1e-5)
        torch.cuda.synchronize()
        assert torch.equal(y, ops.rms_norm(x, w, 1e-5))
        ry, rs, rz = oracle.dynamic_quantize_linear(y.cpu().numpy().reshape(-1))
        assert np.array_equal(yq.cpu().numpy().reshape(-1), ry) and scale.item() == rs and zp.item() == rz
        ref = oracle.rms_norm(x.cpu().numpy(), w.cpu().numpy(), 1e-5)
        assert np.all(np.abs(y.cpu().numpy() - ref) <= 1e-5 * np.abs(ref) + 1e-30)
    # shapes the pair is not fused for are reported as such
    assert ops.lib().rg_hip_rms_norm_quantize_workspace(16, 130) == 0
    assert ops.lib().rg_hip_rms_norm_quantize_workspace(1 << 20, 256) == 0
    assert ops.lib().rg_hip_rms_norm_quantize_workspace(4096, 4096) == 1024 * 8


def test_dynamic_quantize_reference_kats():
    # src/04kernel/test/kernels/dynamic_quantize_linear/test_cpu.cpp:21-38 and test_cuda.cpp:36-39
    y, scale, zp = _dql_check(np.array([0, 2, -3, -2.5, 1.34, 0.5], np.float32))
    assert scale == np.float32(5) / np.float32(255) and zp == 153 and y.tolist() == [153, 255, 0, 26, 221, 179]
    y, scale, zp = _dql_check((3 * np.arange(20) + 15).astype(np.float32))
    assert zp == 0 and y[-1] == 255


@pytest.mark.parametrize("n", [1, 7, 255, 4096, 4097, (1 << 20) + 3, 3 * 5 * 7 * 1024])
@pytest.mark.parametrize("lo,hi", [(-3.0, 5.0), (0.5, 9.0), (-7.0, -0.25)])
def test_dynamic_quantize_bit_exact(n, lo, hi):
    x = np.random.default_rng(n).uniform(lo, hi, n).astype(np.float32)
    _dql_check(x)


def test_dynamic_quantize_ties_zeros_and_unaligned():
    y, scale, zp = _dql_check(np.array([0.0, 255.0, 2.5, 0.5, 1.5, 254.5], np.float32))
    assert y.tolist() == [0, 255, 3, 1, 2, 255]           # ties away from zero
    y, scale, zp = _dql_check(np.zeros(1000, np.float32))
    assert not y.any() and zp == 0
    # operands that are not 16-byte aligned take the element-wise path
    x = np.random.default_rng(5).normal(0, 2, 10001).astype(np.float32)
    xd = dev(x)
    out = torch.empty(10003, dtype=torch.uint8, device=DEV)
    y, scale, zp = ops.dynamic_quantize_linear(xd[1:], out=out[3:3 + 10000])
    ry, rs, rz = oracle.dynamic_quantize_linear(x[1:])
    assert np.array_equal(host(y), ry) and host(scale)[0] == rs and host(zp)[0] == rz


def test_dynamic_quantize_full_config():
    # the producer of MatMulInteger's A operand: fp32 [4096, 4096]
    x = np.random.default_rng(15).normal(0, 1, (4096, 4096)).astype(np.float32)
    y, scale, zp = _dql_check(x)
    back = (y.astype(np.float32) - np.float32(zp)) * scale
    assert np.max(np.abs(back - x)) <= 0.5 * scale * (1 + 1e-5)


# ------------------------------------------------------------------ DequantizeLinear (bit-exact)

def test_dequantize_reference_kat():
    y = ops.dequantize_linear(dev(np.array([0, 3, 128, 255], np.uint8)), dev(np.array([2.0], np.float32)),
                              dev(np.array([128], np.uint8)))
    assert host(y).tolist() == [-256, -250, 0, 254]


@pytest.mark.parametrize("dt", [np.uint8, np.int8, np.int16, np.int32])
@pytest.mark.parametrize("shape,axis", [((4096,), 0), ((3, 5, 4), 1), ((16, 64), 1), ((7, 33), 1), ((8, 12, 6), 0),
                                        ((256, 1024), 1), ((300, 1024), 0), ((5, 7, 128), 1), ((6, 40, 10), 0)])
def test_dequantize_bit_exact(dt, shape, axis):
    rng = np.random.default_rng(7)
    info = np.iinfo(dt)
    lo, hi = max(info.min, -(1 << 20)), min(info.max, 1 << 20)
    x = rng.integers(lo, hi + 1, shape, dtype=dt)
    # scalar (reference path), with and without zero point
    s1 = np.array([0.0123], np.float32)
    z1 = rng.integers(lo, hi + 1, (1,), dtype=dt)
    assert np.array_equal(host(ops.dequantize_linear(dev(x), dev(s1), dev(z1))), oracle.dequantize_linear(x, s1, z1))
    assert np.array_equal(host(ops.dequantize_linear(dev(x), dev(s1))), oracle.dequantize_linear(x, s1))
    # per-axis
    n = shape[axis]
    s = np.random.default_rng(8).uniform(1e-3, 1e-2, n).astype(np.float32)
    z = rng.integers(lo, hi + 1, (n,), dtype=dt)
    assert np.array_equal(host(ops.dequantize_linear(dev(x), dev(s), dev(z), axis=axis)),
                          oracle.dequantize_linear(x, s, z, axis=axis))
    assert np.array_equal(host(ops.dequantize_linear(dev(x), dev(s), axis=axis)),
                          oracle.dequantize_linear(x, s, None, axis=axis))


def test_dequantize_full_config_bit_exact():
    x = np.random.default_rng(7).integers(-128, 128, (4096, 4096), dtype=np.int8)
    s = np.random.default_rng(8).uniform(1e-3, 1e-2, 4096).astype(np.float32)
    y = host(ops.dequantize_linear(dev(x), dev(s), axis=1))
    assert np.array_equal(y, oracle.dequantize_linear(x, s, None, axis=1, threads=8))


# ------------------------------------------------------------------ MatMulInteger (bit-exact)

def test_matmul_integer_reference_kats():
    a = np.array([[1, 2, 3], [4, 5, 6]], np.uint8)
    b = np.array([[1], [2], [3]], np.uint8)
    assert host(ops.matmul_integer(dev(a), dev(b))).reshape(-1).tolist() == [14, 32]
    a = np.arange(1, 5, dtype=np.uint8).reshape(1, 4)
    b = np.tile(np.arange(1, 13, dtype=np.uint8), (4, 1))
    assert host(ops.matmul_integer(dev(a), dev(b))).reshape(-1).tolist() == [10 * i for i in range(1, 13)]
    a = np.array([0, 128, 255, 1, 127, 200], np.uint8).reshape(2, 3)
    b = np.array([-128, 127, 1, -1, 5, 7], np.int8).reshape(3, 2)
    y = ops.matmul_integer(dev(a), dev(b), dev(np.array([128], np.uint8)), dev(np.array([0], np.int8)))
    assert host(y).reshape(-1).tolist() == [17019, -15367, 16615, -15624]
    assert host(ops.matmul_integer(dev(a), dev(b))).reshape(-1).tolist() == [-133, 121, -281, -392]


@pytest.mark.parametrize("m,k,n", [(37, 53, 29), (256, 64, 256), (256, 192, 512), (512, 1024, 256), (300, 64, 256),
                                   (1, 4096, 1), (768, 128, 768), (256, 256, 256), (512, 640, 256)])
def test_matmul_integer_bit_exact_config_zero_points(m, k, n):
    a = np.random.default_rng(5).integers(0, 256, (m, k), dtype=np.uint8)
    b = np.random.default_rng(6).integers(-128, 128, (k, n), dtype=np.int8)
    az, bz = np.array([128], np.uint8), np.array([0], np.int8)
    y = host(ops.matmul_integer(dev(a), dev(b), dev(az), dev(bz)))
    assert np.array_equal(y, oracle.matmul_integer(a, b, az, bz, threads=8))


@pytest.mark.parametrize("m,k,n", [(20, 33, 17), (256, 128, 256), (256, 384, 512), (512, 1024, 256), (200, 512, 512)])
def test_matmul_integer_zero_point_variants_and_broadcast(m, k, n):
    rng = np.random.default_rng(6)
    a = rng.integers(0, 256, (2, 1, m, k), dtype=np.uint8)
    b = rng.integers(0, 256, (1, 3, k, n), dtype=np.uint8)
    variants = [
        (None, None),
        (rng.integers(0, 256, (1,), dtype=np.uint8), rng.integers(-128, 128, (1,), dtype=np.int8)),
        (rng.integers(0, 256, (2 * m,), dtype=np.uint8), rng.integers(-128, 128, (3 * k,), dtype=np.int8)),
        (rng.integers(-128, 128, (2 * m,), dtype=np.int8), None),
    ]
    for az, bz in variants:
        y = host(ops.matmul_integer(dev(a), dev(b), None if az is None else dev(az), None if bz is None else dev(bz)))
        assert y.shape == (2, 3, m, n)
        assert np.array_equal(y, oracle.matmul_integer(a, b, az, bz, threads=8))
    # B's per-row zero points from an address that is no multiple of 4 (the tile kernel then loads them from memory
    # instead of copying them along with the tiles)
    az, bz = rng.integers(0, 256, (2 * m,), dtype=np.uint8), rng.integers(-128, 128, (3 * k,), dtype=np.int8)
    bz_odd = dev(np.concatenate([np.zeros(1, np.int8), bz]))[1:]
    assert bz_odd.data_ptr() % 4 != 0
    y = host(ops.matmul_integer(dev(a), dev(b), dev(az), bz_odd))
    assert np.array_equal(y, oracle.matmul_integer(a, b, az, bz, threads=8))
    # equal batch shapes: the strided (grid.z) path
    a2 = rng.integers(0, 256, (3, m, k), dtype=np.uint8)
    b2 = rng.integers(-128, 128, (3, k, n), dtype=np.int8)
    az = rng.integers(0, 256, (3 * m,), dtype=np.uint8)
    y = host(ops.matmul_integer(dev(a2), dev(b2), dev(az), None))
    assert np.array_equal(y, oracle.matmul_integer(a2, b2, az, None, threads=8))


@pytest.mark.parametrize("m,k,n", [(37, 53, 29), (256, 128, 256), (512, 640, 768)])
def test_matmul_integer_with_dequantize_epilogue(m, k, n):
    # float(sum) * scale in the epilogue == MatMulInteger followed by DequantizeLinear, bit for bit
    rng = np.random.default_rng(m + n)
    a = rng.integers(0, 256, (2, m, k), dtype=np.uint8)
    b = rng.integers(-128, 128, (2, k, n), dtype=np.int8)
    az = rng.integers(0, 256, (1,), dtype=np.uint8)
    acc = oracle.matmul_integer(a, b, az, None, threads=8)
    per_column = rng.uniform(1e-4, 1e-2, n).astype(np.float32)
    scalar = np.array([3.1e-3], np.float32)
    y = host(ops.matmul_integer(dev(a), dev(b), dev(az), None, dequant_scale=dev(per_column)))
    assert y.dtype == np.float32
    assert np.array_equal(y, oracle.dequantize_linear(acc, per_column, None, axis=2))
    y = host(ops.matmul_integer(dev(a), dev(b), dev(az), None, dequant_scale=dev(scalar)))
    assert np.array_equal(y, oracle.dequantize_linear(acc, scalar, None))
    # and equal to the two GPU operators run one after the other
    two = ops.dequantize_linear(ops.matmul_integer(dev(a), dev(b), dev(az), None), dev(per_column), None, axis=2)
    assert torch.equal(two, ops.matmul_integer(dev(a), dev(b), dev(az), None, dequant_scale=dev(per_column)))


def test_matmul_integer_dequantize_large_sums_round_once():
    # |sum| up to 2^26 > 2^24: the int -> float conversion rounds (to nearest even), then one multiplication
    rng = np.random.default_rng(2)
    a = rng.integers(0, 40, (256, 4096), dtype=np.uint8)        # a - 128 in [-128, -89]
    b = rng.integers(-128, -64, (4096, 256), dtype=np.int8)
    az = np.array([128], np.uint8)
    scale = np.array([0.37], np.float32)
    acc = oracle.matmul_integer(a, b, az, None, threads=8)
    assert acc.min() > 2 ** 25 and np.any(acc.astype(np.float32).astype(np.int64) != acc)   # not representable
    y = host(ops.matmul_integer(dev(a), dev(b), dev(az), None, dequant_scale=dev(scale)))
    assert np.array_equal(y, acc.astype(np.float32) * scale[0])


@pytest.mark.parametrize("m,k,n", [(256, 2048, 256), (1024, 1024, 512), (256, 640, 1024), (512, 4096, 256)])
def test_matmul_integer_few_tiles_split_k(m, k, n):
    # too few 256 x 256 tiles for the chip: ranges of k go to different workgroups and meet in a zeroed Y by
    # integer atomics (exact in any order); every zero-point form, batches, the dequantising form
    rng = np.random.default_rng(m + k + n)
    a = rng.integers(0, 256, (2, m, k), dtype=np.uint8)
    b = rng.integers(-128, 128, (2, k, n), dtype=np.int8)
    for az, bz in [(None, None), (np.array([128], np.uint8), np.array([0], np.int8)),
                   (rng.integers(0, 256, (1,), dtype=np.uint8), rng.integers(-128, 128, (1,), dtype=np.int8)),
                   (rng.integers(0, 256, (2 * m,), dtype=np.uint8), rng.integers(-128, 128, (2 * k,), dtype=np.int8))]:
        out = torch.full((2, m, n), -7, dtype=torch.int32, device=DEV)         # the output is zeroed by the call itself
        y = ops.matmul_integer(dev(a), dev(b), None if az is None else dev(az), None if bz is None else dev(bz), out=out)
        assert np.array_equal(host(y), oracle.matmul_integer(a, b, az, bz, threads=8))
    scale = rng.uniform(1e-4, 1e-2, n).astype(np.float32)
    yd = ops.matmul_integer(dev(a), dev(b), dev(az), dev(bz), dequant_scale=dev(scale))
    assert np.array_equal(host(yd), oracle.dequantize_linear(oracle.matmul_integer(a, b, az, bz, threads=8), scale, None, axis=2))
    b1 = np.ascontiguousarray(b[:1])                                            # broadcast weights: one launch per matrix
    assert np.array_equal(host(ops.matmul_integer(dev(a), dev(b1))), oracle.matmul_integer(a, b1, None, None, threads=8))


@pytest.mark.parametrize("m,k,n", [(300, 128, 256), (256, 128, 272), (700, 256, 1008), (513, 384, 528), (257, 128, 257)])
def test_matmul_integer_ragged_rows_and_columns(m, k, n):
    # m and n beyond 256 that are no multiples of the MFMA tile: the last tiles are moved back and overlap
    # their neighbours ((257, 128, 257): n is no multiple of 16, the 128 x 128 tile kernel takes it)
    rng = np.random.default_rng(m * n)
    a = rng.integers(0, 256, (2, m, k), dtype=np.uint8)
    b = rng.integers(-128, 128, (2, k, n), dtype=np.int8)
    az = rng.integers(0, 256, (2 * m,), dtype=np.uint8)        # one per (batch, row)
    bz = rng.integers(-128, 128, (2 * k,), dtype=np.int8)
    ref = oracle.matmul_integer(a, b, az, bz, threads=8)
    assert np.array_equal(host(ops.matmul_integer(dev(a), dev(b), dev(az), dev(bz))), ref)
    scale = rng.uniform(1e-4, 1e-2, n).astype(np.float32)
    y = host(ops.matmul_integer(dev(a), dev(b), dev(az), dev(bz), dequant_scale=dev(scale)))
    assert np.array_equal(y, oracle.dequantize_linear(ref, scale, None, axis=2))


@pytest.mark.parametrize("m,k,n", [(300, 144, 128), (130, 1008, 77), (64, 16, 5), (513, 272, 250), (9, 208, 1031), (257, 128, 16),
                                   (200, 336, 5003)])
def test_matmul_integer_any_shape_on_the_matrix_cores(m, k, n):
    # fewer than 256 columns, column counts that are no multiple of 16 (rows of B then start on odd addresses), k that
    # is no multiple of 128, one to three k tiles: the 128 x 128 tile kernel, every zero-point form, both epilogues
    rng = np.random.default_rng(m * n + k)
    a = rng.integers(0, 256, (2, m, k), dtype=np.uint8)
    b = rng.integers(-128, 128, (2, k, n), dtype=np.int8)
    az = rng.integers(0, 256, (2 * m,), dtype=np.uint8)        # one per (batch, row)
    bz = rng.integers(-128, 128, (2 * k,), dtype=np.int8)
    ref = oracle.matmul_integer(a, b, az, bz, threads=8)
    assert np.array_equal(host(ops.matmul_integer(dev(a), dev(b), dev(az), dev(bz))), ref)
    scale = rng.uniform(1e-4, 1e-2, n).astype(np.float32)
    y = host(ops.matmul_integer(dev(a), dev(b), dev(az), dev(bz), dequant_scale=dev(scale)))
    assert np.array_equal(y, oracle.dequantize_linear(ref, scale, None, axis=2))
    assert np.array_equal(host(ops.matmul_integer(dev(a), dev(b))), oracle.matmul_integer(a, b, None, None, threads=8))
    # B from an address that is no multiple of 4: the aligned words around it belong to the same buffer
    flat = dev(np.concatenate([np.zeros(1, np.int8), b[0].reshape(-1)]))
    b_odd = flat[1:].view(k, n)
    got = host(ops.matmul_integer(dev(a[0]), b_odd, dev(az[:m]), dev(bz[:k])))
    assert np.array_equal(got, ref[0])


@pytest.mark.parametrize("m,k,n", [(1, 128, 256), (7, 1024, 512), (32, 4096, 4096), (33, 256, 256), (64, 256, 256), (100, 384, 512),
                                   (200, 384, 768), (255, 128, 256), (129, 256, 512), (250, 1024, 256), (100, 128, 272),
                                   (40, 256, 1040), (5, 384, 528)])
def test_matmul_integer_few_rows_weight_streaming(m, k, n):
    # fewer than 256 rows of A: B is streamed once per 32 rows, the k-tiles of a column block are added up with
    # integer atomics (exact in any order); every zero-point form, equal and broadcast batches.  More than 128
    # rows, and column counts that are no multiple of 256, run on one row of 256 x 256 tiles instead (with k split
    # between workgroups where n is a multiple of the tile)
    rng = np.random.default_rng(m + k)
    a = rng.integers(0, 256, (2, m, k), dtype=np.uint8)
    b = rng.integers(-128, 128, (2, k, n), dtype=np.int8)
    for az, bz in [(None, None), (np.array([128], np.uint8), np.array([0], np.int8)),
                   (rng.integers(0, 256, (1,), dtype=np.uint8), rng.integers(-128, 128, (1,), dtype=np.int8)),
                   (rng.integers(0, 256, (2 * m,), dtype=np.uint8), rng.integers(-128, 128, (2 * k,), dtype=np.int8))]:
        y = ops.matmul_integer(dev(a), dev(b), None if az is None else dev(az), None if bz is None else dev(bz))
        assert np.array_equal(host(y), oracle.matmul_integer(a, b, az, bz, threads=8))
    scale = rng.uniform(1e-4, 1e-2, n).astype(np.float32)
    yd = ops.matmul_integer(dev(a), dev(b), dev(az), dev(bz), dequant_scale=dev(scale))
    assert np.array_equal(host(yd), oracle.dequantize_linear(oracle.matmul_integer(a, b, az, bz, threads=8), scale, None, axis=2))
    b1 = b[:1]
    out = torch.full((2, m, n), 12345, dtype=torch.int32, device=DEV)          # the output is zeroed by the call itself
    y = ops.matmul_integer(dev(a), dev(np.ascontiguousarray(b1)), out=out)
    assert np.array_equal(host(y), oracle.matmul_integer(a, b1, None, None, threads=8))


@pytest.mark.parametrize("m,k,n", [(1, 16, 16), (1, 4096, 4096), (2, 48, 272), (3, 1008, 1040), (4, 4096, 1024), (4, 16384, 64),
                                   (1, 80, 4112)])
def test_matmul_integer_one_to_four_rows_matrix_vector(m, k, n):
    # at most four rows of A: dot products of four bytes on the vector ALUs, B streamed once; k from one step of 16
    # to many workgroups' ranges (added up with atomics), n that ends inside a strip of 256 columns; every zero-point
    # form (wrap-around of the byte difference included: all byte values occur), equal and broadcast batches
    rng = np.random.default_rng(3 * m + k)
    a = rng.integers(0, 256, (2, m, k), dtype=np.uint8)
    b = rng.integers(-128, 128, (2, k, n), dtype=np.int8)
    for az, bz in [(None, None), (np.array([128], np.uint8), np.array([0], np.int8)),
                   (rng.integers(0, 256, (1,), dtype=np.uint8), rng.integers(-128, 128, (1,), dtype=np.int8)),
                   (rng.integers(0, 256, (2 * m,), dtype=np.uint8), rng.integers(-128, 128, (2 * k,), dtype=np.int8))]:
        y = ops.matmul_integer(dev(a), dev(b), None if az is None else dev(az), None if bz is None else dev(bz))
        assert np.array_equal(host(y), oracle.matmul_integer(a, b, az, bz, threads=8))
    scale = rng.uniform(1e-4, 1e-2, n).astype(np.float32)
    yd = ops.matmul_integer(dev(a), dev(b), dev(az), dev(bz), dequant_scale=dev(scale))
    assert np.array_equal(host(yd), oracle.dequantize_linear(oracle.matmul_integer(a, b, az, bz, threads=8), scale, None, axis=2))
    b1 = b[:1]
    out = torch.full((2, m, n), 12345, dtype=torch.int32, device=DEV)          # the output is zeroed by the call itself
    y = ops.matmul_integer(dev(a), dev(np.ascontiguousarray(b1)), out=out)
    assert np.array_equal(host(y), oracle.matmul_integer(a, b1, None, None, threads=8))
    # extremes: every product (-128) * (-128), the largest sum this k can make
    ae, be = np.zeros((m, k), np.uint8), np.full((k, n), -128, np.int8)
    ye = host(ops.matmul_integer(dev(ae), dev(be), dev(np.array([128], np.uint8)), None))
    assert np.all(ye == k * 16384)


def test_matmul_integer_extremes():
    a = np.zeros((256, 4096), np.uint8)
    b = np.full((4096, 256), -128, np.int8)
    y = host(ops.matmul_integer(dev(a), dev(b), dev(np.array([128], np.uint8)), None))
    assert np.all(y == 2 ** 26)


def test_matmul_integer_full_config():
    # 4096^3: exact float64 BLAS product as the full-size check (all partial sums < 2^53), a
    # sample of rows against the oracle itself
    a = np.random.default_rng(5).integers(0, 256, (4096, 4096), dtype=np.uint8)
    b = np.random.default_rng(6).integers(-128, 128, (4096, 4096), dtype=np.int8)
    az, bz = np.array([128], np.uint8), np.array([0], np.int8)
    y = host(ops.matmul_integer(dev(a), dev(b), dev(az), dev(bz)))
    ref = (a.astype(np.float64) - 128.0) @ b.astype(np.float64)
    assert np.array_equal(y.astype(np.float64), ref)
    rows = [0, 1, 255, 256, 2047, 4095]
    assert np.array_equal(y[rows], oracle.matmul_integer(a[rows], b, az, bz, threads=8))


# ------------------------------------------------------------------ empty inputs and rejected arguments

def test_empty_inputs_are_no_ops_and_bad_arguments_are_refused():
    """Through the C ABI itself: every launcher returns 0 for a tensor without elements and leaves the
    output alone, and refuses (negative code, nothing enqueued) null operands, types it has no kernel
    for and workspaces that are too small."""
    L, p = ops.lib(), ops._ptr
    E_UNSUPPORTED, E_ARGUMENT, E_WORKSPACE = -1, -2, -3
    buf = torch.full((4096,), 7.0, device=DEV)               # stands in for every operand
    out = torch.full((4096,), -3.0, device=DEV)
    i64 = torch.zeros(64, device=DEV, dtype=torch.int64)
    d, o = p(buf), p(out)
    parts = (C.c_void_p * 2)(out.data_ptr(), out.data_ptr() + 8192)     # two parts inside `out`
    null_part = (C.c_void_p * 2)(out.data_ptr(), None)
    seg = np.array([8, 8], np.uint32).ctypes.data_as(C.c_void_p)
    calls = {
        "rms_norm rows=0": L.rg_hip_rms_norm(o, d, d, 0, 64, 1e-5, abi.F32, None),
        "softmax mid=0": L.rg_hip_softmax(o, d, 4, 0, 1, abi.F32, 0, None),
        "rope seq=0": L.rg_hip_rope(o, d, p(i64), 0, 2, 0, 4, 64, 1e4, abi.FP16, None),
        "dequantize inner=0": L.rg_hip_dequantize_linear(o, d, d, None, 1, 4, 0, abi.I8, 1, None),
        "cast size=0": L.rg_hip_cast(o, d, 0, abi.F32, abi.FP16, None),
        "matmul batch=0": L.rg_hip_matmul(o, d, d, None, abi.FP16, 0, 0, 1.0, 0.0, 0, 4, 4, 4, None, None, 0, 0, 0, None),
        "matmul_integer m=0": L.rg_hip_matmul_integer(o, d, d, None, None, 0, 1, 0, 8, 8, None, None, None, None),
        "transpose no blocks": L.rg_hip_transpose(o, d, p(i64), p(i64), 1, 16, 0, None),
        "split no blocks": L.rg_hip_split(parts, d, seg, 2, 0, 16, None),
        "concat no parts": L.rg_hip_concat(o, parts, seg, 0, 4, 16, None),
        "expand no blocks": L.rg_hip_expand(o, d, p(i64), p(i64), 1, 16, 0, None),
        "where no outputs": L.rg_hip_where(o, d, d, d, None, 0, 0, 4, None),
        "attention N=0": L.rg_hip_attention_kvcache(o, d, d, d, None, None, None, 0, 0, 8, 2, 1, 0, 128, 0.1, abi.FP16,
                                                     None, 0, None, None),
    }
    assert all(rc == 0 for rc in calls.values()), calls
    torch.cuda.synchronize()
    assert torch.all(out == -3.0)

    one = np.array([1], np.uint32).ctypes.data_as(C.c_void_p)
    refused = {
        "rms_norm null": (L.rg_hip_rms_norm(o, None, d, 4, 64, 1e-5, abi.F32, None), E_ARGUMENT),
        "rms_norm of integers": (L.rg_hip_rms_norm(o, d, d, 4, 64, 1e-5, abi.I32, None), E_UNSUPPORTED),
        "softmax null": (L.rg_hip_softmax(None, d, 4, 8, 1, abi.F32, 0, None), E_ARGUMENT),
        "softmax of bytes": (L.rg_hip_softmax(o, d, 4, 8, 1, abi.U8, 0, None), E_UNSUPPORTED),
        "rope odd dim": (L.rg_hip_rope(o, d, p(i64), 0, 1, 2, 2, 63, 1e4, abi.FP16, None), E_UNSUPPORTED),
        "dequantize from float": (L.rg_hip_dequantize_linear(o, d, d, None, 1, 1, 8, abi.F32, 0, None), E_UNSUPPORTED),
        "dequantize null scale": (L.rg_hip_dequantize_linear(o, d, None, None, 1, 1, 8, abi.I8, 0, None), E_ARGUMENT),
        "dynamic quantize without workspace": (L.rg_hip_dynamic_quantize_linear(o, o, o, d, 64, None, 0, None), E_WORKSPACE),
        "dynamic quantize size 0": (L.rg_hip_dynamic_quantize_linear(o, o, o, d, 0, d, 1 << 14, None), E_ARGUMENT),
        "cast from strings": (L.rg_hip_cast(o, d, 8, 8, abi.F32, None), E_UNSUPPORTED),
        "matmul of bytes": (L.rg_hip_matmul(o, d, d, None, abi.U8, 0, 0, 1.0, 0.0, 1, 4, 4, 4, None, None, 0, 0, 0, None),
                            E_UNSUPPORTED),
        "matmul null": (L.rg_hip_matmul(o, None, d, None, abi.FP16, 0, 0, 1.0, 0.0, 1, 4, 4, 4, None, None, 0, 0, 0, None),
                        E_ARGUMENT),
        "matmul_integer null": (L.rg_hip_matmul_integer(None, d, d, None, None, 0, 1, 8, 8, 8, None, None, None, None), E_ARGUMENT),
        "fused dequantize without scale": (L.rg_hip_matmul_integer_dequantize(o, d, d, None, None, 0, 1, 8, 8, 8, None, None,
                                                                              None, 0, None, None), E_ARGUMENT),
        "transpose in place": (L.rg_hip_transpose(d, d, one, one, 1, 16, 4, None), E_ARGUMENT),
        "transpose of nine dimensions": (L.rg_hip_transpose(o, d, p(i64), p(i64), 9, 16, 4, None), E_UNSUPPORTED),
        "split segments that do not add up": (L.rg_hip_split(parts, d, seg, 2, 4, 24, None), E_ARGUMENT),
        "split into a null part": (L.rg_hip_split(null_part, d, seg, 2, 4, 16, None), E_ARGUMENT),
        "concat into null": (L.rg_hip_concat(None, parts, seg, 2, 4, 16, None), E_ARGUMENT),
        "expand in place": (L.rg_hip_expand(d, d, one, one, 1, 16, 4, None), E_ARGUMENT),
        "expand of nine dimensions": (L.rg_hip_expand(o, d, p(i64), p(i64), 9, 16, 4, None), E_UNSUPPORTED),
        "where of three-byte elements": (L.rg_hip_where(o, d, d, d, None, 0, 16, 3, None), E_UNSUPPORTED),
        "where without a condition": (L.rg_hip_where(o, None, d, d, None, 0, 16, 4, None), E_ARGUMENT),
        "attention head dim 48": (L.rg_hip_attention_kvcache(o, d, d, d, None, None, None, 0, 1, 8, 2, 1, 0, 48, 0.1, abi.FP16,
                                                              d, 1 << 14, None, None), E_UNSUPPORTED),
        "attention heads not a multiple": (L.rg_hip_attention_kvcache(o, d, d, d, None, None, None, 0, 1, 8, 3, 1, 0, 128, 0.1,
                                                                       abi.FP16, d, 1 << 14, None, None), E_ARGUMENT),
        "attention one cache only": (L.rg_hip_attention_kvcache(o, d, d, d, d, None, None, 0, 1, 8, 2, 1, 16, 128, 0.1, abi.FP16,
                                                                 d, 1 << 14, None, None), E_ARGUMENT),
        "attention without workspace": (L.rg_hip_attention_kvcache(o, d, d, d, None, None, None, 0, 1, 8, 2, 1, 0, 128, 0.1,
                                                                    abi.FP16, None, 0, None, None), E_WORKSPACE),
    }
    wrong = {k: v for k, v in refused.items() if v[0] != v[1]}
    assert not wrong, wrong
    torch.cuda.synchronize()
    assert torch.all(out == -3.0) and torch.all(buf == 7.0)
    for code in (E_UNSUPPORTED, E_ARGUMENT, E_WORKSPACE):
        assert L.rg_hip_error_string(code).startswith(b"rg_hip:")


# ------------------------------------------------------------------ Transpose (bit-exact: data movement)

def test_transpose_driver_digest_equals_the_oracles():
    rng = np.random.default_rng(1)
    for _ in range(300):
        rank = int(rng.integers(1, 7))
        shape = [int(v) for v in rng.integers(1, 5, rank)]
        perm = [int(v) for v in rng.permutation(rank)]
        si, so, block, count = ops.transpose_info(shape, perm, 2)
        dims, oblock, ocount = oracle.transpose_info(shape, perm, 2)
        assert (list(zip(si, so)), block, count) == (dims, oblock, ocount), (shape, perm)


@pytest.mark.parametrize("shape,perm", [
    ((1, 3, 2, 5), (2, 3, 0, 1)),            # src/04kernel/test/kernels/transpose/test_cpu.cpp:9-15
    ((2, 3, 4, 5), (0, 1, 2, 3)), ((7,), (0,)), ((5, 9), (1, 0)), ((3, 5, 7), (2, 1, 0)), ((3, 5, 7), (1, 2, 0)),
    ((2, 48, 8, 128), (0, 2, 1, 3)), ((4, 6, 33, 17), (0, 2, 1, 3)), ((2, 3, 4, 5, 6), (4, 0, 3, 1, 2)),
    ((2, 1, 3, 1, 4), (3, 2, 4, 1, 0)), ((64, 40, 24), (1, 0, 2)), ((129, 257), (1, 0)),
    ((3, 130, 70), (2, 0, 1)), ((3, 130, 70), (0, 2, 1)), ((2, 65, 3, 67), (3, 1, 2, 0))])
@pytest.mark.parametrize("dt", [np.uint8, np.float16, np.float32, np.float64])
def test_transpose_bit_exact(shape, perm, dt):
    x = np.random.default_rng(len(shape)).integers(0, 200, shape).astype(dt)
    y = ops.transpose(dev(x), perm)
    ref = oracle.transpose(x, perm)
    assert tuple(y.shape) == ref.shape and np.array_equal(host(y), ref) and np.array_equal(ref, np.transpose(x, perm))


@pytest.mark.parametrize("shape,perm", [
    ((200, 136), (1, 0)), ((208, 144), (1, 0)), ((2, 4, 72, 64), (0, 1, 3, 2)), ((3, 80, 5, 48), (0, 3, 2, 1)),
    ((2, 3, 160, 256), (1, 3, 0, 2)), ((16, 4096), (1, 0)), ((4096, 16), (1, 0)), ((5, 128, 128), (2, 0, 1))])
@pytest.mark.parametrize("dt", [np.uint8, np.float16])
def test_transpose_of_8_and_16_bit_elements_with_aligned_rows(shape, perm, dt):
    # the innermost dimension moves and every row of either tensor starts on a 16-byte boundary: tiles of 128-byte
    # rows turned in registers and LDS (whole tiles, tiles that reach beyond either extent, outer dimensions on both
    # sides); the same from addresses 16 bytes into a buffer
    x = np.random.default_rng(len(shape) + shape[0]).integers(0, 250, shape).astype(dt)
    y = ops.transpose(dev(x), perm)
    assert tuple(y.shape) == tuple(x.shape[p] for p in perm) and np.array_equal(host(y), np.transpose(x, perm))
    n = x.size
    elems = 16 // x.itemsize
    src = torch.empty(n + elems, device=DEV, dtype=dev(x).dtype)
    src[elems:] = dev(x).reshape(-1)
    dst = torch.empty(n + elems, device=DEV, dtype=src.dtype)
    y2 = ops.transpose(src[elems:].view(*shape), perm, out=dst[elems:].view(*[shape[p] for p in perm]))
    assert np.array_equal(host(y2), np.transpose(x, perm))


def test_transpose_unaligned_views_and_involution():
    x = torch.arange(3 * 37 * 11, device=DEV, dtype=torch.int16).reshape(3, 37, 11)
    buf = torch.empty(3 * 37 * 11 + 1, device=DEV, dtype=torch.int16)
    y = ops.transpose(x, (1, 0, 2), out=buf[1:].view(37, 3, 11))     # output 2 bytes off a 4-byte boundary
    assert torch.equal(y, x.permute(1, 0, 2))
    assert torch.equal(ops.transpose(ops.transpose(x, (2, 0, 1)), (1, 2, 0)), x)


def test_transpose_full_config():
    # heads and sequence swap around attention: [32, 512, 32, 128] fp16 <-> [32, 32, 512, 128]
    x = torch.randn((32, 512, 32, 128), device=DEV).half()
    y = ops.transpose(x, (0, 2, 1, 3))
    assert torch.equal(y, x.permute(0, 2, 1, 3).contiguous())
    assert torch.equal(ops.transpose(y, (0, 2, 1, 3)), x)
    sl = np.s_[5:6]
    assert np.array_equal(host(y[sl]), oracle.transpose(host(x[sl]), (0, 2, 1, 3)))


# ------------------------------------------------------------------ Split / Concat / Expand / Where
_MOVER_DTYPES = [np.uint8, np.int16, np.float32, np.float64]


@pytest.mark.parametrize("shape,axis,sizes", [
    ((2, 3, 1, 20, 7, 7), 3, [1, 9, 3, 7]),          # the reference's test shape
    ((4096, 12288), 1, [4096, 4096, 4096]),           # fused q, k, v of 4096 tokens: segments of 8 KiB
    ((64, 6144), 1, [4096, 1024, 1024]),              # grouped-query projection (32 + 8 + 8 heads of 128)
    ((5, 7, 33), 2, [1, 0, 30, 2]),                   # odd sizes, an empty part
    ((3, 40, 5), 1, list(range(1, 9)) + [4]),         # nine parts
    ((2, 50, 3), 1, [2] * 25),                        # more parts than one launch takes
    ((10,), 0, [3, 7]),                               # one block
    ((7, 2, 4), 0, [5, 2]),                           # split of the slowest axis: two contiguous halves
])
def test_split_and_concat_bit_exact(shape, axis, sizes):
    rng = np.random.default_rng(len(shape) * 100 + axis)
    for dt in _MOVER_DTYPES:
        x = rng.integers(0, 1 << 15, shape).astype(dt)
        want = oracle.split(x, sizes, axis)
        got = ops.split(dev(x), sizes, axis)
        for g, w in zip(got, want):
            assert np.array_equal(host(g), w)
        assert np.array_equal(host(ops.concat([dev(w) for w in want], axis)), oracle.concat(want, axis))
        assert np.array_equal(host(ops.concat(got, axis)), x)          # inverse of each other


def test_split_concat_misaligned_views():
    # parts and joined tensor two bytes off a four-byte boundary: the unit falls back to 2 bytes
    x = torch.arange(3 * 10 * 6, device=DEV, dtype=torch.int16).reshape(3, 10, 6)
    buf = torch.empty(3 * 4 * 6 + 1, device=DEV, dtype=torch.int16)
    a = buf[1:].view(3, 4, 6)
    b = torch.empty((3, 6, 6), device=DEV, dtype=torch.int16)
    ops.split(x, [4, 6], 1, outs=[a, b])
    assert torch.equal(a, x[:, :4]) and torch.equal(b, x[:, 4:])
    jb = torch.empty(3 * 10 * 6 + 1, device=DEV, dtype=torch.int16)
    y = ops.concat([a, b], 1, out=jb[1:].view(3, 10, 6))
    assert torch.equal(y, x)


@pytest.mark.parametrize("inp,out", [
    ((3, 4, 1, 6), (2, 3, 4, 5, 6)),                  # the reference's test shape
    ((4096,), (512, 4096)),                           # a bias over rows
    ((32, 1, 128), (32, 512, 128)),
    ((1, 8, 1, 128), (4, 8, 16, 128)),                # a kv head repeated
    ((5, 1), (3, 5, 7)),                              # innermost dimension broadcast: blocks of 7 elements
    ((1,), (9, 11)),
    ((2, 3, 4), (2, 3, 4)),                           # nothing to do: a copy
    ((), (4, 5)),
    ((300, 1), (300, 64)),                            # single elements along rows of whole 16-byte words
    ((1,), (4096,)), ((3, 1, 5, 1), (3, 2, 5, 16)), ((2, 7, 1), (3, 2, 7, 48)), ((), (2, 3, 32)),
])
def test_expand_bit_exact(inp, out):
    rng = np.random.default_rng(sum(out))
    for dt in _MOVER_DTYPES:
        x = rng.integers(0, 1 << 15, inp).astype(dt)
        assert np.array_equal(host(ops.expand(dev(x), out)), oracle.expand(x, out))


@pytest.mark.parametrize("c_shape,x_shape,y_shape", [
    ((2, 5), (2, 3, 2, 5), (3, 2, 5)),                # the reference's test shape
    ((512, 512), (8, 512, 512), (1,)),                # a causal mask over scores, scalar fill
    ((64, 1024), (64, 1024), (64, 1024)),             # nothing broadcast: the vector kernel
    ((1000,), (1000,), (1000,)),
    ((3, 1, 5), (1, 4, 5), (3, 4, 1)),
    ((), (7, 9), (9,)),
    ((4, 1, 64), (1, 6, 64), (4, 6, 1)),              # 16-byte groups: c and x run along the last axis, y does not
    ((5, 1), (5, 48), (3, 1, 48)),                    # c constant within a group
    ((8,), (3, 5, 8), (5, 8)),                        # groups for elements of 2 bytes and wider only
    ((2, 1, 3, 32), (1, 7, 1, 32), (32,)),
])
def test_where_bit_exact(c_shape, x_shape, y_shape):
    rng = np.random.default_rng(len(x_shape))
    for dt in _MOVER_DTYPES:
        c = rng.integers(0, 2, c_shape).astype(bool)
        x = rng.integers(0, 100, x_shape).astype(dt)
        y = rng.integers(100, 200, y_shape).astype(dt)
        assert np.array_equal(host(ops.where(dev(c), dev(x), dev(y))), oracle.where(c, x, y))


def test_data_movers_full_size():
    # the fused q, k, v projection of 32 x 128 tokens split into its three tensors and joined again
    # (numpy.split is the checker at this size, the oracle on a slab)
    x = torch.randn((4096, 3 * 4096), device=DEV).half()
    q, k, v = ops.split(x, [4096, 4096, 4096], 1)
    assert torch.equal(q, x[:, :4096]) and torch.equal(k, x[:, 4096:8192]) and torch.equal(v, x[:, 8192:])
    assert torch.equal(ops.concat([q, k, v], 1), x)
    slab = host(x[:64])
    assert all(np.array_equal(host(t[:64]), w) for t, w in zip((q, k, v), oracle.split(slab, [4096] * 3, 1)))


# ------------------------------------------------------------------ AttentionKVCache

def _attention_case(N, H, Hkv, seq, cap, D, past, dt=torch.float16, seed=9, per_row=True, pairs=None,
                    sync_state=None):
    rng = np.random.default_rng(seed)
    mk = lambda shape: dev(rng.standard_normal(shape).astype(np.float32)).to(dt)
    q, k, v = mk((N, H, seq, D)), mk((N, Hkv, seq, D)), mk((N, Hkv, seq, D))
    kc, vc = mk((N, Hkv, cap, D)), mk((N, Hkv, cap, D))
    past = np.asarray(past, dtype=np.int64).reshape(-1)
    kc0, vc0 = kc.clone(), vc.clone()
    o = ops.attention_kvcache(q, k, v, kc, vc, dev(past), 1 / math.sqrt(D), sync_state=sync_state)
    f = lambda t: host(t.float())
    ref_o, ref_kc, ref_vc = oracle.attention_kvcache(f(q), f(k), f(v), f(kc0), f(vc0), past, 1 / math.sqrt(D),
                                                     heads=pairs)
    return f(o), ref_o, f(kc), ref_kc, f(vc), ref_vc


@pytest.mark.parametrize("N,H,Hkv,seq,cap,D,past", [
    (2, 4, 2, 1, 64, 64, [5, 40]),
    (3, 8, 2, 1, 300, 128, [0, 17, 299]),
    (4, 32, 8, 1, 1024, 128, [1, 100, 640, 1023]),
    (2, 6, 2, 1, 128, 128, [64, 3]),        # group of 3 heads: 2 + 1 launches
    (2, 4, 4, 1, 128, 64, [100, 9]),        # MHA
    (2, 8, 2, 5, 64, 128, [0, 20]),         # several new rows with history
    (1, 4, 1, 16, 16, 64, [0]),             # prefill into an exactly fitting cache
    (1, 6, 2, 8, 64, 128, [7]),             # history shorter than one step: some key rows meet their
    (1, 2, 1, 48, 64, 64, [7]),             #   first valid key only among the new rows
    (2, 5, 1, 12, 64, 128, [3, 40]),
    (1, 1, 1, 9, 32, 64, [1]),
])
def test_attention_decode_and_small_prefill(N, H, Hkv, seq, cap, D, past):
    o, ref_o, kc, ref_kc, vc, ref_vc = _attention_case(N, H, Hkv, seq, cap, D, past)
    assert np.max(np.abs(o - ref_o)) <= ABS_F16
    assert np.array_equal(kc, ref_kc) and np.array_equal(vc, ref_vc)  # appended rows, rest untouched


@pytest.mark.parametrize("N,H,Hkv,seq,cap,D,dt", [
    (16, 8, 8, 8, 32, 64, torch.float16),     # many short segments: several pieces per range, several passes
    (70, 4, 2, 1, 96, 128, torch.float16),    # more than 64 batch rows: the partition is built by the whole workgroup
    (24, 12, 4, 3, 40, 128, torch.bfloat16),  # group of 3 heads (two launches), short segments, bf16
    (4, 8, 8, 200, 256, 64, torch.float16),   # head dim 64, 200 new rows (the tiled kernel)
    (200, 2, 1, 1, 48, 64, torch.float16),    # 200 batch rows
])
def test_attention_split_many_segments(N, H, Hkv, seq, cap, D, dt):
    past = np.random.default_rng(21).integers(0, cap - seq + 1, N)
    o, ref_o, kc, ref_kc, vc, ref_vc = _attention_case(N, H, Hkv, seq, cap, D, past, dt=dt, seed=22)
    assert np.max(np.abs(o - ref_o)) <= (ABS_F16 if dt == torch.float16 else 2e-2)
    assert np.array_equal(kc, ref_kc) and np.array_equal(vc, ref_vc)


def test_attention_scalar_past_no_cache_and_bf16():
    o, ref_o, kc, ref_kc, _, _ = _attention_case(2, 8, 2, 1, 200, 128, [77])
    assert np.max(np.abs(o - ref_o)) <= ABS_F16 and np.array_equal(kc, ref_kc)
    o, ref_o, kc, ref_kc, _, _ = _attention_case(2, 8, 4, 1, 256, 128, [200, 13], dt=torch.bfloat16)
    assert np.max(np.abs(o - ref_o)) <= 2e-2 and np.array_equal(kc, ref_kc)
    # no cache: plain causal self-attention over the new rows
    rng = np.random.default_rng(10)
    mk = lambda shape: dev(rng.standard_normal(shape).astype(np.float32)).half()
    q, k, v = mk((2, 4, 9, 64)), mk((2, 2, 9, 64)), mk((2, 2, 9, 64))
    o = host(ops.attention_kvcache(q, k, v, scale=0.125).float())
    f = lambda t: host(t.float())
    ref, _, _ = oracle.attention_kvcache(f(q), f(k), f(v), np.zeros((2, 2, 9, 64), np.float32),
                                         np.zeros((2, 2, 9, 64), np.float32), [0, 0], 0.125)
    assert np.max(np.abs(o - ref)) <= ABS_F16


def test_attention_decode_full_config():
    # N=32, 32 q heads / 8 kv heads, D=128, cap 4096, past ~ U{1024..4095}
    past = np.random.default_rng(14).integers(1024, 4096, 32)
    pairs = [(b, h) for b in (0, 7, 19, 31) for h in (0, 5, 14, 31)]
    o, ref_o, kc, ref_kc, vc, ref_vc = _attention_case(32, 32, 8, 1, 4096, 128, past, pairs=pairs)
    for b, h in pairs:
        assert np.max(np.abs(o[b, h] - ref_o[b, h])) <= ABS_F16
    assert np.array_equal(kc, ref_kc) and np.array_equal(vc, ref_vc)
    assert np.isfinite(o).all()


def test_attention_decode_run_to_run_difference_is_bounded():
    # Which blocks a wavefront pulls is decided at run time (a counter in LDS), so the order in which the pieces of a
    # segment are summed may change from run to run: the caches must come out bit for bit the same, the outputs
    # within two units in the last place of the 16-bit result (each run rounds a float that differs by reordering)
    N, H, Hkv, cap, D = 32, 32, 8, 4096, 128
    g = torch.Generator(device=DEV).manual_seed(21)
    rnd = lambda shape: torch.randn(shape, generator=g, device=DEV).half()
    q, k, v = rnd((N, H, 1, D)), rnd((N, Hkv, 1, D)), rnd((N, Hkv, 1, D))
    kc0, vc0 = rnd((N, Hkv, cap, D)), rnd((N, Hkv, cap, D))
    past = torch.from_numpy(np.random.default_rng(14).integers(1024, 4096, N)).to(DEV)
    runs = []
    for _ in range(3):
        kc, vc = kc0.clone(), vc0.clone()
        o = ops.attention_kvcache(q, k, v, kc, vc, past)
        torch.cuda.synchronize()
        runs.append((o, kc, vc))
    o0, kc_a, vc_a = runs[0]
    ulp = torch.maximum(o0.float().abs(), torch.tensor(2.0 ** -14, device=DEV)).log2().floor().exp2() * 2.0 ** -10
    for o, kc, vc in runs[1:]:
        assert torch.equal(kc, kc_a) and torch.equal(vc, vc_a)
        assert bool(((o.float() - o0.float()).abs() <= 2 * ulp).all())


def test_attention_persistent_sync_state_is_left_zero():
    # with caller-owned ticket counters the call is one launch; the counters must come back zero
    # so that consecutive calls (different shapes) can share them
    state = ops.attention_state(DEV)
    for shape in [(4, 32, 8, 1, 1024, 128, [1, 100, 640, 1023]), (2, 8, 2, 5, 64, 128, [0, 20]),
                  (32, 32, 8, 1, 4096, 128, np.random.default_rng(14).integers(1024, 4096, 32))]:
        pairs = [(0, 0), (1, 3)] if shape[0] == 32 else None
        o, ref_o, kc, ref_kc, vc, ref_vc = _attention_case(*shape, pairs=pairs, sync_state=state)
        ok = np.isfinite(ref_o)
        assert np.max(np.abs(o[ok] - ref_o[ok])) <= ABS_F16
        assert np.array_equal(kc, ref_kc) and np.array_equal(vc, ref_vc)
        assert int(state.sum()) == 0


def test_attention_decode_invariants_full_size():
    # uniform K => O = mean(V); permuting history positions leaves O unchanged (to rounding)
    N, H, Hkv, cap, D = 4, 32, 8, 4096, 128
    g = torch.Generator(device=DEV).manual_seed(12)
    rnd = lambda shape: torch.randn(shape, generator=g, device=DEV).half()
    q, k, v = rnd((N, H, 1, D)), rnd((N, Hkv, 1, D)), rnd((N, Hkv, 1, D))
    vc = rnd((N, Hkv, cap, D))
    past = torch.tensor([4095, 2048, 1024, 3000], device=DEV)
    kc = k.expand(N, Hkv, cap, D).contiguous()
    o = ops.attention_kvcache(q, k, v, kc, vc.clone(), past)
    for b in range(N):
        L = int(past[b]) + 1
        vv = torch.cat([vc[b, :, :L - 1], v[b]], dim=1).float().mean(1)          # [Hkv, D]
        assert float((o[b, :, 0].float() - vv.repeat_interleave(4, 0)).abs().max()) <= ABS_F16
    kc = rnd((N, Hkv, cap, D))
    o1 = ops.attention_kvcache(q, k, v, kc.clone(), vc.clone(), past)
    perm = torch.randperm(1024, generator=torch.Generator().manual_seed(1)).to(DEV)
    kc2, vc2 = kc.clone(), vc.clone()
    kc2[:, :, :1024] = kc[:, :, perm]
    vc2[:, :, :1024] = vc[:, :, perm]
    o2 = ops.attention_kvcache(q, k, v, kc2, vc2, past)
    assert float((o1.float() - o2.float()).abs().max()) <= ABS_F16


@pytest.mark.parametrize("N,H,Hkv,seq,cap,D,past,dt", [
    (2, 8, 2, 40, 128, 128, [0, 20], torch.float16),      # ragged: 40 rows, history on one row
    (2, 4, 4, 33, 64, 128, [5, 31], torch.float16),       # MHA (one head per workgroup)
    (1, 4, 2, 64, 200, 128, [100], torch.float16),        # group of 2
    (2, 16, 2, 96, 96, 128, [0, 0], torch.float16),       # group of 8: two head chunks per kv head
    (2, 8, 2, 70, 256, 128, [3, 150], torch.bfloat16),
    (1, 6, 2, 48, 64, 128, [7], torch.float16),           # group of 3: a short chunk of heads
    (1, 8, 2, 129, 512, 128, [300], torch.float16),
    (2, 8, 2, 40, 128, 64, [0, 20], torch.float16),       # head dim 64: the same kernel on half rows
    (2, 4, 4, 33, 64, 64, [5, 31], torch.float16),        # MHA
    (1, 4, 2, 64, 200, 64, [100], torch.float16),         # group of 2
    (2, 16, 2, 96, 96, 64, [0, 0], torch.float16),        # group of 8
    (2, 10, 2, 70, 256, 64, [3, 150], torch.bfloat16),    # group of 5
    (1, 8, 2, 129, 512, 64, [300], torch.float16),
    (3, 4, 1, 200, 333, 64, [0, 70, 133], torch.float16), # odd capacity and history lengths: the seam inside tiles
    (2, 8, 2, 40, 128, 96, [0, 20], torch.float16),       # head dim 96: twelve chunks a row, three blocks of O^T
    (2, 4, 4, 33, 64, 80, [5, 31], torch.float16),        # head dim 80: the third block of O^T half used
    (1, 10, 2, 129, 512, 80, [300], torch.bfloat16),      # group of 5
    (3, 4, 1, 200, 333, 96, [0, 70, 133], torch.float16),
    (2, 8, 8, 1, 300, 80, [17, 299], torch.float16),      # a decode step: these head dims have the tiled kernel only
    (3, 6, 2, 1, 64, 96, [0, 5, 63], torch.bfloat16),
    (1, 32, 32, 7, 40, 96, [33], torch.float16),
])
def test_attention_prefill_tiled_kernel(N, H, Hkv, seq, cap, D, past, dt):
    o, ref_o, kc, ref_kc, vc, ref_vc = _attention_case(N, H, Hkv, seq, cap, D, past, dt=dt)
    assert np.max(np.abs(o - ref_o)) <= (ABS_F16 if dt == torch.float16 else 2e-2)
    assert np.array_equal(kc, ref_kc) and np.array_equal(vc, ref_vc)


@pytest.mark.parametrize("N,H,Hkv,seq,cap,D,dt", [
    (40, 32, 8, 2, 200, 128, torch.float16),    # two new rows per sequence, many sequences: the tiled kernel pays
    (36, 8, 8, 3, 96, 128, torch.float16),      # MHA, three rows
    (24, 12, 4, 5, 70, 128, torch.bfloat16),    # group of 3: the last wavefront of a chunk repeats a head, stores nothing
    (12, 40, 8, 4, 130, 128, torch.float16),    # group of 5: two chunks, the second with one head
    (10, 28, 4, 7, 64, 128, torch.float16),     # group of 7
    (3, 8, 2, 9, 300, 128, torch.float16),      # few sequences: the split kernel (one segment per query row)
    (40, 24, 8, 1, 96, 128, torch.float16),     # one new row, group of 3: the split kernel would take two launches
    (36, 64, 8, 1, 200, 128, torch.float16),    # one new row, group of 8
    (40, 16, 8, 3, 150, 64, torch.float16),     # head dim 64
    (12, 20, 4, 6, 90, 64, torch.bfloat16),     # head dim 64, group of 5
])
def test_attention_few_new_rows_either_kernel(N, H, Hkv, seq, cap, D, dt):
    # up to 31 new rows per sequence run through the tiled kernel when there are enough sequences and kv heads to
    # occupy the chip with one item each (a single new row only where the split kernel would need several launches
    # for the head group), else through the split kernel; any head group size
    past = np.random.default_rng(33).integers(0, cap - seq + 1, N)
    o, ref_o, kc, ref_kc, vc, ref_vc = _attention_case(N, H, Hkv, seq, cap, D, past, dt=dt, seed=34)
    assert np.max(np.abs(o - ref_o)) <= (ABS_F16 if dt == torch.float16 else 2e-2)
    assert np.array_equal(kc, ref_kc) and np.array_equal(vc, ref_vc)


@pytest.mark.parametrize("N,H,Hkv,seq,cap,D,past,dt", [
    (1, 32, 8, 128, 4128, 128, [4000], torch.float16),      # a chunk of a long prompt: 32 items, 16 key ranges each
    (1, 32, 8, 33, 4033, 128, [4000], torch.float16),       # ragged query rows
    (1, 32, 8, 128, 8128, 128, [10], torch.float16),        # a long cache with a short history: ranges beyond the keys
    (1, 32, 8, 200, 3200, 128, [0], torch.float16),         # no history at all
    (2, 8, 8, 100, 2600, 128, [2500, 17], torch.float16),   # one head per kv head, histories that differ
    (1, 16, 2, 77, 3077, 64, [2999], torch.bfloat16),       # head dim 64, group of 8 (two chunks of four heads)
    (1, 12, 4, 64, 5064, 128, [4321], torch.bfloat16),      # group of 3
    (3, 4, 2, 8, 1508, 64, [1500, 0, 700], torch.float16),  # eight new rows: the tiled kernel by the cost rule
    (1, 32, 8, 16, 6016, 128, [6000], torch.float16),       # sixteen new rows
])
def test_attention_long_history_keys_shared_between_workgroups(N, H, Hkv, seq, cap, D, past, dt):
    # few items (one sequence, a chunk of a prompt or a new turn of a conversation) against a long cache: the tiled
    # kernel shares an item's keys between workgroups and a second launch merges their partial results
    o, ref_o, kc, ref_kc, vc, ref_vc = _attention_case(N, H, Hkv, seq, cap, D, past, dt=dt, seed=61)
    assert not np.isnan(o).any()
    assert np.max(np.abs(o - ref_o)) <= (ABS_F16 if dt == torch.float16 else 2e-2)
    assert np.array_equal(kc, ref_kc) and np.array_equal(vc, ref_vc)


def test_attention_prefill_no_cache_tiled():
    rng = np.random.default_rng(21)
    mk = lambda shape: dev(rng.standard_normal(shape).astype(np.float32)).half()
    q, k, v = mk((2, 8, 50, 128)), mk((2, 2, 50, 128)), mk((2, 2, 50, 128))
    o = host(ops.attention_kvcache(q, k, v, scale=0.1).float())
    f = lambda t: host(t.float())
    z = np.zeros((2, 2, 50, 128), np.float32)
    ref, _, _ = oracle.attention_kvcache(f(q), f(k), f(v), z, z, [0, 0], 0.1)
    assert np.max(np.abs(o - ref)) <= ABS_F16


def test_attention_prefill_config_sample():
    # seq 512, past 0, causal, 32/8 heads, D=128 (batch cut to 2 so the oracle finishes in seconds)
    pairs = [(0, 0), (0, 13), (1, 31)]
    o, ref_o, kc, ref_kc, vc, ref_vc = _attention_case(2, 32, 8, 512, 4096, 128, [0, 0], pairs=pairs)
    for b, h in pairs:
        assert np.max(np.abs(o[b, h] - ref_o[b, h])) <= ABS_F16
    assert np.array_equal(kc, ref_kc) and np.array_equal(vc, ref_vc)


def test_attention_prefill_full_config():
    # the whole configuration: N=32, seq 512, past 0, causal, 32/8 heads, D=128, cap 4096 (4096 workgroups,
    # 256 (batch row, kv head) streams dealt to the XCDs).  Whole-cache append bit-exact, eight (b, h) pairs
    # spread over the batch against the oracle, every output finite, and rows 0 (which see one key: O = V)
    g = torch.Generator(device=DEV).manual_seed(31)
    rnd = lambda shape: torch.randn(shape, generator=g, device=DEV).half()
    N, H, Hkv, seq, cap, D = 32, 32, 8, 512, 4096, 128
    q, k, v = rnd((N, H, seq, D)), rnd((N, Hkv, seq, D)), rnd((N, Hkv, seq, D))
    kc, vc = rnd((N, Hkv, cap, D)), rnd((N, Hkv, cap, D))
    kc0, vc0 = kc.clone(), vc.clone()
    past = torch.zeros(N, device=DEV, dtype=torch.int64)
    scale = 1 / math.sqrt(D)
    o = ops.attention_kvcache(q, k, v, kc, vc, past, scale)
    torch.cuda.synchronize()
    assert torch.equal(kc[:, :, :seq], k) and torch.equal(vc[:, :, :seq], v)
    assert torch.equal(kc[:, :, seq:], kc0[:, :, seq:]) and torch.equal(vc[:, :, seq:], vc0[:, :, seq:])
    assert bool(torch.isfinite(o).all())
    assert torch.equal(o[:, :, 0], v[:, :, 0].repeat_interleave(H // Hkv, 1))
    f = lambda t: host(t.float())
    for b, h in [(0, 0), (3, 9), (8, 31), (13, 4), (17, 22), (22, 15), (27, 2), (31, 31)]:
        kh = h // (H // Hkv)
        ref = oracle.attention_head(f(q[b, h]), f(k[b, kh]), f(v[b, kh]), 0, scale, True)
        assert np.max(np.abs(f(o[b, h]) - ref)) <= ABS_F16, (b, h)


@pytest.mark.parametrize("N,H,Hkv,seq,cap,D,past", [
    (3, 8, 2, 1, 64, 128, [63, 64, 1000]),     # decode: the cache is full (63 fits, the others are moved back)
    (2, 4, 2, 5, 32, 64, [30, -3]),            # several new rows through the split kernel; a negative length is 0
    (2, 8, 2, 40, 64, 128, [30, 24]),          # tiled prefill kernel: 30 + 40 > 64 is moved back to 24
])
def test_attention_history_length_outside_the_cache(N, H, Hkv, seq, cap, D, past):
    # the lengths are device data, so the kernels cannot refuse them: they are moved into [0, cap - seq]
    # and the oracle states the same rule
    o, ref_o, kc, ref_kc, vc, ref_vc = _attention_case(N, H, Hkv, seq, cap, D, past)
    assert np.max(np.abs(o - ref_o)) <= ABS_F16
    assert np.array_equal(kc, ref_kc) and np.array_equal(vc, ref_vc)


# ------------------------------------------------------------------ Cast
_CAST_TORCH = {"u8": torch.uint8, "i8": torch.int8, "i16": torch.int16, "i32": torch.int32, "i64": torch.int64,
               "f32": torch.float32, "f64": torch.float64, "bool": torch.bool, "fp16": torch.float16,
               "bf16": torch.bfloat16, "u16": torch.uint16, "u32": torch.uint32, "u64": torch.uint64}
_CAST_BITS = {"u8": 8, "i8": 8, "u16": 16, "i16": 16, "u32": 32, "i32": 32, "u64": 64, "i64": 64}


def _cast_input(src, dst, n, rng):
    """Values of type `src` whose conversion to `dst` is defined (float -> integer stays inside
    the target's range; everything else is unrestricted)."""
    np_t = oracle._CAST_NP[src]
    if src == "bool":
        return rng.integers(0, 2, n).astype(np.bool_)
    if src in _CAST_BITS:
        info = np.iinfo(np_t)
        x = rng.integers(info.min, info.max, n, dtype=np_t, endpoint=True)
        x[:4] = [info.min, info.max, 0, 1]
        return x
    # floating sources
    if dst in _CAST_BITS:
        bits = _CAST_BITS[dst]
        hi = float(2 ** (bits - (0 if dst[0] == "u" else 1)))
        hi = min(hi, 60000.0 if src == "fp16" else hi, 2.0 ** 62)
        lo = 0.0 if dst[0] == "u" else -hi
        f = rng.uniform(lo * 0.999, hi * 0.999, n)
        if src in ("fp16", "bf16"):
            hi, lo = min(hi, 2.0 ** 31) * 0.99, max(lo, -2.0 ** 31) * 0.99   # these go through `int`
            f = rng.uniform(lo, hi, n)
    else:
        f = rng.standard_normal(n) * np.exp(rng.uniform(-20, 12, n))
        f[:6] = [0.0, -0.0, 2049.0, 2051.0, 65519.9, 65520.0]
    if src == "f64":
        return f.astype(np.float64)
    f32 = f.astype(np.float32)
    if src == "f32":
        return f32
    with np.errstate(over="ignore"):
        return f32.astype(np.float16) if src == "fp16" else oracle.cast(f32, "f32", "bf16")


def _cast_to_torch(x, name):
    if name == "bf16":
        return dev(x).view(torch.bfloat16)
    return dev(x)


def _cast_bits(t, name):
    """Result tensor -> numpy array comparable bit for bit."""
    if name == "bf16":
        return host(t.view(torch.uint16))
    a = host(t)
    return a.view(np.uint16) if name == "fp16" else a


@pytest.mark.parametrize("src", oracle.CAST_TYPES)
def test_cast_all_pairs_bit_exact(src):
    rng = np.random.default_rng(hash(src) % 1000)
    for dst in oracle.CAST_TYPES:
        n = 10007                                     # odd: vector body and scalar tail
        x = _cast_input(src, dst, n, rng)
        want = oracle.cast(x, src, dst)
        got = _cast_bits(ops.cast(_cast_to_torch(x, src), _CAST_TORCH[dst]), dst)
        want = want.view(np.uint16) if dst == "fp16" else want
        assert got.shape == want.shape and np.array_equal(got, want), (src, dst)


def test_cast_reference_kat_and_edges():
    x = np.arange(120, dtype=np.float64).reshape(2, 3, 4, 5)      # cast/test_cpu.cpp
    assert np.array_equal(host(ops.cast(dev(x), torch.int8)).reshape(-1), np.arange(120))
    # misaligned views (scalar path), same-type copy, in-place no-op
    base = dev(np.arange(1, 4098, dtype=np.float32))
    view = base[1:]
    assert np.array_equal(host(ops.cast(view, torch.float16)).view(np.uint16),
                          oracle.cast(host(view), "f32", "fp16").view(np.uint16))
    out = torch.empty(4099, dtype=torch.int32, device="cuda")[3:]
    ops.cast(view, torch.int32, out=out)
    assert np.array_equal(host(out), host(view).astype(np.int32))
    assert np.array_equal(host(ops.cast(view, torch.float32)), host(view))
    same = ops.cast(view, torch.float32, out=view)
    assert same.data_ptr() == view.data_ptr() and np.array_equal(host(view), np.arange(2, 4098, dtype=np.float32))
    # double -> half goes through float (two roundings, like the reference's expression)
    assert host(ops.cast(dev(np.array([1 + 2.0 ** -11 + 2.0 ** -26])), torch.float16)).view(np.uint16).tolist() == [0x3C00]
    # integers are taken as `int` and rounded toward zero
    assert host(ops.cast(dev(np.array([2049, 2051, -2049, 70000, 16777217], np.int32)), torch.float16)).tolist() == \
        [2048.0, 2050.0, -2048.0, 65504.0, 65504.0]
    assert host(ops.cast(dev(np.array([3000000000], np.uint32)), torch.float16)).tolist() == [-65504.0]


def test_cast_full_config_f32_to_fp16_and_back():
    x = np.random.default_rng(8).standard_normal(32 * 128 * 4096).astype(np.float32)
    h = ops.cast(dev(x), torch.float16)
    assert np.array_equal(host(h).view(np.uint16), x.astype(np.float16).view(np.uint16))
    back = host(ops.cast(h, torch.float32))
    assert np.array_equal(back, x.astype(np.float16).astype(np.float32))     # widening is exact


# ------------------------------------------------------------------ MatMul
# Tolerances: F32 products are summed in a different order than the CPU loop: |y - ref| <= 1e-5 * sum|a||b|
# (covers 1e-5 relative on well-conditioned sums).  FP16 / BF16: float accumulation, one rounding of the
# result: one half-precision ulp of the reference plus the same accumulation term.
def _matmul_check(got, ref, a_abs_b_abs, rel_out):
    tol = rel_out * np.abs(ref) + 1e-5 * a_abs_b_abs + 1e-30
    assert got.shape == ref.shape
    assert np.all(np.abs(got.astype(np.float64) - ref.astype(np.float64)) <= tol), \
        float(np.max(np.abs(got.astype(np.float64) - ref.astype(np.float64)) / tol))


def _absprod(a, b, ta, tb):
    A = np.abs(np.swapaxes(a, -1, -2) if ta else a).astype(np.float64)
    B = np.abs(np.swapaxes(b, -1, -2) if tb else b).astype(np.float64)
    return A @ B


def test_matmul_reference_vectors():
    for c in GOLDEN["mat_mul"]:
        if "y" not in c:
            continue
        a = np.array(c["a"], np.float32).reshape(c["a_shape"])
        b = np.array(c["b"], np.float32).reshape(c["b_shape"])
        bias = np.array(c["c"], np.float32).reshape(c["c_shape"] or [1])
        y = host(ops.matmul(dev(a), dev(b), dev(bias), alpha=c["alpha"], beta=c["beta"]))
        assert y.reshape(-1).tolist() == c["y"]


@pytest.mark.parametrize("dt", ["f32", "f64"])
def test_matmul_generic_transposes_bias_broadcast(dt):
    rng = np.random.default_rng(13)
    np_t = np.float32 if dt == "f32" else np.float64
    for ta in (False, True):
        for tb in (False, True):
            m, k, n = 37, 53, 29
            a = rng.standard_normal((2, 1) + ((k, m) if ta else (m, k))).astype(np_t)
            b = rng.standard_normal((1, 3) + ((n, k) if tb else (k, n))).astype(np_t)
            for bias in (None, rng.standard_normal((m, 1)).astype(np_t), rng.standard_normal((n,)).astype(np_t),
                         rng.standard_normal((2, 3, m, n)).astype(np_t)):
                ref = oracle.matmul(a, b, bias, ta, tb, 0.5, 2.0, dt)
                got = host(ops.matmul(dev(a), dev(b), None if bias is None else dev(bias), ta, tb, 0.5, 2.0))
                _matmul_check(got, ref, _absprod(a, b, ta, tb), 1e-5 if dt == "f32" else 1e-12)


@pytest.mark.parametrize("tb", [False, True])
@pytest.mark.parametrize("m,k,n", [(130, 64, 260), (65, 16, 4), (256, 128, 128), (100, 48, 36), (70, 32, 8), (300, 4096, 132),
                                   (1, 64, 16), (3, 4096, 64), (7, 192, 48), (13, 128, 6400), (16, 1024, 32), (31, 320, 80),
                                   (32, 4096, 256), (50, 128, 32), (64, 64, 16), (5, 128, 16), (40, 256, 48), (2, 4096, 64)])
def test_matmul_f32_on_the_matrix_cores(m, k, n, tb):
    # float operands.  More than 64 rows, k a multiple of 16 (and n of 4 for B as [k, n]): 128 x 128 tiles of 32x32x2
    # products, rows and columns beyond the matrix loaded from its last ones.  Up to 64 rows against B as [n, k]
    # (k a multiple of 64, n of 16): 4x4x1 block products, 32 rows a pass.  Batches, bias forms, alpha and beta as
    # everywhere
    rng = np.random.default_rng(m + n)
    a = rng.standard_normal((2, m, k)).astype(np.float32)
    b = rng.standard_normal((2, n, k) if tb else (2, k, n)).astype(np.float32)
    for bias in (None, rng.standard_normal((n,)).astype(np.float32), rng.standard_normal((2, m, n)).astype(np.float32)):
        ref = oracle.matmul(a, b, bias, False, tb, 0.5, 2.0, "f32")
        got = host(ops.matmul(dev(a), dev(b), None if bias is None else dev(bias), False, tb, 0.5, 2.0))
        _matmul_check(got, ref, _absprod(a, b, False, tb), 1e-5)
    # integer-valued operands: every product and sum is exact
    ai = rng.integers(-8, 9, (m, k)).astype(np.float32)
    bi = rng.integers(-8, 9, (n, k) if tb else (k, n)).astype(np.float32)
    want = ai.astype(np.int64) @ (bi.T if tb else bi).astype(np.int64)
    assert np.array_equal(host(ops.matmul(dev(ai), dev(bi), trans_b=tb)), want.astype(np.float32))


@pytest.mark.parametrize("tb", [False, True])
@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16])
# (300, 64, 256) to (513, 192, 520): m and n that are no multiples of the 256 x 256 tile (last tiles moved back,
# overlapping); after them fewer than 256 rows on one row of tiles (where the passes of the few-rows kernels would
# take longer, or k and n fit none of them)
@pytest.mark.parametrize("m,k,n", [(256, 64, 256), (256, 192, 512), (512, 128, 256), (300, 64, 256), (256, 128, 264),
                                   (513, 192, 520), (200, 128, 2560), (100, 64, 264), (40, 192, 512), (10, 64, 256),
                                   (255, 128, 11008), (129, 320, 1032)])
def test_matmul_mfma_path_fp16_bf16(m, k, n, dt, tb):
    rng = np.random.default_rng(14)
    a = rng.standard_normal((2, m, k)).astype(np.float32)
    b = rng.standard_normal((2, n, k) if tb else (2, k, n)).astype(np.float32)
    bias = rng.standard_normal((n,)).astype(np.float32)
    ad, bd, cd = (dev(t).to(dt) for t in (a, b, bias))
    name = "fp16" if dt == torch.float16 else "bf16"
    f = lambda t: host(t.float())
    to_oracle = (lambda t: host(t)) if name == "fp16" else (lambda t: host(t.view(torch.uint16)))
    ref = oracle.matmul(to_oracle(ad), to_oracle(bd), to_oracle(cd), False, tb, 0.25, 1.0, name)
    ref = ref.astype(np.float32) if name == "fp16" else oracle._bf16_to_f32(ref)
    got = f(ops.matmul(ad, bd, cd, False, tb, 0.25, 1.0))
    _matmul_check(got, ref, 0.25 * _absprod(f(ad), f(bd), False, tb), 2.0 ** -10 if name == "fp16" else 2.0 ** -7)
    # broadcast B over the batch (per-matrix launches) and no bias
    got = f(ops.matmul(ad, bd[:1].contiguous(), None, False, tb))
    ref = oracle.matmul(to_oracle(ad), to_oracle(bd[:1].contiguous()), None, False, tb, dtype=name)
    ref = ref.astype(np.float32) if name == "fp16" else oracle._bf16_to_f32(ref)
    _matmul_check(got, ref, _absprod(f(ad), f(bd[:1]), False, tb), 2.0 ** -10 if name == "fp16" else 2.0 ** -7)


@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("tb", [False, True])
@pytest.mark.parametrize("m,k,n", [(300, 72, 128), (130, 1000, 77), (64, 8, 5), (513, 136, 250), (9, 200, 1031), (257, 64, 8)])
def test_matmul_any_shape_on_the_matrix_cores(m, k, n, dt, tb):
    # fewer than 256 columns, column counts that are no multiple of 8 (rows of B as [k, n] then start on odd
    # addresses), k that is no multiple of 64, one to three k tiles: the 128 x 128 tile kernel, against the oracle
    rng = np.random.default_rng(41)
    a = rng.standard_normal((2, m, k)).astype(np.float32)
    b = rng.standard_normal((2, n, k) if tb else (2, k, n)).astype(np.float32)
    bias = rng.standard_normal((2, m, n)).astype(np.float32)
    ad, bd, cd = (dev(t).to(dt) for t in (a, b, bias))
    name = "fp16" if dt == torch.float16 else "bf16"
    f = lambda t: host(t.float())
    to_oracle = (lambda t: host(t)) if name == "fp16" else (lambda t: host(t.view(torch.uint16)))
    ref = oracle.matmul(to_oracle(ad), to_oracle(bd), to_oracle(cd), False, tb, 0.5, 2.0, name)
    ref = ref.astype(np.float32) if name == "fp16" else oracle._bf16_to_f32(ref)
    got = f(ops.matmul(ad, bd, cd, False, tb, 0.5, 2.0))
    mag = 0.5 * _absprod(f(ad), f(bd), False, tb) + 2.0 * np.abs(f(cd))
    _matmul_check(got, ref, mag, 2.0 ** -10 if name == "fp16" else 2.0 ** -7)
    if not tb:
        # B from an address that is no multiple of 4: same values, the aligned words around it are the buffer's own
        flat = torch.cat([torch.zeros(1, dtype=dt, device="cuda"), bd.reshape(-1)])
        got_odd = f(ops.matmul(ad, flat[1:].view(bd.shape), cd, False, tb, 0.5, 2.0))
        assert np.array_equal(got_odd, got)


def test_matmul_any_shape_exact_on_small_integers():
    # integer-valued operands: every result is exact in fp16, so rows, columns and k beyond the matrix must
    # contribute nothing, bit for bit (vocabulary-sized column count, both layouts of B)
    rng = np.random.default_rng(42)
    a = rng.integers(-2, 3, (200, 328)).astype(np.float32)
    b = rng.integers(-2, 3, (328, 5003)).astype(np.float32)
    want = (a.astype(np.int64) @ b.astype(np.int64)).astype(np.float32)
    assert np.max(np.abs(want)) < 2048
    assert np.array_equal(host(ops.matmul(dev(a).half(), dev(b).half()).float()), want)
    assert np.array_equal(host(ops.matmul(dev(a).half(), dev(np.ascontiguousarray(b.T)).half(), trans_b=True).float()), want)


@pytest.mark.parametrize("m,k,n", [(1, 256, 512), (16, 128, 256), (100, 64, 264), (300, 192, 512)])
def test_matmul_one_b_for_the_whole_batch(m, k, n):
    # activations [batch, m, k] against one weight matrix: the C ABI turns the batch into rows of one product; every
    # bias form the reference expands (per column, per output element, and one [m, n] for all, which keeps the
    # per-matrix launches), a batch whose A matrices are not consecutive, and MatMulInteger with zero points per row
    rng = np.random.default_rng(51)
    B = 5
    a = rng.integers(-2, 3, (B, m, k)).astype(np.float32)
    b = rng.integers(-2, 3, (1, k, n)).astype(np.float32)
    want = (a.astype(np.int64) @ b[0].astype(np.int64)).astype(np.float32)
    assert np.max(np.abs(want)) < 1024
    for bias in (None, rng.integers(-3, 4, (n,)).astype(np.float32), rng.integers(-3, 4, (B, m, n)).astype(np.float32),
                 rng.integers(-3, 4, (m, n)).astype(np.float32)):
        got = host(ops.matmul(dev(a).half(), dev(b).half(), None if bias is None else dev(bias).half()).float())
        assert np.array_equal(got, want if bias is None else want + bias), None if bias is None else bias.shape
        bt = dev(np.ascontiguousarray(np.swapaxes(b, -1, -2))).half()
        got = host(ops.matmul(dev(a).half(), bt, None if bias is None else dev(bias).half(), trans_b=True).float())
        assert np.array_equal(got, want if bias is None else want + bias)
    # A broadcast as well ([2, 1, m, k] against [1, 3, k, n]: B differs within the batch, nothing to fold)
    a4 = rng.integers(-2, 3, (2, 1, m, k)).astype(np.float32)
    b4 = rng.integers(-2, 3, (1, 3, k, n)).astype(np.float32)
    got = host(ops.matmul(dev(a4).half(), dev(b4).half()).float())
    assert np.array_equal(got, (a4.astype(np.int64) @ b4.astype(np.int64)).astype(np.float32))
    ai = rng.integers(0, 256, (B, m, k), dtype=np.uint8)
    bi = rng.integers(-128, 128, (1, k, n), dtype=np.int8)
    az, bz = rng.integers(0, 256, (B * m,), dtype=np.uint8), rng.integers(-128, 128, (k,), dtype=np.int8)
    ref = oracle.matmul_integer(ai, bi, az, bz, threads=8)
    assert np.array_equal(host(ops.matmul_integer(dev(ai), dev(bi), dev(az), dev(bz))), ref)
    scale = rng.uniform(1e-4, 1e-2, n).astype(np.float32)
    y = host(ops.matmul_integer(dev(ai), dev(bi), dev(az), dev(bz), dequant_scale=dev(scale)))
    assert np.array_equal(y, oracle.dequantize_linear(ref, scale, None, axis=2))


def test_matmul_one_b_for_a_batch_of_many_small_matrices():
    # 3000 matrices of 24 rows against one [64, 40] matrix: 72000 rows of one product (1125 tiles of 64 rows)
    rng = np.random.default_rng(52)
    a = rng.integers(-2, 3, (3000, 24, 64)).astype(np.float32)
    b = rng.integers(-2, 3, (1, 64, 40)).astype(np.float32)
    want = (a.astype(np.int64) @ b[0].astype(np.int64)).astype(np.float32)
    assert np.array_equal(host(ops.matmul(dev(a).half(), dev(b).half()).float()), want)
    ai = rng.integers(0, 256, (3000, 24, 64), dtype=np.uint8)
    bi = rng.integers(-128, 128, (1, 64, 40), dtype=np.int8)
    az = rng.integers(0, 256, (3000 * 24,), dtype=np.uint8)
    assert np.array_equal(host(ops.matmul_integer(dev(ai), dev(bi), dev(az), None)), oracle.matmul_integer(ai, bi, az, None, threads=8))


@pytest.mark.parametrize("m, k, n", [(1, 128, 24576), (1, 136, 24584), (3, 128, 24592), (4, 72, 25000), (1, 256, 32000),
                                     (1, 1024, 32768), (2, 128, 24577)])
def test_matmul_few_rows_against_a_vocabulary_of_rows(m, k, n):
    # one to four rows against W as [n, k] with more than 23000 rows: the kernels that read W once, whatever n
    # is (a workgroup of the one-row kernel walks several blocks of rows); exact on small integers, with a bias
    rng = np.random.default_rng(m * 1000 + k)
    a = rng.integers(-2, 3, (m, k)).astype(np.float32)
    w = rng.integers(-2, 3, (n, k)).astype(np.float32)
    c = rng.integers(-8, 9, (n,)).astype(np.float32)
    want = (a.astype(np.int64) @ w.T.astype(np.int64)).astype(np.float32)
    for dt in (torch.float16, torch.bfloat16):
        if dt == torch.bfloat16 and np.max(np.abs(want)) + 8 >= 256:
            continue
        got = host(ops.matmul(dev(a).to(dt), dev(w).to(dt), trans_b=True).float())
        assert np.array_equal(got, want)
        got = host(ops.matmul(dev(a).to(dt), dev(w).to(dt), dev(c).to(dt), trans_b=True).float())
        assert np.array_equal(got, want + c)


@pytest.mark.parametrize("m, k, n", [(1, 64, 50257), (5, 80, 50257), (8, 64, 40001), (7, 4096, 5003)])
def test_matmul_up_to_8_rows_against_an_odd_vocabulary(m, k, n):
    # n odd (no kernel with 16-byte loads along n takes it) and so large that the 128 x 128 tiles with most of
    # their rows masked beat the plain kernel: both layouts of B, and MatMulInteger with every kind of zero point
    rng = np.random.default_rng(m * 100 + k)
    a = rng.integers(-1, 2, (m, k)).astype(np.float32)
    b = rng.integers(-1, 2, (k, n)).astype(np.float32)
    c = rng.integers(-8, 9, (n,)).astype(np.float32)
    want = (a.astype(np.int64) @ b.astype(np.int64)).astype(np.float32)
    assert np.max(np.abs(want)) + 8 < 256
    for dt in (torch.float16, torch.bfloat16):
        assert np.array_equal(host(ops.matmul(dev(a).to(dt), dev(b).to(dt), dev(c).to(dt)).float()), want + c)
        bt = dev(np.ascontiguousarray(b.T)).to(dt)
        assert np.array_equal(host(ops.matmul(dev(a).to(dt), bt, trans_b=True).float()), want)
    ai = rng.integers(0, 256, (m, k), dtype=np.uint8)
    bi = rng.integers(-128, 128, (k, n), dtype=np.int8)
    az, bz = rng.integers(0, 256, (m,), dtype=np.uint8), rng.integers(-128, 128, (k,), dtype=np.int8)
    for za, zb in ((None, None), (az[:1], bz[:1]), (az, bz)):
        got = host(ops.matmul_integer(dev(ai), dev(bi), None if za is None else dev(za), None if zb is None else dev(zb)))
        assert np.array_equal(got, oracle.matmul_integer(ai, bi, za, zb, threads=8))


@pytest.mark.parametrize("B, S, T, D", [(32, 32, 32, 128), (32, 128, 128, 128), (32, 128, 512, 128), (6, 40, 264, 64),
                                        (32, 1, 512, 128), (5, 3, 300, 128), (4, 512, 512, 128), (3, 20, 48, 128)])
def test_matmul_batches_of_attention_products(B, S, T, D):
    # scores Q K^T (short k) and their product with V (few columns), one pair of matrices per head: batches whose
    # matrices together decide between the few-rows kernels and one launch of small tiles; exact on small integers
    rng = np.random.default_rng(B * 1000 + S)
    q = rng.integers(-1, 2, (B, S, D)).astype(np.float32)
    kk = rng.integers(-1, 2, (B, T, D)).astype(np.float32)
    p = rng.integers(-1, 2, (B, S, T)).astype(np.float32)
    v = rng.integers(-1, 2, (B, T, D)).astype(np.float32)
    want_s = np.einsum("bsd,btd->bst", q, kk)
    want_o = np.einsum("bst,btd->bsd", p, v)
    assert max(np.max(np.abs(want_s)), np.max(np.abs(want_o))) < 256
    for dt in (torch.float16, torch.bfloat16):
        assert np.array_equal(host(ops.matmul(dev(q).to(dt), dev(kk).to(dt), trans_b=True).float()), want_s)
        assert np.array_equal(host(ops.matmul(dev(p).to(dt), dev(v).to(dt)).float()), want_o)


@pytest.mark.parametrize("S, T, D", [(1, 300, 128), (4, 264, 64), (40, 136, 128), (130, 96, 72)])
def test_matmul_groups_of_matrices_that_share_one_b(S, T, D):
    # the query heads of a key / value head: [2, 3, 4, S, D] against [2, 3, 1, T, D] is six products of 4 S rows;
    # a bias over the whole output; then shapes whose matrices only partly follow each other in both operands
    rng = np.random.default_rng(S * 10 + D)
    q = rng.integers(-1, 2, (2, 3, 4, S, D)).astype(np.float32)
    kk = rng.integers(-1, 2, (2, 3, 1, T, D)).astype(np.float32)
    p = rng.integers(-1, 2, (2, 3, 4, S, T)).astype(np.float32)
    v = rng.integers(-1, 2, (2, 3, 1, T, D)).astype(np.float32)
    c = rng.integers(-8, 9, (2, 3, 4, S, T)).astype(np.float32)
    want_s = np.einsum("abgsd,abtd->abgst", q, kk[:, :, 0])
    want_o = np.einsum("abgst,abtd->abgsd", p, v[:, :, 0])
    assert max(np.max(np.abs(want_s)) + 8, np.max(np.abs(want_o))) < 256
    for dt in (torch.float16, torch.bfloat16):
        assert np.array_equal(host(ops.matmul(dev(q).to(dt), dev(kk).to(dt), trans_b=True).float()), want_s)
        assert np.array_equal(host(ops.matmul(dev(q).to(dt), dev(kk).to(dt), dev(c).to(dt), trans_b=True).float()), want_s + c)
        assert np.array_equal(host(ops.matmul(dev(p).to(dt), dev(v).to(dt)).float()), want_o)
    a = rng.integers(-1, 2, (3, 1, S, D)).astype(np.float32)
    b = rng.integers(-1, 2, (1, 5, D, T)).astype(np.float32)
    assert np.array_equal(host(ops.matmul(dev(a).half(), dev(b).half()).float()), np.einsum("asd,bdt->abst", a[:, 0], b[0]))
    a = rng.integers(-1, 2, (1, 5, S, D)).astype(np.float32)
    b = rng.integers(-1, 2, (3, 5, D, T)).astype(np.float32)
    assert np.array_equal(host(ops.matmul(dev(a).half(), dev(b).half()).float()), np.einsum("bsd,abdt->abst", a[0], b))
    got = host(ops.matmul(dev(q).float(), dev(kk).float(), trans_b=True))
    assert np.array_equal(got, want_s)


def test_matmul_fp16_exact_on_small_integers_full_tile_grid():
    # integer-valued operands with |sum| < 2048: every fp16 result is exact, so the MFMA path must
    # reproduce numpy's integer product bit for bit over a 3 x 2 grid of tiles and 5 k-tiles
    rng = np.random.default_rng(15)
    a = rng.integers(-2, 3, (768, 320)).astype(np.float32)
    b = rng.integers(-2, 3, (320, 512)).astype(np.float32)
    want = a.astype(np.int64) @ b.astype(np.int64)
    assert np.max(np.abs(want)) < 2048
    got = host(ops.matmul(dev(a).half(), dev(b).half()).float())
    assert np.array_equal(got, want.astype(np.float32))
    got_t = host(ops.matmul(dev(a).half(), dev(np.ascontiguousarray(b.T)).half(), trans_b=True).float())
    assert np.array_equal(got_t, want.astype(np.float32))
    # generic kernel on the same data (transposed A) and odd shapes
    got_g = host(ops.matmul(dev(np.ascontiguousarray(a.T)).half(), dev(b).half(), trans_a=True).float())
    assert np.array_equal(got_g, want.astype(np.float32))


def test_matmul_full_config_fp16():
    # 4096 x 4096 x 4096 (a decoder layer's projection at 4096 tokens): float64 BLAS on the fp16
    # values as the full-size check, a sample of rows against the oracle
    rng = np.random.default_rng(16)
    a = (rng.standard_normal((4096, 4096)) * 0.5).astype(np.float16)
    b = (rng.standard_normal((4096, 4096)) * 0.05).astype(np.float16)
    got = host(ops.matmul(dev(a), dev(b), trans_b=True).float())
    ref64 = a.astype(np.float64) @ b.astype(np.float64).T
    bound = 2.0 ** -10 * np.abs(ref64) + 1e-5 * (np.abs(a).astype(np.float64) @ np.abs(b).astype(np.float64).T)
    assert np.all(np.abs(got - ref64) <= bound)
    rows = [0, 255, 256, 4095]
    ref = oracle.matmul(a[rows], b, None, False, True, dtype="fp16").astype(np.float32)
    _matmul_check(got[rows], ref, _absprod(a[rows].astype(np.float32), b.astype(np.float32), False, True), 2.0 ** -10)


@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("m,k,n", [(1, 256, 32), (7, 1024, 96), (32, 4096, 4096), (33, 512, 64), (100, 768, 160), (200, 256, 96),
                                   (5, 128, 16), (16, 11008, 48), (17, 384, 80), (31, 4224, 1040), (9, 2176, 32),
                                   (2, 4096, 1024), (4, 384, 48), (3, 128, 16), (8, 256, 4096), (13, 256, 6400),
                                   (16, 2176, 16), (12, 1152, 6160), (1, 11008, 64), (3, 16384, 32)])
def test_matmul_few_rows_weight_streaming(m, k, n, dt):
    # weights as [n, k] (trans_b), fewer than 256 rows of A: the kernels that read W once (block products with
    # operands straight from memory up to 16 rows, in every workgroup size they are launched with; tiles through
    # LDS for slabs of 32 rows beyond)
    rng = np.random.default_rng(17)
    a = rng.standard_normal((2, m, k)).astype(np.float32)
    w = (rng.standard_normal((2, n, k)) * 0.1).astype(np.float32)
    bias = rng.standard_normal((n,)).astype(np.float32)
    ad, wd, cd = (dev(t).to(dt) for t in (a, w, bias))
    name = "fp16" if dt == torch.float16 else "bf16"
    f = lambda t: host(t.float())
    to_oracle = (lambda t: host(t)) if name == "fp16" else (lambda t: host(t.view(torch.uint16)))
    ref = oracle.matmul(to_oracle(ad), to_oracle(wd), to_oracle(cd), False, True, 0.5, 1.0, name)
    ref = ref.astype(np.float32) if name == "fp16" else oracle._bf16_to_f32(ref)
    got = f(ops.matmul(ad, wd, cd, False, True, 0.5, 1.0))
    _matmul_check(got, ref, 0.5 * _absprod(f(ad), f(wd), False, True), 2.0 ** -10 if name == "fp16" else 2.0 ** -7)
    # exact on integer-valued operands (every partial sum of every wavefront is exact)
    ai = rng.integers(-2, 3, (m, k)).astype(np.float32)
    wi = rng.integers(-2, 3, (n, k)).astype(np.float32)
    want = ai.astype(np.int64) @ wi.astype(np.int64).T
    if np.max(np.abs(want)) < (2048 if name == "fp16" else 256):
        assert np.array_equal(f(ops.matmul(dev(ai).to(dt), dev(wi).to(dt), trans_b=True)), want.astype(np.float32))


@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("m,k,n", [(1, 8, 8), (1, 4096, 4096), (2, 520, 40), (3, 1000, 248), (4, 4096, 1024), (4, 11008, 72),
                                   (1, 8200, 16), (2, 12288, 104), (2, 264, 10248), (3, 512, 5120), (4, 136, 2568),
                                   (5, 520, 40), (13, 4096, 264), (32, 1000, 248), (30, 264, 10248),
                                   (1, 128, 16), (3, 256, 48), (5, 128, 16), (8, 1152, 272), (13, 256, 6400), (16, 2176, 16),
                                   (17, 384, 80), (31, 4224, 1040), (32, 1024, 2048), (9, 11008, 64), (12, 256, 8192),
                                   (3, 384, 8224), (6, 128, 8224), (33, 256, 64), (64, 384, 48), (40, 128, 8192),
                                   (255, 128, 32)])
def test_matmul_few_rows_weights_as_k_by_n(m, k, n, dt):
    # B as [k, n] (not transposed), fewer than 256 rows of A.  With k a multiple of 128 and n of 16: block products
    # behind a transposition in registers, 32 rows a pass, strips of 16 or (n from 8192) 32 columns.  Otherwise at
    # most four rows of A at a time (up to 32 rows as passes of four, the last
    # one of fewer): a workgroup walks all of k for a strip of columns
    # (fixed order of summation, no atomics); k beyond one LDS segment of A (4096), k and n that end inside a
    # workgroup's step and strip; strips of 16, 32 and 64 columns (the widest that still gives 160 workgroups
    # over the two matrices of the batch: n = 4096 takes 32, 10248 and 5120 take 64), with a number of strips
    # that is a multiple of eight (numbered per XCD) and one that is not
    rng = np.random.default_rng(31)
    a = rng.standard_normal((2, m, k)).astype(np.float32)
    w = (rng.standard_normal((2, k, n)) * 0.1).astype(np.float32)
    bias = rng.standard_normal((m, n)).astype(np.float32)
    ad, wd, cd = (dev(t).to(dt) for t in (a, w, bias))
    name = "fp16" if dt == torch.float16 else "bf16"
    f = lambda t: host(t.float())
    to_oracle = (lambda t: host(t)) if name == "fp16" else (lambda t: host(t.view(torch.uint16)))
    ref = oracle.matmul(to_oracle(ad), to_oracle(wd), to_oracle(cd), False, False, 0.5, -1.5, name)
    ref = ref.astype(np.float32) if name == "fp16" else oracle._bf16_to_f32(ref)
    got = f(ops.matmul(ad, wd, cd, False, False, 0.5, -1.5))
    _matmul_check(got, ref, 0.5 * _absprod(f(ad), f(wd), False, False), 2.0 ** -10 if name == "fp16" else 2.0 ** -7)
    # exact on integer-valued operands; and the same call twice gives the same bits (fixed order of summation)
    ai = rng.integers(-2, 3, (m, k)).astype(np.float32)
    wi = rng.integers(-2, 3, (k, n)).astype(np.float32)
    want = ai.astype(np.int64) @ wi.astype(np.int64)
    if np.max(np.abs(want)) < (2048 if name == "fp16" else 256):
        assert np.array_equal(f(ops.matmul(dev(ai).to(dt), dev(wi).to(dt))), want.astype(np.float32))
    assert torch.equal(ops.matmul(ad, wd, cd, False, False, 0.5, -1.5), ops.matmul(ad, wd, cd, False, False, 0.5, -1.5))


@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("m,k,n", [(1, 4096, 4096), (2, 4096, 4096), (3, 1000, 4104), (4, 4096, 11008), (1, 8192, 2048),
                                   (4, 520, 2056), (1, 33000, 256), (2, 256, 4096), (4, 20000, 1024), (3, 4096, 65536 + 8),
                                   (8, 4096, 4096), (32, 4096, 4096), (13, 1000, 4224), (32, 520, 2048), (5, 4096, 11008),
                                   (17, 33000, 256), (32, 256, 4096), (20, 20000, 1024), (31, 136, 32768)])
def test_matmul_few_rows_k_by_n_with_workspace(m, k, n, dt):
    # one to four rows against weights as [k, n] through rg_hip_matmul_ws: strips of 256 columns, k shared between
    # workgroups, their float sums in a workspace that is handed over full of ones (nothing may need clearing) and
    # reused by the second call; shares that end inside k, a last strip that ends inside its 256 columns, one share
    # only (k = 256), more strips than CUs (n = 65544: two shares, a share holding at most 2048 k-rows); k beyond 255 shares never
    # arises below 2^23, so the longest k here has shares of the maximum 2048 rows.  Five to 32 rows: the same sharing
    # on the matrix cores (strips of 128 columns, shares of at most 512 k-rows copied straight into LDS), k that ends
    # inside a share and inside a quarter of it, rows of A that the 32-row operand repeats.  Same bar as without
    # the workspace, the same bits on every call, and exact on integer-valued operands.
    rng = np.random.default_rng(37)
    a = rng.standard_normal((m, k)).astype(np.float32)
    w = (rng.standard_normal((k, n)) * 0.1).astype(np.float32)
    bias = rng.standard_normal((m, n)).astype(np.float32)
    ad, wd, cd = (dev(t).to(dt) for t in (a, w, bias))
    name = "fp16" if dt == torch.float16 else "bf16"
    code = ops._T2CODE[dt]
    need = ops.lib().rg_hip_matmul_workspace(code, 0, 0, 1, m, k, n)
    assert need > 0
    ws = torch.full((need + 64,), 0xff, dtype=torch.uint8, device="cuda")
    f = lambda t: host(t.float())
    to_oracle = (lambda t: host(t)) if name == "fp16" else (lambda t: host(t.view(torch.uint16)))
    ref = oracle.matmul(to_oracle(ad), to_oracle(wd), to_oracle(cd), False, False, 0.5, -1.5, name)
    ref = ref.astype(np.float32) if name == "fp16" else oracle._bf16_to_f32(ref)
    first = ops.matmul(ad, wd, cd, False, False, 0.5, -1.5, workspace=ws)
    _matmul_check(f(first), ref, 0.5 * _absprod(f(ad), f(wd), False, False), 2.0 ** -10 if name == "fp16" else 2.0 ** -7)
    assert torch.equal(first, ops.matmul(ad, wd, cd, False, False, 0.5, -1.5, workspace=ws))
    assert torch.equal(first, ops.matmul(ad, wd, cd, False, False, 0.5, -1.5))      # a fresh workspace of the size asked for
    # a workspace that is too small is not an error: the call runs what rg_hip_matmul runs
    small = torch.empty(64, dtype=torch.uint8, device="cuda")
    _matmul_check(f(ops.matmul(ad, wd, cd, False, False, 0.5, -1.5, workspace=small)), ref,
                  0.5 * _absprod(f(ad), f(wd), False, False), 2.0 ** -10 if name == "fp16" else 2.0 ** -7)
    ai = rng.integers(-2, 3, (m, k)).astype(np.float32)
    wi = rng.integers(-2, 3, (k, n)).astype(np.float32)
    want = ai.astype(np.int64) @ wi.astype(np.int64)
    if np.max(np.abs(want)) < (2048 if name == "fp16" else 256):
        assert np.array_equal(f(ops.matmul(dev(ai).to(dt), dev(wi).to(dt), workspace=ws)), want.astype(np.float32))


@pytest.mark.parametrize("dt", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("m,k,n", [(1, 8, 1), (1, 4096, 4096), (2, 520, 37), (3, 1000, 250), (4, 4096, 1024), (4, 11008, 72),
                                   (1, 32768, 16), (4, 20480, 24), (3, 20488, 8), (1, 40000, 8), (2, 33008, 5), (5, 2048, 33), (7, 1000, 130),
                                   (8, 4096, 512), (6, 11008, 64)])
def test_matmul_one_to_four_rows_matrix_vector(m, k, n, dt):
    # weights as [n, k] (trans_b), at most four rows of A: products on the vector ALUs, W streamed once;
    # k that is not a multiple of a wavefront's step (512), n that is not a multiple of a workgroup's rows,
    # rows of A longer than the 64 KiB of LDS a workgroup uses (k walked in segments, whole and ragged);
    # five to eight rows (the matrix-core kernel) for comparison
    rng = np.random.default_rng(29)
    a = rng.standard_normal((2, m, k)).astype(np.float32)
    w = (rng.standard_normal((2, n, k)) * 0.1).astype(np.float32)
    bias = rng.standard_normal((m, n)).astype(np.float32)
    ad, wd, cd = (dev(t).to(dt) for t in (a, w, bias))
    name = "fp16" if dt == torch.float16 else "bf16"
    f = lambda t: host(t.float())
    to_oracle = (lambda t: host(t)) if name == "fp16" else (lambda t: host(t.view(torch.uint16)))
    ref = oracle.matmul(to_oracle(ad), to_oracle(wd), to_oracle(cd), False, True, 0.5, -1.5, name)
    ref = ref.astype(np.float32) if name == "fp16" else oracle._bf16_to_f32(ref)
    got = f(ops.matmul(ad, wd, cd, False, True, 0.5, -1.5))
    _matmul_check(got, ref, 0.5 * _absprod(f(ad), f(wd), False, True), 2.0 ** -10 if name == "fp16" else 2.0 ** -7)
    # exact on integer-valued operands, and the same answer as the row inside a taller product (another kernel)
    ai = rng.integers(-2, 3, (m, k)).astype(np.float32)
    wi = rng.integers(-2, 3, (n, k)).astype(np.float32)
    want = ai.astype(np.int64) @ wi.astype(np.int64).T
    if np.max(np.abs(want)) < (2048 if name == "fp16" else 256):
        assert np.array_equal(f(ops.matmul(dev(ai).to(dt), dev(wi).to(dt), trans_b=True)), want.astype(np.float32))
