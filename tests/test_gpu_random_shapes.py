"""Parity on randomly drawn shapes: every operator of the path against the CPU oracle (numpy's own
indexing for the data movers), with seeded generators so that a failure names its case.

The drawn sizes straddle the dispatch boundaries of the kernels (vector widths, tile sizes, row
counts that switch kernels); the bars are those of the fixed-shape tests: bit-exact for integer and
byte work, 1e-5 relative for fp32 rows, 2e-3 absolute for fp16 (2e-2 for bf16 attention).
"""
import math

import numpy as np
import pytest
import torch

import oracle
from refactorgraph_amd import ops

pytestmark = pytest.mark.gpu

DEV = "cuda"


def dev(a):
    a = np.asarray(a)
    return torch.from_numpy(np.ascontiguousarray(a)).reshape(a.shape).to(DEV)


def host(t):
    torch.cuda.synchronize()
    return t.cpu().numpy()


_SIZES = [1, 2, 3, 4, 5, 7, 8, 16, 31, 32, 33, 64, 100, 128, 255, 256, 1000, 2048, 4100]


def _shape(rng, max_rank, max_elems=1 << 18, sizes=_SIZES):
    while True:
        s = tuple(int(rng.choice(sizes)) for _ in range(int(rng.integers(1, max_rank + 1))))
        if np.prod(s) <= max_elems:
            return s


@pytest.mark.parametrize("seed", [101, 102])
def test_rows_operators_on_random_shapes(seed):
    rng = np.random.default_rng(seed)
    for case in range(40):
        s = _shape(rng, 3)
        x = rng.standard_normal(s).astype(np.float32)
        w = rng.uniform(0.5, 1.5, s[-1]).astype(np.float32)
        y = host(ops.rms_norm(dev(x), dev(w), 1e-5))
        assert np.allclose(y, oracle.rms_norm(x, w, 1e-5, threads=8), rtol=1e-5, atol=1e-7), ("rms_norm", case, s)

        s = _shape(rng, 4)
        axis = int(rng.integers(0, len(s)))
        x = (3 * rng.standard_normal(s)).astype(np.float32)
        y = host(ops.softmax(dev(x), axis))
        assert np.allclose(y, oracle.softmax(x, axis, threads=8), rtol=1e-5, atol=1e-9), ("softmax", case, s, axis)
        x16 = dev(x).half()
        x32 = host(x16.float())
        y = host(ops.softmax(x16).float())
        assert np.max(np.abs(y - oracle.softmax(x32, threads=8))) <= 2e-3, ("softmax fp16", case, s)
        if len(s) >= 2 and s[-1] >= s[-2]:
            y = host(ops.softmax(x16, causal=True).float())
            assert np.max(np.abs(y - oracle.softmax_causal(x32, threads=8))) <= 2e-3, ("softmax causal", case, s)

        B, S, H = int(rng.integers(1, 4)), int(rng.integers(1, 70)), int(rng.integers(1, 9))
        D = int(rng.choice([2, 8, 16, 64, 128, 256]))
        x16 = dev(rng.standard_normal((B, S, H, D)).astype(np.float32)).half()
        pos = rng.integers(0, 5000, (B, S)).astype(np.int64)
        y = host(ops.rope(x16, dev(pos), 10000.0).float())
        assert np.max(np.abs(y - oracle.rope(host(x16.float()), pos, 10000.0, threads=8))) <= 4e-3, ("rope", case, (B, S, H, D))


@pytest.mark.parametrize("seed", [201, 202])
def test_quantisation_operators_on_random_shapes(seed):
    rng = np.random.default_rng(seed)
    for case in range(40):
        s = _shape(rng, 3)
        axis = int(rng.integers(0, len(s)))
        dt = rng.choice([np.uint8, np.int8, np.int16, np.int32])
        info = np.iinfo(dt)
        x = rng.integers(max(info.min, -100000), min(info.max, 100000) + 1, s).astype(dt)
        n_scales = s[axis] if rng.integers(0, 2) else 1
        scale = rng.uniform(1e-3, 1e-2, n_scales).astype(np.float32)
        zp = None if rng.integers(0, 2) else rng.integers(max(info.min, -50), min(info.max, 50) + 1, n_scales).astype(dt)
        y = host(ops.dequantize_linear(dev(x), dev(scale), None if zp is None else dev(zp), axis))
        assert np.array_equal(y, oracle.dequantize_linear(x, scale, zp, axis, threads=8)), ("dequantize", case, s, axis)

        n = int(rng.choice([1, 5, 100, 4095, 4096, 70001, 300000]))
        x = rng.uniform(rng.uniform(-9, 1), rng.uniform(1, 9), n).astype(np.float32)
        y, sc, z = ops.dynamic_quantize_linear(dev(x))
        ry, rs, rz = oracle.dynamic_quantize_linear(x)
        assert np.array_equal(host(y), ry) and host(sc).reshape(-1)[0] == np.float32(rs), ("dynamic quantize", case, n)
        assert int(host(z).reshape(-1)[0]) == int(rz), ("dynamic quantize zero point", case, n)


def _gemm_dim(rng, kind):
    if kind == 0:
        return int(rng.integers(1, 40))
    if kind == 1:
        return max(1, int(rng.choice([8, 16, 32, 64, 128, 256, 512, 1024])) + int(rng.choice([0, 0, 0, 1, 8, -8, 16, 24])))
    return int(rng.integers(1, 700))


@pytest.mark.parametrize("seed", [301, 302])
def test_matmul_integer_on_random_shapes(seed):
    rng = np.random.default_rng(seed)
    draw = lambda size, signed: (rng.integers(-128, 128, size).astype(np.int8) if signed
                                 else rng.integers(0, 256, size).astype(np.uint8))
    for case in range(50):
        m, k, n = _gemm_dim(rng, rng.integers(0, 3)), _gemm_dim(rng, rng.integers(1, 3)), _gemm_dim(rng, rng.integers(0, 3))
        batch = int(rng.choice([1, 1, 1, 2, 3]))
        a, b = draw((batch, m, k), rng.integers(0, 2)), draw((batch, k, n), rng.integers(0, 2))
        kinds = rng.integers(0, 3, 2)
        # per-row zero points as the reference reads them: one per (batch, row) of the operand
        a_zp = None if kinds[0] == 0 else draw(1 if kinds[0] == 1 else batch * m, rng.integers(0, 2))
        b_zp = None if kinds[1] == 0 else draw(1 if kinds[1] == 1 else batch * k, rng.integers(0, 2))
        y = host(ops.matmul_integer(dev(a), dev(b), None if a_zp is None else dev(a_zp), None if b_zp is None else dev(b_zp)))
        assert np.array_equal(y, oracle.matmul_integer(a, b, a_zp, b_zp, threads=8)), (case, batch, m, k, n, kinds.tolist())


@pytest.mark.parametrize("seed", [401, 402])
def test_matmul_on_random_shapes(seed):
    rng = np.random.default_rng(seed)
    for case in range(50):
        m, k, n = _gemm_dim(rng, rng.integers(0, 3)), _gemm_dim(rng, rng.integers(1, 3)), _gemm_dim(rng, rng.integers(0, 3))
        batch = int(rng.choice([1, 1, 1, 2, 3]))
        dt = torch.float16 if rng.integers(0, 3) else torch.bfloat16
        trans_b = bool(rng.integers(0, 2))
        a = dev(rng.standard_normal((batch, m, k)).astype(np.float32)).to(dt)
        b = dev(rng.standard_normal((batch, n, k) if trans_b else (batch, k, n)).astype(np.float32)).to(dt)
        bias_kind = rng.integers(0, 3)
        c = None if bias_kind == 0 else dev(rng.standard_normal((n,) if bias_kind == 1 else (batch, m, n)).astype(np.float32)).to(dt)
        alpha, beta = (1.0, 1.0) if rng.integers(0, 2) else (0.5, 2.0)
        y = host(ops.matmul(a, b, c, trans_b=trans_b, alpha=alpha, beta=beta).float())
        af, bf = host(a.float()).astype(np.float64), host(b.float()).astype(np.float64)
        if trans_b:
            bf = np.swapaxes(bf, -1, -2)
        ref, mag = alpha * (af @ bf), alpha * (np.abs(af) @ np.abs(bf))
        if c is not None:
            cf = host(c.float()).astype(np.float64)
            ref, mag = ref + beta * cf, mag + np.abs(beta * cf)
        # one rounding of the result to the data type, float accumulation of the products before it
        eps = 2.0 ** -10 if dt == torch.float16 else 2.0 ** -7
        limit = eps * np.abs(ref) + mag * 2.0 ** -20 + 1e-6
        assert np.all(np.abs(y - ref) <= 1.01 * limit), (case, batch, m, k, n, str(dt), trans_b, int(bias_kind))


@pytest.mark.parametrize("seed", [451, 452])
def test_matmul_few_rows_with_workspace_on_random_shapes(seed):
    # at most 32 rows against weights kept as [k, n], through the workspace (shares of k between workgroups): shapes
    # whose k ends inside a share, a load round and a quarter of a share; one workspace, full of junk at first, serves
    # every case of a seed in turn, so each case finds what another shape left there
    rng = np.random.default_rng(seed)
    ws = torch.full((24 << 20,), 0x5a, dtype=torch.uint8, device=DEV)
    for case in range(24):
        m = int(rng.integers(1, 33))
        step_k, step_n = (2, 8) if m <= 4 else (8, 64)
        n = int(rng.integers(1, 5000 // step_n + 1)) * step_n
        k = max(int(rng.integers(1, 6000 // step_k + 1)) * step_k, -(-(1 << 20) // n // step_k) * step_k)
        dt = torch.float16 if rng.integers(0, 3) else torch.bfloat16
        need = ops.lib().rg_hip_matmul_workspace(ops._T2CODE[dt], 0, 0, 1, m, k, n)
        assert 0 < need <= ws.numel(), (case, m, k, n)
        a = dev(rng.standard_normal((m, k)).astype(np.float32)).to(dt)
        b = dev((rng.standard_normal((k, n)) * 0.25).astype(np.float32)).to(dt)
        bias_kind = rng.integers(0, 3)
        c = None if bias_kind == 0 else dev(rng.standard_normal((n,) if bias_kind == 1 else (m, n)).astype(np.float32)).to(dt)
        alpha, beta = (1.0, 1.0) if rng.integers(0, 2) else (0.5, 2.0)
        got = ops.matmul(a, b, c, alpha=alpha, beta=beta, workspace=ws)
        assert torch.equal(got, ops.matmul(a, b, c, alpha=alpha, beta=beta, workspace=ws)), (case, m, k, n)
        y = host(got.float())
        af, bf = host(a.float()).astype(np.float64), host(b.float()).astype(np.float64)
        ref, mag = alpha * (af @ bf), alpha * (np.abs(af) @ np.abs(bf))
        if c is not None:
            cf = host(c.float()).astype(np.float64)
            ref, mag = ref + beta * cf, mag + np.abs(beta * cf)
        eps = 2.0 ** -10 if dt == torch.float16 else 2.0 ** -7
        limit = eps * np.abs(ref) + mag * 2.0 ** -20 + 1e-6
        assert np.all(np.abs(y - ref) <= 1.01 * limit), (case, m, k, n, str(dt), int(bias_kind))


@pytest.mark.parametrize("seed", [501, 502])
def test_data_movers_on_random_shapes(seed):
    rng = np.random.default_rng(seed)
    dtypes = [np.uint8, np.int16, np.float32, np.float64]
    for case in range(50):
        rank = int(rng.integers(1, 6))
        s = _shape(rng, rank, sizes=[1, 2, 3, 4, 5, 8, 16, 17, 32, 64, 65, 128, 130])
        perm = tuple(int(p) for p in rng.permutation(len(s)))
        x = rng.integers(0, 200, s).astype(rng.choice(dtypes))
        assert np.array_equal(host(ops.transpose(dev(x), perm)), np.transpose(x, perm)), ("transpose", case, s, perm)

        s = list(_shape(rng, 3, 1 << 16))
        axis = int(rng.integers(0, len(s)))
        sizes = [int(v) for v in rng.integers(0, 40, int(rng.integers(1, 6)))]
        sizes[0] += 3 if sum(sizes) == 0 else 0
        s[axis] = sum(sizes)
        x = rng.integers(0, 200, s).astype(rng.choice(dtypes))
        got = ops.split(dev(x), sizes, axis)
        for g, want in zip(got, np.split(x, np.cumsum(sizes)[:-1], axis=axis)):
            assert np.array_equal(host(g), want), ("split", case, s, axis, sizes)
        assert np.array_equal(host(ops.concat(got, axis)), x), ("concat", case, s, axis, sizes)

        full = [int(rng.choice([1, 2, 3, 5, 8, 16, 33, 64, 100])) for _ in range(int(rng.integers(1, 5)))]
        part = lambda: tuple(d if rng.integers(0, 3) else 1 for d in full[len(full) - int(rng.integers(0, len(full) + 1)):])
        cs, xs, ys = part(), part(), part()
        dt = rng.choice(dtypes)
        cond = rng.integers(0, 2, cs).astype(bool)
        xv, yv = rng.integers(0, 100, xs).astype(dt), rng.integers(100, 200, ys).astype(dt)
        y = host(ops.where(dev(cond), dev(xv), dev(yv)))
        assert np.array_equal(y, np.where(cond, xv, yv)), ("where", case, cs, xs, ys)
        assert np.array_equal(host(ops.expand(dev(xv), tuple(full))), np.broadcast_to(xv, tuple(full))), ("expand", case, xs, full)


@pytest.mark.parametrize("seed", [601, 602])
def test_attention_on_random_shapes(seed):
    rng = np.random.default_rng(seed)
    for case in range(60):
        N = int(rng.integers(1, 7))
        Hkv = int(rng.choice([1, 2, 3, 4, 8]))
        H = Hkv * int(rng.choice([1, 2, 3, 4, 5, 8, 12]))
        D = int(rng.choice([64, 80, 96, 128]))
        kind = rng.integers(0, 4)
        seq = 1 if kind == 0 else int(rng.integers(1, 20)) if kind == 1 else int(rng.integers(16, 150))
        if kind == 3 and rng.integers(0, 3) == 0:
            seq = int(rng.integers(150, 400))
        room = int(rng.choice([0, 1, 7, 64, 300, 1500]))
        cap = seq + room
        past = rng.integers(0, room + 1, N)
        if rng.integers(0, 4) == 0:
            past[:] = 0
        if rng.integers(0, 6) == 0:
            past[:] = room
        dt = torch.float16 if rng.integers(0, 4) else torch.bfloat16
        one_length = rng.integers(0, 5) == 0        # a single history length for all batch rows
        if one_length:
            past[:] = past[0]
        mk = lambda shape: dev(rng.standard_normal(shape).astype(np.float32)).to(dt)
        q, k, v = mk((N, H, seq, D)), mk((N, Hkv, seq, D)), mk((N, Hkv, seq, D))
        kc, vc = mk((N, Hkv, cap, D)), mk((N, Hkv, cap, D))
        kc0, vc0 = kc.clone(), vc.clone()
        lens = dev(past[:1].astype(np.int64)) if one_length else dev(past.astype(np.int64))
        o = ops.attention_kvcache(q, k, v, kc, vc, lens, 1 / math.sqrt(D))
        f = lambda t: host(t.float())
        ref_o, ref_kc, ref_vc = oracle.attention_kvcache(f(q), f(k), f(v), f(kc0), f(vc0), past, 1 / math.sqrt(D))
        what = (case, N, H, Hkv, seq, cap, D, past.tolist(), str(dt), bool(one_length))
        assert np.max(np.abs(f(o) - ref_o)) <= (2e-3 if dt == torch.float16 else 2e-2), what
        assert np.array_equal(f(kc), ref_kc) and np.array_equal(f(vc), ref_vc), what


@pytest.mark.parametrize("seed", [611])
def test_attention_long_caches_on_random_shapes(seed):
    # few sequences against long caches: the tiled kernel with an item's keys shared between workgroups (ranges that
    # lie beyond a short history included), the decode kernel with eight heads of a group per launch
    rng = np.random.default_rng(seed)
    for case in range(40):
        N = int(rng.integers(1, 4))
        Hkv = int(rng.choice([1, 2, 4, 8]))
        H = Hkv * int(rng.choice([1, 2, 4, 7, 8, 16]))
        D = int(rng.choice([64, 128]))
        seq = int(rng.choice([1, 2, 5, 16, 31, 32, 33, 70, 128, 200]))
        room = int(rng.choice([1000, 2500, 4000, 9000]))
        cap = seq + room
        past = rng.integers(0, room + 1, N)
        if rng.integers(0, 3) == 0:
            past[:] = room
        if rng.integers(0, 5) == 0:
            past[:] = rng.integers(0, 40)
        dt = torch.float16 if rng.integers(0, 4) else torch.bfloat16
        mk = lambda shape: dev(rng.standard_normal(shape).astype(np.float32)).to(dt)
        q, k, v = mk((N, H, seq, D)), mk((N, Hkv, seq, D)), mk((N, Hkv, seq, D))
        kc, vc = mk((N, Hkv, cap, D)), mk((N, Hkv, cap, D))
        kc0, vc0 = kc.clone(), vc.clone()
        o = ops.attention_kvcache(q, k, v, kc, vc, dev(past.astype(np.int64)), 1 / math.sqrt(D))
        f = lambda t: host(t.float())
        ref_o, ref_kc, ref_vc = oracle.attention_kvcache(f(q), f(k), f(v), f(kc0), f(vc0), past, 1 / math.sqrt(D))
        what = (case, N, H, Hkv, seq, cap, D, past.tolist(), str(dt))
        assert not np.isnan(f(o)).any(), what
        assert np.max(np.abs(f(o) - ref_o)) <= (2e-3 if dt == torch.float16 else 2e-2), what
        assert np.array_equal(f(kc), ref_kc) and np.array_equal(f(vc), ref_vc), what
