"""ctypes binding of the CPU oracle (oracle/oracle.c).

TEST INFRASTRUCTURE ONLY: imported by tests/, by ``__graft_entry__.smoke()`` and by the
``cpu_baseline`` leg of ``bench.py``.  The product (``refactorgraph_amd``) never imports it.

Each wrapper takes and returns numpy arrays; the reference file:line every function follows
is listed in oracle/oracle.h.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "_build", "liboracle.so")

F32, U8, I8, U16, I16, I32, F64 = 1, 2, 3, 4, 5, 6, 11
_NP2CODE = {np.dtype(np.uint8): U8, np.dtype(np.int8): I8, np.dtype(np.uint16): U16,
            np.dtype(np.int16): I16, np.dtype(np.int32): I32}


def build() -> str:
    """Compile oracle.c with the committed Makefile."""
    subprocess.run(["make", "-C", _HERE, "-s"], check=True)
    return _LIB_PATH


_lib = None


def lib() -> C.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(_LIB_PATH):
            build()
        L = C.CDLL(_LIB_PATH)
        sz, vp, i32, f32 = C.c_size_t, C.c_void_p, C.c_int, C.c_float
        L.oracle_rms_norm_f32.argtypes = [vp, vp, vp, sz, sz, f32, i32]
        L.oracle_rms_norm_f64.argtypes = [vp, vp, vp, sz, sz, f32, i32]
        L.oracle_softmax_f32.argtypes = [vp, vp, sz, sz, sz, i32]
        L.oracle_softmax_f64.argtypes = [vp, vp, sz, sz, sz, i32]
        L.oracle_softmax_literal_f32.argtypes = [vp, vp, sz, sz, sz]
        L.oracle_softmax_causal_f32.argtypes = [vp, vp, sz, sz, sz, i32]
        L.oracle_matmul_integer.argtypes = [vp, vp, vp, vp, i32, i32, vp, i32, i32,
                                            sz, sz, sz, sz, vp, vp, sz, sz, i32]
        L.oracle_dequantize_linear.argtypes = [vp, vp, vp, vp, sz, sz, sz, i32, sz, i32]
        L.oracle_dequantize_linear.restype = i32
        L.oracle_dynamic_quantize_linear.argtypes = [vp, vp, vp, vp, sz]
        L.oracle_dynamic_quantize_linear.restype = None
        L.oracle_matmul_f32.argtypes = [vp, vp, vp, sz, sz, sz, sz, sz, sz, sz, f32]
        L.oracle_mul_f32.argtypes = [vp, vp, vp, sz, sz]
        L.oracle_matmul_bias_f32.argtypes = [vp, vp, vp, sz, sz, sz, sz, sz, sz, sz, f32, f32]
        L.oracle_matmul_bias_f64.argtypes = [vp, vp, vp, sz, sz, sz, sz, sz, sz, sz, C.c_double, C.c_double]
        L.oracle_matmul_bias_f32.restype = L.oracle_matmul_bias_f64.restype = None
        L.oracle_attention_head_f32.argtypes = [vp, vp, vp, vp, sz, sz, sz, f32, i32, vp]
        L.oracle_rope_f32.argtypes = [vp, vp, vp, i32, sz, sz, sz, sz, f32, i32]
        L.oracle_transpose_info.argtypes = [vp, vp, vp, vp, vp, vp, i32, C.c_uint32]
        L.oracle_transpose_info.restype = i32
        L.oracle_transpose.argtypes = [vp, vp, vp, vp, i32, C.c_uint32]
        L.oracle_transpose.restype = None
        u32 = C.c_uint32
        L.oracle_split_info.argtypes = [vp, vp, vp, vp, i32, i32, i32, u32]
        L.oracle_split.argtypes = [vp, vp, vp, sz, sz, sz]
        L.oracle_concat.argtypes = [vp, vp, vp, sz, sz, sz]
        L.oracle_expand_info.argtypes = [vp, vp, vp, vp, vp, i32, vp, i32, u32]
        L.oracle_expand_info.restype = i32
        L.oracle_expand.argtypes = [vp, vp, vp, vp, i32, u32, u32]
        L.oracle_broadcaster.argtypes = [vp, vp, vp, vp, i32]
        L.oracle_broadcaster.restype = i32
        L.oracle_where.argtypes = [vp, vp, vp, vp, vp, i32, u32, u32]
        for name in ("oracle_split_info", "oracle_split", "oracle_concat", "oracle_expand", "oracle_where"):
            getattr(L, name).restype = None
        for name in ("oracle_rms_norm_f32", "oracle_rms_norm_f64", "oracle_softmax_f32",
                     "oracle_softmax_f64", "oracle_softmax_literal_f32", "oracle_softmax_causal_f32",
                     "oracle_matmul_integer", "oracle_matmul_f32", "oracle_mul_f32",
                     "oracle_attention_head_f32", "oracle_rope_f32"):
            getattr(L, name).restype = None
        _lib = L
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _c(a, dtype=None):
    return np.ascontiguousarray(a, dtype=dtype)


def rms_norm(x, w, eps, threads=1):
    x = _c(x)
    assert x.dtype in (np.float32, np.float64)
    w = _c(w, x.dtype)
    cols = x.shape[-1]
    rows = x.size // cols if cols else 0
    y = np.empty_like(x)
    fn = lib().oracle_rms_norm_f32 if x.dtype == np.float32 else lib().oracle_rms_norm_f64
    fn(_p(y), _p(x), _p(w), rows, cols, float(eps), threads)
    return y


def _pre_mid_post(shape, axis):
    pre = int(np.prod(shape[:axis], dtype=np.int64))
    post = int(np.prod(shape[axis + 1:], dtype=np.int64))
    return pre, int(shape[axis]), post


def softmax(x, axis=-1, threads=1):
    x = _c(x)
    assert x.dtype in (np.float32, np.float64)
    axis = axis % x.ndim
    pre, mid, post = _pre_mid_post(x.shape, axis)
    y = np.empty_like(x)
    fn = lib().oracle_softmax_f32 if x.dtype == np.float32 else lib().oracle_softmax_f64
    fn(_p(y), _p(x), pre, mid, post, threads)
    return y


def softmax_literal(x, axis=-1):
    x = _c(x, np.float32)
    axis = axis % x.ndim
    pre, mid, post = _pre_mid_post(x.shape, axis)
    y = np.empty_like(x)
    lib().oracle_softmax_literal_f32(_p(y), _p(x), pre, mid, post)
    return y


def softmax_causal(x, threads=1):
    x = _c(x, np.float32)
    rows, cols = x.shape[-2], x.shape[-1]
    batch = x.size // (rows * cols)
    y = np.empty_like(x)
    lib().oracle_softmax_causal_f32(_p(y), _p(x), batch, rows, cols, threads)
    return y


def batch_offsets(a_batch_shape, b_batch_shape):
    """Operand matrix index for every output batch under multidirectional broadcasting
    (independent of the host-side Broadcaster: numpy's own broadcasting does the work)."""
    na = int(np.prod(a_batch_shape, dtype=np.int64))
    nb = int(np.prod(b_batch_shape, dtype=np.int64))
    ia = np.arange(na, dtype=np.uint32).reshape(a_batch_shape)
    ib = np.arange(nb, dtype=np.uint32).reshape(b_batch_shape)
    oa, ob = np.broadcast_arrays(ia, ib)
    return _c(oa.reshape(-1)), _c(ob.reshape(-1)), na, nb


def matmul_integer(a, b, a_zp=None, b_zp=None, threads=1):
    """a [..., m, k], b [..., k, n] of uint8/int8; zero points: None, 1-element array, or
    per-row arrays as the reference reads them (A: [batch*m], B: [batch*k])."""
    a, b = _c(a), _c(b)
    assert a.dtype in (np.uint8, np.int8) and b.dtype in (np.uint8, np.int8)
    m, k = a.shape[-2:]
    k2, n = b.shape[-2:]
    assert k == k2
    oa, ob, na, nb = batch_offsets(a.shape[:-2], b.shape[:-2])
    batch = oa.size
    out_batch_shape = np.broadcast_shapes(a.shape[:-2], b.shape[:-2])
    y = np.empty(out_batch_shape + (m, n), dtype=np.int32)

    def zp_args(zp):
        if zp is None:
            return None, 1, 1
        zp = _c(zp)
        assert zp.dtype in (np.uint8, np.int8)
        return zp, int(zp.dtype == np.int8), int(zp.size == 1)

    az, az_s, az_sc = zp_args(a_zp)
    bz, bz_s, bz_sc = zp_args(b_zp)
    lib().oracle_matmul_integer(_p(y), _p(a), _p(b), _p(az), az_s, az_sc, _p(bz), bz_s, bz_sc,
                                batch, m, k, n, _p(oa), _p(ob), na, nb, threads)
    return y


def dequantize_linear(x, scale, zp=None, axis=1, threads=1):
    x = _c(x)
    code = _NP2CODE[x.dtype]
    scale = _c(scale, np.float32).reshape(-1)
    if zp is not None:
        zp = _c(zp, x.dtype).reshape(-1)
        assert zp.size == scale.size
    if scale.size == 1:
        outer, axis_len, inner = 1, 1, x.size
    else:
        axis = axis % x.ndim
        outer, axis_len, inner = _pre_mid_post(x.shape, axis)
        assert scale.size == axis_len
    y = np.empty(x.shape, dtype=np.float32)
    rc = lib().oracle_dequantize_linear(_p(y), _p(x), _p(scale), _p(zp), outer, axis_len, inner,
                                        code, scale.size, threads)
    assert rc == 0
    return y


def dynamic_quantize_linear(x):
    """float32 tensor -> (uint8 tensor, float32 scale, uint8 zero point)."""
    x = _c(x, np.float32)
    y = np.empty(x.shape, dtype=np.uint8)
    scale = np.empty(1, dtype=np.float32)
    zp = np.empty(1, dtype=np.uint8)
    lib().oracle_dynamic_quantize_linear(_p(y), _p(scale), _p(zp), _p(x), x.size)
    return y, scale[0], zp[0]


def matmul_f32(a, b, trans_b=False, alpha=1.0):
    a, b = _c(a, np.float32), _c(b, np.float32)
    M, K = a.shape
    if trans_b:
        N = b.shape[0]
        sb0, sb1 = 1, K
    else:
        N = b.shape[1]
        sb0, sb1 = N, 1
    y = np.empty((M, N), dtype=np.float32)
    lib().oracle_matmul_f32(_p(y), _p(a), _p(b), M, K, N, K, 1, sb0, sb1, float(alpha))
    return y


def mul_f32(a, b):
    a, b = _c(a, np.float32), _c(b, np.float32)
    y = np.empty(a.shape if a.size >= b.size else b.shape, dtype=np.float32)
    lib().oracle_mul_f32(_p(y), _p(a), _p(b), a.size, b.size)
    return y


def attention_head(q, kc, vc, past, scale, causal=True):
    """q [seq, D]; kc/vc [past+seq, D] (history followed by the new rows), float32."""
    q, kc, vc = _c(q, np.float32), _c(kc, np.float32), _c(vc, np.float32)
    seq, D = q.shape
    assert kc.shape == (past + seq, D) and vc.shape == (past + seq, D)
    o = np.empty((seq, D), dtype=np.float32)
    scratch = np.empty(2 * seq * (past + seq), dtype=np.float32)
    lib().oracle_attention_head_f32(_p(o), _p(q), _p(kc), _p(vc), seq, int(past), D,
                                    float(scale), int(causal), _p(scratch))
    return o


def attention_kvcache(q, k, v, k_cache, v_cache, past_lens, scale, heads=None):
    """Composed attention with cache append, fp32 math on already up-cast inputs.

    q [N,H,seq,D]; k,v [N,Hkv,seq,D]; caches [N,Hkv,S,D] (updated copies are returned);
    past_lens: int array [N] (or one value); a length outside [0, S - seq] is moved to the nearer
    end of that interval, the rule the device kernels apply to lengths they cannot refuse.
    ``heads``: optional iterable of (b, h) pairs to evaluate (others are left as NaN) so large
    shapes can be spot-checked.
    Returns (o, k_cache_out, v_cache_out)."""
    q = _c(q, np.float32)
    N, H, seq, D = q.shape
    Hkv = k.shape[1]
    g = H // Hkv
    past_lens = np.broadcast_to(np.asarray(past_lens, dtype=np.int64).reshape(-1), (N,))
    past_lens = np.clip(past_lens, 0, max(k_cache.shape[2] - seq, 0))
    kc = np.array(k_cache, copy=True)
    vc = np.array(v_cache, copy=True)
    for b in range(N):
        p = int(past_lens[b])
        kc[b, :, p:p + seq, :] = k[b]
        vc[b, :, p:p + seq, :] = v[b]
    o = np.full(q.shape, np.nan, dtype=np.float32)
    pairs = heads if heads is not None else [(b, h) for b in range(N) for h in range(H)]
    for b, h in pairs:
        p = int(past_lens[b])
        kh = h // g
        o[b, h] = attention_head(q[b, h], kc[b, kh, :p + seq].astype(np.float32),
                                 vc[b, kh, :p + seq].astype(np.float32), p, scale, True)
    return o, kc, vc


def rope(x, pos, theta=10000.0, threads=1):
    """x [batch, seq, heads, D] float32 (already up-cast); pos int64 [batch, seq] or [seq]."""
    x = _c(x, np.float32)
    batch, seq, heads, D = x.shape
    pos = _c(pos, np.int64)
    per_batch = int(pos.ndim == 2)
    assert pos.shape == ((batch, seq) if per_batch else (seq,))
    y = np.empty_like(x)
    lib().oracle_rope_f32(_p(y), _p(x), _p(pos), per_batch, batch, seq, heads, D, float(theta), threads)
    return y


# ---------------------------------------------------------------------------------------------
# Cast.  numpy restatement (no C): the conversions are single machine operations.
#   - types of the reference's CPU kernel (u8 u16 u32 u64 i8 i16 i32 i64 f32 f64 bool):
#     `static_cast<U>(a)` of src/04kernel/src/kernels/cast/cpu_kernel.cc:28-40 = numpy `astype`
#     (C conversion rules: integer narrowing wraps, float -> integer truncates, integer -> float
#     rounds to nearest even), `-> bool` is `a != 0`;
#   - fp16 / bf16: the expressions the reference's CUDA kernel generates,
#     src/04kernel/src/kernels/cast/cuda_kernel.cc:55-96: float/double -> fp16|bf16 round to
#     nearest even (a double through float first); integer -> fp16|bf16 takes the value as `int`
#     and rounds toward zero; fp16|bf16 -> integer truncates as `int`; fp16 <-> bf16 through float.
#     `-> bool` from a floating source is written `x == 0` there (true for zeros): NOT followed,
#     `x != 0` is used for every source (cast_bool_reference_literal keeps the literal form).
# bf16 tensors are uint16 arrays of bit patterns (numpy has no bfloat16).
CAST_TYPES = ("u8", "u16", "u32", "u64", "i8", "i16", "i32", "i64", "f32", "f64", "bool", "fp16", "bf16")
_CAST_NP = {"u8": np.uint8, "u16": np.uint16, "u32": np.uint32, "u64": np.uint64, "i8": np.int8,
            "i16": np.int16, "i32": np.int32, "i64": np.int64, "f32": np.float32, "f64": np.float64,
            "bool": np.bool_, "fp16": np.float16, "bf16": np.uint16}


def _bf16_to_f32(bits):
    return (bits.astype(np.uint32) << 16).view(np.float32)


def _f32_to_bf16_rn(f):
    u = np.ascontiguousarray(f, np.float32).view(np.uint32)
    rounded = (u + (0x7FFF + ((u >> 16) & 1))) >> 16          # nearest, ties to even
    nan = np.isnan(f)
    return np.where(nan, (u >> 16) | 0x40, rounded).astype(np.uint16)


def _int_to_f32_rz(v):
    """int32 values -> float32 rounded toward zero."""
    f = v.astype(np.float32)                                     # nearest
    away = np.abs(f.astype(np.float64)) > np.abs(v.astype(np.float64))
    return np.where(away, np.nextafter(f, np.float32(0)), f).astype(np.float32)


def _f32_to_fp16_rz(f):
    with np.errstate(over="ignore"):
        h = f.astype(np.float16)                                 # nearest, may overflow to inf
    away = np.abs(h.astype(np.float64)) > np.abs(f.astype(np.float64))
    return np.where(away, np.nextafter(h, np.float16(0)), h).astype(np.float16)


def cast(x, src, dst):
    """x: numpy array holding `src` values (CAST_TYPES names); returns the `dst` array."""
    x = np.ascontiguousarray(x, _CAST_NP[src])
    narrow = ("fp16", "bf16")
    if src == dst:
        return x.copy()
    if src not in narrow and dst not in narrow:
        if dst == "bool":
            return x != 0
        with np.errstate(invalid="ignore", over="ignore"):
            return x.astype(_CAST_NP[dst])
    if src in narrow:
        f = x.astype(np.float32) if src == "fp16" else _bf16_to_f32(x)
        if dst == "bool":
            return f != 0
        if dst == "fp16":
            with np.errstate(over="ignore"):
                return f.astype(np.float16)
        if dst == "bf16":
            return _f32_to_bf16_rn(f)
        if dst in ("f32", "f64"):
            return f.astype(_CAST_NP[dst])
        with np.errstate(invalid="ignore"):
            return np.trunc(f).astype(np.int32).astype(_CAST_NP[dst])   # as int, then the implicit conversion
    # dst narrow, src one of the CPU types
    if src in ("f32", "f64"):
        with np.errstate(over="ignore"):
            f = x.astype(np.float32)
            return f.astype(np.float16) if dst == "fp16" else _f32_to_bf16_rn(f)
    v = x.astype(np.int32)                                        # bool -> 0/1; wider integers wrap, as `int`
    f = _int_to_f32_rz(v)
    if dst == "fp16":
        return _f32_to_fp16_rz(f)
    return (f.view(np.uint32) >> 16).astype(np.uint16)            # dropping the low half is rounding toward zero


def cast_bool_reference_literal(x, src):
    """The `-> Bool` expression the reference's CUDA kernel generates for floating sources
    (cuda_kernel.cc:73-88): `x == 0`.  Kept as a named fixture of the defect; not used as oracle."""
    f = cast(x, src, "f64") if src in ("fp16", "bf16") else np.asarray(x)
    return f == 0


# ---------------------------------------------------------------------------------------------
# MatMul: Y = alpha * op(A) @ op(B) + beta * C (src/04kernel/src/kernels/mat_mul/cpu_kernel.cc:27-66,
# mat_mul_common/cpu_template.hpp:19-31; shapes and broadcasting of
# src/04kernel/src/attributes/mat_mul_info.cc:27-43).  `dtype` names the element type: "f32", "f64"
# computed as the CPU kernel does; "fp16" / "bf16" (no CPU kernel in the reference: the cuBLAS
# kernel takes them) computed in float on the up-cast values with alpha / beta rounded to the type
# first and one rounding of the result.  bf16 tensors are uint16 bit patterns.
def matmul(a, b, c=None, trans_a=False, trans_b=False, alpha=1.0, beta=1.0, dtype="f32"):
    def widen(t):
        if dtype == "bf16":
            return _bf16_to_f32(np.ascontiguousarray(t, np.uint16))
        return np.ascontiguousarray(t, np.float64 if dtype == "f64" else np.float32)

    def through(v):  # alpha, beta converted to the data type (cpu_kernel.cc:46-47)
        if dtype == "fp16":
            return float(np.float16(v))
        if dtype == "bf16":
            return float(_bf16_to_f32(_f32_to_bf16_rn(np.array([v], np.float32)))[0])
        return float(np.float32(v)) if dtype == "f32" else float(v)

    a, b = widen(a), widen(b)
    wide = np.float64 if dtype == "f64" else np.float32
    m, k = (a.shape[-1], a.shape[-2]) if trans_a else (a.shape[-2], a.shape[-1])
    n = b.shape[-2] if trans_b else b.shape[-1]
    assert k == (b.shape[-1] if trans_b else b.shape[-2])
    batch_shape = np.broadcast_shapes(a.shape[:-2], b.shape[:-2])
    out_shape = tuple(batch_shape) + (m, n)
    if c is None:
        y, beta = np.zeros(out_shape, wide), 0.0
    else:
        y = np.ascontiguousarray(np.broadcast_to(widen(c), out_shape)).copy()   # the Expand of the bias
    a_b = np.broadcast_to(a, tuple(batch_shape) + a.shape[-2:]).reshape((-1,) + a.shape[-2:])
    b_b = np.broadcast_to(b, tuple(batch_shape) + b.shape[-2:]).reshape((-1,) + b.shape[-2:])
    y2 = y.reshape(-1, m, n)
    fn = lib().oracle_matmul_bias_f64 if dtype == "f64" else lib().oracle_matmul_bias_f32
    sa = (1, m) if trans_a else (k, 1)
    sb = (1, k) if trans_b else (n, 1)
    for i in range(y2.shape[0]):
        ai, bi, yi = np.ascontiguousarray(a_b[i]), np.ascontiguousarray(b_b[i]), np.ascontiguousarray(y2[i])
        fn(_p(yi), _p(ai), _p(bi), m, k, n, sa[0], sa[1], sb[0], sb[1], through(alpha), through(beta))
        y2[i] = yi
    y = y2.reshape(out_shape)
    if dtype == "fp16":
        with np.errstate(over="ignore"):
            return y.astype(np.float16)
    if dtype == "bf16":
        return _f32_to_bf16_rn(y)
    return y


def transpose_info(shape, perm, elem_size):
    """The reference's digest of a transposition: ([(strideI, strideO), ...], block bytes, block count)."""
    rank = len(shape)
    assert rank == len(perm) and rank <= 8
    sh, pm = np.asarray(shape, np.uint32), np.asarray(perm, np.uint32)
    si, so = np.zeros(8, np.uint32), np.zeros(8, np.uint32)
    block, count = np.zeros(1, np.uint32), np.zeros(1, np.uint32)
    dims = lib().oracle_transpose_info(_p(si), _p(so), _p(block), _p(count), _p(sh), _p(pm), rank, elem_size)
    return [(int(si[i]), int(so[i])) for i in range(dims)], int(block[0]), int(count[0])


def transpose(x, perm):
    """np.transpose(x, perm) made contiguous, computed the reference's way (any dtype, moved as bytes)."""
    x = np.ascontiguousarray(x)
    sh, pm = np.asarray(x.shape, np.uint32), np.asarray(perm, np.uint32)
    y = np.empty(tuple(x.shape[p] for p in perm), dtype=x.dtype)
    lib().oracle_transpose(_p(y), _p(x), _p(sh), _p(pm), x.ndim, x.dtype.itemsize)
    return y


def split_info(part_shapes, axis, elem_size):
    """The reference's SplitInfo of parts with the given shapes: (block count, bytes per joined block, segment bytes)."""
    shapes = np.asarray(part_shapes, np.uint32)
    count, rank = shapes.shape
    blocks, total = np.zeros(1, np.uint32), np.zeros(1, np.uint32)
    segments = np.zeros(count, np.uint32)
    lib().oracle_split_info(_p(blocks), _p(total), _p(segments), _p(shapes), count, rank, axis, elem_size)
    return int(blocks[0]), int(total[0]), [int(v) for v in segments]


def split(x, sizes, axis):
    """numpy.split(x, cumsum(sizes)[:-1], axis) made contiguous, computed the reference's way."""
    x = np.ascontiguousarray(x)
    shapes = [x.shape[:axis] + (n,) + x.shape[axis + 1:] for n in sizes]
    blocks, total, segments = split_info(shapes, axis, x.dtype.itemsize)
    outs = [np.empty(sh, x.dtype) for sh in shapes]
    ptrs = (C.c_void_p * len(outs))(*[o.ctypes.data for o in outs])
    seg = np.asarray(segments, np.uint32)
    lib().oracle_split(ptrs, _p(x), _p(seg), len(outs), blocks, total)
    return outs


def concat(parts, axis):
    """numpy.concatenate(parts, axis), computed the reference's way."""
    parts = [np.ascontiguousarray(p) for p in parts]
    blocks, total, segments = split_info([p.shape for p in parts], axis, parts[0].dtype.itemsize)
    shape = list(parts[0].shape)
    shape[axis] = sum(p.shape[axis] for p in parts)
    y = np.empty(shape, parts[0].dtype)
    ptrs = (C.c_void_p * len(parts))(*[p.ctypes.data for p in parts])
    seg = np.asarray(segments, np.uint32)
    lib().oracle_concat(_p(y), ptrs, _p(seg), len(parts), blocks, total)
    return y


def expand_info(in_shape, out_shape, elem_size):
    """The reference's ExpandInfo: ([(i, o), ...], block bytes, block count)."""
    a, b = np.asarray(in_shape, np.uint32).reshape(-1), np.asarray(out_shape, np.uint32).reshape(-1)
    si, so = np.zeros(18, np.uint32), np.zeros(18, np.uint32)
    block, count = np.zeros(1, np.uint32), np.zeros(1, np.uint32)
    dims = lib().oracle_expand_info(_p(si), _p(so), _p(block), _p(count), _p(a), len(a), _p(b), len(b), elem_size)
    return [(int(si[d]), int(so[d])) for d in range(dims)], int(block[0]), int(count[0])


def expand(x, out_shape):
    """numpy.broadcast_to(x, out_shape) made contiguous, computed the reference's way."""
    x = np.require(x, requirements="C")
    pairs, block, count = expand_info(x.shape, out_shape, x.dtype.itemsize)
    y = np.empty(out_shape, x.dtype)
    si = np.asarray([p[0] for p in pairs] + [0], np.uint32)
    so = np.asarray([p[1] for p in pairs] + [1], np.uint32)
    lib().oracle_expand(_p(y), _p(x), _p(si), _p(so), len(pairs), block, count)
    return y


def broadcaster(shapes):
    """The reference's Broadcaster of the given input shapes: (rows of strides: one per input, then the output's;
    output element count).  No rows: nothing is broadcast."""
    n = len(shapes)
    table = np.ones((n, 8), np.uint32)
    ranks = np.zeros(n, np.int32)
    for i, sh in enumerate(shapes):
        ranks[i] = len(sh)
        table[i, :len(sh)] = sh
    strides, count = np.zeros(16 * (n + 1), np.uint32), np.zeros(1, np.uint32)
    dims = lib().oracle_broadcaster(_p(strides), _p(count), _p(table), _p(ranks), n)
    return strides[:dims * (n + 1)].reshape(dims, n + 1).astype(np.int64).tolist(), int(count[0])


def where(c, x, y):
    """numpy.where(c, x, y) with multidirectional broadcasting, computed the reference's way."""
    c = np.require(np.asarray(c).astype(np.bool_), requirements="C")   # (keeps 0-d arrays 0-d)
    x, y = np.require(x, requirements="C"), np.require(y, requirements="C")
    assert x.dtype == y.dtype
    rows, count = broadcaster([c.shape, x.shape, y.shape])
    out = np.empty(np.broadcast_shapes(c.shape, x.shape, y.shape), x.dtype)
    assert out.size == count
    st = np.asarray(rows, np.uint32).reshape(-1) if rows else np.zeros(4, np.uint32)
    lib().oracle_where(_p(out), _p(c.view(np.uint8)), _p(x), _p(y), _p(st), len(rows), count, x.dtype.itemsize)
    return out
