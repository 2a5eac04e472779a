"""Test/benchmark driver: calls the C ABI on torch CUDA(HIP) tensors.

Every function hands raw device pointers to librg_hip.so and enqueues on torch's current
stream.  Argument meaning follows include/rg_hip.h; outputs are allocated with torch.
"""
from __future__ import annotations

import ctypes as C
import math

import numpy as np
import torch

from . import abi
from .abi import check, lib

_T2CODE = {
    torch.float32: abi.F32, torch.float64: abi.F64, torch.float16: abi.FP16, torch.bfloat16: abi.BF16,
    torch.uint8: abi.U8, torch.int8: abi.I8, torch.int16: abi.I16, torch.int32: abi.I32,
    torch.int64: abi.I64,
}
_T2CODE[torch.bool] = abi.BOOL
for _name, _code in (("uint16", abi.U16), ("uint32", abi.U32), ("uint64", abi.U64)):
    if hasattr(torch, _name):
        _T2CODE[getattr(torch, _name)] = _code


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _ptr(t):
    return None if t is None else C.c_void_p(t.data_ptr())


def _need_gpu(*ts):
    for t in ts:
        if t is not None and (not t.is_cuda or not t.is_contiguous()):
            raise ValueError("operands must be contiguous device tensors")


def rms_norm(x, w, eps=1e-5, out=None):
    _need_gpu(x, w)
    y = torch.empty_like(x) if out is None else out
    cols = x.shape[-1]
    rows = x.numel() // cols
    check(lib().rg_hip_rms_norm(_ptr(y), _ptr(x), _ptr(w), rows, cols, float(eps), _T2CODE[x.dtype], _stream()),
          "rg_hip_rms_norm")
    return y


def rms_norm_quantize(x, w, eps=1e-5):
    """RmsNormalization followed by DynamicQuantizeLinear of its output, fused: returns (y, yq, scale, zero_point)."""
    _need_gpu(x, w)
    assert x.dtype == torch.float32
    cols = x.shape[-1]
    rows = x.numel() // cols
    nbytes = lib().rg_hip_rms_norm_quantize_workspace(rows, cols)
    if nbytes == 0:
        raise ValueError("rg_hip_rms_norm_quantize does not take this shape")
    ws = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
    y = torch.empty_like(x)
    yq = torch.empty(x.shape, dtype=torch.uint8, device=x.device)
    scale = torch.empty((), dtype=torch.float32, device=x.device)
    zp = torch.empty((), dtype=torch.uint8, device=x.device)
    check(lib().rg_hip_rms_norm_quantize(_ptr(yq), _ptr(scale), _ptr(zp), _ptr(y), _ptr(x), _ptr(w), rows, cols, float(eps),
                                         _ptr(ws), nbytes, _stream()), "rg_hip_rms_norm_quantize")
    return y, yq, scale, zp


def softmax(x, axis=-1, causal=False, out=None):
    _need_gpu(x)
    axis = axis % x.dim()
    pre = math.prod(x.shape[:axis])
    mid = x.shape[axis]
    post = math.prod(x.shape[axis + 1:])
    causal_rows = x.shape[-2] if causal else 0
    y = torch.empty_like(x) if out is None else out
    check(lib().rg_hip_softmax(_ptr(y), _ptr(x), pre, mid, post, _T2CODE[x.dtype], causal_rows, _stream()),
          "rg_hip_softmax")
    return y


def rope(x, pos, theta=10000.0, out=None):
    _need_gpu(x, pos)
    assert pos.dtype == torch.int64
    batch, seq, heads, dim = x.shape
    per_batch = int(pos.dim() == 2)
    y = torch.empty_like(x) if out is None else out
    check(lib().rg_hip_rope(_ptr(y), _ptr(x), _ptr(pos), per_batch, batch, seq, heads, dim, float(theta),
                            _T2CODE[x.dtype], _stream()), "rg_hip_rope")
    return y


def dequantize_linear(x, scale, zp=None, axis=1, out=None):
    _need_gpu(x, scale, zp)
    assert scale.dtype == torch.float32
    per_axis = int(scale.numel() != 1)
    if per_axis:
        axis = axis % x.dim()
        outer, axis_len, inner = math.prod(x.shape[:axis]), x.shape[axis], math.prod(x.shape[axis + 1:])
        assert scale.numel() == axis_len
    else:
        outer, axis_len, inner = 1, 1, x.numel()
    y = torch.empty(x.shape, dtype=torch.float32, device=x.device) if out is None else out
    check(lib().rg_hip_dequantize_linear(_ptr(y), _ptr(x), _ptr(scale), _ptr(zp), outer, axis_len, inner,
                                         _T2CODE[x.dtype], per_axis, _stream()), "rg_hip_dequantize_linear")
    return y


def dynamic_quantize_linear(x, out=None, workspace=None):
    """x float32 (any shape) -> (y uint8 like x, scale float32 [1], zero_point uint8 [1])."""
    _need_gpu(x)
    assert x.dtype == torch.float32 and x.is_contiguous()
    n = x.numel()
    y = torch.empty(x.shape, dtype=torch.uint8, device=x.device) if out is None else out
    assert y.dtype == torch.uint8 and y.numel() == n and y.is_contiguous()
    scale = torch.empty(1, dtype=torch.float32, device=x.device)
    zp = torch.empty(1, dtype=torch.uint8, device=x.device)
    nbytes = lib().rg_hip_dynamic_quantize_linear_workspace(n)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=x.device) if workspace is None else workspace
    check(lib().rg_hip_dynamic_quantize_linear(_ptr(y), _ptr(scale), _ptr(zp), _ptr(x), n, _ptr(ws), ws.numel(),
                                               _stream()), "rg_hip_dynamic_quantize_linear")
    return y, scale, zp


def cast(x, dtype, out=None):
    """Element-wise conversion of x to `dtype` (a torch dtype)."""
    _need_gpu(x)
    assert x.is_contiguous()
    y = torch.empty(x.shape, dtype=dtype, device=x.device) if out is None else out
    assert y.dtype == dtype and y.numel() == x.numel() and y.is_contiguous()
    check(lib().rg_hip_cast(_ptr(y), _ptr(x), x.numel(), _T2CODE[x.dtype], _T2CODE[dtype], _stream()), "rg_hip_cast")
    return y


def matmul(a, b, c=None, trans_a=False, trans_b=False, alpha=1.0, beta=1.0, out=None, workspace=None):
    """Y = alpha * op(A) @ op(B) + beta * C.  a [..., m, k] ([..., k, m] when trans_a), b [..., k, n]
    ([..., n, k] when trans_b), batch dimensions broadcast; c broadcasts to [m, n] (any leading
    dimensions of size 1) or has the output's full shape.  float32/float64/float16/bfloat16."""
    _need_gpu(a, b, c)
    assert a.dtype == b.dtype and a.is_contiguous() and b.is_contiguous()
    m, k = (a.shape[-1], a.shape[-2]) if trans_a else (a.shape[-2], a.shape[-1])
    n = b.shape[-2] if trans_b else b.shape[-1]
    assert k == (b.shape[-1] if trans_b else b.shape[-2])
    ab, bb = tuple(a.shape[:-2]), tuple(b.shape[:-2])
    ob = tuple(np.broadcast_shapes(ab, bb))
    batch = math.prod(ob)
    a_idx = b_idx = None
    if ab != bb:
        ia = np.arange(math.prod(ab), dtype=np.uint32).reshape(ab)
        ib = np.arange(math.prod(bb), dtype=np.uint32).reshape(bb)
        oa, obb = np.broadcast_arrays(ia, ib)
        a_idx = np.ascontiguousarray(oa.reshape(-1))
        b_idx = np.ascontiguousarray(obb.reshape(-1))
    sb = sm = sn = 0
    if c is not None:
        assert c.dtype == a.dtype and c.is_contiguous()
        cs = (1,) * (len(ob) + 2 - c.dim()) + tuple(c.shape)
        if cs[:-2] == ob and batch > 1:
            sb = cs[-2] * cs[-1]
        else:
            assert all(d == 1 for d in cs[:-2]), "bias batch dimensions must be 1 or the output's"
        assert cs[-2] in (1, m) and cs[-1] in (1, n)
        sm = cs[-1] if cs[-2] == m else 0
        sn = 1 if cs[-1] == n else 0
        if cs[-2] == 1:
            sm = 0
    y = torch.empty(ob + (m, n), dtype=a.dtype, device=a.device) if out is None else out
    if workspace is None:
        # what the routine's lowering would ask the allocator for (a uint8 tensor passed as `workspace` is used as is)
        need = lib().rg_hip_matmul_workspace(_T2CODE[a.dtype], int(trans_a), int(trans_b), batch, m, k, n)
        workspace = torch.empty(need, dtype=torch.uint8, device=a.device) if need else None
    check(lib().rg_hip_matmul_ws(
        _ptr(y), _ptr(a), _ptr(b), _ptr(c), _T2CODE[a.dtype], int(trans_a), int(trans_b), float(alpha), float(beta),
        batch, m, k, n,
        None if a_idx is None else a_idx.ctypes.data_as(C.c_void_p),
        None if b_idx is None else b_idx.ctypes.data_as(C.c_void_p),
        sb, sm, sn, _ptr(workspace), 0 if workspace is None else workspace.numel(), _stream()), "rg_hip_matmul_ws")
    return y


def transpose_info(shape, perm, itemsize):
    """(stride_i, stride_o, block bytes, block count): the digest of a transposition that
    rg_hip_transpose takes (TransposeInfo of the host layer, restated for this driver): size-1
    dimensions dropped, dimensions that stay neighbours merged, a last dimension that stays last
    folded into the block."""
    dims = [(s, p) for p, s in enumerate(shape)]
    keep = [i for i, s in enumerate(shape) if s != 1]
    new_of = {old: new for new, old in enumerate(keep)}
    shape = [shape[i] for i in keep]
    perm = [new_of[p] for p in perm if p in new_of]
    # merge runs perm[i], perm[i]+1, ... into one dimension
    runs = []
    for p in perm:
        if runs and p == runs[-1][-1] + 1:
            runs[-1].append(p)
        else:
            runs.append([p])
    runs_in_input_order = sorted(runs, key=lambda r: r[0])
    shape = [math.prod(shape[i] for i in r) for r in runs_in_input_order]
    perm = [runs_in_input_order.index(r) for r in runs]
    block, count = itemsize, math.prod(shape)
    if len(shape) <= 1:
        return [1], [1], block * count, 1
    if perm[-1] == len(shape) - 1:
        block *= shape[-1]
        count //= shape[-1]
        shape, perm = shape[:-1], perm[:-1]
    in_stride = [math.prod(shape[i + 1:]) for i in range(len(shape))]
    out_shape = [shape[p] for p in perm]
    stride_o = [math.prod(out_shape[i + 1:]) for i in range(len(shape))]
    stride_i = [in_stride[p] for p in perm]
    return stride_i, stride_o, block, count


def transpose(x, perm, out=None):
    """Contiguous x with its dimensions permuted (any dtype: bytes are moved)."""
    _need_gpu(x)
    assert x.is_contiguous() and sorted(perm) == list(range(x.dim()))
    si, so, block, count = transpose_info(list(x.shape), list(perm), x.element_size())
    y = torch.empty([x.shape[p] for p in perm], dtype=x.dtype, device=x.device) if out is None else out
    si_, so_ = np.asarray(si, np.uint32), np.asarray(so, np.uint32)
    check(lib().rg_hip_transpose(_ptr(y), _ptr(x), si_.ctypes.data_as(C.c_void_p), so_.ctypes.data_as(C.c_void_p),
                                 len(si), block, count, _stream()), "rg_hip_transpose")
    return y


def split_info(part_shapes, axis, itemsize):
    """(block count, bytes of a joined block, segment bytes): SplitInfo of the host layer, restated for this driver."""
    first = part_shapes[0]
    blocks = math.prod(first[:axis])
    postfix = itemsize * math.prod(first[axis + 1:])
    segments = [sh[axis] * postfix for sh in part_shapes]
    return blocks, sum(segments), segments


def _pointer_array(tensors):
    return (C.c_void_p * len(tensors))(*[t.data_ptr() for t in tensors])


def split(x, sizes, axis, outs=None):
    """The parts of x along `axis` with the given sizes, each contiguous (any dtype: bytes are moved)."""
    _need_gpu(x)
    axis %= x.dim()
    assert sum(sizes) == x.shape[axis]
    shapes = [tuple(x.shape[:axis]) + (n,) + tuple(x.shape[axis + 1:]) for n in sizes]
    if outs is None:
        outs = [torch.empty(sh, dtype=x.dtype, device=x.device) for sh in shapes]
    blocks, total, segments = split_info(shapes, axis, x.element_size())
    seg = np.asarray(segments, np.uint32)
    check(lib().rg_hip_split(_pointer_array(outs), _ptr(x), seg.ctypes.data_as(C.c_void_p), len(outs), blocks, total,
                             _stream()), "rg_hip_split")
    return outs


def concat(parts, axis, out=None):
    _need_gpu(*parts)
    axis %= parts[0].dim()
    shape = list(parts[0].shape)
    shape[axis] = sum(p.shape[axis] for p in parts)
    y = torch.empty(shape, dtype=parts[0].dtype, device=parts[0].device) if out is None else out
    blocks, total, segments = split_info([tuple(p.shape) for p in parts], axis, parts[0].element_size())
    seg = np.asarray(segments, np.uint32)
    check(lib().rg_hip_concat(_ptr(y), _pointer_array(parts), seg.ctypes.data_as(C.c_void_p), len(parts), blocks, total,
                              _stream()), "rg_hip_concat")
    return y


def expand_info(in_shape, out_shape, itemsize):
    """(stride_i, stride_o, block bytes, block count): ExpandInfo of the host layer, restated for this driver.
    Walks the dimensions from the last one; runs of dimensions that are all broadcast or all kept become one
    stride pair; the innermost run becomes the block."""
    pairs, count, stride, broadcast_run = [], 1, 1, None
    ins = [1] * (len(out_shape) - len(in_shape)) + list(in_shape)
    for i_, o_ in zip(reversed(ins), reversed(list(out_shape))):
        if o_ == 1:
            continue
        is_broadcast = i_ == 1
        if broadcast_run is None:
            if is_broadcast:            # the innermost run is a broadcast one: it starts a pair of its own
                pairs.append((0, count))
        elif is_broadcast != broadcast_run:
            pairs.append((0 if is_broadcast else stride, count))
        broadcast_run = is_broadcast
        if not is_broadcast:
            stride *= i_
        count *= o_
    if not any(p[0] == 0 for p in pairs):
        return [], [], itemsize * count, 1
    # slowest dimension first; the innermost explicit pair is a broadcast one (a kept innermost run is the
    # implicit pair (1, 1)) and becomes the block
    pairs.reverse()
    tail_o = pairs[-1][1]
    return [p[0] // tail_o for p in pairs], [p[1] // tail_o for p in pairs], itemsize * tail_o, count // tail_o


def expand(x, out_shape, out=None):
    _need_gpu(x)
    y = torch.empty(tuple(out_shape), dtype=x.dtype, device=x.device) if out is None else out
    si, so, block, count = expand_info(list(x.shape), list(out_shape), x.element_size())
    si_, so_ = np.asarray(si + [0], np.uint32), np.asarray(so + [1], np.uint32)
    check(lib().rg_hip_expand(_ptr(y), _ptr(x), si_.ctypes.data_as(C.c_void_p), so_.ctypes.data_as(C.c_void_p), len(si),
                              block, count, _stream()), "rg_hip_expand")
    return y


def broadcaster(shapes):
    """(rows of strides: one per input, then the output's; output element count): the host layer's Broadcaster,
    restated for this driver.  Dimensions where every input is 1 vanish; neighbouring dimensions in which the same
    inputs are broadcast merge.  No rows: nothing is broadcast."""
    n, rank = len(shapes), max((len(sh) for sh in shapes), default=0)
    padded = [[1] * (rank - len(sh)) + list(sh) for sh in shapes]
    rows, muls, count, state = [], [1] * n, 1, [False] * n
    for d in reversed(range(rank)):
        dims = [padded[i][d] for i in range(n)]
        extent = max(dims)
        if extent == 1:
            continue
        nxt = [v != 1 for v in dims]
        if nxt != state:
            state = nxt
            rows.append([muls[i] if state[i] else 0 for i in range(n)] + [count])
        for i in range(n):
            if state[i]:
                muls[i] *= extent
        count *= extent
    rows.reverse()
    if len(rows) == 1 and all(v == 1 for v in rows[0]):
        rows = []
    return rows, count


def where(c, x, y, out=None):
    """torch.where(c, x, y) with multidirectional broadcasting; c: bool."""
    _need_gpu(c, x, y)
    assert c.dtype == torch.bool and x.dtype == y.dtype
    rows, count = broadcaster([list(c.shape), list(x.shape), list(y.shape)])
    shape = torch.broadcast_shapes(c.shape, x.shape, y.shape)
    o = torch.empty(shape, dtype=x.dtype, device=x.device) if out is None else out
    st = np.asarray(rows if rows else [[0, 0, 0, 1]], np.uint32).reshape(-1)
    check(lib().rg_hip_where(_ptr(o), _ptr(c), _ptr(x), _ptr(y), st.ctypes.data_as(C.c_void_p), len(rows), count,
                             x.element_size(), _stream()), "rg_hip_where")
    return o


def matmul_integer(a, b, a_zp=None, b_zp=None, out=None, dequant_scale=None):
    """a [..., m, k], b [..., k, n] (uint8/int8).  Zero points: None, one element, or one per
    (batch, row) of the operand as the reference's CPU kernel reads them.  dequant_scale (float32,
    one element or n): the result leaves as float32 = float(sum) * scale instead of int32."""
    _need_gpu(a, b, a_zp, b_zp, dequant_scale)
    m, k = a.shape[-2:]
    k2, n = b.shape[-2:]
    assert k == k2
    ab, bb = tuple(a.shape[:-2]), tuple(b.shape[:-2])
    ob = tuple(np.broadcast_shapes(ab, bb))
    batch = math.prod(ob)
    a_idx = b_idx = None
    if ab != bb:
        na, nb = math.prod(ab), math.prod(bb)
        ia = np.arange(na, dtype=np.uint32).reshape(ab)
        ib = np.arange(nb, dtype=np.uint32).reshape(bb)
        oa, obb = np.broadcast_arrays(ia, ib)
        a_idx = np.ascontiguousarray(oa.reshape(-1))
        b_idx = np.ascontiguousarray(obb.reshape(-1))
    flags = 0
    if a_zp is not None and a_zp.numel() == 1:
        flags |= abi.MMI_A_ZP_SCALAR
    if b_zp is not None and b_zp.numel() == 1:
        flags |= abi.MMI_B_ZP_SCALAR
    if dequant_scale is not None:
        assert dequant_scale.dtype == torch.float32 and dequant_scale.numel() in (1, n)
        y = torch.empty(ob + (m, n), dtype=torch.float32, device=a.device) if out is None else out
        check(lib().rg_hip_matmul_integer_dequantize(
            _ptr(y), _ptr(a), _ptr(b), _ptr(a_zp), _ptr(b_zp), flags, batch, m, k, n,
            None if a_idx is None else a_idx.ctypes.data_as(C.c_void_p),
            None if b_idx is None else b_idx.ctypes.data_as(C.c_void_p),
            _ptr(dequant_scale), int(dequant_scale.numel() != 1), None, _stream()), "rg_hip_matmul_integer_dequantize")
        return y
    y = torch.empty(ob + (m, n), dtype=torch.int32, device=a.device) if out is None else out
    check(lib().rg_hip_matmul_integer(
        _ptr(y), _ptr(a), _ptr(b), _ptr(a_zp), _ptr(b_zp), flags, batch, m, k, n,
        None if a_idx is None else a_idx.ctypes.data_as(C.c_void_p),
        None if b_idx is None else b_idx.ctypes.data_as(C.c_void_p),
        None, _stream()), "rg_hip_matmul_integer")
    return y


_ws_cache = {}


def attention_workspace(N, H, Hkv, seq, cap, D, device):
    nbytes = lib().rg_hip_attention_kvcache_workspace(N, H, Hkv, seq, cap, D)
    key = (nbytes, str(device))
    if key not in _ws_cache:
        _ws_cache[key] = torch.empty(nbytes, dtype=torch.uint8, device=device)
    return _ws_cache[key]


_state_cache = {}


def attention_state(device):
    """Persistent, zero-initialised ticket counters (one buffer per device, calls must not overlap)."""
    key = str(device)
    if key not in _state_cache:
        _state_cache[key] = torch.zeros(lib().rg_hip_attention_kvcache_state_bytes(), dtype=torch.uint8, device=device)
    return _state_cache[key]


def attention_kvcache(q, k, v, k_cache=None, v_cache=None, past_lens=None, scale=None, out=None,
                      workspace=None, sync_state=None):
    """q [N,H,seq,D]; k, v [N,Hkv,seq,D]; caches [N,Hkv,cap,D] are updated in place;
    past_lens: int64 device tensor with 1 or N elements (None = 0)."""
    _need_gpu(q, k, v, k_cache, v_cache, past_lens)
    N, H, seq, D = q.shape
    Hkv = k.shape[1]
    cap = k_cache.shape[2] if k_cache is not None else 0
    if scale is None:
        scale = 1.0 / math.sqrt(D)
    per_row = 0
    if past_lens is not None:
        assert past_lens.dtype == torch.int64 and past_lens.numel() in (1, N)
        per_row = int(past_lens.numel() == N and N > 1)
    o = torch.empty_like(q) if out is None else out
    ws = attention_workspace(N, H, Hkv, seq, cap, D, q.device) if workspace is None else workspace
    check(lib().rg_hip_attention_kvcache(
        _ptr(o), _ptr(q), _ptr(k), _ptr(v), _ptr(k_cache), _ptr(v_cache), _ptr(past_lens), per_row,
        N, H, Hkv, seq, cap, D, float(scale), _T2CODE[q.dtype], _ptr(ws), ws.numel(), _ptr(sync_state),
        _stream()),
        "rg_hip_attention_kvcache")
    return o
