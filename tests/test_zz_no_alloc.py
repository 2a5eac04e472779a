"""The entry point that allocates nothing (rg_hip_attention_kvcache_static) against the existing
rg_hip_attention_kvcache, through the C ABI: two calls in a row, the second on a smaller input, so
that whatever the first call left in the library's scratch array is still there.  Outputs within
the fp16 bar (2e-3 absolute; the order of summation is decided at run time in both entries), the
appended cache rows bit for bit."""
import math

import numpy as np
import pytest
import torch

from refactorgraph_amd import abi, ops

pytestmark = pytest.mark.gpu
DEV = "cuda"
ABS_F16 = 2e-3


def _inputs(N, H, Hkv, seq, cap, D, past, seed):
    g = torch.Generator(device=DEV).manual_seed(seed)
    rnd = lambda shape: torch.randn(shape, generator=g, device=DEV).half()
    return dict(q=rnd((N, H, seq, D)), k=rnd((N, Hkv, seq, D)), v=rnd((N, Hkv, seq, D)),
                kc=rnd((N, Hkv, cap, D)), vc=rnd((N, Hkv, cap, D)),
                past=torch.as_tensor(np.asarray(past, dtype=np.int64)).to(DEV))


def _static(t, scale):
    N, H, seq, D = t["q"].shape
    Hkv, cap = t["k"].shape[1], t["kc"].shape[2]
    o = torch.empty_like(t["q"])
    kc, vc = t["kc"].clone(), t["vc"].clone()
    torch.cuda.synchronize()
    p = lambda x: x.data_ptr()
    rc = abi.lib().rg_hip_attention_kvcache_static(
        p(o), p(t["q"]), p(t["k"]), p(t["v"]), p(kc), p(vc), p(t["past"]), int(N > 1), N, H, Hkv, seq, cap, D,
        float(scale), abi.FP16, torch.cuda.current_stream().cuda_stream)
    assert rc == 0, abi.lib().rg_hip_error_string(rc)
    torch.cuda.synchronize()
    return o, kc, vc


def _existing(t, scale):
    kc, vc = t["kc"].clone(), t["vc"].clone()
    o = ops.attention_kvcache(t["q"], t["k"], t["v"], kc, vc, t["past"], scale)
    torch.cuda.synchronize()
    return o, kc, vc


def test_static_scratch_entry_matches_the_workspace_entry_twice():
    assert abi.lib().rg_hip_attention_kvcache_static_scratch_bytes() <= 4 << 20
    rng = np.random.default_rng(5)
    # the decode configuration (every range cuts segments: partials and tickets in use), then a smaller batch
    big = _inputs(32, 32, 8, 1, 4096, 128, rng.integers(1024, 4096, 32), seed=1)
    small = _inputs(3, 8, 2, 1, 700, 128, [699 - 1, 17, 300], seed=2)
    scale = 1 / math.sqrt(128)
    for t in (big, small):
        o, kc, vc = _static(t, scale)
        ro, rkc, rvc = _existing(t, scale)
        assert torch.equal(kc, rkc) and torch.equal(vc, rvc)
        assert float((o.float() - ro.float()).abs().max()) <= ABS_F16
        assert bool(torch.isfinite(o).all())
    # several new rows per batch row (more segments than workgroups) and the tiled prefill path, which needs no scratch
    for t in (_inputs(4, 8, 8, 40, 64, 64, [0, 5, 24, 11], seed=3), _inputs(2, 8, 2, 48, 128, 128, [0, 60], seed=4)):
        o, kc, vc = _static(t, 0.11)
        ro, rkc, rvc = _existing(t, 0.11)
        assert torch.equal(kc, rkc) and torch.equal(vc, rvc)
        assert float((o.float() - ro.float()).abs().max()) <= ABS_F16


def test_static_scratch_entry_with_a_long_cache_and_few_query_tiles():
    # a prompt chunk against a long cache: the tiled kernel shares an item's keys between workgroups as far as the
    # library's 2 MiB of scratch hold their records (fewer ranges than with the caller's workspace), then a call
    # whose records do not fit at all; same results either way
    scale = 1 / math.sqrt(128)
    for t in (_inputs(1, 32, 8, 64, 4160, 128, [4000], seed=3), _inputs(2, 32, 8, 100, 3100, 128, [3000, 5], seed=4),
              _inputs(1, 8, 2, 16, 2064, 128, [2048], seed=5)):
        o, kc, vc = _static(t, scale)
        ro, rkc, rvc = _existing(t, scale)
        assert torch.equal(kc, rkc) and torch.equal(vc, rvc)
        assert float((o.float() - ro.float()).abs().max()) <= ABS_F16


def test_static_scratch_entry_on_the_other_head_groups_and_head_dims():
    # eight query heads per kv head against a long history (the launch of half as many workgroups), groups of 3 and 5
    # with one new row (the tiled kernel with key ranges, as far as the scratch holds their records), head dims 80
    # and 96 (tiled kernel only, no key ranges)
    cases = [(_inputs(2, 64, 8, 1, 4097, 128, [4096, 1500], seed=6), 1 / math.sqrt(128)),
             (_inputs(3, 24, 8, 1, 2100, 128, [2099, 40, 1024], seed=7), 1 / math.sqrt(128)),
             (_inputs(2, 20, 4, 1, 1500, 64, [1499, 700], seed=8), 0.125),
             (_inputs(2, 16, 4, 1, 600, 80, [599, 100], seed=9), 0.11),
             (_inputs(1, 12, 4, 40, 300, 96, [200], seed=10), 0.1),
             (_inputs(2, 16, 2, 1, 90, 128, [3, 89], seed=11), 0.09)]
    for t, scale in cases:
        o, kc, vc = _static(t, scale)
        ro, rkc, rvc = _existing(t, scale)
        assert torch.equal(kc, rkc) and torch.equal(vc, rvc)
        assert float((o.float() - ro.float()).abs().max()) <= ABS_F16
        assert bool(torch.isfinite(o).all())


def test_static_scratch_entry_refuses_what_the_workspace_entry_refuses():
    d = torch.zeros(4096, device=DEV, dtype=torch.float16)
    p = d.data_ptr()
    L = abi.lib()
    assert L.rg_hip_attention_kvcache_static(p, p, p, p, None, None, None, 0, 1, 8, 2, 1, 0, 48, 0.1, abi.FP16, None) == -1
    assert L.rg_hip_attention_kvcache_static(p, p, p, p, None, None, None, 0, 1, 8, 2, 1, 0, 256, 0.1, abi.FP16, None) == -3
    assert L.rg_hip_attention_kvcache_static(p, p, p, p, None, None, None, 0, 1, 8, 3, 1, 0, 128, 0.1, abi.FP16, None) == -2
