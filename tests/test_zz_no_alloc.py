"""ns_attn_decode_static - the decode entry point that allocates nothing (its partials live in an array inside the
library's code object) - against ns_attn_decode_t on the same inputs: the same kernels, so the same bits. Two calls in a
row share the array; the second, smaller one must not see anything of the first."""
import numpy as np
import pytest

from helpers import gpu_decode, make_kv, make_q
from nextsycl_amd import DevBuf
from nextsycl_amd.attn import BF16, F16, F32
from nextsycl_amd.core import Error

pytestmark = pytest.mark.gpu


def _static(ops, qt, kt, qd, bufs, T, Hq, Hkv, D, cap, p0, win=0):
    g = ops.gpu
    ob = DevBuf(g, T * Hq * D * (4 if qt == F32 else 2))
    ob.fill(0xFF)
    ops.decode_static(qt, kt, DevBuf.of(g, qd), Hq * D, bufs[0], bufs[1], T, Hq, Hkv, D, cap, p0, ob, win=win)
    return ob.read(np.float32 if qt == F32 else np.uint16)


def test_static_scratch_decode_matches_the_buffer_form(ops):
    g = ops.gpu
    # a large pass first (many splits, 4 rows), then smaller ones of other shapes: each against ns_attn_decode_t's bits
    shapes = [(4, 32, 4, 128, 30000, 0, 0, F16), (1, 8, 2, 128, 700, 0, 0, F32), (2, 16, 2, 256, 2500, 0, 1, F32), (3, 16, 4, 128, 5000, 1024, 3, BF16),
              (1, 32, 8, 128, 129, 0, 2, F16)]
    for rep in range(2):
        for i, (T, Hq, Hkv, D, p0, win, kt, qt) in enumerate(shapes):
            cap = p0 + T
            kc, vc = make_kv(kt, Hkv, D, cap, cap, cfg=i)
            qd, _ = make_q(qt, T, Hq, D, cfg=i)
            bufs = (DevBuf.of(g, kc), DevBuf.of(g, vc))
            _, want = gpu_decode(ops, qt, kt, qd, kc, vc, T, Hq, Hkv, D, cap, p0, win=win, bufs=bufs)
            got = _static(ops, qt, kt, qd, bufs, T, Hq, Hkv, D, cap, p0, win=win)
            assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), (rep, i)


def test_static_scratch_decode_rejects_what_does_not_fit(ops):
    g = ops.gpu
    b = DevBuf(g, 1 << 16)
    # 16 rows x 64 heads over 128 splits: 68 MB of partials against the array's 16 MiB - refused before any launch
    T, Hq, Hkv, D, p0 = 16, 64, 4, 128, 200000
    assert ops.k.attn_decode_scratch(T, Hq, Hkv, D, p0, 0) > (4 << 20)
    rc = ops.k.attn_decode_static(g.raw, 0, 0, 0, b.ptr, Hq * D, b.ptr, b.ptr, T, Hq, Hkv, D, p0 + T, p0, 0, 0.0, b.ptr)
    assert rc == -1 and "the array holds" in ops.k.api.error()
    with pytest.raises(Error):
        ops.decode_static(F32, 0, b, Hq * D, b, b, 17, Hq, Hkv, D, 64, 0, b)
