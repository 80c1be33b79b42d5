"""GPU test of tf_flash_decode_static_f16, the flash-decoding entry point that allocates
nothing: its per-split partials live in a static device array inside the library instead of a
caller-provided workspace.  It runs the same two kernels as tf_flash_decode_f16, so its output
must be bit-identical to that entry point's (and therefore within rel-L2 <= 1e-3 / max-abs <=
2e-2 of the fp32 oracle, which is also checked).  Two calls in a row share the one array; the
second is smaller, so stale partials of the first lie behind and between its own."""

import math

import pytest
import torch

import oracle
from oracle import numerics as N
from tests.gpu_util import DEV, c_decode, stream
from tilefusion_amd import _capi

pytestmark = pytest.mark.gpu


def _slices(bh, lkv):
    qs, ks, vs = zip(*[oracle.make_c5_decode_slice(i // 32, i % 32, kv_len=lkv) for i in range(bh)])
    return torch.stack(qs), torch.stack(ks), torch.stack(vs)


def c_decode_static(q, k, v, num_splits, scale=None):
    lib = _capi.load()
    bh, lkv, d = k.shape
    scale = 1.0 / math.sqrt(d) if scale is None else scale
    o = torch.full((bh, d), float("nan"), device=q.device, dtype=torch.float16)
    _capi.check(lib.tf_flash_decode_static_f16(q.data_ptr(), k.data_ptr(), v.data_ptr(), o.data_ptr(), bh, lkv, d,
                                               num_splits, scale, stream()), "tf_flash_decode_static_f16")
    return o


def test_static_scratch_matches_workspace_entry_point_on_two_calls():
    lib = _capi.load()
    assert lib.tf_flash_decode_static_max_partials() == 32768
    for bh, lkv, splits in [(24, 6000, 48), (5, 777, 7)]:      # the second call is the smaller one
        q, k, v = _slices(bh, lkv)
        qd, kd, vd = q.to(DEV), k.to(DEV), v.to(DEV)
        got = c_decode_static(qd, kd, vd, splits)
        want = c_decode(qd, kd, vd, splits)
        torch.cuda.synchronize()
        assert not torch.isnan(got).any()
        assert torch.equal(got, want), f"bh={bh} lkv={lkv} splits={splits}: differs from tf_flash_decode_f16"
        ok, r, m = N.check_close(got, N.flash_decode_ref(q, k, v))
        assert ok, f"bh={bh} lkv={lkv} splits={splits}: rel_l2={r:.3e} max_abs={m:.3e}"


def test_static_entry_point_allocates_nothing_and_runs_on_any_stream():
    # after the one-time address lookup a call must leave the device's free memory untouched (torch's
    # caching allocator is bypassed by asking the driver), on the default and on a second stream
    lib = _capi.load()
    assert lib.tf_flash_decode_static_prepare() == 0
    q, k, v = _slices(8, 3000)
    qd, kd, vd = q.to(DEV), k.to(DEV), v.to(DEV)
    want = c_decode(qd, kd, vd, 12)
    o = torch.full((8, 128), float("nan"), device=DEV, dtype=torch.float16)
    side = torch.cuda.Stream()

    def both_streams():
        for st in (stream(), side.cuda_stream):
            o.fill_(float("nan"))
            torch.cuda.synchronize()
            rc = lib.tf_flash_decode_static_f16(qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), o.data_ptr(), 8, 3000, 128,
                                                12, 1.0 / math.sqrt(128), st)
            assert rc == 0
            torch.cuda.synchronize()
            assert torch.equal(o, want)

    # The first pass pays what the runtime sets up once per stream and per kernel (queues, code
    # objects, torch's own staging for the comparison); the second pass is the one measured.
    both_streams()
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    both_streams()
    free_after, _ = torch.cuda.mem_get_info()
    # the runtime may hand memory of earlier work back in the meantime; a call that allocated and
    # kept anything would show as less free memory
    assert free_after >= free_before


def test_static_scratch_rejects_sizes_beyond_the_array():
    lib = _capi.load()
    q, k, v = _slices(2, 64)
    qd, kd, vd = q.to(DEV), k.to(DEV), v.to(DEV)
    o = torch.zeros(2, 128, device=DEV, dtype=torch.float16)
    rc = lib.tf_flash_decode_static_f16(qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), o.data_ptr(), 2, 64, 128,
                                        16385, 0.1, stream())    # 2 x 16385 partials > 32768
    assert rc == _capi.TF_ERR_INVALID_ARG
    assert b"exceeds the static scratch array" in lib.tf_last_error()
    rc = lib.tf_flash_decode_static_f16(qd.data_ptr(), kd.data_ptr(), vd.data_ptr(), o.data_ptr(), 2, 64, 64,
                                        4, 0.1, stream())
    assert rc == _capi.TF_ERR_UNSUPPORTED
    torch.cuda.synchronize()
    assert (o == 0).all()
