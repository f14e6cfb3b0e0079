"""The decode entry point that allocates nothing (static scratch array) against the one that takes a caller
workspace: both are called through the C ABI on the same inputs, twice in a row, the second call smaller."""
import ctypes
import math

import pytest
import torch

from tests.gpu_util import say
from tests.test_gpu_decode import ragged_cache

pytestmark = pytest.mark.gpu


def both_entry_points(lib, q, k, v, valid, n_rows, row_end, tail_start):
    """(workspace form, static-scratch form) of one decode step, as raw C-ABI calls."""
    from neuralattentionsearch_amd._lib import check, i64_array
    B, Hq, _, D = q.shape
    Hkv = k.shape[1]
    code = 0 if q.dtype == torch.bfloat16 else 1
    qc = q.reshape(B, Hq, D).contiguous()
    v8 = valid.view(torch.uint8)
    scale = 1.0 / math.sqrt(D)
    stream = torch.cuda.current_stream().cuda_stream or None
    re_ptr = None if row_end is None else row_end.data_ptr()
    common = (qc.data_ptr(), k.data_ptr(), v.data_ptr(), v8.data_ptr(), re_ptr, int(tail_start))
    shape = (B, Hq, Hkv, D, n_rows, i64_array(k.stride()[:3]), i64_array(v8.stride()[:2]), scale, code)
    nbytes = lib.nats_decode_workspace_bytes(B, Hq, Hkv, D, n_rows)
    ws = torch.empty(nbytes, dtype=torch.uint8, device="cuda")
    out_ws = torch.full((B, Hq, D), float("nan"), dtype=q.dtype, device="cuda")
    out_static = torch.full((B, Hq, D), float("nan"), dtype=q.dtype, device="cuda")
    check(lib.nats_decode_fwd(*common, out_ws.data_ptr(), *shape, ws.data_ptr(), ws.numel(), stream))
    check(lib.nats_decode_fwd_static(*common, out_static.data_ptr(), *shape, stream))
    torch.cuda.synchronize()
    return out_ws, out_static


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32])
def test_static_scratch_equals_caller_workspace_twice_second_smaller(dtype):
    from neuralattentionsearch_amd import _lib
    lib = _lib.load()
    assert lib.nats_decode_static_scratch_bytes() == 8 << 20
    # (B, Hq, Hkv, D, W, C, longest head in chunks, open-chunk rows): the second call is the smaller one and
    # finds the first call's partial results in the shared array
    cases = [(4, 16, 4, 128, 128, 64, 40, 9), (2, 8, 2, 128, 128, 64, 6, 3)]
    for i, (B, Hq, Hkv, D, W, C, n_chunks, fill) in enumerate(cases):
        say("decode static scratch", dtype, B, Hq, Hkv, D, W, C, n_chunks, fill)
        k, v, valid, n_rows = ragged_cache(40 + i, B, Hkv, D, W, C, n_chunks, dtype, fill=fill)
        row_end, tail_start = ragged_cache.row_end, ragged_cache.tail_start
        q = torch.randn(B, Hq, 1, D, generator=torch.Generator().manual_seed(7 + i)).to(dtype)
        for hint in (False, True):
            re = row_end.cuda() if hint and dtype == torch.bfloat16 else None
            a, b = both_entry_points(lib, q.cuda(), k.cuda(), v.cuda(), valid.cuda(), n_rows, re, tail_start if hint else 0)
            assert torch.isfinite(a).all() and torch.isfinite(b).all()
            assert torch.equal(a, b), f"static-scratch result differs: max abs {(a.float() - b.float()).abs().max().item()}"


def test_static_scratch_rejects_a_shape_beyond_its_size():
    """Validation only: the call fails before anything is launched."""
    from neuralattentionsearch_amd import _lib
    lib = _lib.load()
    B, Hq, Hkv, D, n_rows = 64, 64, 8, 128, 70000
    assert lib.nats_decode_workspace_bytes(B, Hq, Hkv, D, n_rows) > lib.nats_decode_static_scratch_bytes()
    t = torch.zeros(64, dtype=torch.uint8, device="cuda")
    fake = t.data_ptr()
    st = _lib.i64_array([8, 8, 8])
    rc = lib.nats_decode_fwd_static(fake, fake, fake, fake, None, 0, fake, B, Hq, Hkv, D, n_rows, st, st, 1.0, 0, None)
    assert rc == -5
    assert b"static array" in lib.nats_last_error()
    with pytest.raises(ValueError):
        _lib.check(rc)
