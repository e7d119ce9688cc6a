"""The entry point that allocates nothing (flh_decode_attention_f16_static: partial results in a static device array)
against flh_decode_attention_f16 with a caller workspace, through the C ABI: the same bits, on two calls in a row, the
second with a smaller input; a call beyond the static array's size is rejected before anything is launched."""
import ctypes

import pytest
import torch

from flh_amd import _lib

pytestmark = pytest.mark.gpu


def call(lib, static, q, k, v, kv_len):
    b, hq, d = q.shape
    hkv, max_len = k.size(1), k.size(2)
    out = torch.full_like(q, float("nan"))
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    common = (ctypes.c_void_p(q.data_ptr()), ctypes.c_void_p(k.data_ptr()), ctypes.c_void_p(v.data_ptr()),
              ctypes.c_void_p(out.data_ptr()), b, hq, hkv, d, kv_len, max_len, ctypes.c_float(d ** -0.5))
    if static:
        rc = lib.flh_decode_attention_f16_static(*common, stream)
    else:
        need = lib.flh_decode_attention_workspace_bytes(b, hq, d, kv_len)
        ws = torch.empty(need, dtype=torch.uint8, device="cuda")
        rc = lib.flh_decode_attention_f16(*common, ctypes.c_void_p(ws.data_ptr()), need, stream)
    torch.cuda.synchronize()
    return rc, out


def test_static_scratch_entry_point_equals_the_workspace_one():
    lib = _lib.load()
    assert lib.flh_init() == 0, lib.flh_last_error()
    gen = torch.Generator(device="cuda").manual_seed(1)
    for b, hq, hkv, d, kv_len, max_len in ((16, 32, 8, 128, 2048, 2048), (3, 8, 4, 64, 100, 128),   # the second smaller
                                           (24, 32, 32, 128, 1000, 1024)):                       # ... and a larger one again
        q = torch.randn(b, hq, d, device="cuda", generator=gen).half()
        k = (torch.randn(b, hkv, max_len, d, device="cuda", generator=gen) * 0.5).half()
        v = torch.randn(b, hkv, max_len, d, device="cuda", generator=gen).half()
        print(f"case static scratch b={b} hq={hq} d={d} kv_len={kv_len}", flush=True)
        rc_s, out_s = call(lib, True, q, k, v, kv_len)
        rc_w, out_w = call(lib, False, q, k, v, kv_len)
        assert rc_s == 0 and rc_w == 0, lib.flh_last_error()
        assert not torch.isnan(out_s).any()
        assert torch.equal(out_s, out_w)
    # beyond the static array: rejected, nothing written
    cap = lib.flh_decode_attention_static_scratch_bytes()
    b, hq, d, kv_len = 64, 32, 128, 4096
    assert lib.flh_decode_attention_workspace_bytes(b, hq, d, kv_len) > cap
    q = torch.zeros(b, hq, d, device="cuda", dtype=torch.float16)
    k = torch.zeros(b, 8, kv_len, d, device="cuda", dtype=torch.float16)
    rc, out = call(lib, True, q, k, k, kv_len)
    assert rc == -1 and b"static" in lib.flh_last_error() and bool(torch.isnan(out).all())
