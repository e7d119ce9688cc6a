"""The PyTorch-ROCm C++ extension (flh_amd/_flh_torch.so) against the ctypes ops: both call the same C ABI, so every
op must return the same bits for the same inputs (the ctypes ops are what the other test files check against the
oracle); the reference's error behaviour (RuntimeError from the tensor checks); the dispatcher registrations; and
that flh_amd._CUDA really is the extension."""
import numpy as np
import pytest
import torch

import flh_amd
from flh_amd import _ops
from flh_amd import synthetic as syn

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ext():
    from flh_amd import _ext_ops
    return _ext_ops


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def same(a, b):
    if isinstance(a, (list, tuple)):
        return len(a) == len(b) and all(same(x, y) for x, y in zip(a, b))
    return a.dtype == b.dtype and a.shape == b.shape and torch.equal(a, b)


def test_cuda_handle_is_the_extension(ext):
    assert flh_amd._CUDA.gemm_i4_dequant_o16 is ext.gemm_i4_dequant_o16
    assert "flh_amd/_flh_torch" in ext._ext.__file__.replace("\\", "/")
    assert flh_amd._CUDA.encode_f6 is _ops.encode_f6          # ops the extension does not wrap fall through


@pytest.mark.parametrize("m,n,k", [(1, 4096, 4096), (16, 1024, 4096), (300, 520, 1024), (2048, 4096, 512)])
def test_gemm_ops_equal_ctypes(ext, m, n, k):
    rng = np.random.default_rng(m + n + k)
    a = dev(syn.pack_codes(rng.integers(-8, 8, size=(m, k), dtype=np.int8)))
    b = dev(syn.pack_codes(rng.integers(-8, 8, size=(n, k), dtype=np.int8)))
    sa1, sb1 = dev(rng.uniform(0.01, 0.5, size=(m, 1)).astype(np.float16)), dev(syn.weight_scales(n, 1, 1))
    print(f"case ext gemm m={m} n={n} k={k}", flush=True)
    assert same(ext.gemm_i4_dequant_o16(a, b, sa1, sb1), _ops.gemm_i4_dequant_o16(a, b, sa1, sb1))
    for g in (128, 64, 32):
        sag, sbg = dev(rng.uniform(0.01, 0.5, size=(m, k // g)).astype(np.float16)), dev(syn.weight_scales(n, k // g, g))
        assert same(ext.gemm_i4_dequant_o16_gs(a, b, sag, sbg, g), _ops.gemm_i4_dequant_o16_gs(a, b, sag, sbg, g))
        assert same(ext.gemm_i4_dequant(a, b, sa1, sbg, g), _ops.gemm_i4_dequant(a, b, sa1, sbg, g))
        assert same(torch.ops.flh_hip.gemm_i4_dequant_o16_gs(a, b, sag, sbg, g), _ops.gemm_i4_dequant_o16_gs(a, b, sag, sbg, g))
    b2 = dev(syn.pack_codes(rng.integers(-8, 8, size=(n // 2 + 3, k), dtype=np.int8)))
    sb2 = dev(syn.weight_scales(n // 2 + 3, 1, 2))
    assert same(ext.gemm_i4_dequant_multi(a, [b, b2], sa1, [sb1, sb2], 128), _ops.gemm_i4_dequant_multi(a, [b, b2], sa1, [sb1, sb2], 128))


def test_quantiser_ops_equal_ctypes(ext):
    x = dev(syn.activations(777, 128, seed=1))
    assert same(ext.hadamard_and_quantize_i4(x), _ops.hadamard_and_quantize_i4(x))
    assert same(ext.hadamard_and_quantize_i4(x, scale_mul=0.25), _ops.hadamard_and_quantize_i4(x, scale_mul=0.25))
    assert same(ext.quant_and_pack_i4(x), _ops.quant_and_pack_i4(x))
    for g in (32, 64, 128):
        xg = x.view(-1, g)
        assert same(ext.hadamard_and_quantize_i4_gs(xg, g), _ops.hadamard_and_quantize_i4_gs(xg, g))
        assert same(ext.quant_and_pack_i4_gs(xg, g), _ops.quant_and_pack_i4_gs(xg, g))
        y1, y2 = xg.clone(), xg.clone()
        fn = {32: "hadamard_transform_32_half", 64: "hadamard_transform_64_half", 128: "hadamard_transform_half"}[g]
        out = getattr(ext, fn)(y1)
        assert out.data_ptr() == y1.data_ptr() and same(y1, getattr(_ops, fn)(y2))
    for k, mode in ((4096, "exact"), (4096, "fast"), (11008, True), (14336, True), (1024, "exact"), (4096, False)):
        xr = dev(syn.activations(130, k, seed=k))
        assert same(ext.rotate_and_quantize_i4(xr, hadamard=mode), _ops.rotate_and_quantize_i4(xr, hadamard=mode))
    xr = dev(syn.activations(65, 4096, seed=3))
    assert same(ext.rotate_and_quantize_i4(xr, "exact", 0, 128, 0.9, True), _ops.rotate_and_quantize_i4(xr, "exact", 0, 128, 0.9, True))
    w = dev((np.random.default_rng(0).uniform(0.5, 1.5, 4096)).astype(np.float16))
    assert same(ext.rmsnorm_rotate_and_quantize_i4(xr, w, 1e-5), _ops.rmsnorm_rotate_and_quantize_i4(xr, w, 1e-5))
    assert same(ext.rmsnorm_rotate_and_quantize_i4(xr, None, 1e-6, True, 1.0, True), _ops.rmsnorm_rotate_and_quantize_i4(xr, None, 1e-6, True, 1.0, True))
    assert same(ext.rmsnorm_and_quantize_i4_gs(xr, w, 1e-5, 128), _ops.rmsnorm_and_quantize_i4_gs(xr, w, 1e-5, 128))
    g8, u8 = dev(syn.activations(40, 1024, seed=5)).view(2, 20, 1024), dev(syn.activations(40, 1024, seed=6)).view(2, 20, 1024)
    assert same(ext.silu_mul_and_quantize_i4_gs(g8, u8, 128), _ops.silu_mul_and_quantize_i4_gs(g8, u8, 128))


def test_decode_gemm_with_quantiser_inside_equal_ctypes(ext):
    rng = np.random.default_rng(9)
    x = dev(syn.activations(2, 4096, seed=2))
    bs = [dev(syn.pack_codes(rng.integers(-8, 8, size=(n, 4096), dtype=np.int8))) for n in (4096, 1024, 1000)]
    ss = [dev(syn.weight_scales(b.size(0), 32, i)) for i, b in enumerate(bs)]
    assert same(ext.rotate_quantize_gemm_i4(x, bs[0], ss[0]), _ops.rotate_quantize_gemm_i4(x, bs[0], ss[0]))
    assert same(ext.rotate_quantize_gemm_i4_multi(x, bs, ss), _ops.rotate_quantize_gemm_i4_multi(x, bs, ss))


def test_residual_gemm_and_prefill_attention_equal_ctypes(ext):
    rng = np.random.default_rng(11)
    m, n, k = 300, 264, 512
    print("case ext residual gemm / prefill attention", flush=True)
    a = dev(syn.pack_codes(rng.integers(-8, 8, size=(m, k), dtype=np.int8)))
    b = dev(syn.pack_codes(rng.integers(-8, 8, size=(n, k), dtype=np.int8)))
    sa, sb = dev(rng.uniform(0.01, 0.5, size=(m, 1)).astype(np.float16)), dev(syn.weight_scales(n, 1, 1))
    r = dev((rng.standard_normal((m, n)) * 2).astype(np.float16))
    want = _ops.gemm_i4_dequant_add(a, b, sa, sb, r, 128)
    assert same(ext.gemm_i4_dequant_add(a, b, sa, sb, r), want)
    r2 = r.clone()
    got = ext.gemm_i4_dequant_add(a, b, sa, sb, r2, 128, out=r2)         # in place on the residual stream
    assert got.data_ptr() == r2.data_ptr() and same(r2, want)
    assert same(ext.gemm_i4_dequant_add(a, b, sa, sb, r.view(3, 100, n), 128), want)
    with pytest.raises(RuntimeError):
        ext.gemm_i4_dequant_add(a, b, sa, sb, r[:, :32])
    with pytest.raises(RuntimeError):
        ext.gemm_i4_dequant_add(a, b, sa, sb, r.float())
    gen = torch.Generator(device="cuda").manual_seed(4)
    q = torch.randn(2, 150, 8, 128, device="cuda", generator=gen).half()
    kc = torch.randn(2, 2, 200, 128, device="cuda", generator=gen).half()
    vc = torch.randn(2, 2, 200, 128, device="cuda", generator=gen).half()
    assert same(ext.prefill_attention(q, kc, vc, 50), _ops.prefill_attention(q, kc, vc, 50))
    assert same(ext.prefill_attention(q, kc, vc, 0, scale=0.05), _ops.prefill_attention(q, kc, vc, 0, scale=0.05))
    with pytest.raises(RuntimeError):
        ext.prefill_attention(q, kc, vc, 51)                              # past + T exceeds the cache
    with pytest.raises(RuntimeError):
        ext.prefill_attention(q[..., :64].contiguous(), kc[..., :64].contiguous(), vc[..., :64].contiguous(), 0)
    assert flh_amd._CUDA.prefill_attention is ext.prefill_attention


def test_tensor_checks_raise_runtime_error(ext):
    a = torch.zeros(4, 64, dtype=torch.uint8, device="cuda")
    s = torch.ones(4, 1, dtype=torch.float16, device="cuda")
    with pytest.raises(RuntimeError):
        ext.gemm_i4_dequant_o16(a.cpu(), a, s, s)                      # not on the device
    with pytest.raises(RuntimeError):
        ext.gemm_i4_dequant_o16(a, a, s.float(), s)                    # wrong dtype
    with pytest.raises(RuntimeError):
        ext.gemm_i4_dequant_o16(a, a[:, :32], s, s)                    # K mismatch (and not contiguous)
    with pytest.raises(RuntimeError):
        ext.gemm_i4_dequant_o16(a, a, s[:2], s)                        # scale rows
    with pytest.raises(RuntimeError):
        ext.gemm_i4_dequant_o16_gs(a, a, s, s, 48)                     # group size
    with pytest.raises(RuntimeError):
        ext.hadamard_transform_half(torch.zeros(4, 64, dtype=torch.float16, device="cuda"))
    with pytest.raises(RuntimeError):
        ext.quant_and_pack_i4_gs(torch.zeros(4, 64, dtype=torch.float16, device="cuda"), 128)
    assert ext.gemm_i4_dequant_o16(a[:0], a, s[:0], s).shape == (0, 4)


def test_launches_follow_the_current_stream(ext):
    """Work goes to torch's current stream of the tensor's device: a result produced on a side stream and consumed
    after waiting for that stream equals the one from the default stream."""
    x = dev(syn.activations(512, 4096, seed=8))
    want = ext.rotate_and_quantize_i4(x, hadamard="exact")
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        got = ext.rotate_and_quantize_i4(x, hadamard="exact")
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    assert same(got, want)
