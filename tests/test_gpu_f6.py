"""The int4 GEMM on the 6-bit (e3m2) matrix instruction: encoder bytes against the oracle's definition of
the operand format, int32 sums and fp16 outputs bit for bit against the oracle of the integer GEMM (the
float32 accumulator holds exact integers), through the C ABI."""
import numpy as np
import pytest
import torch

from flh_amd import synthetic as syn

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    assert torch.cuda.is_available(), "these tests need the GPU"
    from flh_amd import _ops
    return _ops


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    return t.detach().cpu().numpy()


@pytest.mark.parametrize("rows,k", [(1, 128), (5, 384), (33, 1024), (64, 640), (300, 4096), (7, 11008)])
def test_encode_f6_bytes(ops, rows, k):
    from oracle.pack import encode_f6
    rng = np.random.default_rng(rows + k)
    q = rng.integers(-8, 8, size=(rows, k), dtype=np.int8)
    q[0, :16] = np.arange(-8, 8)                       # every code at least once
    got = host(ops.encode_f6(dev(syn.pack_codes(q))))
    assert got.shape == (rows, k // 128 * 96)
    assert np.array_equal(got, encode_f6(q))


SHAPES = [(1, 128, 128), (16, 256, 512), (33, 100, 384), (257, 129, 256), (300, 520, 1024), (64, 1024, 11008),
          (700, 4200, 512), (2048, 4096, 256), (1000, 4096, 1152), (130, 8200, 128)]


@pytest.mark.parametrize("m,n,k", SHAPES)
def test_gemm_f6_int32_bit_exact(ops, m, n, k):
    from oracle import gemm as G
    rng = np.random.default_rng(m * 7 + n * 3 + k)
    a = rng.integers(-8, 8, size=(m, k), dtype=np.int8)
    b = rng.integers(-8, 8, size=(n, k), dtype=np.int8)
    print(f"case f6 int32 m={m} n={n} k={k}", flush=True)
    c = host(ops.gemm_f6_int32(ops.encode_f6(dev(syn.pack_codes(a))), ops.encode_f6(dev(syn.pack_codes(b)))))
    assert np.array_equal(c, G.int_gemm(a, b))


@pytest.mark.parametrize("tile", [256, 128, 64])
@pytest.mark.parametrize("k", [1536, 1408, 128])      # even / odd number of K steps, a single step
def test_gemm_f6_every_tile(ops, tile, k, gemm_tuning):
    from oracle import gemm as G
    gemm_tuning(tile)
    m, n = 300, 264
    rng = np.random.default_rng(tile + k)
    a = rng.integers(-8, 8, size=(m, k), dtype=np.int8)
    b = rng.integers(-8, 8, size=(n, k), dtype=np.int8)
    sa, sb = syn.weight_scales(m, 1, 5), syn.weight_scales(n, 1, 6)
    a6, b6 = ops.encode_f6(dev(syn.pack_codes(a))), ops.encode_f6(dev(syn.pack_codes(b)))
    print(f"case f6 tile={tile} k={k}", flush=True)
    assert np.array_equal(host(ops.gemm_f6_int32(a6, b6)), G.int_gemm(a, b))
    ref, _ = G.gemm_i4_dequant(syn.pack_codes(a), syn.pack_codes(b), sa, sb)
    d = host(ops.gemm_f6_dequant_o16(a6, b6, dev(sa), dev(sb)))
    assert np.array_equal(d.view(np.uint16), ref.view(np.uint16))


def test_gemm_f6_extreme_codes_stay_exact(ops):
    """All products +64 (or -56): the largest partial sums the float32 accumulator sees, 64 K = 917504 at
    K = 14336, far below 2^24."""
    for k in (4096, 14336):
        a = np.full((40, k), -8, np.int8)
        b = np.full((72, k), -8, np.int8)
        b[1::2] = 7
        c = host(ops.gemm_f6_int32(ops.encode_f6(dev(syn.pack_codes(a))), ops.encode_f6(dev(syn.pack_codes(b)))))
        assert np.all(c[:, 0::2] == 64 * k) and np.all(c[:, 1::2] == -56 * k)


@pytest.mark.parametrize("m,n,k", [(16, 256, 512), (300, 520, 1024), (2048, 1024, 4096), (257, 4096, 11008)])
def test_gemm_f6_row_scale_equals_the_int8_path_and_the_oracle(ops, m, n, k):
    from oracle import gemm as G
    rng = np.random.default_rng(m + n + k)
    a = rng.integers(-8, 8, size=(m, k), dtype=np.int8)
    b = rng.integers(-8, 8, size=(n, k), dtype=np.int8)
    sa, sb = syn.weight_scales(m, 1, 5), syn.weight_scales(n, 1, 6)
    ap, bp = dev(syn.pack_codes(a)), dev(syn.pack_codes(b))
    print(f"case f6 row scale m={m} n={n} k={k}", flush=True)
    d6 = ops.gemm_f6_dequant_o16(ops.encode_f6(ap), ops.encode_f6(bp), dev(sa), dev(sb))
    assert torch.equal(d6, ops.gemm_i4_dequant_o16(ap, bp, dev(sa), dev(sb)))
    if m * n * k <= 300 * 520 * 1024 * 8:
        ref, _ = G.gemm_i4_dequant(syn.pack_codes(a), syn.pack_codes(b), sa, sb)
        assert np.array_equal(host(d6).view(np.uint16), ref.view(np.uint16))


def test_gemm_f6_argument_errors(ops):
    a6 = torch.zeros(4, 96, dtype=torch.uint8, device="cuda")
    with pytest.raises(RuntimeError):
        ops.gemm_f6_int32(a6, torch.zeros(4, 192, dtype=torch.uint8, device="cuda"))
    with pytest.raises(RuntimeError):
        ops.gemm_f6_int32(a6, torch.zeros(4, 100, dtype=torch.uint8, device="cuda")[:, :96])
    with pytest.raises(RuntimeError):
        ops.encode_f6(torch.zeros(4, 100, dtype=torch.uint8, device="cuda"))
    s = torch.ones(4, 1, dtype=torch.float16, device="cuda")
    with pytest.raises(RuntimeError):
        ops.gemm_f6_dequant_o16(a6, a6, s[:2], s)
    assert ops.gemm_f6_int32(a6[:0], a6).shape == (0, 4)
    assert ops.encode_f6(torch.zeros(0, 64, dtype=torch.uint8, device="cuda")).shape == (0, 96)


@pytest.mark.parametrize("m,n,k", [(1, 128, 128), (33, 200, 640), (300, 384, 2048), (130, 520, 1152), (2048, 1024, 4096),
                                   (16, 256, 8 * 128), (16, 256, 9 * 128), (700, 4200, 17 * 128), (64, 256, 18 * 128),
                                   (130, 260, 11008)])
@pytest.mark.parametrize("a_token", [False, True])
def test_gemm_f6_group_scale_equals_the_int8_kernel(ops, m, n, k, a_token):
    """Group scales of 128 on the 6-bit instruction: same bits as the int8 group kernel (both fold
    float(sum_g) * scale in ascending g with one FMA), and within the path's tolerance of the oracle; K step
    counts around the eight-group blocks in which the scales are staged."""
    from oracle import gemm as G
    rng = np.random.default_rng(m + n + k + a_token)
    a = rng.integers(-8, 8, size=(m, k), dtype=np.int8)
    b = rng.integers(-8, 8, size=(n, k), dtype=np.int8)
    ng = k // 128
    sa = rng.uniform(0.01, 0.5, size=(m, 1 if a_token else ng)).astype(np.float16)
    sb = rng.uniform(0.005, 0.02, size=(n, ng)).astype(np.float16)
    ap, bp = dev(syn.pack_codes(a)), dev(syn.pack_codes(b))
    print(f"case f6 group m={m} n={n} k={k} a_token={a_token}", flush=True)
    d6 = ops.gemm_f6_dequant_o16_gs(ops.encode_f6(ap), ops.encode_f6(bp), dev(sa), dev(sb))
    d8 = ops.gemm_i4_dequant(ap, bp, dev(sa), dev(sb), 128)
    assert torch.equal(d6, d8)
    # the same scales from storage that is only 2-byte aligned (rows of scales are then fetched piece by piece)
    sa_odd, sb_odd = dev(np.concatenate([[0], sa.ravel()]).astype(np.float16))[1:].view(sa.shape), \
        dev(np.concatenate([[0], sb.ravel()]).astype(np.float16))[1:].view(sb.shape)
    assert torch.equal(ops.gemm_f6_dequant_o16_gs(ops.encode_f6(ap), ops.encode_f6(bp), sa_odd, sb_odd), d8)
    if m * n * k <= 300 * 520 * 2048:
        ref, _ = G.gemm_i4_dequant(syn.pack_codes(a), syn.pack_codes(b), sa, sb, group=128)
        assert np.allclose(host(d6).astype(np.float32), ref.astype(np.float32), rtol=1e-3, atol=1e-2)
        assert np.mean(host(d6).view(np.uint16) != ref.view(np.uint16)) < 2e-3


@pytest.mark.parametrize("m,k", [(1, 128), (7, 384), (33, 4096), (300, 11008), (2048, 1024)])
@pytest.mark.parametrize("had", [False, True])
def test_group_quantiser_writes_the_6bit_format(ops, m, k, had):
    """The group quantiser's 6-bit output mode: same scales, and the bytes that encode_f6 makes of its int4 codes."""
    rng = np.random.default_rng(m + k + had)
    x = (rng.standard_normal((m, k)) * rng.uniform(0.1, 8, (m, 1))).astype(np.float16)
    x[0, :128] = 0                                       # an all-zero group: scale 1, codes 0
    xd = dev(x)
    q4, s4 = (ops.hadamard_and_quantize_i4 if had else ops.quant_and_pack_i4)(xd.view(-1, 128), **({"scale_mul": 0.5} if had else {}))
    q6, s6 = ops.group_quantize_f6(xd, had, scale_mul=0.5 if had else 1.0)
    assert torch.equal(s6.view(-1), s4)
    assert torch.equal(q6, ops.encode_f6(q4.view(m, k // 2)))


@pytest.mark.parametrize("m,ns,k", [(2048, (4096, 1024, 1024), 4096), (300, (520, 136, 200, 64), 1024), (257, (129, 1), 256),
                                    (1024, (11008, 11008), 512)])
@pytest.mark.parametrize("scales", ["rows", "token_group", "group_group"])
def test_several_weight_matrices_in_one_launch(ops, m, ns, k, scales):
    """flh_gemm_f6_o16_multi: every output the bits of its own single call, for the three scale layouts."""
    rng = np.random.default_rng(m + k)
    ng = k // 128
    A6 = ops.encode_f6(dev(rng.integers(0, 256, size=(m, k // 2), dtype=np.uint8)))
    As = dev(rng.uniform(0.01, 0.1, size=(m, ng if scales == "group_group" else 1)).astype(np.float16))
    B6s = [ops.encode_f6(dev(rng.integers(0, 256, size=(n, k // 2), dtype=np.uint8))) for n in ns]
    Bss = [dev(rng.uniform(0.005, 0.02, size=(n, 1 if scales == "rows" else ng)).astype(np.float16)) for n in ns]
    got = ops.gemm_f6_dequant_multi(A6, B6s, As, Bss)
    single = ops.gemm_f6_dequant_o16 if scales == "rows" else ops.gemm_f6_dequant_o16_gs
    for D, B6, Bs in zip(got, B6s, Bss):
        assert torch.equal(D, single(A6, B6, As, Bs))
