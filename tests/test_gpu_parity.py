"""Parity of the HIP kernels (through the C ABI) with the CPU oracle on seeded inputs.
All tests need the MI355X: run with  -m gpu ."""
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


# ------------------------------------------------------------------ GEMM
GEMM_SHAPES = [(1, 128, 128), (16, 256, 512), (33, 100, 384), (256, 128, 128), (300, 520, 1024),
               (257, 129, 256), (16, 4096, 4096), (64, 1024, 11008),
               # decode kernel: 1 / 2 / 4 token tiles, odd number of 128-code steps, ragged N
               (5, 17, 640), (17, 4096, 4096), (48, 200, 1152),
               # prefill kernel, every tile shape: 64 x 64, 128 x 128, 256 x 128
               (65, 64, 256), (700, 4200, 512), (1024, 4096, 256), (2048, 4096, 256),
               # ... and the in-workgroup K split: two quads on 256 x 128 and 128 x 128, four on 64 x 64
               (2048, 4096, 1024), (1000, 4096, 512), (256, 4096, 1024), (2048, 4000, 768),
               # two tile sizes in one launch (whole waves of large tiles, small tiles for the rest)
               (2048, 11008, 256), (4096, 8320, 128)]


@pytest.mark.parametrize("m,n,k", GEMM_SHAPES)
def test_gemm_int32_bit_exact(ops, m, n, k):
    from oracle import gemm as G
    rng = np.random.default_rng(m * 7 + n * 3 + k)
    a = rng.integers(-8, 8, size=(m, k), dtype=np.int8)
    b = rng.integers(-8, 8, size=(n, k), dtype=np.int8)
    print(f"case int32 m={m} n={n} k={k}", flush=True)
    c = host(ops.gemm_i4_int32(dev(syn.pack_codes(a)), dev(syn.pack_codes(b))))
    assert np.array_equal(c, G.int_gemm(a, b))


@pytest.mark.parametrize("tile,ks", [(256, 1), (256, 2), (128, 1), (128, 2), (64, 1), (64, 2), (64, 4)])
@pytest.mark.parametrize("k", [1536, 1408])     # 12 resp. 11 K steps: even and uneven splits
def test_gemm_every_tile_and_k_split(ops, tile, ks, k, gemm_tuning):
    """The tuning overrides select each tile shape and in-workgroup K split directly; all of them
    must give the same exact integers and the same bit-exact fp16 outputs."""
    from oracle import gemm as G
    gemm_tuning(tile, ks)
    m, n = 300, 264
    rng = np.random.default_rng(tile + ks + k)
    a = rng.integers(-8, 8, size=(m, k), dtype=np.int8)
    b = rng.integers(-8, 8, size=(n, k), dtype=np.int8)
    ap, bp = syn.pack_codes(a), syn.pack_codes(b)
    print(f"case tile={tile} ks={ks} k={k}", flush=True)
    assert np.array_equal(host(ops.gemm_i4_int32(dev(ap), dev(bp))), G.int_gemm(a, b))
    sa = rng.uniform(0.01, 0.5, size=(m, 1)).astype(np.float16)
    sb = syn.weight_scales(n, 1, seed=k)
    d = host(ops.gemm_i4_dequant_o16(dev(ap), dev(bp), dev(sa), dev(sb)))
    ref, _ = G.gemm_i4_dequant(ap, bp, sa, sb)
    assert np.array_equal(d.view(np.uint16), ref.view(np.uint16))


def test_gemm_int32_extreme_codes(ops):
    k = 14336
    a = np.full((5, k), -8, dtype=np.int8)
    b = np.full((7, k), -8, dtype=np.int8)
    b[1::2] = 7
    c = host(ops.gemm_i4_int32(dev(syn.pack_codes(a)), dev(syn.pack_codes(b))))
    assert (c[:, 0::2] == 64 * k).all() and (c[:, 1::2] == -56 * k).all()


@pytest.mark.parametrize("m,n,k", GEMM_SHAPES)
def test_gemm_row_scale_bit_exact(ops, m, n, k):
    from oracle import gemm as G
    rng = np.random.default_rng(m + n + k)
    ap = syn.pack_codes(rng.integers(-8, 8, size=(m, k), dtype=np.int8))
    bp = syn.pack_codes(rng.integers(-8, 8, size=(n, k), dtype=np.int8))
    sa = rng.uniform(0.01, 0.5, size=(m, 1)).astype(np.float16)
    sb = syn.weight_scales(n, 1, seed=k)
    print(f"case rowscale m={m} n={n} k={k}", flush=True)
    d = host(ops.gemm_i4_dequant_o16(dev(ap), dev(bp), dev(sa), dev(sb)))
    ref, _ = G.gemm_i4_dequant(ap, bp, sa, sb)
    assert np.array_equal(d.view(np.uint16), ref.view(np.uint16))


@pytest.mark.parametrize("m,n,k", [(1, 1024, 2048), (16, 256, 512), (130, 200, 1024), (256, 256, 4096),
                                   (16, 64, 14336), (3, 50, 384), (17, 128, 1024)])
@pytest.mark.parametrize("a_token", [False, True])
def test_gemm_group_scale(ops, m, n, k, a_token):
    from oracle import gemm as G
    rng = np.random.default_rng(m * n + k)
    ap = syn.pack_codes(rng.integers(-8, 8, size=(m, k), dtype=np.int8))
    bp = syn.pack_codes(rng.integers(-8, 8, size=(n, k), dtype=np.int8))
    ng = k // 128
    sa = rng.uniform(0.01, 0.5, size=(m, 1 if a_token else ng)).astype(np.float16)
    sb = syn.weight_scales(n, ng, seed=k + 1)
    print(f"case group m={m} n={n} k={k} a_token={a_token}", flush=True)
    d = host(ops.gemm_i4_dequant_o16(dev(ap), dev(bp), dev(sa), dev(sb)))
    ref, _ = G.gemm_i4_dequant(ap, bp, sa, sb)
    # stated tolerance of the path: rtol 1e-3 / atol 1e-2 ; the fused-multiply-add order is
    # the reference kernel's, so the outputs equal the fused-multiply-add oracle bit for bit
    assert np.allclose(d.astype(np.float64), ref.astype(np.float64), rtol=1e-3, atol=1e-2)
    assert np.array_equal(d.view(np.uint16), ref.view(np.uint16))      # and in fact the same bits
    # reference-native signature with randn scales as in test/test_gemm_dequant.py:24-25
    if not a_token:
        sa = rng.standard_normal((m, ng)).astype(np.float16)
        sb = rng.standard_normal((n, ng)).astype(np.float16)
        d = host(ops.gemm_i4_dequant_o16_gs(dev(ap), dev(bp), dev(sa), dev(sb), 128))
        ref, _ = G.gemm_i4_dequant(ap, bp, sa, sb)
        assert np.allclose(d.astype(np.float64), ref.astype(np.float64), rtol=1e-3, atol=1e-2)


@pytest.mark.parametrize("gs", [32, 64, 128])
@pytest.mark.parametrize("m,n,k", [(1, 128, 128), (33, 200, 640), (300, 384, 2048), (2048, 2048, 512)])
def test_gemm_group_sizes(ops, gs, m, n, k):
    """gemm_i4_dequant_o16_gs with every group size the reference accepts
    (flh_cuda_bindings.cpp:254-299); one activation scale per token is also exercised."""
    from oracle import gemm as G
    rng = np.random.default_rng(gs + m + n + k)
    ap = syn.pack_codes(rng.integers(-8, 8, size=(m, k), dtype=np.int8))
    bp = syn.pack_codes(rng.integers(-8, 8, size=(n, k), dtype=np.int8))
    ng = k // gs
    sa = rng.uniform(0.01, 0.5, size=(m, ng)).astype(np.float16)
    sb = syn.weight_scales(n, ng, seed=k + gs)
    print(f"case group-size gs={gs} m={m} n={n} k={k}", flush=True)
    d = host(ops.gemm_i4_dequant_o16_gs(dev(ap), dev(bp), dev(sa), dev(sb), gs))
    ref, _ = G.gemm_i4_dequant(ap, bp, sa, sb, gs)
    assert np.allclose(d.astype(np.float64), ref.astype(np.float64), rtol=1e-3, atol=1e-2)
    assert np.array_equal(d.view(np.uint16), ref.view(np.uint16))      # and in fact the same bits
    # unit scales: the result is the integer contraction itself, any group size
    one_a, one_b = np.ones((m, ng), np.float16), np.ones((n, ng), np.float16)
    d = host(ops.gemm_i4_dequant_o16_gs(dev(ap), dev(bp), dev(one_a), dev(one_b), gs))
    from oracle.pack import unpack_i4
    exact = G.int_gemm(unpack_i4(ap), unpack_i4(bp)).astype(np.float32).astype(np.float16)
    assert np.array_equal(d.view(np.uint16), exact.view(np.uint16))
    # per-token activation scale with grouped weight scales
    sa1 = rng.uniform(0.01, 0.5, size=(m, 1)).astype(np.float16)
    d = host(ops.gemm_i4_dequant(dev(ap), dev(bp), dev(sa1), dev(sb), gs))
    ref, _ = G.gemm_i4_dequant(ap, bp, sa1, sb, gs)
    assert np.allclose(d.astype(np.float64), ref.astype(np.float64), rtol=1e-3, atol=1e-2)
    assert np.array_equal(d.view(np.uint16), ref.view(np.uint16))


@pytest.mark.parametrize("m", [4, 200])
def test_gemm_group_activations_per_channel_weights(ops, m):
    """Group-scaled activations against one weight scale per output channel (the mirror image of the
    per-token x group case), decode and prefill kernels."""
    from oracle import gemm as G
    n, k, gs = 136, 1024, 128
    rng = np.random.default_rng(m)
    ap = syn.pack_codes(rng.integers(-8, 8, size=(m, k), dtype=np.int8))
    bp = syn.pack_codes(rng.integers(-8, 8, size=(n, k), dtype=np.int8))
    sa = rng.uniform(0.01, 0.5, size=(m, k // gs)).astype(np.float16)
    sb = syn.weight_scales(n, 1, seed=3)
    d = host(ops.gemm_i4_dequant(dev(ap), dev(bp), dev(sa), dev(sb), gs))
    ref, _ = G.gemm_i4_dequant(ap, bp, sa, sb, gs)
    assert np.allclose(d.astype(np.float64), ref.astype(np.float64), rtol=1e-3, atol=1e-2)
    assert np.array_equal(d.view(np.uint16), ref.view(np.uint16))      # and in fact the same bits


def test_gemm_unit_scales_give_integers(ops):
    rng = np.random.default_rng(9)
    m, n, k = 40, 136, 256
    a = rng.integers(-8, 8, size=(m, k), dtype=np.int8)
    b = rng.integers(-8, 8, size=(n, k), dtype=np.int8)
    one = lambda r, c: dev(np.ones((r, c), dtype=np.float16))
    exact = a.astype(np.int64) @ b.astype(np.int64).T
    d = host(ops.gemm_i4_dequant_o16(dev(syn.pack_codes(a)), dev(syn.pack_codes(b)), one(m, 2), one(n, 2)))
    assert np.array_equal(d.astype(np.int64), exact)
    d = host(ops.gemm_i4_dequant_o16(dev(syn.pack_codes(a)), dev(syn.pack_codes(b)), one(m, 1), one(n, 1)))
    assert np.array_equal(d.astype(np.int64), exact)


def test_gemm_argument_errors(ops):
    a = torch.zeros((4, 64), dtype=torch.uint8, device="cuda")
    s = torch.ones((4, 1), dtype=torch.float16, device="cuda")
    with pytest.raises(RuntimeError):
        ops.gemm_i4_dequant_o16(a, a.to(torch.int8), s, s)
    with pytest.raises(RuntimeError):
        ops.gemm_i4_dequant_o16(a, a[:, :32].contiguous(), s, s)
    with pytest.raises(RuntimeError):
        ops.gemm_i4_dequant_o16(a[:, :48].contiguous(), a[:, :48].contiguous(), s, s)   # K = 96
    with pytest.raises(RuntimeError):
        ops.gemm_i4_dequant_o16(a.cpu(), a, s, s)
    with pytest.raises(RuntimeError):
        ops.gemm_i4_dequant_o16_gs(a, a, s, s, 48)
    assert ops.gemm_i4_dequant_o16(a[:0], a, s[:0], s).shape == (0, 4)


# ------------------------------------------------------------------ group kernels (reference kernel arithmetic)
@pytest.mark.parametrize("g", [32, 64, 128])
@pytest.mark.parametrize("had", [True, False])
@pytest.mark.parametrize("rows", [1, 7, 64, 1000])
def test_group_quant_bit_exact(ops, g, had, rows):
    from oracle import quant as Q
    from oracle.pack import pack_i4
    x = syn.activations(rows, g, seed=rows + g)
    x[rows // 2] = 0                     # an all-zero row
    if rows > 3:
        x[3] = np.float16(6e-6)          # scale below the kernel's 1e-6 threshold -> 1.0
    print(f"case group_quant g={g} had={had} rows={rows}", flush=True)
    xd = dev(x)
    if g == 128:
        q, s = (ops.hadamard_and_quantize_i4 if had else ops.quant_and_pack_i4)(xd)
    else:
        q, s = (ops.hadamard_and_quantize_i4_gs if had else ops.quant_and_pack_i4_gs)(xd, g)
    qr, sr, _ = Q.kernel_had_and_quant(x, g, had)
    assert np.array_equal(host(s).view(np.uint16), sr.view(np.uint16))
    assert np.array_equal(host(q), pack_i4(qr))


def test_group_quant_every_row_maximum(ops):
    """One row for every positive finite fp16 value as the row maximum (subnormals included), the other values
    spread over [-m, m]: the kernels take the scale as m * fl32(1/7) and the quotients through the hardware
    reciprocal; codes and scales must still be the oracle's (exact division) for every possible scale."""
    from oracle import quant as Q
    from oracle.pack import pack_i4
    m = np.arange(1, 0x7C00, dtype=np.uint16).view(np.float16)
    rng = np.random.default_rng(5)
    x = (rng.uniform(-1, 1, size=(m.size, 32)).astype(np.float32) * m.astype(np.float32)[:, None]).astype(np.float16)
    x[:, 0] = m
    x[:, 1] = -m
    x[:, 2:9] = (m.astype(np.float32)[:, None] * ((np.arange(1, 8, dtype=np.float32) - 0.5) / 7.0)).astype(np.float16)  # near the rounding ties
    q, s = ops.quant_and_pack_i4_gs(dev(x), 32)
    qr, sr, _ = Q.kernel_had_and_quant(x, 32, False)
    assert np.array_equal(host(s).view(np.uint16), sr.view(np.uint16))
    assert np.array_equal(host(q), pack_i4(qr))
    # whole-row path (one wave per row): the same maxima, rows of 512
    x512 = np.tile(x, (1, 16))
    q, s = ops.rotate_and_quantize_i4(dev(x512), hadamard=False)
    qr, sr = Q.quantize_rows(x512)
    assert np.array_equal(host(s).reshape(-1).view(np.uint16), sr.reshape(-1).view(np.uint16))
    assert np.array_equal(host(q), pack_i4(qr))


@pytest.mark.parametrize("g", [32, 64, 128])
def test_fwht_inplace_bit_exact(ops, g):
    from oracle import hadamard as H
    x = syn.activations(333, g, seed=g)
    xd = dev(x)
    fn = {32: ops.hadamard_transform_32_half, 64: ops.hadamard_transform_64_half, 128: ops.hadamard_transform_half}[g]
    out = fn(xd)
    assert out.data_ptr() == xd.data_ptr()
    assert np.array_equal(host(xd).view(np.uint16), H.fwht_butterfly(x, np.float16, g).view(np.uint16))
    with pytest.raises(RuntimeError):
        fn(dev(x[:, : g // 2]))


# ------------------------------------------------------------------ whole-row rotate + quantise
@pytest.mark.parametrize("k", [512, 1024, 2048, 4096, 8192])
@pytest.mark.parametrize("m", [1, 5, 64])
def test_rotate_quant_pow2_bit_exact(ops, m, k):
    from oracle import linear as L
    x = syn.activations(m, k, seed=m + k)
    if m > 2:
        x[1] = 0
    print(f"case rotate_quant m={m} k={k}", flush=True)
    q, s, y = ops.rotate_and_quantize_i4(dev(x), return_rotated=True)
    qr, sr, yr = L.rotate_and_quantize(x, "f32")
    assert np.array_equal(host(y).view(np.uint16), yr.view(np.uint16))
    assert np.array_equal(host(s).view(np.uint16), sr.view(np.uint16))
    assert np.array_equal(host(q), qr)
    # mismatch rate against the exactly rounded (float64) transform is reported, not required to be 0
    qe, _, _ = L.rotate_and_quantize(x, "exact")
    rate = (host(q) != qe).mean()
    print(f"  byte mismatch rate vs exact transform: {rate:.2e}", flush=True)
    assert rate < 2e-3


@pytest.mark.parametrize("m", [1, 3, 512])
def test_rotate_quant_4096_few_rows_bit_exact(ops, m):
    """Up to 512 rows of 4096 take the kernel with eight waves per row: same bytes as the oracle and as the
    wave-per-row kernel (which a call with more rows takes) on the same rows; zero, tiny and outlier rows."""
    from oracle import linear as L
    x = syn.activations(1024, 4096, seed=77 + m)
    x[1] = 0
    x[2] = (x[2].astype(np.float32) * 1e-6).astype(np.float16)      # subnormal values: the clamping path
    print(f"case rotate_quant few rows m={m}", flush=True)
    q, s = ops.rotate_and_quantize_i4(dev(x[:m]), hadamard="exact")
    qr, sr, _ = L.rotate_and_quantize(x[:m], "f32")
    assert np.array_equal(host(s).view(np.uint16), sr.view(np.uint16))
    assert np.array_equal(host(q), qr)
    qw, sw = ops.rotate_and_quantize_i4(dev(x), hadamard="exact")
    assert np.array_equal(host(q), host(qw)[:m]) and np.array_equal(host(s).view(np.uint16), host(sw)[:m].view(np.uint16))


def test_rotate_quant_golden_4096(ops, golden):
    x = golden["fo_pt_h_4096_x"]
    q, s = ops.rotate_and_quantize_i4(dev(x))
    # reference output (float64 transform): scales equal, codes equal up to rare double roundings
    assert np.array_equal(host(s).reshape(-1), golden["fo_pt_h_4096_scale"].reshape(-1))
    assert (host(q) != golden["fo_pt_h_4096_packed"]).mean() < 2e-3


@pytest.mark.parametrize("k", [512, 4096])
@pytest.mark.parametrize("clip", [1.0, 0.9])
def test_quant_only_and_clip(ops, k, clip):
    from oracle import linear as L
    x = syn.activations(9, k, seed=k)
    for had in (False, True):
        q, s = ops.rotate_and_quantize_i4(dev(x), hadamard=had, clip_ratio=clip)
        qr, sr, _ = L.rotate_and_quantize(x, "f32" if had else "none", None, clip)
        assert np.array_equal(host(s).view(np.uint16), sr.view(np.uint16))
        assert np.array_equal(host(q), qr)


@pytest.mark.parametrize("k,hg,sg", [(256, 0, 0), (64, 0, 0), (1024, 128, 128), (512, 64, 64), (4096, 0, 128),
                                       (16384, 0, 0), (1024, 128, 0)])
def test_rotate_quant_generic_paths(ops, k, hg, sg):
    from oracle import hadamard as H
    from oracle import quant as Q
    from oracle.pack import pack_i4
    x = syn.activations(6, k, seed=k + hg + sg)
    q, s, y = ops.rotate_and_quantize_i4(dev(x), had_group=hg, scale_group=sg, clip_ratio=0.95, return_rotated=True)
    yr = H.had_transform_f32(x, hg if hg else None)
    qr, sr = Q.quantize_rows(yr, sg if sg else None, 0.95)
    assert np.array_equal(host(y).view(np.uint16), yr.view(np.uint16))
    assert np.array_equal(host(s).view(np.uint16), sr.view(np.uint16))
    assert np.array_equal(host(q), pack_i4(qr))


@pytest.mark.parametrize("k", [28 * 16, 172 * 16, 14336, 11008, 12 * 8, 40 * 128])
def test_rotate_quant_non_pow2(ops, k):
    from oracle import hadamard as H
    from oracle import quant as Q
    from oracle.pack import pack_i4
    rng = np.random.default_rng(k)
    # integer data: every summation order gives the same float32 result -> pins the wiring
    xi = rng.integers(-3, 4, size=(3, k)).astype(np.float16)
    q, s, y = ops.rotate_and_quantize_i4(dev(xi), return_rotated=True)
    yr = H.hadamard_full(xi, exact=True)
    assert np.array_equal(host(y).view(np.uint16), yr.view(np.uint16))
    qr, sr = Q.quantize_rows(yr)
    assert np.array_equal(host(s).view(np.uint16), sr.view(np.uint16)) and np.array_equal(host(q), pack_i4(qr))
    # random data: the dense factor's summation order is not defined by the reference
    x = syn.activations(4, k, seed=k)
    q, s, y = ops.rotate_and_quantize_i4(dev(x), return_rotated=True)
    ye = H.hadamard_full(x, exact=True)
    ulp_off = (host(y).view(np.uint16) != ye.view(np.uint16)).mean()
    qe, se = Q.quantize_rows(ye)
    rate = (host(q) != pack_i4(qe)).mean()
    print(f"k={k}: rotated fp16 values differing from exact: {ulp_off:.2e}, packed byte mismatch: {rate:.2e}", flush=True)
    assert ulp_off < 5e-3 and rate < 5e-3
    assert np.allclose(host(s).astype(np.float32), se.astype(np.float32), rtol=2e-3)


@pytest.mark.parametrize("k", [172 * 16, 11008, 14336, 28 * 16, 40 * 128, 12 * 8, 156 * 32, 108 * 64])
def test_rotate_quant_non_pow2_summation_order(ops, k):
    """The dense factor's summation order is this build's own choice (the reference's is whatever its BLAS
    does): float32, sequential over the columns of the literal matrix.  The kernel must keep exactly that,
    whatever it does to be fast."""
    from oracle import hadamard as H
    x = np.random.default_rng(k).standard_normal((5, k)).astype(np.float16)
    kd, p = H.get_hadK(k)
    blocks = H.fwht_butterfly(x, np.float32, p).reshape(5, kd, p)
    h = H.had_literal(kd).astype(np.float32)
    acc = np.zeros_like(blocks)
    for jj in range(kd):
        acc = acc + h[:, jj][None, :, None] * blocks[:, jj][:, None, :]
    want = (acc.reshape(5, k) / np.sqrt(np.float32(k))).astype(np.float16)
    _, _, y = ops.rotate_and_quantize_i4(dev(x), "exact", return_rotated=True)
    assert np.array_equal(host(y).view(np.uint16), want.view(np.uint16))


# ------------------------------------------------------------------ matrix-core rotation mode
@pytest.mark.parametrize("k", [4096, 11008, 14336])
def test_rotate_quant_fast_mode_integer_data_bit_exact(ops, k):
    """Integer inputs make every partial sum exact in any order and any intermediate precision the
    kernel uses, so the matrix-core path must agree with the exact transform bit for bit: this
    pins the operand layouts, the dense factors (had172, had28 (x) H8) and the nibble packing."""
    from oracle import hadamard as H
    from oracle import quant as Q
    from oracle.pack import pack_i4
    rng = np.random.default_rng(k)
    for m in (1, 6, 300):
        print(f"case fast-mode integer m={m} k={k}", flush=True)
        xi = rng.integers(-3, 4, size=(m, k)).astype(np.float16)
        xi[m // 2] = 0                                        # an all-zero row: scale 1, codes 0
        q, s = ops.rotate_and_quantize_i4(dev(xi), hadamard="fast")
        qe, se = Q.quantize_rows(H.hadamard_full(xi, exact=True))
        assert np.array_equal(host(s).reshape(-1).view(np.uint16), se.reshape(-1).view(np.uint16))
        assert np.array_equal(host(q), pack_i4(qe))


@pytest.mark.parametrize("k,code_rate,scale_rate", [(4096, 2e-5, 5e-3), (11008, 2e-3, 0.25), (14336, 2e-3, 0.25)])
@pytest.mark.parametrize("clip", [1.0, 0.9])
def test_rotate_quant_fast_mode_mismatch_rate(ops, k, code_rate, scale_rate, clip):
    """Random activations with outlier channels: the matrix-core path is not bit-exact; its codes
    may differ from the exactly rounded transform by one step at a small measured rate, and a scale
    by one or two fp16 ulps (K = 4096 keeps 22 bits of the intermediate, the dense-factor sizes 11)."""
    from oracle import hadamard as H
    from oracle import quant as Q
    from oracle.pack import unpack_i4
    x = syn.activations(96, k, seed=k + 7)
    q, s = ops.rotate_and_quantize_i4(dev(x), hadamard="fast", clip_ratio=clip)
    qe, se = Q.quantize_rows(H.hadamard_full(x, exact=True), None, clip)
    codes = unpack_i4(host(q))
    diff = np.abs(codes.astype(np.int32) - qe.astype(np.int32))
    s_bits, se_bits = host(s).reshape(-1).view(np.uint16).astype(np.int32), se.reshape(-1).view(np.uint16).astype(np.int32)
    print(f"k={k} clip={clip}: code mismatch rate {np.mean(diff != 0):.2e} (max step {diff.max()}), "
          f"scale mismatch rate {np.mean(s_bits != se_bits):.2e}", flush=True)
    assert diff.max() <= 1 and np.mean(diff != 0) < code_rate
    # a row maximum one ulp off moves max / 7 by up to two ulps when the quotient sits high in its binade
    assert np.abs(s_bits - se_bits).max() <= 2 and np.mean(s_bits != se_bits) <= scale_rate


def test_rotate_quant_fast_mode_feeds_gemm(ops):
    """End to end at the down-projection shape: fast-mode codes through the int4 GEMM stay within
    the fp16 output tolerance of the exact-mode result."""
    m, n, k = 64, 256, 11008
    x = syn.activations(m, k, seed=3)
    w = dev(syn.pack_codes(syn.weight_codes(n, k, seed=4)))
    sw = dev(syn.weight_scales(n, 1, seed=5))
    outs = []
    for mode in ("exact", "fast"):
        q, s = ops.rotate_and_quantize_i4(dev(x), hadamard=mode)
        outs.append(host(ops.gemm_i4_dequant_o16(q, w, s, sw)).astype(np.float32))
    scale = np.abs(outs[0]).max()
    assert np.abs(outs[0] - outs[1]).max() <= 2e-2 * scale


def test_rotate_quant_fast_mode_falls_back(ops):
    """Shapes the matrix-core kernels do not cover run the float32-butterfly kernels."""
    from oracle import linear as L
    x = syn.activations(5, 2048, seed=11)
    q, s = ops.rotate_and_quantize_i4(dev(x), hadamard="fast")
    qr, sr, _ = L.rotate_and_quantize(x, "f32")
    assert np.array_equal(host(q), qr) and np.array_equal(host(s).view(np.uint16), sr.view(np.uint16))


def test_gemm_random_shapes_sweep(ops):
    """Forty random (M, N, K) with ragged M and N, every K step count from 1 to 16: int32 sums, the
    per-token x per-channel epilogue and the 6-bit path, all bit for bit against the oracle."""
    from oracle import gemm as G
    rng = np.random.default_rng(2024)
    for case in range(40):
        m = int(rng.integers(1, 600))
        n = int(rng.integers(1, 600))
        k = 128 * int(rng.integers(1, 17))
        a = rng.integers(-8, 8, size=(m, k), dtype=np.int8)
        b = rng.integers(-8, 8, size=(n, k), dtype=np.int8)
        sa = rng.uniform(0.01, 0.5, size=(m, 1)).astype(np.float16)
        sb = rng.uniform(0.005, 0.02, size=(n, 1)).astype(np.float16)
        ap, bp = dev(syn.pack_codes(a)), dev(syn.pack_codes(b))
        print(f"case sweep {case}: m={m} n={n} k={k}", flush=True)
        want = G.int_gemm(a, b)
        assert np.array_equal(host(ops.gemm_i4_int32(ap, bp)), want)
        ref, _ = G.gemm_i4_dequant(syn.pack_codes(a), syn.pack_codes(b), sa, sb)
        d = host(ops.gemm_i4_dequant_o16(ap, bp, dev(sa), dev(sb)))
        assert np.array_equal(d.view(np.uint16), ref.view(np.uint16))
        a6, b6 = ops.encode_f6(ap), ops.encode_f6(bp)
        assert np.array_equal(host(ops.gemm_f6_int32(a6, b6)), want)
        d6 = host(ops.gemm_f6_dequant_o16(a6, b6, dev(sa), dev(sb)))
        assert np.array_equal(d6.view(np.uint16), ref.view(np.uint16))


def test_gemm_group_scale_random_shapes_sweep(ops):
    """Twenty random shapes x group sizes for the group-scale epilogue (both scale layouts), within the
    tolerance the path specifies and with exact agreement on unit scales."""
    from oracle import gemm as G
    rng = np.random.default_rng(77)
    for case in range(20):
        g = int(rng.choice([32, 64, 128]))
        m, n = int(rng.integers(1, 300)), int(rng.integers(1, 300))
        k = 128 * int(rng.integers(1, 9))
        a = rng.integers(-8, 8, size=(m, k), dtype=np.int8)
        b = rng.integers(-8, 8, size=(n, k), dtype=np.int8)
        sa = rng.uniform(0.01, 0.5, size=(m, k // g)).astype(np.float16)
        sb = rng.uniform(0.005, 0.02, size=(n, k // g)).astype(np.float16)
        ap, bp = syn.pack_codes(a), syn.pack_codes(b)
        print(f"case group sweep {case}: m={m} n={n} k={k} g={g}", flush=True)
        ref, _ = G.gemm_i4_dequant(ap, bp, sa, sb, group=g)
        d = host(ops.gemm_i4_dequant_o16_gs(dev(ap), dev(bp), dev(sa), dev(sb), g))
        assert np.allclose(d.astype(np.float32), ref.astype(np.float32), rtol=1e-3, atol=1e-2)
        ones_a, ones_b = np.ones_like(sa), np.ones_like(sb)
        d1 = host(ops.gemm_i4_dequant_o16_gs(dev(ap), dev(bp), dev(ones_a), dev(ones_b), g))
        exact = G.int_gemm(a, b).astype(np.float32).astype(np.float16)
        assert np.array_equal(d1.view(np.uint16), exact.view(np.uint16))


@pytest.mark.parametrize("k", [11008, 14336])
def test_rotate_quant_fast_mode_short_and_long_batches_agree(ops, k):
    """Short batches run the matrix-core rotation with one row per workgroup and the output tiles split over
    the wave pairs, long batches with four rows per workgroup: the same row must give the same bytes either way
    (decode and prefill of one token stream must not disagree)."""
    x = dev(syn.activations(600, k, seed=k))
    q_long, s_long = ops.rotate_and_quantize_i4(x, hadamard="fast")             # 600 rows: unsplit
    for lo, hi in ((0, 1), (1, 17), (17, 273), (344, 600)):                     # 1, 16, 256, 256 rows: split
        q, s = ops.rotate_and_quantize_i4(x[lo:hi].contiguous(), hadamard="fast")
        assert torch.equal(q, q_long[lo:hi]) and torch.equal(s, s_long[lo:hi]), (lo, hi)
