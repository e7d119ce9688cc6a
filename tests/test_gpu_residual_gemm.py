"""The GEMM launches that add a decoder layer's residual in their epilogue (flh_gemm_i4_add_o16, flh_gemm_f6_add_o16):
D = fp16(residual + fp16(gemm)) must be the oracle GEMM's fp16 output followed by numpy's fp16 addition, bit for bit,
on every kernel the shape can select -- prefill tiles and K splits, the decode kernel, per-row and group scales, ragged
and odd N -- and in place on the residual."""
import numpy as np
import pytest
import torch

from flh_amd import synthetic as syn

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    import flh_amd
    return flh_amd._CUDA


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    return t.detach().cpu().numpy()


def case(m, n, k, seed, a_cols, b_cols, group):
    rng = np.random.default_rng(seed)
    ap = syn.pack_codes(rng.integers(-8, 8, size=(m, k), dtype=np.int8))
    bp = syn.pack_codes(rng.integers(-8, 8, size=(n, k), dtype=np.int8))
    ng = k // group
    sa = rng.uniform(0.01, 0.1, size=(m, ng if a_cols > 1 else 1)).astype(np.float16)
    sb = syn.weight_scales(n, ng if b_cols > 1 else 1, seed + 1)
    res = (rng.standard_normal((m, n)) * 2).astype(np.float16)
    return ap, bp, sa, sb, res


def expected(ap, bp, sa, sb, res, group):
    from oracle import gemm as G
    d, _ = G.gemm_i4_dequant(ap, bp, sa, sb, group)
    return (d + res).astype(np.float16)          # numpy adds fp16 values with one rounding


SHAPES = [(1, 4096, 4096), (8, 512, 1024), (16, 100, 256), (64, 264, 512), (65, 64, 256), (300, 264, 1024),
          (130, 1000, 512), (1024, 704, 384), (70, 36, 128), (257, 515, 640)]


@pytest.mark.parametrize("m,n,k", SHAPES)
@pytest.mark.parametrize("scales", ["row", "token_group", "group_group"])
def test_residual_epilogue_against_the_oracle(ops, m, n, k, scales):
    a_cols, b_cols = {"row": (1, 1), "token_group": (1, 2), "group_group": (2, 2)}[scales]
    print(f"case residual gemm m={m} n={n} k={k} {scales}", flush=True)
    ap, bp, sa, sb, res = case(m, n, k, m + n + k, a_cols, b_cols, 128)
    want = expected(ap, bp, sa, sb, res, 128)
    r = dev(res)
    got = ops.gemm_i4_dequant_add(dev(ap), dev(bp), dev(sa), dev(sb), r, 128)
    assert np.array_equal(host(got).view(np.uint16), want.view(np.uint16))
    assert np.array_equal(host(r).view(np.uint16), res.view(np.uint16))          # the residual itself is left alone
    # in place on the residual stream
    same = ops.gemm_i4_dequant_add(dev(ap), dev(bp), dev(sa), dev(sb), r, 128, out=r)
    assert same.data_ptr() == r.data_ptr()
    assert np.array_equal(host(r).view(np.uint16), want.view(np.uint16))
    # the launch without a residual is unchanged: torch's fp16 addition on its output gives the same bits
    plain = ops.gemm_i4_dequant(dev(ap), dev(bp), dev(sa), dev(sb), 128)
    assert np.array_equal(host(plain + dev(res)).view(np.uint16), want.view(np.uint16))


@pytest.mark.parametrize("group", [32, 64])
def test_residual_epilogue_small_groups(ops, group):
    print(f"case residual gemm group={group}", flush=True)
    ap, bp, sa, sb, res = case(200, 264, 512, group, 2, 2, group)
    want = expected(ap, bp, sa, sb, res, group)
    got = ops.gemm_i4_dequant_add(dev(ap), dev(bp), dev(sa), dev(sb), dev(res), group)
    assert np.array_equal(host(got).view(np.uint16), want.view(np.uint16))


@pytest.mark.parametrize("tile,ks", [(256, 1), (256, 2), (128, 1), (128, 2), (64, 1), (64, 2), (64, 4)])
def test_residual_epilogue_every_tile(ops, tile, ks, gemm_tuning):
    print(f"case residual gemm tile={tile} ks={ks}", flush=True)
    ap, bp, sa, sb, res = case(300, 264, 1408, 7, 1, 1, 128)
    want = expected(ap, bp, sa, sb, res, 128)
    gemm_tuning(tile, ks)
    got = ops.gemm_i4_dequant_add(dev(ap), dev(bp), dev(sa), dev(sb), dev(res), 128)
    gemm_tuning(0)
    assert np.array_equal(host(got).view(np.uint16), want.view(np.uint16))


@pytest.mark.parametrize("m,n,k", [(65, 64, 256), (300, 264, 1024), (130, 1000, 512), (2048, 1408, 512), (40, 36, 128)])
@pytest.mark.parametrize("scales", ["row", "token_group", "group_group"])
def test_residual_epilogue_on_the_six_bit_instruction(ops, m, n, k, scales):
    a_cols, b_cols = {"row": (1, 1), "token_group": (1, 2), "group_group": (2, 2)}[scales]
    print(f"case residual gemm f6 m={m} n={n} k={k} {scales}", flush=True)
    ap, bp, sa, sb, res = case(m, n, k, m + n + k + 1, a_cols, b_cols, 128)
    want = expected(ap, bp, sa, sb, res, 128)
    a6, b6 = ops.encode_f6(dev(ap)), ops.encode_f6(dev(bp))
    r = dev(res)
    got = ops.gemm_f6_dequant_add(a6, b6, dev(sa), dev(sb), r)
    assert np.array_equal(host(got).view(np.uint16), want.view(np.uint16))
    ops.gemm_f6_dequant_add(a6, b6, dev(sa), dev(sb), r, out=r)
    assert np.array_equal(host(r).view(np.uint16), want.view(np.uint16))


def test_residual_epilogue_argument_checks(ops):
    ap, bp, sa, sb, res = case(70, 64, 128, 3, 1, 1, 128)
    with pytest.raises(RuntimeError):
        ops.gemm_i4_dequant_add(dev(ap), dev(bp), dev(sa), dev(sb), dev(res[:, :32]), 128)
    with pytest.raises(RuntimeError):
        ops.gemm_i4_dequant_add(dev(ap), dev(bp), dev(sa), dev(sb), dev(res).float(), 128)


@pytest.mark.parametrize("six_bit", [False, True])
@pytest.mark.parametrize("group,bias", [(-1, False), (128, False), (128, True)])
def test_linear_module_residual_argument(ops, six_bit, group, bias):
    """LinearFLH.forward(..., residual=r) == r + LinearFLH.forward(...), bit for bit, on both matrix instructions."""
    from flh_amd.nn import LinearFLH
    torch.manual_seed(5)
    lin = torch.nn.Linear(512, 384, bias=bias).half().cuda()
    layer = LinearFLH.from_float(lin, weight_group_size=group)
    layer.six_bit = six_bit
    x = torch.randn(3, 100, 512, device="cuda").half()
    q, s = ops.rotate_and_quantize_i4(x.view(-1, 512), hadamard="exact")
    q, s = q.view(3, 100, -1), s.view(3, 100, 1)
    r = torch.randn(3, 100, 384, device="cuda").half()
    want = r + layer(q, s, None, x_is_packed=True)
    got = layer(q, s, None, x_is_packed=True, residual=r)
    assert got.shape == want.shape and torch.equal(got, want)
