"""Parity at the full sizes of the benchmark configurations (Llama-2-7B and Llama-3-8B linears, M = 2048 prefill and
M = 1 / 16 decode).  Where the oracle would take too long on the whole output, size-independent properties carry the
check: row and column checksums of the integer contraction (exact, O(MK + NK) on the host), a random sample of
complete rows against the oracle, and invariants of symmetric int4 quantisation."""
import numpy as np
import pytest
import torch

from flh_amd import synthetic as syn

pytestmark = pytest.mark.gpu

LLAMA2 = [(4096, 4096), (11008, 4096), (4096, 11008)]
LLAMA3 = [(4096, 4096), (1024, 4096), (14336, 4096), (4096, 14336)]


@pytest.fixture(scope="module")
def ops():
    from flh_amd import _ops
    return _ops


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    return t.detach().cpu().numpy()


def codes(rows, k, seed):
    return np.random.default_rng(seed).integers(-8, 8, size=(rows, k), dtype=np.int8)


@pytest.mark.parametrize("n,k", sorted(set(LLAMA2 + LLAMA3)))
def test_prefill_int32_checksums_and_sampled_rows(ops, n, k):
    from oracle import gemm as G
    m = 2048
    a, b = codes(m, k, n + k), codes(n, k, n + k + 1)
    print(f"case full-size int32 m={m} n={n} k={k}", flush=True)
    c = host(ops.gemm_i4_int32(dev(syn.pack_codes(a)), dev(syn.pack_codes(b)))).astype(np.int64)
    a64, b64 = a.astype(np.int64), b.astype(np.int64)
    assert np.array_equal(c.sum(axis=1), a64 @ b64.sum(axis=0))        # row checksums: sum_n C[m, n]
    assert np.array_equal(c.sum(axis=0), b64 @ a64.sum(axis=0))        # column checksums: sum_m C[m, n]
    rows = np.random.default_rng(0).choice(m, size=24, replace=False)
    assert np.array_equal(c[rows], G.int_gemm(a[rows], b))


@pytest.mark.parametrize("n,k", LLAMA2)
def test_prefill_row_scale_sampled_rows_bit_exact(ops, n, k):
    from oracle import gemm as G
    m = 2048
    ap, bp = syn.pack_codes(codes(m, k, 3 * n + k)), syn.pack_codes(codes(n, k, 5 * n + k))
    rng = np.random.default_rng(n)
    sa = rng.uniform(0.01, 0.5, size=(m, 1)).astype(np.float16)
    sb = syn.weight_scales(n, 1, seed=k)
    print(f"case full-size row-scale m={m} n={n} k={k}", flush=True)
    d = host(ops.gemm_i4_dequant_o16(dev(ap), dev(bp), dev(sa), dev(sb)))
    rows = rng.choice(m, size=32, replace=False)
    ref, _ = G.gemm_i4_dequant(ap[rows], bp, sa[rows], sb)
    assert np.array_equal(d[rows].view(np.uint16), ref.view(np.uint16))
    assert np.isfinite(d.astype(np.float32)).all()


@pytest.mark.parametrize("n,k", LLAMA3)
@pytest.mark.parametrize("a_token", [True, False])
def test_prefill_group_scale_sampled_rows(ops, n, k, a_token):
    """Llama-3 shapes, weight scales per group of 128; activations per token or per group."""
    from oracle import gemm as G
    m, ng = 2048, k // 128
    ap, bp = syn.pack_codes(codes(m, k, n + 7 * k)), syn.pack_codes(codes(n, k, n + 9 * k))
    rng = np.random.default_rng(k)
    sa = rng.uniform(0.01, 0.5, size=(m, 1 if a_token else ng)).astype(np.float16)
    sb = syn.weight_scales(n, ng, seed=n)
    print(f"case full-size group-scale m={m} n={n} k={k} a_token={a_token}", flush=True)
    d = host(ops.gemm_i4_dequant_o16(dev(ap), dev(bp), dev(sa), dev(sb)))
    rows = rng.choice(m, size=16, replace=False)
    ref, _ = G.gemm_i4_dequant(ap[rows], bp, sa[rows], sb)
    assert np.allclose(d[rows].astype(np.float64), ref.astype(np.float64), rtol=1e-3, atol=1e-2)
    assert np.array_equal(d[rows].view(np.uint16), ref.view(np.uint16))


@pytest.mark.parametrize("m", [1, 16])
@pytest.mark.parametrize("n,k", sorted(set(LLAMA2 + LLAMA3)))
def test_decode_full_matrices_bit_exact(ops, m, n, k):
    from oracle import gemm as G
    a, b = codes(m, k, m + n), codes(n, k, m + k)
    ap, bp = syn.pack_codes(a), syn.pack_codes(b)
    print(f"case full-size decode m={m} n={n} k={k}", flush=True)
    assert np.array_equal(host(ops.gemm_i4_int32(dev(ap), dev(bp))), G.int_gemm(a, b))
    rng = np.random.default_rng(n + m)
    sa = rng.uniform(0.01, 0.5, size=(m, 1)).astype(np.float16)
    sb = syn.weight_scales(n, 1, seed=k)
    d = host(ops.gemm_i4_dequant_o16(dev(ap), dev(bp), dev(sa), dev(sb)))
    ref, _ = G.gemm_i4_dequant(ap, bp, sa, sb)
    assert np.array_equal(d.view(np.uint16), ref.view(np.uint16))
    ng = k // 128
    sbg = syn.weight_scales(n, ng, seed=k + 1)
    for sag in (sa, rng.uniform(0.01, 0.5, size=(m, ng)).astype(np.float16)):
        d = host(ops.gemm_i4_dequant_o16(dev(ap), dev(bp), dev(sag), dev(sbg)))
        ref, _ = G.gemm_i4_dequant(ap, bp, sag, sbg)
        assert np.allclose(d.astype(np.float64), ref.astype(np.float64), rtol=1e-3, atol=1e-2)
        assert np.array_equal(d.view(np.uint16), ref.view(np.uint16))


@pytest.mark.parametrize("m", [8, 256])
@pytest.mark.parametrize("n,k", sorted(set(LLAMA2 + LLAMA3)))
def test_batch_8_and_256_full_width(ops, m, n, k):
    """M = 8 (decode batch of the Llama-3 step) and M = 256 (the short prefill, which selects the 64 x 64 tile with K
    split over four wave quads) at the full Llama widths: whole int32 matrices against the oracle, the one-scale-per-row
    epilogue bit for bit, the group epilogue (one scale per token, weight groups of 128) bit-equal to the FMA oracle."""
    from oracle import gemm as G
    a, b = codes(m, k, 11 * m + n), codes(n, k, 13 * m + k)
    ap, bp = syn.pack_codes(a), syn.pack_codes(b)
    print(f"case full-width m={m} n={n} k={k}", flush=True)
    acc = G.int_gemm(a, b)
    assert np.array_equal(host(ops.gemm_i4_int32(dev(ap), dev(bp))), acc)
    rng = np.random.default_rng(n + m + k)
    sa = rng.uniform(0.01, 0.5, size=(m, 1)).astype(np.float16)
    sb = syn.weight_scales(n, 1, seed=k)
    d = host(ops.gemm_i4_dequant_o16(dev(ap), dev(bp), dev(sa), dev(sb)))
    ref, _ = G.gemm_i4_dequant(ap, bp, sa, sb)
    assert np.array_equal(d.view(np.uint16), ref.view(np.uint16))
    sbg = syn.weight_scales(n, k // 128, seed=k + 1)
    d = host(ops.gemm_i4_dequant_o16(dev(ap), dev(bp), dev(sa), dev(sbg)))
    ref, _ = G.gemm_i4_dequant(ap, bp, sa, sbg)
    assert np.allclose(d.astype(np.float64), ref.astype(np.float64), rtol=1e-3, atol=1e-2)
    assert np.array_equal(d.view(np.uint16), ref.view(np.uint16))


def test_rotate_quant_exact_mode_whole_batch(ops):
    """M = 2048, K = 4096: every row against the float32-butterfly oracle, bit for bit."""
    from oracle import linear as L
    x = syn.activations(2048, 4096, seed=5)
    q, s, y = ops.rotate_and_quantize_i4(dev(x), return_rotated=True)
    qr, sr, yr = L.rotate_and_quantize(x, "f32")
    assert np.array_equal(host(y).view(np.uint16), yr.view(np.uint16))
    assert np.array_equal(host(s).view(np.uint16), sr.view(np.uint16))
    assert np.array_equal(host(q), qr)


@pytest.mark.parametrize("k", [4096, 11008, 14336])
def test_rotate_quant_fast_mode_invariants_whole_batch(ops, k):
    """M = 2048 in the matrix-core mode: invariants that hold for every row whatever the summation order --
    the largest code of a row is +-7 (its scale is max / 7), codes times scale reproduce a rotation of the
    input (norm preserved within the quantisation noise), and sampled rows agree with the exact transform
    up to one code step."""
    from oracle import hadamard as H
    from oracle import quant as Q
    from oracle.pack import unpack_i4
    m = 2048
    x = syn.activations(m, k, seed=k)
    q, s = ops.rotate_and_quantize_i4(dev(x), hadamard="fast")
    c = unpack_i4(host(q)).astype(np.int32)
    sc = host(s).astype(np.float32).reshape(m, 1)
    assert np.abs(c).max(axis=1).min() == 7 and c.min() >= -8 and c.max() <= 7
    deq = c * sc
    nx, nd = np.linalg.norm(x.astype(np.float32), axis=1), np.linalg.norm(deq, axis=1)
    # rounding noise of variance s^2 / 12 per element on top of an orthogonal transform
    assert np.allclose(nd, nx, rtol=0.05)
    rows = np.random.default_rng(1).choice(m, size=16, replace=False)
    qe, se = Q.quantize_rows(H.hadamard_full(x[rows], exact=True))
    assert np.abs(c[rows] - qe).max() <= 1 and (c[rows] != qe).mean() < 2e-3
    assert np.abs(host(s)[rows].reshape(-1).view(np.uint16).astype(np.int32) - se.reshape(-1).view(np.uint16).astype(np.int32)).max() <= 2


@pytest.mark.parametrize("n,k", sorted(set(LLAMA2 + LLAMA3)))
def test_prefill_6bit_path_checksums_and_equality(ops, n, k):
    """The GEMM on the 6-bit matrix instruction at full size: exact row / column checksums of the int32 sums,
    sampled rows against the oracle, and fp16 outputs identical to the int8 kernel's over the whole matrix."""
    from oracle import gemm as G
    m = 2048
    a, b = codes(m, k, 7 * n + k), codes(n, k, 7 * n + k + 1)
    ap, bp = dev(syn.pack_codes(a)), dev(syn.pack_codes(b))
    a6, b6 = ops.encode_f6(ap), ops.encode_f6(bp)
    print(f"case full-size 6-bit m={m} n={n} k={k}", flush=True)
    c = host(ops.gemm_f6_int32(a6, b6)).astype(np.int64)
    a64, b64 = a.astype(np.int64), b.astype(np.int64)
    assert np.array_equal(c.sum(axis=1), a64 @ b64.sum(axis=0))
    assert np.array_equal(c.sum(axis=0), b64 @ a64.sum(axis=0))
    rows = np.random.default_rng(1).choice(m, size=16, replace=False)
    assert np.array_equal(c[rows], G.int_gemm(a[rows], b))
    sa = dev(np.random.default_rng(n).uniform(0.01, 0.5, size=(m, 1)).astype(np.float16))
    sb = dev(syn.weight_scales(n, 1, seed=k))
    assert torch.equal(ops.gemm_f6_dequant_o16(a6, b6, sa, sb), ops.gemm_i4_dequant_o16(ap, bp, sa, sb))


@pytest.mark.parametrize("m", [2048, 16384])
def test_fused_producers_whole_batch(ops, m):
    """SwiGLU product + quantise at [m, 11008] and RMSNorm + quantise at [m, 4096]: sampled rows against the
    oracle (last-bit tolerance of the device's exp / rsqrt / summation order), and over the whole batch the
    invariants of the symmetric quantiser: every group uses the full code range on at least one side unless
    it is all zero, and no code leaves [-8, 7]."""
    from oracle import prologue as P, quant as Q
    from oracle.pack import unpack_i4
    gen = torch.Generator(device="cuda").manual_seed(m)
    gate = torch.randn(m, 11008, device="cuda", dtype=torch.float16, generator=gen) * 2
    up = torch.randn(m, 11008, device="cuda", dtype=torch.float16, generator=gen)
    x = torch.randn(m, 4096, device="cuda", dtype=torch.float16, generator=gen) * 3
    wn = torch.rand(4096, device="cuda", dtype=torch.float16, generator=gen) + 0.5
    print(f"case fused producers whole batch m={m}", flush=True)
    rows = np.random.default_rng(m).choice(m, size=12, replace=False)
    rt = torch.from_numpy(rows).cuda()
    for name, (q, s), y_rows in (
            ("silu_mul", ops.silu_mul_and_quantize_i4_gs(gate, up, 128), P.silu_mul_f16(host(gate[rt]), host(up[rt]))),
            ("rmsnorm", ops.rmsnorm_and_quantize_i4_gs(x, wn, 1e-5, 128), P.rmsnorm_f16(host(x[rt]), host(wn), 1e-5))):
        k = q.shape[1] * 2
        qr, sr, _ = Q.kernel_had_and_quant(y_rows.reshape(-1, 128), 128, False)
        got_q = unpack_i4(host(q[rt])).reshape(-1, 128)
        got_s = host(s[rt]).reshape(-1)
        ds = np.abs(got_s.view(np.uint16).astype(np.int32) - sr.view(np.uint16).astype(np.int32))
        assert ds.max() <= 1 and np.mean(ds != 0) < 5e-3, (name, ds.max(), np.mean(ds != 0))
        dq = np.abs(got_q - qr)[ds == 0]
        assert dq.max() <= 1 and np.mean(dq != 0) < 1e-4, (name, dq.max(), np.mean(dq != 0))
        # whole batch, on the device: nibbles as signed codes, per-group extreme
        lo = (q & 0xF).to(torch.int8)
        hi = (q >> 4).to(torch.int8)
        lo = torch.where(lo > 7, lo - 16, lo)
        hi = torch.where(hi > 7, hi - 16, hi)
        amax = torch.maximum(lo.abs().view(m, k // 128, 64).amax(-1), hi.abs().view(m, k // 128, 64).amax(-1))
        nonzero = s.view(m, k // 128) != 1.0
        assert bool(((amax == 7) | (amax == 8) | ~nonzero).all()), name       # max |y| / scale rounds to 7 (or -8 after rounding up)
        assert bool(torch.isfinite(s.float()).all()) and bool((s > 0).all())


def test_group_kernels_beyond_4_gib_use_wide_offsets(ops):
    """The group kernels address with 32-bit offsets when the launch fits and with 64-bit ones beyond: 2^24 + 300
    rows of 128 (4.3 GB of fp16) take the wide path; the same rows in two launches that each fit must give the
    same codes and scales, and the in-place transform the same values."""
    rows = (1 << 24) + 300
    gen = torch.Generator(device="cuda").manual_seed(9)
    x = torch.empty(rows, 128, dtype=torch.float16, device="cuda")
    x.normal_(generator=gen)
    x[-1] = 3.0                                         # a recognisable last row
    half = 1 << 23
    for fn in (ops.hadamard_and_quantize_i4, ops.quant_and_pack_i4):
        q, s = fn(x)
        for lo, hi in ((0, half), (half, rows)):
            qp, sp = fn(x[lo:hi])
            assert torch.equal(q[lo:hi], qp) and torch.equal(s.view(-1)[lo:hi], sp.view(-1))
        del q, s, qp, sp
    y = x.clone()
    ops.hadamard_transform_half(y)
    for lo, hi in ((0, half), (half, rows)):
        part = x[lo:hi].clone()
        ops.hadamard_transform_half(part)
        assert torch.equal(y[lo:hi], part)
        del part
