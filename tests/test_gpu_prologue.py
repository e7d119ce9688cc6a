"""Fused SwiGLU-product and RMSNorm prologues of the group quantiser against the CPU oracle
(through the C ABI).  exp, rsqrt and the float32 summation order belong to the device, so on
random data the fp16 intermediate may differ from the CPU evaluation in its last bit for a few
values per million: the tolerance below is a mismatch RATE on codes (by one step at most) and
scales (by one fp16 ulp at most); on data where the arithmetic is exact the comparison is
bit for bit."""
import numpy as np
import pytest
import torch

from flh_amd import synthetic as syn

pytestmark = pytest.mark.gpu

CODE_RATE = 1e-4     # fraction of codes allowed to differ (by one step)
SCALE_RATE = 2e-3    # fraction of group scales allowed to differ (by one fp16 ulp)


@pytest.fixture(scope="module")
def ops():
    assert torch.cuda.is_available(), "these tests need the GPU"
    from flh_amd import _ops
    return _ops


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    return t.detach().cpu().numpy()


def oracle_group_quant(y, g, had, scale_mul=1.0):
    from oracle import quant as Q
    lead, k = y.shape[:-1], y.shape[-1]
    q, s, _ = Q.kernel_had_and_quant(y.reshape(-1, g), g, had)
    if scale_mul != 1.0:
        s = (s.astype(np.float32) * np.float32(scale_mul)).astype(np.float16)
    return q.reshape(lead + (k,)), s.reshape(lead + (k // g,))


def compare(q_dev, s_dev, q_ref, s_ref, exact, scale_ulps=1):
    from oracle.pack import unpack_i4
    codes = unpack_i4(host(q_dev)).astype(np.int32)
    scales = host(s_dev)
    if exact:
        assert np.array_equal(scales.view(np.uint16), s_ref.view(np.uint16))
        assert np.array_equal(codes, q_ref)
        return
    ds = np.abs(scales.view(np.uint16).astype(np.int32) - s_ref.view(np.uint16).astype(np.int32))
    assert ds.max() <= scale_ulps and np.mean(ds != 0) <= SCALE_RATE, (ds.max(), np.mean(ds != 0))
    same_scale = np.repeat(ds == 0, q_ref.shape[-1] // s_ref.shape[-1], axis=-1)
    dq = np.abs(codes - q_ref)[same_scale]
    assert dq.max() <= 1 and np.mean(dq != 0) <= CODE_RATE, (dq.max(), np.mean(dq != 0))


@pytest.mark.parametrize("g", [32, 64, 128])
@pytest.mark.parametrize("had", [False, True])
@pytest.mark.parametrize("shape", [(1, 128), (7, 384), (3, 5, 256), (300, 11008)])
def test_silu_mul_group_quant(ops, g, had, shape):
    from oracle import prologue as P
    rng = np.random.default_rng(g + had + sum(shape))
    gate = (rng.standard_normal(shape) * 2.5).astype(np.float16)
    up = (rng.standard_normal(shape) * 1.5).astype(np.float16)
    print(f"case silu_mul g={g} had={had} shape={shape}", flush=True)
    q, s = ops.silu_mul_and_quantize_i4_gs(dev(gate), dev(up), g, had, scale_mul=0.25)
    assert q.shape == shape[:-1] + (shape[-1] // 2,) and s.shape == shape[:-1] + (shape[-1] // g,)
    q_ref, s_ref = oracle_group_quant(P.silu_mul_f16(gate, up), g, had, 0.25)
    # behind the transform a last-bit difference of one input can be two ulps of a group maximum (binade boundary)
    compare(q, s, q_ref, s_ref, exact=False, scale_ulps=2 if had else 1)


@pytest.mark.parametrize("g", [32, 64, 128])
@pytest.mark.parametrize("had", [False, True])
def test_silu_mul_exact_data_bit_exact(ops, g, had):
    """gate >= 17: the sigmoid is 1 in float32, silu(gate) = gate; integer products below 2048 are exact in
    fp16, so every value of the intermediate is fixed and the outputs must match bit for bit.  Includes an
    all-zero group (scale 1, codes 0) and the extreme inputs."""
    from oracle import prologue as P
    rng = np.random.default_rng(g * 2 + had)
    gate = rng.integers(17, 41, size=(65, 4 * g)).astype(np.float16)
    up = rng.integers(-12, 13, size=(65, 4 * g)).astype(np.float16)
    up[3, :g] = 0
    gate[4, :8] = [-65504.0, 65504.0, -30.0, 0.0, -0.0, 17.0, 40.0, 20.0]
    up[4, :8] = [1.0, 2.0 ** -10, 100.0, 5.0, -5.0, 0.0, -0.0, 6.1e-5]
    q, s = ops.silu_mul_and_quantize_i4_gs(dev(gate), dev(up), g, had)
    q_ref, s_ref = oracle_group_quant(P.silu_mul_f16(gate, up), g, had)
    compare(q, s, q_ref, s_ref, exact=True)


@pytest.mark.parametrize("g", [32, 64, 128])
@pytest.mark.parametrize("had", [False, True])
@pytest.mark.parametrize("m,k", [(1, 128), (5, 512), (64, 4096), (33, 11008), (9, 14336), (3, 16384), (6, 2176)])
@pytest.mark.parametrize("weighted", [False, True])
def test_rmsnorm_group_quant(ops, g, had, m, k, weighted):
    from oracle import prologue as P
    rng = np.random.default_rng(g + had + m + k + weighted)
    x = (rng.standard_normal((m, k)) * rng.uniform(0.05, 30, (m, 1))).astype(np.float16)
    w = rng.uniform(0.3, 2.5, k).astype(np.float16) if weighted else None
    print(f"case rmsnorm g={g} had={had} m={m} k={k} weighted={weighted}", flush=True)
    q, s = ops.rmsnorm_and_quantize_i4_gs(dev(x), dev(w) if weighted else None, 1e-5, g, had)
    assert q.shape == (m, k // 2) and s.shape == (m, k // g)
    q_ref, s_ref = oracle_group_quant(P.rmsnorm_f16(x, w, 1e-5), g, had)
    # behind the transform a last-bit difference of one input can be two ulps of a group maximum (binade boundary)
    compare(q, s, q_ref, s_ref, exact=False, scale_ulps=2 if had else 1)


@pytest.mark.parametrize("g", [32, 64, 128])
@pytest.mark.parametrize("had", [False, True])
@pytest.mark.parametrize("k", [256, 4096, 11008])
def test_rmsnorm_exact_data_bit_exact(ops, g, had, k):
    """Rows of +-1 with eps = 0: the mean square is exactly 1, every output is sign * weight, so the
    outputs are fixed bit for bit.  One row of zeros (stays zero: scale 1, codes 0)."""
    from oracle import prologue as P
    rng = np.random.default_rng(g + had + k)
    x = rng.choice([-1.0, 1.0], size=(19, k)).astype(np.float16)
    x[7] = 0
    w = rng.uniform(0.3, 2.5, k).astype(np.float16)
    q, s = ops.rmsnorm_and_quantize_i4_gs(dev(x), dev(w), 0.0, g, had, scale_mul=float(np.float32(1 / np.sqrt(g))))
    y = P.rmsnorm_f16(np.where(x == 0, np.float16(0), x), w, 0.0)
    y[7] = 0                                            # 0 * inf is NaN on the CPU and on the device alike ...
    q_ref, s_ref = oracle_group_quant(y, g, had, float(np.float32(1 / np.sqrt(g))))
    keep = np.arange(19) != 7                           # ... so the zero row with eps = 0 is outside the contract
    compare(q[torch.from_numpy(keep).cuda()], s[torch.from_numpy(keep).cuda()], q_ref[keep], s_ref[keep], exact=True)
    # with eps > 0 the zero row is defined: zeros, scale 1
    q, s = ops.rmsnorm_and_quantize_i4_gs(dev(x[7:8]), dev(w), 1e-5, g, had)
    assert not host(q).any() and np.all(host(s) == np.float16(1.0))


@pytest.mark.parametrize("k", [512, 1024, 2048, 4096, 8192])
@pytest.mark.parametrize("had", [False, True])
@pytest.mark.parametrize("weighted", [False, True])
def test_rmsnorm_rotate_quant(ops, k, had, weighted):
    """RMSNorm in front of the whole-row rotation.  A last-bit difference in one normalised value moves
    every rotated value by at most 2^-11 / sqrt(K) of it, so codes differ rarely and by one step, the row
    scale by one ulp at most."""
    from oracle import linear as L, prologue as P
    from oracle.pack import unpack_i4
    rng = np.random.default_rng(k + had + 2 * weighted)
    m = 37
    x = (rng.standard_normal((m, k)) * rng.uniform(0.05, 30, (m, 1))).astype(np.float16)
    x[:, rng.integers(0, k, 4)] *= 12        # outlier channels
    w = rng.uniform(0.3, 2.5, k).astype(np.float16) if weighted else None
    print(f"case rmsnorm_rotate k={k} had={had} weighted={weighted}", flush=True)
    q, s, y = ops.rmsnorm_rotate_and_quantize_i4(dev(x), dev(w) if weighted else None, 1e-5, had, return_rotated=True)
    qp_ref, s_ref, y_ref = L.rotate_and_quantize(P.rmsnorm_f16(x, w, 1e-5), "f32" if had else "none")
    # rotated row: a last-bit difference of a few inputs shows as a small absolute difference (many ulps
    # where the rotated value is near zero), bounded by the inputs' ulp over sqrt(K) plus the final rounding
    yd, yr = host(y).astype(np.float64), y_ref.astype(np.float64)
    bound = 2.0 ** -10 * np.abs(yr) + 2.0 ** -11 * np.abs(yr).max(-1, keepdims=True)
    assert np.all(np.abs(yd - yr) <= bound) and np.mean(yd != yr) < (5e-2 if had else 2e-3), np.mean(yd != yr)
    ds = np.abs(host(s).view(np.uint16).astype(np.int32) - s_ref.view(np.uint16).astype(np.int32))
    assert ds.max() <= 1, ds.max()
    same = (ds == 0).reshape(-1)
    dq = np.abs(unpack_i4(host(q)).astype(np.int32) - unpack_i4(qp_ref).astype(np.int32))[same]
    assert dq.max() <= 1 and np.mean(dq != 0) < 1e-3, (dq.max(), np.mean(dq != 0))


@pytest.mark.parametrize("k", [512, 4096, 8192])
@pytest.mark.parametrize("had", [False, True])
def test_rmsnorm_rotate_quant_exact_data_bit_exact(ops, k, had):
    """Rows of +-1, eps = 0: the normalised row is sign * weight exactly, so everything downstream must
    match the oracle bit for bit (clip included)."""
    from oracle import linear as L, prologue as P
    rng = np.random.default_rng(k + had)
    x = rng.choice([-1.0, 1.0], size=(21, k)).astype(np.float16)
    w = rng.uniform(0.3, 2.5, k).astype(np.float16)
    for clip in (1.0, 0.9):
        q, s, y = ops.rmsnorm_rotate_and_quantize_i4(dev(x), dev(w), 0.0, had, clip_ratio=clip, return_rotated=True)
        qp_ref, s_ref, y_ref = L.rotate_and_quantize(P.rmsnorm_f16(x, w, 0.0), "f32" if had else "none", None, clip)
        assert np.array_equal(host(y).view(np.uint16), y_ref.view(np.uint16))
        assert np.array_equal(host(s).view(np.uint16), s_ref.view(np.uint16))
        assert np.array_equal(host(q), qp_ref)
    # and the same launch without the weight equals the plain kernel on the same +-1 rows
    q0, s0 = ops.rmsnorm_rotate_and_quantize_i4(dev(x), None, 0.0, had)
    q1, s1 = ops.rotate_and_quantize_i4(dev(x), hadamard="exact" if had else False)
    assert torch.equal(q0, q1) and torch.equal(s0, s1)


def test_prologue_feeds_the_gemm(ops):
    """MLP tail as the model runs it: SwiGLU product, group quantiser, group-scale GEMM, against the
    oracle's linear layer on the oracle's intermediate."""
    from oracle import gemm as G, prologue as P
    rng = np.random.default_rng(11)
    m, inter, n, g = 48, 1024, 256, 128
    gate = (rng.standard_normal((m, inter)) * 2).astype(np.float16)
    up = rng.standard_normal((m, inter)).astype(np.float16)
    wq = rng.integers(-8, 8, size=(n, inter), dtype=np.int8)
    ws = rng.uniform(0.005, 0.02, (n, inter // g)).astype(np.float16)
    q, s = ops.silu_mul_and_quantize_i4_gs(dev(gate), dev(up), g)
    out = host(ops.gemm_i4_dequant_o16_gs(q, dev(syn.pack_codes(wq)), s, dev(ws), g))
    q_ref, s_ref = oracle_group_quant(P.silu_mul_f16(gate, up), g, False)
    ref, _ = G.gemm_i4_dequant(syn.pack_codes(q_ref.astype(np.int8)), syn.pack_codes(wq), s_ref, ws, g)
    assert np.allclose(out.astype(np.float32), ref.astype(np.float32), rtol=1e-3, atol=1e-2)


def test_prologue_argument_errors(ops):
    x = torch.zeros(4, 256, dtype=torch.float16, device="cuda")
    with pytest.raises(RuntimeError):
        ops.silu_mul_and_quantize_i4_gs(x, x[:2], 128)
    with pytest.raises(RuntimeError):
        ops.silu_mul_and_quantize_i4_gs(x, x, 48)
    with pytest.raises(RuntimeError):
        ops.silu_mul_and_quantize_i4_gs(x.float(), x.float(), 128)
    with pytest.raises(RuntimeError):
        ops.rmsnorm_and_quantize_i4_gs(x, x[0, :128].contiguous(), 1e-5, 128)
    with pytest.raises(RuntimeError):
        ops.rmsnorm_and_quantize_i4_gs(torch.zeros(2, 32768, dtype=torch.float16, device="cuda"), None, 1e-5, 128)
    with pytest.raises(RuntimeError):
        ops.rmsnorm_rotate_and_quantize_i4(torch.zeros(2, 1536, dtype=torch.float16, device="cuda"), None, 1e-5)
    q, s = ops.rmsnorm_and_quantize_i4_gs(x[:0], None, 1e-5, 128)
    assert q.shape == (0, 128) and s.shape == (0, 2)


def test_rmsnorm_rotate_short_batches_give_the_long_batch_bytes(ops):
    """Up to 512 rows of 4096 take one workgroup of eight waves per row, more take one wave per row: the same sums in
    the same order (statistics included), so a row's codes and scale do not depend on the batch it arrives in."""
    x = dev(syn.activations(700, 4096, seed=11))
    w = dev(np.random.default_rng(12).uniform(0.5, 1.5, 4096).astype(np.float16))
    for weight in (w, None):
        q_long, s_long = ops.rmsnorm_rotate_and_quantize_i4(x, weight, 1e-5)
        for rows in (1, 8, 16, 300, 512):
            q, s = ops.rmsnorm_rotate_and_quantize_i4(x[:rows].contiguous(), weight, 1e-5)
            assert torch.equal(q, q_long[:rows]) and torch.equal(s, s_long[:rows]), rows


@pytest.mark.parametrize("k", [512, 4096, 8192])
@pytest.mark.parametrize("m", [1, 5, 512, 700])
@pytest.mark.parametrize("had", [True, False])
def test_residual_add_in_front_of_rmsnorm_rotate_gives_the_separate_launches_bytes(ops, k, m, had):
    """x + add in fp16 is one correctly rounded addition per value on the device as in torch, so the fused launch must
    give torch's sum and, from it, the bytes of the launch without the addition (both row layouts: eight waves per row up
    to 512 rows of 4096, one wave per row otherwise)."""
    print(f"case add_rmsnorm m={m} k={k} had={had}", flush=True)
    x = dev(syn.activations(m, k, seed=k + m))
    add = dev((np.random.default_rng(m).standard_normal((m, k)) * 0.3).astype(np.float16))
    w = dev(np.random.default_rng(3).uniform(0.5, 1.5, k).astype(np.float16))
    total, q, s = ops.add_rmsnorm_rotate_and_quantize_i4(x, add, w, 1e-5, had)
    assert torch.equal(total, x + add)
    assert np.array_equal(host(total), (host(x).astype(np.float64) + host(add).astype(np.float64)).astype(np.float16))
    q_ref, s_ref = ops.rmsnorm_rotate_and_quantize_i4(total, w, 1e-5, had)
    assert torch.equal(q, q_ref) and torch.equal(s.view(torch.int16), s_ref.view(torch.int16))


def test_residual_add_argument_errors(ops):
    x = torch.zeros(4, 4096, dtype=torch.float16, device="cuda")
    with pytest.raises(RuntimeError):
        ops.add_rmsnorm_rotate_and_quantize_i4(x, x[:2], None, 1e-5)
    with pytest.raises(RuntimeError):
        ops.add_rmsnorm_rotate_and_quantize_i4(x[:, :768].contiguous(), x[:, :768].contiguous(), None, 1e-5)
    with pytest.raises(RuntimeError):
        ops.add_rmsnorm_rotate_and_quantize_i4(x, x.float(), None, 1e-5)


# ---- RMSNorm on its own (a model's final norm), optionally behind the residual addition ---------------------------------

VALUE_RATE = 1e-3    # fraction of fp16 outputs allowed to differ from the CPU evaluation (by one ulp: summation order)


@pytest.mark.parametrize("m,k", [(1, 4096), (16, 4096), (5, 5120), (3, 8192), (7, 16384), (9, 264), (33, 8)])
@pytest.mark.parametrize("weighted", [False, True])
@pytest.mark.parametrize("with_add", [False, True])
def test_add_rmsnorm(ops, m, k, weighted, with_add):
    from oracle import prologue as P
    rng = np.random.default_rng(m + k + weighted + 2 * with_add)
    x = (rng.standard_normal((m, k)) * rng.uniform(0.05, 30, (m, 1))).astype(np.float16)
    a = (rng.standard_normal((m, k)) * rng.uniform(0.05, 30, (m, 1))).astype(np.float16) if with_add else None
    w = rng.uniform(0.3, 2.5, k).astype(np.float16) if weighted else None
    print(f"case add_rmsnorm m={m} k={k} weighted={weighted} add={with_add}", flush=True)
    if with_add:
        total, y = ops.add_rmsnorm(dev(x), dev(w) if weighted else None, 1e-5, add=dev(a), return_sum=True)
        s = (x.astype(np.float32) + a.astype(np.float32)).astype(np.float16)      # one rounding per value
        assert np.array_equal(host(total).view(np.uint16), s.view(np.uint16))
        assert np.array_equal(host(ops.add_rmsnorm(dev(x), dev(w) if weighted else None, 1e-5, add=dev(a))).view(np.uint16),
                              host(y).view(np.uint16))
    else:
        s, y = x, ops.add_rmsnorm(dev(x), dev(w) if weighted else None, 1e-5)
    ref = P.rmsnorm_f16(s, w, 1e-5)
    d = np.abs(host(y).view(np.int16).astype(np.int32) - ref.view(np.int16).astype(np.int32))
    assert d.max() <= 1 and np.mean(d != 0) <= VALUE_RATE, (d.max(), np.mean(d != 0))


@pytest.mark.parametrize("k", [8, 4096, 16384])
def test_add_rmsnorm_exact_data_bit_exact(ops, k):
    """Rows of +-1 with eps = 0 (as the sum of +-3 and -+2): the mean square is exactly 1 and every output is
    sign * weight bit for bit; a row of zeros with eps > 0 stays zero."""
    rng = np.random.default_rng(k)
    sign = rng.choice([-1.0, 1.0], size=(11, k)).astype(np.float16)
    w = rng.uniform(0.3, 2.5, k).astype(np.float16)
    y = ops.add_rmsnorm(dev(sign * np.float16(3)), dev(w), 0.0, add=dev(sign * np.float16(-2)))
    assert np.array_equal(host(y).view(np.uint16), (sign * w).astype(np.float16).view(np.uint16))
    z = ops.add_rmsnorm(torch.zeros(2, k, dtype=torch.float16, device="cuda"), dev(w), 1e-5)
    assert not host(z).any()


def test_add_rmsnorm_argument_errors(ops):
    x = torch.zeros(4, 4096, dtype=torch.float16, device="cuda")
    for bad in (lambda: ops.add_rmsnorm(x, None, 1e-5, add=x[:2]),
                lambda: ops.add_rmsnorm(x[:, :4092].contiguous()),
                lambda: ops.add_rmsnorm(torch.zeros(2, 16392, dtype=torch.float16, device="cuda")),
                lambda: ops.add_rmsnorm(x.float()),
                lambda: ops.add_rmsnorm(x, x[0, :100].contiguous()),
                lambda: ops.add_rmsnorm(x, None, 1e-5, return_sum=True)):
        with pytest.raises(RuntimeError):
            bad()
    from flh_amd import _lib
    lib = _lib.load()
    assert lib.flh_add_rmsnorm_f16(x.data_ptr(), None, None, 1e-5, x.data_ptr(), x.data_ptr(), 4, 4096, None) != 0   # sum_out without add
    assert b"sum_out" in lib.flh_last_error()
    assert ops.add_rmsnorm(x[:0]).shape == (0, 4096)
