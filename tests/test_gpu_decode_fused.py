"""The decode GEMM that rotates and quantises its own activations (one launch instead of two): outputs against
the oracle of the whole path, and bit for bit against the two stand-alone launches, through the C ABI."""
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


def weights(n, k, cols, seed):
    rng = np.random.default_rng(seed)
    w = rng.integers(0, 256, size=(n, k // 2), dtype=np.uint8)
    s = rng.uniform(0.005, 0.02, size=(n, cols)).astype(np.float16)
    return w, s


@pytest.mark.parametrize("m", [1, 2, 3, 4])
@pytest.mark.parametrize("n,k", [(4096, 4096), (11008, 4096), (40, 4096), (22016, 4096)])
@pytest.mark.parametrize("grouped", [False, True])
def test_equals_the_two_launches(ops, m, n, k, grouped):
    x = syn.activations(m, k, seed=100 * m + n % 97)
    w, s = weights(n, k, k // 128 if grouped else 1, seed=n + k)
    xd, wd, sd = dev(x), dev(w), dev(s)
    q, a = ops.rotate_and_quantize_i4(xd, hadamard="exact")
    want = ops.gemm_i4_dequant_o16(q, wd, a, sd)
    got = ops.rotate_quantize_gemm_i4(xd, wd, sd)
    assert got.shape == (m, n) and torch.equal(got, want)


@pytest.mark.parametrize("m", [1, 3])
def test_against_the_oracle(ops, m):
    from oracle import gemm as G
    from oracle import hadamard as H
    from oracle import quant as Q
    from oracle.pack import pack_i4
    n, k = 256, 4096
    x = syn.activations(m, k, seed=m)
    w, s = weights(n, k, 1, seed=5)
    codes, a = Q.quantize_rows(H.hadamard_full(x, exact=False))
    want = G.gemm_i4_dequant(pack_i4(codes), w, a.reshape(m, 1), s)
    want = want[0] if isinstance(want, tuple) else want
    got = host(ops.rotate_quantize_gemm_i4(dev(x), dev(w), dev(s)))
    assert np.array_equal(got.view(np.uint16), np.asarray(want).view(np.uint16))


@pytest.mark.parametrize("m", [1, 3])
@pytest.mark.parametrize("ns", [(4096, 4096, 4096), (4096, 1024, 1024), (11008, 11008), (40, 24, 1000, 16)])
@pytest.mark.parametrize("grouped", [False, True])
def test_several_weight_matrices(ops, m, ns, grouped):
    k = 4096
    xd = dev(syn.activations(m, k, seed=m + len(ns)))
    ws = [weights(n, k, k // 128 if grouped else 1, seed=n + i) for i, n in enumerate(ns)]
    Bs, Ss = [dev(w) for w, _ in ws], [dev(s) for _, s in ws]
    got = ops.rotate_quantize_gemm_i4_multi(xd, Bs, Ss)
    for D, B, S in zip(got, Bs, Ss):
        assert torch.equal(D, ops.rotate_quantize_gemm_i4(xd, B, S))


def test_zero_and_outlier_rows(ops):
    n, k = 64, 4096
    x = np.zeros((4, k), dtype=np.float16)
    x[1, 7] = 60000.0                                  # one huge value
    x[2] = 1e-7                                        # subnormal row
    x[3] = syn.activations(1, k, seed=3)[0]
    w, s = weights(n, k, 1, seed=9)
    xd, wd, sd = dev(x), dev(w), dev(s)
    q, a = ops.rotate_and_quantize_i4(xd, hadamard="exact")
    assert torch.equal(ops.rotate_quantize_gemm_i4(xd, wd, sd), ops.gemm_i4_dequant_o16(q, wd, a, sd))


def test_argument_errors(ops):
    w, s = weights(32, 4096, 1, seed=1)
    wd, sd = dev(w), dev(s)
    with pytest.raises(RuntimeError):
        ops.rotate_quantize_gemm_i4(torch.zeros(5, 4096, dtype=torch.float16, device="cuda"), wd, sd)
    with pytest.raises(RuntimeError):
        ops.rotate_quantize_gemm_i4(torch.zeros(1, 2048, dtype=torch.float16, device="cuda"), wd[:, :1024].contiguous(), sd)
    with pytest.raises(RuntimeError):
        ops.rotate_quantize_gemm_i4(torch.zeros(1, 4096, dtype=torch.float16, device="cuda"), wd, sd.repeat(1, 3))
    assert ops.rotate_quantize_gemm_i4(torch.zeros(0, 4096, dtype=torch.float16, device="cuda"), wd, sd).shape == (0, 32)


@pytest.mark.parametrize("m", [1, 2, 4])
@pytest.mark.parametrize("grouped", [False, True])
@pytest.mark.parametrize("with_add,with_weight", [(False, True), (True, True), (True, False)])
def test_norm_and_residual_prologue_equals_the_separate_launches(ops, m, grouped, with_add, with_weight):
    """RMSNorm (and the residual addition in front of it) inside the decode GEMM: the sum, and every output, bit for bit
    those of [add_]rmsnorm_rotate_and_quantize_i4 followed by the shared-input GEMM launch."""
    k, ns = 4096, (4096, 1024, 1000)
    print(f"case norm prologue m={m} grouped={grouped} add={with_add} weight={with_weight}", flush=True)
    x = dev(syn.activations(m, k, seed=7 * m + grouped))
    add = dev((np.random.default_rng(m).standard_normal((m, k)) * 0.5).astype(np.float16)) if with_add else None
    nw = dev(np.random.default_rng(5).uniform(0.5, 1.5, k).astype(np.float16)) if with_weight else None
    ws = [weights(n, k, k // 128 if grouped else 1, seed=n + m) for n in ns]
    Bs, Ss = [dev(w) for w, _ in ws], [dev(s) for _, s in ws]
    total, outs = ops.rmsnorm_rotate_quantize_gemm_i4_multi(x, add, nw, 1e-5, Bs, Ss)
    if with_add:
        want_total, q, s = ops.add_rmsnorm_rotate_and_quantize_i4(x, add, nw, 1e-5)
        assert torch.equal(total, want_total) and torch.equal(total, x + add)
    else:
        assert total is None
        q, s = ops.rmsnorm_rotate_and_quantize_i4(x, nw, 1e-5)
    want = ops.gemm_i4_dequant_multi(q, Bs, s, Ss, 128)
    for got, ref in zip(outs, want):
        assert torch.equal(got.view(torch.int16), ref.view(torch.int16))


def test_norm_prologue_argument_errors(ops):
    x = torch.zeros(2, 4096, dtype=torch.float16, device="cuda")
    B = torch.zeros(64, 2048, dtype=torch.uint8, device="cuda")
    S = torch.ones(64, 1, dtype=torch.float16, device="cuda")
    with pytest.raises(RuntimeError):
        ops.rmsnorm_rotate_quantize_gemm_i4_multi(torch.zeros(5, 4096, dtype=torch.float16, device="cuda"), None, None, 1e-5, [B], [S])
    with pytest.raises(RuntimeError):
        ops.rmsnorm_rotate_quantize_gemm_i4_multi(x, x[:1], None, 1e-5, [B], [S])
    with pytest.raises(RuntimeError):
        ops.rmsnorm_rotate_quantize_gemm_i4_multi(x, None, torch.ones(100, dtype=torch.float16, device="cuda"), 1e-5, [B], [S])
