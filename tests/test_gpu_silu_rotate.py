"""The SwiGLU product in front of the online rotation of down_proj for decode-sized batches, through the C ABI.

Two statements.  (1) The product kernel against the CPU oracle's float64 evaluation of fp16(fp16(silu(g)) * u): exp and the
reciprocal belong to the device, so a few values per million may differ in the last bit -- the bound is one fp16 ulp on a
mismatch rate; on data where silu is exact (gate >= 17) the comparison is bit for bit.  (2) The fused launch against the
separate launches ON THE DEVICE'S OWN PRODUCT: same codes, same scales, bit for bit (integer / byte work), and on
exact data against the oracle's rotation and quantiser as well."""
import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def ops():
    assert torch.cuda.is_available(), "these tests need the GPU"
    from flh_amd import _ops
    return _ops


def rows(m, k, seed, scale=1.0):
    rng = np.random.default_rng(seed)
    gate = (rng.standard_normal((m, k)) * scale).astype(np.float16)
    up = rng.standard_normal((m, k)).astype(np.float16)
    return gate, up


@pytest.mark.parametrize("shape", [(1, 4096), (3, 11008), (64, 14336), (5, 7, 128)])
def test_product_against_the_oracle(ops, shape):
    from oracle import prologue as P
    print(f"case silu_mul shape={shape}", flush=True)
    rng = np.random.default_rng(11)
    gate = (rng.standard_normal(shape) * 3).astype(np.float16)
    up = rng.standard_normal(shape).astype(np.float16)
    got = ops.silu_mul(torch.from_numpy(gate).cuda(), torch.from_numpy(up).cuda()).cpu().numpy()
    ref = P.silu_mul_f16(gate, up)
    d = np.abs(got.view(np.int16).astype(np.int32) - ref.view(np.int16).astype(np.int32))
    assert d.max() <= 1 and np.mean(d != 0) <= 1e-4, (d.max(), np.mean(d != 0))


def test_product_on_exact_data_bit_for_bit(ops):
    from oracle import prologue as P
    rng = np.random.default_rng(12)
    gate = rng.integers(17, 40, (16, 4096)).astype(np.float16)       # sigmoid(gate) = 1 in float32
    up = rng.integers(-40, 41, (16, 4096)).astype(np.float16)        # products below 2048: exact in fp16
    got = ops.silu_mul(torch.from_numpy(gate).cuda(), torch.from_numpy(up).cuda()).cpu().numpy()
    assert np.array_equal(got, gate * up)
    assert np.array_equal(got.view(np.uint16), P.silu_mul_f16(gate, up).view(np.uint16))


@pytest.mark.parametrize("k", [11008, 14336])
@pytest.mark.parametrize("m", [1, 2, 8, 16, 37, 256])
def test_fused_launch_gives_the_bytes_of_the_separate_launches(ops, m, k):
    print(f"case silu_mul_rotate m={m} k={k}", flush=True)
    gate, up = rows(m, k, 100 + m, scale=2.0)
    g, u = torch.from_numpy(gate).cuda(), torch.from_numpy(up).cuda()
    q, s = ops.silu_mul_rotate_and_quantize_i4(g, u)
    q_ref, s_ref = ops.rotate_and_quantize_i4(ops.silu_mul(g, u), hadamard="fast")
    assert q.shape == (m, k // 2) and s.shape == (m, 1)
    assert torch.equal(s.view(torch.int16), s_ref.view(torch.int16))
    assert torch.equal(q, q_ref)


def test_fused_launch_twice_in_a_row_and_outliers(ops):
    # a second call with fewer rows, and rows with one dominant channel (the scale follows the rotated row, not the input)
    for m in (16, 3):
        gate, up = rows(m, 14336, 7 + m)
        gate[:, 5] = 60.0
        up[:, 5] = -30.0
        g, u = torch.from_numpy(gate).cuda(), torch.from_numpy(up).cuda()
        q, s = ops.silu_mul_rotate_and_quantize_i4(g, u)
        q_ref, s_ref = ops.rotate_and_quantize_i4(ops.silu_mul(g, u), hadamard="fast")
        assert torch.equal(q, q_ref) and torch.equal(s.view(torch.int16), s_ref.view(torch.int16))


@pytest.mark.parametrize("k", [11008, 14336])
def test_fused_launch_on_exact_data_against_the_oracle(ops, k):
    """gate = 17 .. 20 (the sigmoid is 1 in float32, silu(gate) = gate) and up in {-1, 0, 1} at a few positions: the
    product is a small integer, every partial sum of the rotation is exact in any order and precision, so the device must
    give the codes and scales of the exactly rounded transform of the oracle's product bit for bit."""
    from oracle import hadamard as H, prologue as P, quant as Q
    from oracle.pack import pack_i4
    rng = np.random.default_rng(k)
    for m in (1, 9):
        gate = rng.integers(17, 21, (m, k)).astype(np.float16)
        up = np.zeros((m, k), np.float16)
        for r in range(m):
            idx = rng.choice(k, 40, replace=False)
            up[r, idx] = rng.choice([-1.0, 1.0], 40).astype(np.float16)
        prod = P.silu_mul_f16(gate, up)
        assert np.array_equal(prod, gate * up)
        q, s = ops.silu_mul_rotate_and_quantize_i4(torch.from_numpy(gate).cuda(), torch.from_numpy(up).cuda())
        qe, se = Q.quantize_rows(H.hadamard_full(prod, exact=True))
        assert np.array_equal(s.cpu().numpy().reshape(-1).view(np.uint16), se.reshape(-1).view(np.uint16))
        assert np.array_equal(q.cpu().numpy(), pack_i4(qe))


def test_argument_errors(ops):
    x = torch.zeros(4, 14336, dtype=torch.float16, device="cuda")
    with pytest.raises(RuntimeError):
        ops.silu_mul_rotate_and_quantize_i4(x, x[:2])
    with pytest.raises(RuntimeError):
        ops.silu_mul_rotate_and_quantize_i4(x[:, :4096].contiguous(), x[:, :4096].contiguous())
    with pytest.raises(RuntimeError):
        ops.silu_mul_rotate_and_quantize_i4(x.float(), x.float())
    big = torch.zeros(257, 11008, dtype=torch.float16, device="cuda")
    with pytest.raises(RuntimeError):
        ops.silu_mul_rotate_and_quantize_i4(big, big)
    with pytest.raises(RuntimeError):
        ops.silu_mul(x[:, :7], x[:, :7])
