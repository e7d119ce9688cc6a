"""The whole-row rotation + per-token quantiser writing the 6-bit operand format directly (flh_rotate_quant_f6), through
the C ABI: byte / integer work, so the bar is equality -- the encoded bytes equal flh_encode_f6 of the nibble output of
the corresponding nibble-writing call (which the other tests compare with the oracle), the scales are the same bits,
and the 6-bit GEMM on them gives the int8 GEMM's output."""
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


@pytest.mark.parametrize("k", [512, 1024, 4096, 8192])
@pytest.mark.parametrize("m", [1, 300, 700])
@pytest.mark.parametrize("had", [True, False])
def test_power_of_two_rows(ops, m, k, had):
    print(f"case rotate_f6 m={m} k={k} had={had}", flush=True)
    x = dev(syn.activations(m, k, seed=m + k))
    enc, s = ops.rotate_and_quantize_f6(x, hadamard=had, clip_ratio=0.9 if m == 300 else 1.0)
    q, s_ref = ops.rotate_and_quantize_i4(x, hadamard="exact" if had else False, clip_ratio=0.9 if m == 300 else 1.0)
    assert enc.shape == (m, k // 128 * 96)
    assert torch.equal(s.view(torch.int16), s_ref.view(torch.int16))
    assert torch.equal(enc, ops.encode_f6(q))


@pytest.mark.parametrize("m", [2, 513, 1000])
@pytest.mark.parametrize("with_add,with_weight", [(False, True), (True, True), (True, False)])
def test_norm_and_residual_prologues(ops, m, with_add, with_weight):
    k = 4096
    print(f"case rotate_f6 prologue m={m} add={with_add} weight={with_weight}", flush=True)
    x = dev(syn.activations(m, k, seed=3 * m))
    add = dev((np.random.default_rng(m).standard_normal((m, k)) * 0.4).astype(np.float16)) if with_add else None
    w = dev(np.random.default_rng(1).uniform(0.5, 1.5, k).astype(np.float16)) if with_weight else None
    if with_add:
        total, enc, s = ops.rotate_and_quantize_f6(x, norm_weight=w, eps=1e-5, add=add)
        want_total, q, s_ref = ops.add_rmsnorm_rotate_and_quantize_i4(x, add, w, 1e-5)
        assert torch.equal(total, want_total)
    else:
        enc, s = ops.rotate_and_quantize_f6(x, norm_weight=w, eps=1e-5)
        q, s_ref = ops.rmsnorm_rotate_and_quantize_i4(x, w, 1e-5)
    assert torch.equal(s.view(torch.int16), s_ref.view(torch.int16))
    assert torch.equal(enc, ops.encode_f6(q))


@pytest.mark.parametrize("k", [11008, 14336])
@pytest.mark.parametrize("m", [5, 256, 601])
def test_dense_factor_rows_on_the_matrix_cores(ops, m, k):
    print(f"case rotate_f6 dense m={m} k={k}", flush=True)
    x = dev(syn.activations(m, k, seed=k + m))
    enc, s = ops.rotate_and_quantize_f6(x, clip_ratio=0.9 if m == 5 else 1.0)
    q, s_ref = ops.rotate_and_quantize_i4(x, hadamard="fast", clip_ratio=0.9 if m == 5 else 1.0)
    assert torch.equal(s.view(torch.int16), s_ref.view(torch.int16))
    assert torch.equal(enc, ops.encode_f6(q))


@pytest.mark.parametrize("k,n,grouped", [(4096, 384, False), (4096, 384, True), (14336, 256, True)])
def test_feeds_the_six_bit_gemm(ops, k, n, grouped):
    m = 300
    x = dev(syn.activations(m, k, seed=9))
    rng = np.random.default_rng(k)
    w = dev(rng.integers(0, 256, size=(n, k // 2), dtype=np.uint8))
    ws = dev(rng.uniform(0.005, 0.02, size=(n, k // 128 if grouped else 1)).astype(np.float16))
    enc, s = ops.rotate_and_quantize_f6(x)
    q, s_ref = ops.rotate_and_quantize_i4(x, hadamard=True)
    w6 = ops.encode_f6(w)
    got = ops.gemm_f6_dequant_o16_gs(enc, w6, s, ws) if grouped else ops.gemm_f6_dequant_o16(enc, w6, s, ws)
    want = ops.gemm_i4_dequant(q, w, s_ref, ws, 128)
    assert torch.equal(got.view(torch.int16), want.view(torch.int16))


def test_argument_errors(ops):
    x = torch.zeros(4, 4096, dtype=torch.float16, device="cuda")
    with pytest.raises(RuntimeError):
        ops.rotate_and_quantize_f6(x[:, :768].contiguous())
    with pytest.raises(RuntimeError):
        ops.rotate_and_quantize_f6(x, add=x.clone())                      # addition without the norm
    with pytest.raises(RuntimeError):
        ops.rotate_and_quantize_f6(torch.zeros(4, 11008, dtype=torch.float16, device="cuda"), eps=1e-5)
    with pytest.raises(RuntimeError):
        ops.rotate_and_quantize_f6(x.float())


def _unpack(q):
    """[M, K/2] u8 -> signed codes [M, K] int32 (low nibble first)"""
    b = q.to(torch.int32)
    lo, hi = b & 15, b >> 4
    c = torch.stack((lo, hi), dim=-1).reshape(q.size(0), -1)
    return torch.where(c > 7, c - 16, c)


@pytest.mark.parametrize("m", [3, 300, 2048])
@pytest.mark.parametrize("prologue", ["none", "rms", "rms_weight", "add_rms_weight"])
def test_matrix_core_rotation_of_4096_with_prologues(ops, m, prologue):
    """hadamard="fast" at K = 4096 behind RMSNorm / the residual addition, nibble and 6-bit output: not bit-exact by
    design (the matrix cores sum in their own order; the sum of squares of the norm too), so measured against the
    float32-butterfly launches -- codes one step apart at a rate below 1e-4, scales at most one fp16 step apart in a
    few rows per thousand; the residual sum is the same bits; the 6-bit output is the encoding of the same mode's
    nibble output, byte for byte."""
    k = 4096
    print(f"case fast 4096 m={m} {prologue}", flush=True)
    x = dev(syn.activations(m, k, seed=5 * m + 1))
    add = dev((np.random.default_rng(m).standard_normal((m, k)) * 0.4).astype(np.float16)) if prologue.startswith("add") else None
    w = dev(np.random.default_rng(2).uniform(0.5, 1.5, k).astype(np.float16)) if "weight" in prologue else None
    if prologue == "none":
        q, s = ops.rotate_and_quantize_i4(x, hadamard="fast")
        qe, se = ops.rotate_and_quantize_i4(x, hadamard="exact")
        enc, s6 = ops.rotate_and_quantize_f6(x, hadamard="fast")
    elif add is None:
        q, s = ops.rmsnorm_rotate_and_quantize_i4(x, w, 1e-5, hadamard="fast")
        qe, se = ops.rmsnorm_rotate_and_quantize_i4(x, w, 1e-5, hadamard="exact")
        enc, s6 = ops.rotate_and_quantize_f6(x, hadamard="fast", norm_weight=w, eps=1e-5)
    else:
        total, q, s = ops.add_rmsnorm_rotate_and_quantize_i4(x, add, w, 1e-5, hadamard="fast")
        total_e, qe, se = ops.add_rmsnorm_rotate_and_quantize_i4(x, add, w, 1e-5, hadamard="exact")
        total6, enc, s6 = ops.rotate_and_quantize_f6(x, hadamard="fast", norm_weight=w, eps=1e-5, add=add)
        assert torch.equal(total, total_e) and torch.equal(total6, total_e)       # the residual stream: the same bits
    diff = (_unpack(q) - _unpack(qe)).abs()
    s_step = (s.view(torch.int16).int() - se.view(torch.int16).int()).abs()
    print(f"  code mismatch rate {(diff != 0).float().mean().item():.2e}, scale mismatch rate "
          f"{(s_step != 0).float().mean().item():.2e}", flush=True)
    assert int(diff.max()) <= 1 and (diff != 0).float().mean().item() < 1e-4
    assert int(s_step.max()) <= 1 and (s_step != 0).float().mean().item() <= max(5e-3, 1.0 / m if m < 10 else 0)
    # the 6-bit output of the same mode: byte for byte the encoding of its nibble output
    assert torch.equal(s6.view(torch.int16), s.view(torch.int16))
    assert torch.equal(enc, ops.encode_f6(q))
