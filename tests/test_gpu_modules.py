"""The reference's module-level API on the GPU, checked against the CPU oracle."""
import numpy as np
import pytest
import torch

import flh_amd
from flh_amd import synthetic as syn
from flh_amd.nn import ActQuantizer, LinearFLH
from flh_amd.nn.linear_gs import LinearFLHGS
from flh_amd.nn.quantization_gs import ActQuantizerGS, SimpleActQuantizerGS

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    return t.detach().cpu().numpy()


@pytest.mark.parametrize("had", [True, False])
def test_act_quantizer_forward_matches_kernel_oracle(had):
    from oracle import quant as Q
    from oracle.pack import pack_i4
    x = syn.activations(2 * 5, 512, seed=3).reshape(2, 5, 512)
    scale, zp, q = ActQuantizer(bits=4, group_size=128, use_hadamard=had)(dev(x))
    sr, qr = Q.act_quantizer_forward(x, 128, had)
    assert zp is None and scale.shape == (2, 5, 4) and q.shape == (2, 5, 256)
    assert np.array_equal(host(scale).view(np.uint16), sr.view(np.uint16))
    assert np.array_equal(host(q), pack_i4(qr))


def test_act_quantizer_kernel_vs_forward_origin_close():
    # the reference's own smoke check (test/test_had_and_quant.py): kernel path vs torch path;
    # they differ by fp16-vs-fp64 butterfly rounding, so compare dequantised values
    x = syn.activations(64, 2048, seed=4)
    aq = ActQuantizer(bits=4, group_size=128, use_hadamard=True, packed_output=True)
    s, _, q = aq(dev(x))
    s0, _, q0 = aq.forward_origin(torch.from_numpy(x))
    from flh_amd.functional import unpack_i4
    a = unpack_i4(q.cpu()).float().view(64, 16, 128) * s.cpu().float().unsqueeze(-1)
    b = unpack_i4(q0).float().view(64, 16, 128) * s0.float().unsqueeze(-1)
    assert (a - b).abs().max() <= 1.01 * s0.float().max()          # at most one quantisation step
    step = s0.float().unsqueeze(-1)
    assert ((a - b).abs() > 0.5 * step).float().mean() < 0.02   # codes differ only near rounding ties


def test_per_token_quantizer_and_linear_config1():
    """The reference's own small case: X [16, 4096], 4096-point rotation, per-token x per-channel."""
    from oracle import linear as L
    m, k, n = 16, 4096, 4096
    x = syn.activations(m, k, seed=0)
    wq = syn.pack_codes(syn.weight_codes(n, k, seed=1))
    ws = syn.weight_scales(n, 1, seed=2)
    layer = LinearFLH(k, n, group_size=-1, device="cuda")
    layer.w_packed.copy_(dev(wq).flatten())
    layer.w_scale.copy_(dev(ws))
    aq = ActQuantizer(bits=4, per_token=True)
    scale, _, q = aq(dev(x))
    y = layer(q, scale, None, x_is_packed=True)
    ref, ap, asc = L.w4a4_linear(x, wq, ws, "f32")
    assert np.array_equal(host(q), ap) and np.array_equal(host(scale).view(np.uint16), asc.view(np.uint16))
    assert np.array_equal(host(y).view(np.uint16), ref.view(np.uint16))
    # and against the exactly rounded (float64) rotation: tolerance of the path
    ref64, _, _ = L.w4a4_linear(x, wq, ws, "exact")
    assert np.allclose(host(y).astype(np.float64), ref64.astype(np.float64), rtol=1e-3, atol=0.35)  # one code flip moves y by ~scale*w
    assert (host(y).view(np.uint16) != ref64.view(np.uint16)).mean() < 0.02


@pytest.mark.parametrize("shape", [(1, 10, 2048, 2048), (3, 7, 512, 384)])
def test_linear_flh_module_flow(shape):
    """ActQuantizer -> LinearFLH as test/test_linear.py does, against the oracle of the same flow
    and against the module's own torch path."""
    from oracle import linear as L
    b, t, k, n = shape
    torch.manual_seed(0)
    lin = torch.nn.Linear(k, n, bias=False).half()
    layer = LinearFLH.from_float(lin, weight_bits=4, weight_group_size=128, weight_sym=True, in_group_size=128)
    layer_gpu = LinearFLH(k, n, group_size=128, in_group_size=128, device="cuda")
    layer_gpu.load_state_dict(layer.state_dict())
    x = syn.activations(b * t, k, seed=5).reshape(b, t, k)
    a_scale, zp, q = ActQuantizer(bits=4, group_size=128, use_hadamard=True)(dev(x))
    y = layer_gpu(q, a_scale, zp, x_is_packed=True)
    assert y.shape == (b, t, n) and y.dtype == torch.float16
    ref, sr, pr = L.flh_module_forward(x, layer.w_packed.numpy().reshape(n, k // 2), layer.w_scale.numpy(), 128, True)
    assert np.array_equal(host(q), pr)
    assert np.allclose(host(y).astype(np.float64), ref.astype(np.float64), rtol=1e-3, atol=1e-2)
    yt = layer_gpu.forward_torch(q, a_scale, zp, x_is_packed=True)
    assert torch.allclose(y.float(), yt.float(), rtol=2e-2, atol=2e-2)
    # the rotation cancels: (H x) . (H w) = x . w  up to quantisation noise
    full = torch.from_numpy(x).float() @ lin.weight.data.float().T
    err = (y.cpu().float() - full).abs().mean() / full.abs().mean()
    assert err < 0.35


@pytest.mark.parametrize("g", [32, 64, 128])
def test_gs_modules(g):
    from oracle import quant as Q
    from oracle.pack import pack_i4
    x = syn.activations(24, 4 * g, seed=g)
    s, zp, q = ActQuantizerGS(group_size=g)(dev(x))
    sr, qr = Q.act_quantizer_forward(x, g, True)
    assert np.array_equal(host(q), pack_i4(qr)) and np.array_equal(host(s).view(np.uint16), sr.view(np.uint16))
    assert zp.dtype == torch.uint8 and int(zp.sum()) == 0
    s2, _, q2 = SimpleActQuantizerGS(group_size=g)(dev(x))
    qk, sk, _ = Q.kernel_had_and_quant(x.reshape(-1, g), g, False)
    assert np.array_equal(host(q2), pack_i4(qk).reshape(24, -1)) and np.array_equal(host(s2).reshape(-1).view(np.uint16), sk.view(np.uint16))
    lin = torch.nn.Linear(4 * g, 256, bias=True).half()
    layer = LinearFLHGS.from_float(lin, weight_group_size=g).cuda()
    y = layer(q, s)
    from oracle import gemm as G
    ref, _ = G.gemm_i4_dequant(host(q), layer.w_packed.cpu().numpy(), host(s), layer.w_scale.cpu().numpy(), g)
    assert np.allclose(host(y).astype(np.float64), ref.astype(np.float64) + lin.bias.data.numpy().astype(np.float64), rtol=2e-3, atol=2e-2)
    with pytest.raises(ValueError):
        layer(q, s[:, :2].contiguous())


def test_cuda_wrappers():
    from flh_amd import cuda as C
    from oracle import hadamard as H
    x = syn.activations(50, 128, seed=9)
    xd = dev(x)
    y = C.hadamard_transform(xd, scale=0.5)
    ref = (H.fwht_butterfly(x, np.float16, 128).astype(np.float32) * np.float32(0.5)).astype(np.float16)
    assert np.array_equal(host(xd), x) and np.array_equal(host(y), ref)
    y64 = C.hadamard_transform_n(dev(x[:, :64].copy()), n=64)
    assert np.array_equal(host(y64), H.fwht_butterfly(x[:, :64], np.float16, 64))
    q, s = C.hadamard_and_quantize_i4(xd)
    assert q.shape == (50, 64) and s.shape == (50,)
    with pytest.raises(ValueError):
        C.quant_and_pack_i4(xd[:, :64])
    assert flh_amd.cuda.load_flh_cuda_ext().gemm_i4_dequant_o16 is flh_amd._CUDA.gemm_i4_dequant_o16


def test_config3_group_weight_scales_per_token_activations():
    """Per-token activation scale x g=128 weight scales (the Llama-3 weight-group configuration)."""
    from oracle import linear as L
    m, k, n = 16, 4096, 1024
    x = syn.activations(m, k, seed=11)
    wq = syn.pack_codes(syn.weight_codes(n, k, seed=12))
    ws = syn.weight_scales(n, k // 128, seed=13)
    q, s = flh_amd._CUDA.rotate_and_quantize_i4(dev(x))
    y = flh_amd._CUDA.gemm_i4_dequant_o16(q, dev(wq), s, dev(ws))
    ref, ap, asc = L.w4a4_linear(x, wq, ws, "f32", 128)
    assert np.array_equal(host(q), ap)
    assert np.allclose(host(y).astype(np.float64), ref.astype(np.float64), rtol=1e-3, atol=1e-2)


@pytest.mark.parametrize("group", [32, 64, 128, -1])
def test_weight_preparation_on_the_gpu_equals_the_tensor_arithmetic(group):
    """LinearFLH.set_weight / from_float on fp16 CUDA weights run the HIP quantise-and-pack kernel; the bytes
    and scales must equal what the same module computes with tensor arithmetic on the CPU."""
    import flh_amd
    torch.manual_seed(group + 40)
    n, k = 96, 1024
    w = (torch.randn(n, k) * 0.05).half()
    lin = torch.nn.Linear(k, n, bias=False).half()
    lin.weight.data.copy_(w)
    cpu = flh_amd.nn.LinearFLH.from_float(lin, weight_group_size=group, in_group_size=128, no_hadamard=True)
    gpu = flh_amd.nn.LinearFLH.from_float(lin.cuda(), weight_group_size=group, in_group_size=128, no_hadamard=True)
    assert gpu.w_packed.is_cuda
    assert torch.equal(gpu.w_packed.cpu(), cpu.w_packed)
    assert torch.equal(gpu.w_scale.cpu().view(torch.int16), cpu.w_scale.view(torch.int16))
    assert not gpu.w_zero.any()


def test_weight_preparation_on_the_gpu_golden(golden):
    """The reference's own from_float bytes (no rotation; the rotated case goes through the 128-group
    kernel on the GPU and the float64 path on the CPU, as in the reference, and is compared elsewhere)."""
    import flh_amd
    w = torch.from_numpy(golden["ff_f16_nohad_w"])
    lin = torch.nn.Linear(w.shape[1], w.shape[0], bias=False).half()
    lin.weight.data.copy_(w)
    q = flh_amd.nn.LinearFLH.from_float(lin.cuda(), weight_bits=4, weight_group_size=128, weight_sym=True,
                                        in_group_size=128, no_hadamard=True)
    assert np.array_equal(q.w_packed.cpu().numpy(), golden["ff_f16_nohad_packed"])
    assert np.array_equal(q.w_scale.cpu().numpy().view(np.uint16), golden["ff_f16_nohad_scale"].view(np.uint16))


def test_fused_producer_modules_feed_linear_gs():
    """RMSNormQuant / SiluMulQuant in place of (RMSNorm | silu * up) + SimpleActQuantizerGS: same triple
    layout, and the linear layer accepts it; outputs agree with the unfused module chain to the quantiser's
    last-bit tolerance."""
    from flh_amd.nn import RMSNorm, RMSNormQuant, SiluMulQuant
    torch.manual_seed(3)
    m, k, inter, g = 64, 512, 1024, 128
    x = (torch.randn(m, k, device="cuda") * 2).half()
    norm = RMSNorm(k).cuda().half()
    norm.weight.data.uniform_(0.5, 1.5)
    fused = RMSNormQuant(k, eps=norm.eps, group_size=g).cuda()
    fused.weight.data.copy_(norm.weight.data)
    quant = SimpleActQuantizerGS(group_size=g)
    s0, z0, q0 = quant(norm(x))
    s1, z1, q1 = fused(x)
    assert s1.shape == s0.shape and q1.shape == q0.shape and z1.shape == z0.shape and not z1.any()
    assert (s1.view(torch.int16) - s0.view(torch.int16)).abs().max() <= 1
    same = (s1 == s0).repeat_interleave(g // 2, dim=-1)
    assert ((q1 != q0) & same).float().mean() < 1e-3
    gate, up = (torch.randn(m, inter, device="cuda") * 2).half(), torch.randn(m, inter, device="cuda").half()
    s2, z2, q2 = SiluMulQuant(group_size=g)(gate, up)
    s3, z3, q3 = quant(torch.nn.functional.silu(gate) * up)
    assert (s2.view(torch.int16) - s3.view(torch.int16)).abs().max() <= 1
    same = (s2 == s3).repeat_interleave(g // 2, dim=-1)
    assert ((q2 != q3) & same).float().mean() < 1e-3
    lin = LinearFLHGS(inter, 256, group_size=g)
    lin.w_packed.copy_(dev(syn.pack_codes(syn.weight_codes(256, inter, seed=5))))
    lin.w_scale.copy_(dev(syn.weight_scales(256, inter // g, seed=6)))
    y_fused, y_chain = lin(q2, s2), lin(q3, s3)
    assert torch.allclose(y_fused.float(), y_chain.float(), rtol=2e-2, atol=2e-2)
    assert (y_fused != y_chain).float().mean() < 0.05


@pytest.mark.parametrize("group", [128, -1])
def test_linear_flh_six_bit_switch_gives_the_same_bits(group):
    """LinearFLH.six_bit = True routes prefill-sized calls through the 6-bit matrix instruction: same
    outputs bit for bit, for per-channel and for group-of-128 weight scales; short batches stay on the int8
    kernels."""
    torch.manual_seed(group + 200)
    n, k, m = 384, 1024, 512
    lin = torch.nn.Linear(k, n, bias=True).half().cuda()
    layer = LinearFLH.from_float(lin, weight_group_size=group, in_group_size=128, no_hadamard=True)
    x = (torch.randn(m, k, device="cuda") * 2).half()
    q, s = flh_amd._CUDA.rotate_and_quantize_i4(x, hadamard=False)             # one scale per token
    layer.six_bit = False
    want = layer(q, s, x_is_packed=True)
    assert layer._w6 is None
    layer.six_bit = True
    got = layer(q, s, x_is_packed=True)
    assert layer._w6 is not None and torch.equal(got, want)
    short = layer(q[:8].contiguous(), s[:8].contiguous(), x_is_packed=True)       # below six_bit_min_rows
    assert torch.equal(short, want[:8])


@pytest.mark.parametrize("had", [False, True])
def test_six_bit_quantiser_feeds_linear_flh(had):
    """ActQuantizerGS(six_bit=True) -> LinearFLH with group-of-128 weight scales: the reference's group
    configuration end to end on the 6-bit matrix instruction, same bits as the int8 kernels."""
    torch.manual_seed(7 + had)
    n, k, m = 256, 1024, 300
    lin = torch.nn.Linear(k, n, bias=False).half().cuda()
    layer = LinearFLH.from_float(lin, weight_group_size=128, in_group_size=128, no_hadamard=True)
    x = (torch.randn(2, m // 2, k, device="cuda") * 2).half()            # a leading batch dimension
    s4, z4, q4 = ActQuantizerGS(group_size=128, use_hadamard=had)(x)
    s6, z6, q6 = ActQuantizerGS(group_size=128, use_hadamard=had, six_bit=True)(x)
    assert torch.equal(s4, s6) and q6.shape == (2, m // 2, k // 128 * 96)
    layer.six_bit = False
    want = layer(q4, s4, z4, x_is_packed=True)
    assert layer._w6 is None
    got = layer(q6, s6, z6, x_is_packed=True)
    assert got.shape == want.shape and torch.equal(got, want)
    layer.six_bit = None           # automatic: group-scaled weights take the 6-bit instruction from 256 rows on
    assert torch.equal(layer(q4, s4, z4, x_is_packed=True), want)


@pytest.mark.parametrize("tokens,group", [(1, 0), (2, 128), (7, 0), (7, 128)])
def test_forward_online_is_rotation_plus_forward(tokens, group):
    """LinearFLH.forward_online = whole-row rotation + per-token quantiser + forward; the one- and two-token
    calls go through the single-launch decode kernel and must give the same bits."""
    torch.manual_seed(tokens + group)
    n, k = 384, 4096
    lin = torch.nn.Linear(k, n, bias=True).half().cuda()
    layer = LinearFLH.from_float(lin, weight_group_size=group if group else k, no_hadamard=True)
    x = (torch.randn(1, tokens, k, device="cuda") * 1.5).half()
    q, s = flh_amd._CUDA.rotate_and_quantize_i4(x.view(-1, k), hadamard="exact")
    want = layer(q.view(1, tokens, k // 2), s.view(1, tokens, 1), None, x_is_packed=True)
    got = layer.forward_online(x)
    assert got.shape == (1, tokens, n) and torch.equal(got, want)


@pytest.mark.parametrize("tokens,group", [(300, 128), (300, 0), (3, 128)])
def test_forward_many_equals_separate_calls(tokens, group):
    """LinearFLH.forward_many: the projections that share a quantised input in one launch, same bits."""
    torch.manual_seed(tokens)
    k = 1024
    layers = [LinearFLH.from_float(torch.nn.Linear(k, n, bias=b).half().cuda(), weight_group_size=group if group else k,
                                   in_group_size=128, no_hadamard=True) for n, b in ((512, False), (128, True), (136, False))]
    x = (torch.randn(2, tokens, k, device="cuda") * 2).half()
    if group:
        s, z, q = ActQuantizerGS(group_size=128, use_hadamard=True)(x)
    else:
        q, s = flh_amd._CUDA.rotate_and_quantize_i4(x.view(-1, k), hadamard="exact")
        q, s = q.view(2, tokens, k // 2), s.view(2, tokens, 1)
    got = LinearFLH.forward_many(layers, q, s)
    for y, layer in zip(got, layers):
        assert torch.equal(y, layer(q, s, None, x_is_packed=True))


@pytest.mark.parametrize("group", [128, 0])
def test_forward_many_on_the_six_bit_path(group):
    """Layers that opted into the 6-bit matrix instruction share one launch there too; same bits as the int8 path."""
    torch.manual_seed(11)
    k, tokens = 1024, 300
    layers = [LinearFLH.from_float(torch.nn.Linear(k, n, bias=False).half().cuda(), weight_group_size=group if group else k,
                                   in_group_size=128, no_hadamard=True) for n in (512, 128, 136)]
    x = (torch.randn(tokens, k, device="cuda") * 2).half()
    if group:
        s, z, q = ActQuantizerGS(group_size=128, use_hadamard=True)(x)
    else:
        q, s = flh_amd._CUDA.rotate_and_quantize_i4(x, hadamard="exact")
    for layer in layers:
        layer.six_bit = False
    want = LinearFLH.forward_many(layers, q, s)
    assert all(layer._w6 is None for layer in layers)
    for layer in layers:
        layer.six_bit = True
    got = LinearFLH.forward_many(layers, q, s)
    assert all(layer._w6 is not None for layer in layers)
    for a, b in zip(got, want):
        assert torch.equal(a, b)


@pytest.mark.parametrize("g", [128, 64])
def test_hql_linear4bit_alias(g):
    """The legacy names of the reference's linear benchmark (benchmark_linear4bit.py:495-508): weights prepared with
    hql.had_and_quant, forward on fp16 activations.  Codes / scales of both operands against the oracle's group kernel,
    the output against the oracle GEMM on them, and against x @ W.T as the benchmark's own error check does."""
    from oracle import gemm as G
    from oracle import quant as Q
    from oracle.pack import pack_i4
    import flh_amd.hql as hql
    hql.install_as_hql()
    from hql.nn import Linear4bit
    k, n, m = 1024, 384, 40
    rng = np.random.default_rng(g)
    w = (rng.standard_normal((n, k)) * 0.02).astype(np.float16)
    x = syn.activations(m, k, seed=3 + g)
    layer = Linear4bit(k, n, bias=False, dtype=torch.float16, group_size=g).cuda()
    qw, sw = hql.had_and_quant(dev(w).view(-1, g))
    layer.weight.copy_(qw.reshape(-1, k // 2))
    layer.weight_scales.copy_(sw.reshape(-1, k // g))
    qwr, swr, _ = Q.kernel_had_and_quant(w.reshape(-1, g), g, True)
    assert np.array_equal(host(layer.weight), pack_i4(qwr).reshape(n, k // 2))
    assert np.array_equal(host(layer.weight_scales).view(np.uint16), swr.reshape(n, -1).view(np.uint16))
    y = host(layer(dev(x)))
    qxr, sxr, _ = Q.kernel_had_and_quant(x.reshape(-1, g), g, True)
    sx = (sxr.astype(np.float32) * np.float32(1.0 / g)).astype(np.float16).reshape(m, -1)
    ref, _ = G.gemm_i4_dequant(pack_i4(qxr).reshape(m, k // 2), pack_i4(qwr).reshape(n, k // 2), sx, swr.reshape(n, -1), group=g)
    assert np.allclose(y.astype(np.float64), ref.astype(np.float64), rtol=1e-3, atol=1e-2)
    full = x.astype(np.float64) @ w.astype(np.float64).T
    assert np.linalg.norm(y - full) / np.linalg.norm(full) < 0.3


def test_checkpoint_load_gives_the_same_forward_bits(tmp_path):
    """A tree of LinearFLH layers saved in the reference's layout (model.pt in pickle protocol 4 +
    quantization_config.json) and loaded into a freshly built tree on the GPU: the same forward bits, also on the
    6-bit path whose second encoding of the weights is rebuilt after the load."""
    from flh_amd.nn import load_quantized, save_quantized
    torch.manual_seed(5)

    def tree(fill):
        mk = lambda k, n: (LinearFLH.from_float(torch.nn.Linear(k, n, bias=False).half(), weight_group_size=128,
                                                in_group_size=128, no_hadamard=True) if fill
                           else LinearFLH(k, n, in_group_size=128, group_size=128))
        return torch.nn.ModuleDict({"up": mk(512, 384), "down": mk(384, 512)})

    src = tree(True).cuda()
    x = dev(syn.activations(300, 512, seed=2))
    quant = ActQuantizer(bits=4, group_size=128, use_hadamard=False, packed_output=True)

    def run(model):
        s, z, q = quant(x)
        h = model["up"](q, s, z, x_is_packed=True)
        s, z, q = quant(h)
        return h, model["down"](q, s, z, x_is_packed=True)
    want = run(src)
    save_quantized(src, tmp_path / "ckpt")
    dst = tree(False)
    dst["up"].six_bit = True
    dst = dst.cuda()
    before = run(dst)                                    # zero weights: builds the 6-bit encoding of the empty layer
    assert float(before[1].abs().max()) == 0.0
    load_quantized(dst, tmp_path / "ckpt", device="cuda")
    got = run(dst)
    assert torch.equal(got[0], want[0]) and torch.equal(got[1], want[1])


def test_gptq_on_the_gpu_matches_the_oracle():
    """FLHGPTQ with the layer and the calibration inputs on the GPU (float32 tensor arithmetic there) against the
    float64 elimination form of oracle/gptq.py, then packed by LinearFLH.from_float and run through the GEMM."""
    from flh_amd.nn import FLHGPTQ
    from oracle import gptq as OG
    from oracle import hadamard as OH
    rng = np.random.default_rng(6)
    cols, rows = 512, 64
    mix = rng.standard_normal((cols, cols)) * 2.0 / np.sqrt(cols) + np.eye(cols)
    x = rng.standard_normal((1500, cols)) @ mix
    w = (rng.standard_normal((rows, cols)) * 0.05).astype(np.float32)
    layer = torch.nn.Linear(cols, rows, bias=False).cuda()
    layer.weight.data.copy_(torch.from_numpy(w))
    g = FLHGPTQ(layer)
    g.add_batch(torch.from_numpy(x).float().cuda(), None, group_size=128)
    g.fasterquant(group_size=128, actorder=True)
    got = layer.weight.data.cpu().numpy().astype(np.float64)
    want = OG.gptq(w.astype(np.float64), OG.hessian([x], 128), group_size=128, actorder=True)
    scales, gsz = OG.grid_scales(OH.had_transform(w.astype(np.float64), 128), 128)
    diff = np.abs(got - want) / np.repeat(scales, gsz, axis=1)
    # float32 on the device against float64: a column that rounds the other way feeds a different error to the columns
    # after it OF THE SAME ROW, which can move a few of them by a step in turn -- whole rows stay equal otherwise
    off = diff > 1e-3
    assert off.mean() < 0.02 and diff.max() < 2.5 and off.any(axis=1).mean() < 0.25
    xr = OH.had_transform(x, 128)
    wr = OH.had_transform(w.astype(np.float64), 128)
    e_got, e_want = np.linalg.norm(xr @ (got - wr).T), np.linalg.norm(xr @ (want - wr).T)
    assert abs(e_got - e_want) < 0.05 * e_want               # the same quality on the calibration inputs
    packed = LinearFLH.from_float(layer.half(), weight_group_size=128, in_group_size=128, no_hadamard=True)
    xs = dev(syn.activations(40, cols, seed=1))
    s, z, q = ActQuantizer(bits=4, group_size=128, use_hadamard=True, packed_output=True)(xs)
    y = packed(q, s, z, x_is_packed=True)
    full = OH.had_transform(host(xs).astype(np.float64), 128) @ got.T       # rotated inputs x rotated GPTQ weights
    assert np.linalg.norm(host(y) - full) / np.linalg.norm(full) < 0.25
    g.free()


def test_gptq_on_the_gpu_against_the_references_weights():
    """The fixture of the reference's own GPTQ (tests/golden/gptq_vectors.npz: groups of 128 / one scale per row,
    activation order on / off, clip 1.0 / 0.9; reproduced bit for bit by the same code on the CPU,
    tests/test_oracle_gptq.py) with layer and calibration inputs on the GPU: float32 sums in the device's order, so a
    column on a rounding boundary may flip and move later codes of ITS ROW by a step -- most rows must equal the
    reference's exactly, every weight must stay within two steps of it, and a wrong group index (a scale of another
    group applied to a column) would show as a whole column off."""
    import pathlib
    import sys
    from flh_amd.nn import FLHGPTQ
    here = pathlib.Path(__file__).parent / "golden"
    sys.path.insert(0, str(here))
    import gptq_inputs as G
    v = np.load(here / "gptq_vectors.npz")
    w = torch.from_numpy(G.weight())
    batches = [torch.from_numpy(b).cuda() for b in G.calibration_batches()]
    for label, g, act, clip in G.CASES:
        layer = torch.nn.Linear(G.COLS, G.ROWS, bias=False).cuda()
        layer.weight.data.copy_(w)
        q = FLHGPTQ(layer)
        for b in batches:
            q.add_batch(b, None, group_size=g)
        q.fasterquant(group_size=g, blocksize=128, percdamp=0.01, actorder=act, sym=True, bits=4, clip_ratio=clip)
        got, ref = layer.weight.data.cpu().numpy().astype(np.float64), v[f"weight_{label}"].astype(np.float64)
        step = np.abs(ref).max(axis=1, keepdims=True) / 7.0 if g < 0 else \
            np.repeat(np.abs(ref.reshape(G.ROWS, -1, g)).max(axis=2) / 7.0, g, axis=1)      # >= the grid step of the element
        off = np.abs(got - ref) > 1e-6
        print(f"case gptq fixture {label}: {off.mean():.4f} of the weights, {off.any(axis=1).mean():.3f} of the rows differ", flush=True)
        assert off.any(axis=1).mean() <= 0.25 and off.mean() < 0.03, label
        assert (np.abs(got - ref) <= 2.01 * np.maximum(step, 1e-12)).all(), label
        assert off.all(axis=0).sum() == 0, label                                          # no column is off as a whole
