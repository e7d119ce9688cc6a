"""CPU-only tests of the host side: torch helpers against the oracle and the reference's
golden vectors, the C ABI library's exports, the exhaustive check behind the kernels'
quantisation step.  Nothing here launches a kernel."""
import pathlib
import re
import subprocess

import numpy as np
import pytest
import torch

import flh_amd
from flh_amd import _lib
from flh_amd.functional import hadamard as FH
from flh_amd.functional import quantization as FQ
from flh_amd.nn import ActQuantizer, LinearFLH, OnlineHadamard, RMSNorm, WeightQuantizer, fast_hadamard_transform
from oracle import hadamard as OH
from oracle import pack as OP

ROOT = pathlib.Path(__file__).resolve().parents[1]


def test_library_exports_every_declared_symbol():
    # the product interface and the header of the test / tuning entry points
    header = (ROOT / "include" / "flh_hip.h").read_text() + (ROOT / "include" / "flh_hip_testing.h").read_text()
    assert "flh_gemm_set_tuning" not in (ROOT / "include" / "flh_hip.h").read_text()
    declared = set(re.findall(r"^(?:int|void|size_t|const char\*)\s+(\w+)\(", header, re.M))
    assert declared == set(_lib.EXPORTS), declared ^ set(_lib.EXPORTS)
    lib = _lib.load()          # raises if the .so is missing or a symbol is not exported
    assert lib.flh_abi_version() == 1
    assert lib.flh_last_error() == b""
    # the reference's C++-linkage functions: one mangled export per declaration of the second header
    native = (ROOT / "include" / "flh_reference_native.h").read_text()
    declared_cxx = set(re.findall(r"^void\s+(\w+)\(", native, re.M))
    assert declared_cxx == set(_lib._SIG_CXX), declared_cxx ^ set(_lib._SIG_CXX)
    for name, mangled in _lib._SIG_CXX.items():
        assert name in mangled and "6__half" in mangled
        assert getattr(lib, mangled) is not None


def test_argument_errors_come_back_before_any_launch():
    """Shape and alignment errors are found on the host: the entry points return FLH_EINVAL with a message and
    never touch the pointers, so this runs without a device (the addresses below are never dereferenced)."""
    lib = _lib.load()
    ok, odd, st = 0x10000, 0x10008, None
    calls = [
        ("flh_gemm_i4_o16", (odd, ok, ok, ok, ok, 16, 128, 128, 1, 1, 128, st), b"16-byte aligned"),
        ("flh_gemm_i4_o16", (ok, ok, ok, ok, odd, 16, 128, 128, 1, 1, 128, st), b"16-byte aligned"),
        ("flh_gemm_i4_o16", (ok, ok, ok, ok, ok, 16, 128, 192, 1, 1, 128, st), b"multiple of 128"),
        ("flh_gemm_i4_o16", (ok, ok, ok, ok, ok, 16, 128, 256, 2, 5, 128, st), b"scale columns"),
        ("flh_gemm_i4_i32", (ok, odd, ok, 16, 128, 128, st), b"16-byte aligned"),
        ("flh_rotate_quant_i4", (odd, ok, ok, None, 4, 4096, 1, 0, 0, 1.0, st), b"16-byte aligned"),
        ("flh_rotate_quant_i4", (ok, ok, ok, odd, 4, 4096, 1, 0, 0, 1.0, st), b"16-byte aligned"),
        ("flh_group_quant_i4", (ok, odd, ok, 4, 128, 1, 1.0, st), b"16-byte aligned"),
        ("flh_fwht_f16_inplace", (odd, 4, 128, st), b"16-byte aligned"),
        ("flh_gemm_i4_swiglu_o16", (ok, ok, odd, ok, ok, ok, ok, 16, 128, 128, 1, 1, 128, st), b"16-byte aligned"),
        ("flh_gemm_i4_swiglu_o16", (ok, ok, ok, ok, ok, ok, ok, 16, 128, 192, 1, 1, 128, st), b"multiple of 128"),
        ("flh_gemm_f6_o16", (ok, odd, ok, ok, ok, 16, 128, 128, st), b"16-byte aligned"),
        ("flh_gemm_f6_o16_gs", (ok, ok, ok, ok, ok, 16, 128, 256, 3, 2, st), b"scale columns"),
        ("flh_gemm_f6_swiglu_o16", (ok, ok, ok, ok, ok, ok, ok, 16, 128, 256, 2, 5, st), b"scale columns"),
        ("flh_gemm_f6_i32", (ok, ok, ok, 16, 128, 100, st), b"multiple of 128"),
        ("flh_encode_f6", (ok, ok, 4, 100, st), b"multiple of 128"),
        ("flh_group_quant_f6", (odd, ok, ok, 4, 128, 1, 1.0, st), b"16-byte aligned"),
        ("flh_rotate_quant_f6", (ok, None, None, 0, None, 1e-5, ok, ok, 4, 1000, 1, 1.0, st), b"K (1000)"),
        ("flh_rotate_quant_f6", (ok, ok, None, 0, None, 1e-5, ok, ok, 4, 4096, 1, 1.0, st), b"come together"),
        ("flh_silu_mul_group_quant_i4", (ok, odd, ok, ok, 4, 128, 1, 1.0, st), b"16-byte aligned"),
        ("flh_rmsnorm_group_quant_i4", (ok, ok, ok, ok, 4, 100, 1e-5, 128, 1, 1.0, st), b"multiple of the group size"),
        ("flh_rmsnorm_rotate_quant_i4", (ok, ok, 1e-5, ok, ok, None, 4, 1000, 1, 1.0, st), b"K (1000)"),
        ("flh_add_rmsnorm_rotate_quant_i4", (ok, ok, ok, ok, 1e-5, ok, ok, 4, 4096, 1, 1.0, st), b"must not be x or add"),
        ("flh_silu_mul_rotate_quant_i4", (ok, ok, ok, ok, 4, 4096, st), b"11008 or 14336"),
        ("flh_silu_mul_rotate_quant_i4", (ok, ok, ok, ok, 1000, 11008, st), b"at most 256 rows"),
        ("flh_silu_mul_f16", (ok, ok, ok, 12, st), b"multiple of 8"),
        ("flh_rotate_quant_gemm_i4_o16", (ok, ok, ok, ok, 8, 128, 4096, 1, st), b"at most 4 tokens"),
        ("flh_rotate_quant_gemm_i4_o16", (ok, ok, ok, ok, 2, 128, 2048, 1, st), b"not supported"),
        ("flh_decode_attention_f16", (ok, ok, ok, ok, 1, 32, 8, 100, 16, 16, 1.0, ok, 1 << 20, st), b"head_dim"),
        ("flh_decode_attention_f16", (ok, ok, ok, ok, 1, 32, 8, 128, 2048, 2048, 1.0, ok, 16, st), b"workspace"),
        ("flh_decode_attention_f16_static", (ok, ok, ok, ok, 4096, 32, 8, 128, 8192, 8192, 1.0, st), b"static array"),
        ("flh_gemm_set_tuning", (100, 0), b"tile must be"),
        ("flh_prefill_attention_f16", (ok, ok, ok, ok, 1, 16, 8, 2, 64, 0, 64, 0.1, st), b"head_dim (64) must be 128"),
        ("flh_prefill_attention_f16", (ok, ok, ok, ok, 1, 16, 8, 3, 128, 0, 64, 0.1, st), b"do not divide"),
        ("flh_prefill_attention_f16", (ok, ok, ok, ok, 1, 16, 8, 2, 128, 60, 64, 0.1, st), b"exceeds the cache length"),
        ("flh_prefill_attention_f16", (ok, odd, ok, ok, 1, 16, 8, 2, 128, 0, 64, 0.1, st), b"16-byte aligned"),
        ("flh_gemm_i4_add_o16", (ok, ok, ok, ok, odd, ok, 16, 128, 128, 1, 1, 128, st), b"residual must be 16-byte aligned"),
        ("flh_gemm_i4_add_o16", (ok, ok, ok, ok, None, ok, 16, 128, 128, 1, 1, 128, st), b"null pointer"),
        ("flh_gemm_f6_add_o16", (ok, ok, ok, ok, ok, ok, 16, 128, 256, 3, 2, st), b"scale columns"),
    ]
    for name, args, message in calls:
        rc = getattr(lib, name)(*args)
        assert rc == -1, (name, args, rc)                       # FLH_EINVAL
        assert message in lib.flh_last_error(), (name, lib.flh_last_error())
    # the q / k / v launch with the rotary epilogue takes its three weight matrices and scales as pointer arrays
    import ctypes
    three = (ctypes.c_void_p * 3)(ok, ok, ok)
    rope = lambda **kw: lib.flh_gemm_i4_qkv_rope_o16(
        ok, ok, three, three, kw.get("cos", ok), ok, ok, ok, ok, ok, 2, 40, 4, kw.get("hkv", 2), 64, kw.get("k", 256),
        1, kw.get("b_cols", 1), kw.get("group", 128), st)
    for kw, message in (({"k": 192}, b"multiple of 128"), ({"hkv": 0}, b"must be positive"), ({"cos": odd}, b"16-byte aligned"),
                        ({"b_cols": 2, "group": 64}, b"groups of 128")):
        assert rope(**kw) == -1 and message in lib.flh_last_error(), (kw, lib.flh_last_error())
    rope6 = lambda **kw: lib.flh_gemm_f6_qkv_rope_o16(
        ok, ok, three, three, kw.get("cos", ok), ok, ok, ok, ok, ok, 2, 40, 4, kw.get("hkv", 2), 64, kw.get("k", 256),
        kw.get("a_cols", 1), kw.get("b_cols", 1), st)
    for kw, message in (({"k": 192}, b"multiple of 128"), ({"hkv": 0}, b"must be positive"), ({"cos": odd}, b"16-byte aligned"),
                        ({"a_cols": 3, "b_cols": 2}, b"scale columns")):
        assert rope6(**kw) == -1 and message in lib.flh_last_error(), (kw, lib.flh_last_error())


def test_ops_fail_loudly_without_library(monkeypatch, tmp_path):
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", tmp_path / "missing.so")
    with pytest.raises(_lib.FLHLibraryError):
        flh_amd._CUDA.gemm_i4_dequant_o16


def test_install_as_flh_aliases():
    flh_amd.install_as_flh()
    import flh
    import flh.nn
    assert flh.nn.LinearFLH is LinearFLH and flh._CUDA is flh_amd._CUDA
    t = flh.PackedQuantizedTensor(torch.zeros(2, 4, dtype=torch.uint8), torch.ones(2, 1))
    assert t.size() == (2, 4) and t.dtype == torch.uint8 and t.device.type == "cpu"


def test_quantisation_formula_exhaustive(tmp_path):
    exe = tmp_path / "divcheck"
    subprocess.run(["gcc", "-O2", "-mf16c", "-mavx", "-fopenmp", str(ROOT / "tests" / "native" / "divcheck.c"),
                    "-o", str(exe), "-lm"], check=True)
    r = subprocess.run([str(exe)], capture_output=True, text=True, timeout=600)
    assert r.returncode == 0, r.stdout
    assert "pairs=633628987" in r.stdout and "=0,0,0 one-step{r,r+,r-}=0,0,0" in r.stdout, r.stdout


def test_pack_unpack_match_oracle():
    rng = np.random.default_rng(0)
    q = rng.integers(-8, 8, size=(5, 3, 64))
    p = FQ.pack_i4(torch.from_numpy(q))
    assert np.array_equal(p.numpy(), OP.pack_i4(q))
    assert np.array_equal(FQ.unpack_i4(p).numpy(), q)
    with pytest.raises(AssertionError):
        FQ.pack_i4(torch.tensor([[9, 0]]))
    with pytest.raises(AssertionError):
        FQ.unpack_i4(torch.zeros(2, 2, dtype=torch.int8))
    assert FQ.two_compl(torch.tensor([-1, 3]), 4).tolist() == [15, 3]
    x = torch.tensor([0.26, -0.9, 2.0])
    assert FQ.sym_quant(x, torch.tensor(0.25), torch.tensor(7))[0].tolist() == [1.0, -4.0, 7.0]


def test_hadamard_helpers(golden):
    for k, digest in OH.HADK_SHA256_PREFIX.items():
        assert np.array_equal(getattr(FH, f"get_had{k}")().numpy(), OH.had_literal(k).astype(np.float32))
    assert FH.get_hadK(11008)[1] == 172 and FH.get_hadK(14336)[1] == 28 and FH.get_hadK(64) == (None, 1)
    for n in (28 * 4, 172 * 2, 4096, 12 * 8):
        x = torch.from_numpy(golden[f"hadU_{n}_x"])
        assert torch.allclose(FH.matmul_hadU(x.double()), torch.from_numpy(golden[f"hadU_{n}_f64"]), rtol=1e-12, atol=1e-12)
        assert torch.allclose(FH.matmul_hadU(x.float()), torch.from_numpy(golden[f"hadU_{n}_f32"]), rtol=2e-5, atol=2e-4)
        hk, k = FH.get_hadK(n)
        # same transform; the scale 1/sqrt(n) is formed in double here, in float32 by matmul_hadU
        assert torch.allclose(FH.matmul_hadU_cuda(x.double(), hk, k), torch.from_numpy(golden[f"hadU_{n}_f64"]), rtol=1e-6, atol=1e-7)
    x = torch.randn(3, 64, dtype=torch.float64)
    assert torch.allclose(FH.hadamard_transform(x), x @ torch.from_numpy(OH.sylvester(64).astype(np.float64)))
    h = FH.random_hadamard_matrix(16, "cpu")
    assert torch.allclose(h @ h.T, torch.eye(16, dtype=torch.float64), atol=1e-12)
    lin = torch.nn.Linear(24, 8, bias=False)   # 24 = 12 * 2
    w0 = lin.weight.data.clone()
    FH.apply_exact_had_to_linear(lin)
    assert torch.allclose(lin.weight.data, FH.matmul_hadU(w0), atol=1e-6)
    oh = OnlineHadamard(32, group_size=8)
    y = oh(torch.randn(2, 32))
    assert y.shape == (2, 32) and torch.equal(oh.hadamard_matrix[:8, :8], OnlineHadamard.hadamard(8))
    with pytest.raises(ValueError):
        OnlineHadamard(32, group_size=12)


def test_fast_hadamard_transform_golden(golden):
    y = fast_hadamard_transform(torch.from_numpy(golden["fht_full_2048_x"]), use_cuda=False)
    assert y.dtype == torch.float16 and np.array_equal(y.numpy(), golden["fht_full_2048_y"])
    y = fast_hadamard_transform(torch.from_numpy(golden["fht_g128_1024_x"]), group_size=128, use_cuda=False)
    assert np.array_equal(y.numpy(), golden["fht_g128_1024_y"])
    with pytest.raises(ValueError):
        fast_hadamard_transform(torch.zeros(2, 24), use_cuda=False)


def test_forward_origin_golden(golden):
    cases = {
        "pt_h_256": dict(group_size=-1, use_hadamard=True), "pt_h_4096": dict(group_size=-1, use_hadamard=True),
        "g128_h_512": dict(group_size=128, use_hadamard=True), "g128_n_512": dict(group_size=128, use_hadamard=False),
        "pt_n_1024": dict(group_size=-1, use_hadamard=False),
        "pt_h_clip_1024": dict(group_size=-1, use_hadamard=True, input_clip_ratio=0.9),
        "g64_h_clip_256": dict(group_size=64, use_hadamard=True, input_clip_ratio=0.85),
    }
    for name, kw in cases.items():
        x = torch.from_numpy(golden[f"fo_{name}_x"])
        scale, zp, packed = ActQuantizer(bits=4, sym=True, packed_output=True, **kw).forward_origin(x)
        assert np.array_equal(scale.numpy(), golden[f"fo_{name}_scale"]), name
        assert np.array_equal(packed.numpy(), golden[f"fo_{name}_packed"]), name
        _, _, codes = ActQuantizer(bits=4, sym=True, **kw).forward_origin(x)
        assert np.array_equal(codes.numpy().astype(np.int8), golden[f"fo_{name}_codes"]), name
    with pytest.raises(ValueError):
        ActQuantizer(bits=8, packed_output=True)
    s, z, q = ActQuantizer(bits=4, sym=False, group_size=64, use_hadamard=False).forward_origin(torch.randn(3, 128))
    assert s.shape == (3, 2) and q.min() >= 0 and q.max() <= 15


def test_weight_quantizer_and_from_float_golden(golden):
    for tag in ("f16", "f32"):
        for gs in (128, 512):
            for clip in (100, 90):
                key = f"wq_{tag}_g{gs}_c{clip}"
                wq = WeightQuantizer(bits=4, group_size=gs, sym=True, channel_wise=False, use_hadamard=False, clip_ratio=clip / 100)
                s, z, wi = wq(torch.from_numpy(golden[key + "_w"]))
                assert np.array_equal(s.numpy(), golden[key + "_scale"]), key
                assert np.array_equal(wi.numpy().astype(np.int8), golden[key + "_codes"]), key
        for mode in ("nohad", "had"):
            key = f"ff_{tag}_{mode}"
            lin = torch.nn.Linear(256, 64, bias=False)
            lin.weight.data = torch.from_numpy(golden[key + "_w"]).clone()
            layer = LinearFLH.from_float(lin, weight_group_size=128, in_group_size=128, no_hadamard=(mode == "nohad"))
            assert np.array_equal(layer.w_packed.numpy(), golden[key + "_packed"]), key
            assert np.array_equal(layer.w_scale.numpy(), golden[key + "_scale"]), key
    wq = WeightQuantizer(bits=4, group_size=-1, channel_wise=True, use_hadamard=False)   # the reference's broken branch works here
    s, _, wi = wq(torch.randn(8, 32))
    assert s.shape == (8, 1) and wi.abs().max() <= 8
    with pytest.raises(RuntimeError):
        WeightQuantizer(use_hadamard=False).quantize(torch.randn(4, 4))


def test_linear_forward_torch_is_dequantised_matmul():
    torch.manual_seed(0)
    lin = torch.nn.Linear(256, 32, bias=True)
    layer = LinearFLH.from_float(lin, weight_group_size=128, in_group_size=128, no_hadamard=True)
    w = layer.get_weight(torch.float32)
    assert w.shape == (32, 256) and (w - lin.weight.data).abs().max() < lin.weight.data.abs().max() / 7
    x = torch.randn(4, 256)
    aq = ActQuantizer(bits=4, group_size=128, use_hadamard=False, packed_output=True)
    s, z, qp = aq.forward_origin(x)
    y = layer.forward_torch(qp, s, None, x_is_packed=True)
    x_deq = (FQ.unpack_i4(qp).float().view(4, 2, 128) * s.unsqueeze(-1)).view(4, 256)
    assert torch.allclose(y, x_deq @ w.T + lin.bias.data, atol=1e-5)
    layer.set_weight(lin.weight.data)
    assert torch.equal(layer.get_weight(torch.float32), w)
    n = RMSNorm(256)
    assert torch.allclose(n(x).pow(2).mean(-1), torch.ones(4), atol=1e-3)


def test_guards_raise_value_error_on_cpu_tensors():
    from flh_amd import cuda as C
    x = torch.zeros(4, 128, dtype=torch.float16)
    for fn in (C.hadamard_transform_half, C.hadamard_and_quantize_i4, C.quant_and_pack_i4):
        with pytest.raises(ValueError):
            fn(x)
    with pytest.raises(ValueError):
        C.hadamard_transform_n(x, n=48)
    y = C.hadamard_transform(torch.ones(2, 8))          # torch path
    assert y[0].tolist() == [8, 0, 0, 0, 0, 0, 0, 0]
    from flh_amd.nn.linear_gs import LinearFLHGS
    from flh_amd.nn.quantization_gs import ActQuantizerGS, SimpleActQuantizerGS
    with pytest.raises(ValueError):
        LinearFLHGS(256, 8, group_size=48, device="cpu")
    with pytest.raises(ValueError):
        ActQuantizerGS(bits=8)
    with pytest.raises(ValueError):
        SimpleActQuantizerGS(group_size=16)
    layer = LinearFLHGS.from_float(torch.nn.Linear(128, 16), weight_group_size=64)
    assert layer.w_packed.shape == (16, 64) and layer.w_scale.shape == (16, 2) and layer.bias is not None


def test_checkpoint_round_trip_in_the_reference_layout(tmp_path):
    """model.pt + quantization_config.json (flh/quantized_model/modeling_llama.py:1079-1137): what a tree of
    LinearFLH layers writes, a freshly built tree reads back bit for bit; float32 tensors are stored as fp16."""
    import json
    from flh_amd.nn import LinearFLH, load_quantized, save_quantized

    def tree(fill):
        torch.manual_seed(3)
        block = torch.nn.ModuleDict({
            "q_proj": LinearFLH.from_float(torch.nn.Linear(256, 64, bias=True).half(), weight_group_size=128,
                                           in_group_size=128, no_hadamard=True) if fill else
            LinearFLH(256, 64, bias=True, in_group_size=128, group_size=128),
            "down_proj": LinearFLH.from_float(torch.nn.Linear(128, 32, bias=False).half(), weight_group_size=128,
                                              in_group_size=128, no_hadamard=True) if fill else
            LinearFLH(128, 32, bias=False, in_group_size=128, group_size=128),
            "norm": torch.nn.LayerNorm(8)})
        return block

    src = tree(True)
    save_quantized(src, tmp_path / "ckpt", weight_group_size=128, clip_ratio=0.9)
    cfg = json.loads((tmp_path / "ckpt" / "quantization_config.json").read_text())
    assert cfg == {"weight_bits": 4, "weight_group_size": 128, "act_bits": 4, "act_group_size": 128,
                   "weight_sym": True, "act_sym": True, "clip_ratio": 0.9, "dtype": "float16"}
    from flh_amd.nn.checkpoint import read_state_dict
    stored = read_state_dict(tmp_path / "ckpt" / "model.pt")
    assert stored["norm.weight"].dtype == torch.float16 and stored["q_proj.w_packed"].dtype == torch.uint8
    dst = tree(False)
    got = load_quantized(dst, tmp_path / "ckpt")
    assert got["clip_ratio"] == 0.9 and not got["missing_keys"] and not got["unexpected_keys"]
    for key, value in src.state_dict().items():
        other = dst.state_dict()[key]
        assert torch.equal(other.float(), value.half().float() if value.dtype == torch.float32 else value.float()), key
    with pytest.raises(ValueError):
        save_quantized(src, tmp_path / "bad", group=64)
    wrong = torch.nn.ModuleDict({"q_proj": LinearFLH(256, 64, bias=True, group_size=64),
                                 "down_proj": LinearFLH(128, 32, group_size=128), "norm": torch.nn.LayerNorm(8)})
    with pytest.raises(ValueError, match="do not fit"):
        load_quantized(wrong, tmp_path / "ckpt")


def test_state_dict_reader_takes_the_references_pickle_protocol_and_nothing_else(tmp_path):
    """The reference writes model.pt with pickle protocol 4 (flh/quantized_model/modeling_llama.py:1107), which
    torch's non-executing loader refuses; the allow-list reader returns the same tensors (shared storages, offsets and
    non-contiguous views included) and refuses a file that names any other global."""
    import collections
    import pickle
    from flh_amd.nn.checkpoint import read_state_dict
    base = torch.arange(48, dtype=torch.float16)
    state = collections.OrderedDict(
        packed=torch.randint(0, 256, (37, 5), dtype=torch.uint8), scale=torch.rand(7, 3).half(),
        view=base[8:32].view(4, 6), strided=base.view(6, 8).t(), other=base, i64=torch.arange(5), empty=torch.zeros(0, 4).half(),
        b=torch.tensor([True, False]), f32=torch.rand(3))
    for proto in (2, 4):
        path = tmp_path / f"m{proto}.pt"
        torch.save(state, path, pickle_protocol=proto)
        got = read_state_dict(path)
        assert list(got) == list(state)
        for k, v in state.items():
            assert got[k].dtype == v.dtype and got[k].shape == v.shape and torch.equal(got[k], v), (proto, k)
    with pytest.raises(pickle.UnpicklingError):
        torch.load(tmp_path / "m4.pt", weights_only=True)        # the reason the reader exists

    class Evil:
        def __reduce__(self):
            import os
            return (os.getcwd, ())
    bad = tmp_path / "bad.pt"
    torch.save({"x": torch.zeros(2), "y": Evil()}, bad, pickle_protocol=4)
    with pytest.raises(pickle.UnpicklingError, match="refused"):
        read_state_dict(bad)
    notdict = tmp_path / "list.pt"
    torch.save([torch.zeros(2)], notdict, pickle_protocol=4)
    with pytest.raises(pickle.UnpicklingError):
        read_state_dict(notdict)


def test_torch_extension_loads_and_checks_tensors_without_a_device():
    """The PyTorch-ROCm extension imports on a machine without a GPU, registers its dispatcher ops, and its tensor
    checks reject CPU tensors before anything touches the device."""
    ext = pytest.importorskip("flh_amd._flh_torch")
    for name in ("gemm_i4_dequant_o16", "gemm_i4_dequant_o16_gs", "hadamard_transform_half", "hadamard_transform_64_half",
                 "hadamard_transform_32_half", "hadamard_and_quantize_i4", "quant_and_pack_i4",
                 "hadamard_and_quantize_i4_gs", "quant_and_pack_i4_gs"):      # flh_cuda_bindings.cpp:301-313
        assert hasattr(ext, name) and hasattr(torch.ops.flh_hip, name)
    a, s = torch.zeros(2, 64, dtype=torch.uint8), torch.zeros(2, 1, dtype=torch.float16)
    with pytest.raises(RuntimeError, match="CUDA"):
        ext.gemm_i4_dequant_o16(a, a, s, s)
    with pytest.raises(RuntimeError, match="CUDA"):
        ext.quant_and_pack_i4(torch.zeros(2, 128, dtype=torch.float16))


def test_model_checkpoint_directory_uses_the_references_key_names(tmp_path):
    """W4A4LlamaModel.save_quantized / from_quantized: the reference's directory layout (model.pt written with pickle
    protocol 4 under the key names of its transformers model, quantization_config.json, config.json), read back without
    executing anything from the file; every tensor survives the round trip."""
    import json
    import torch
    from flh_amd.nn.checkpoint import read_state_dict
    from flh_amd.quantized_model.llama import LlamaShape, W4A4LlamaModel, reference_key
    assert reference_key("layers.3.q_proj.w_packed") == "model.layers.3.self_attn.q_proj.w_packed"
    assert reference_key("layers.0.down_proj.w_scale") == "model.layers.0.mlp.down_proj.w_scale"
    assert reference_key("layers.1.input_layernorm.weight") == "model.layers.1.input_layernorm.weight"
    assert reference_key("norm.weight") == "model.norm.weight" and reference_key("lm_head.weight") == "lm_head.weight"
    assert reference_key("embed_tokens.weight") == "model.embed_tokens.weight"
    shape = LlamaShape(256, 4, 2, 512, 2, 100, 1e-6, 12345.0)
    gen = torch.Generator().manual_seed(0)
    model = W4A4LlamaModel(shape, activation="group", device="cpu")
    with torch.no_grad():
        for t in model.state_dict().values():
            if t.dtype == torch.uint8:
                t.copy_(torch.randint(0, 256, t.shape, dtype=torch.uint8, generator=gen))
            else:
                t.copy_(torch.randn(t.shape, generator=gen).half().to(t.dtype))
    model.save_quantized(tmp_path, clip_ratio=0.9)
    raw = read_state_dict(tmp_path / "model.pt")
    assert "model.layers.1.mlp.gate_proj.w_packed" in raw and "model.norm.weight" in raw
    assert raw["model.norm.weight"].dtype == torch.float16                      # float32 tensors are stored as float16
    assert json.load(open(tmp_path / "quantization_config.json"))["clip_ratio"] == 0.9
    cfg = json.load(open(tmp_path / "config.json"))
    assert cfg["num_key_value_heads"] == 2 and cfg["rope_theta"] == 12345.0
    again = W4A4LlamaModel.from_quantized(tmp_path, device="cpu")
    assert again.shape.num_kv_heads == 2 and again.shape.eps == 1e-6 and again.activation == "group"
    a, b = model.state_dict(), again.state_dict()
    assert set(a) == set(b) and all(torch.equal(a[k], b[k]) for k in a)
    # weight_sym false, or absent (which the reference's loader reads as false): refused unless the caller vouches
    # that the stored codes are signed nibbles
    import pytest
    qc = json.load(open(tmp_path / "quantization_config.json"))
    for variant in ({**qc, "weight_sym": False}, {k: v for k, v in qc.items() if k != "weight_sym"}):
        json.dump(variant, open(tmp_path / "quantization_config.json", "w"))
        with pytest.raises(ValueError, match="weight_sym"):
            W4A4LlamaModel.from_quantized(tmp_path, device="cpu")
        vouched = W4A4LlamaModel.from_quantized(tmp_path, device="cpu", assume_symmetric_weights=True).state_dict()
        assert all(torch.equal(a[k], vouched[k]) for k in a)
    # a checkpoint that lacks a tensor is refused
    del raw["model.layers.0.self_attn.k_proj.w_scale"]
    with pytest.raises(KeyError):
        W4A4LlamaModel(shape, activation="group", device="cpu").load_reference_state_dict(raw)
