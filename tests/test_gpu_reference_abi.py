"""The reference's own native entry points (include/flh_hip.h and include/flh_reference_native.h), launched through
the C ABI on the GPU -- C linkage and the C++-linkage symbols a HIP-compiled flh_cuda_bindings.cpp would link against --
and checked against the oracle.  They launch on the legacy default stream, so each call is bracketed by device syncs."""
import numpy as np
import pytest
import torch

from flh_amd import _lib
from flh_amd import synthetic as syn

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    return t.detach().cpu().numpy()


def entry(name, cxx):
    lib = _lib.load()
    assert lib.flh_init() == 0, lib.flh_last_error()
    return getattr(lib, _lib._SIG_CXX[name] if cxx else name)


def run(fn, *args):
    torch.cuda.synchronize()
    fn(*args)
    torch.cuda.synchronize()


@pytest.mark.parametrize("cxx", [False, True])
@pytest.mark.parametrize("had", [True, False])
@pytest.mark.parametrize("g", [None, 128, 64, 32])      # None: the functions without a group-size parameter
def test_group_quantiser_wrappers(cxx, had, g):
    from oracle import quant as Q
    from oracle.pack import pack_i4
    width = g or 128
    rows = 1000
    x = syn.activations(rows, width, seed=width + had)
    x[17] = 0
    xd = dev(x)
    q = torch.full((rows, width // 2), 0xAA, dtype=torch.uint8, device="cuda")
    s = torch.zeros(rows, dtype=torch.float16, device="cuda")
    base = "had_and_quant_host" if had else "quant_and_pack_host"
    print(f"case wrapper {base} g={g} cxx={cxx}", flush=True)
    if g is None:
        run(entry(base, cxx), xd.data_ptr(), q.data_ptr(), s.data_ptr(), rows)
    else:
        run(entry(base + "_gs", cxx), g, xd.data_ptr(), q.data_ptr(), s.data_ptr(), rows)
    qr, sr, _ = Q.kernel_had_and_quant(x, width, had)
    assert np.array_equal(host(s).view(np.uint16), sr.view(np.uint16))
    assert np.array_equal(host(q), pack_i4(qr))


@pytest.mark.parametrize("variant", ["c", "c_gs", "cxx_gs"])
@pytest.mark.parametrize("g", [128, 64, 32])
def test_gemm_wrappers(variant, g):
    from oracle import gemm as G
    if variant == "c" and g != 128:
        pytest.skip("flhDenseLayerGEMM_i4_o16 has groups of 128 only")
    m, n, k = 128, 256, 512
    rng = np.random.default_rng(g)
    ap = syn.pack_codes(rng.integers(-8, 8, size=(m, k), dtype=np.int8))
    bp = syn.pack_codes(rng.integers(-8, 8, size=(n, k), dtype=np.int8))
    sa = rng.uniform(0.01, 0.5, size=(m, k // g)).astype(np.float16)
    sb = syn.weight_scales(n, k // g, seed=g)
    a, b, das, dbs = dev(ap), dev(bp), dev(sa), dev(sb)
    d = torch.zeros(m, n, dtype=torch.float16, device="cuda")
    print(f"case wrapper gemm {variant} g={g}", flush=True)
    if variant == "c":
        run(entry("flhDenseLayerGEMM_i4_o16", False), a.data_ptr(), b.data_ptr(), das.data_ptr(), dbs.data_ptr(),
            d.data_ptr(), m, n, k)
    else:
        run(entry("flhDenseLayerGEMM_i4_o16_gs", variant == "cxx_gs"), g, a.data_ptr(), b.data_ptr(), d.data_ptr(), m, n, k,
            das.data_ptr(), dbs.data_ptr())
    ref, _ = G.gemm_i4_dequant(ap, bp, sa, sb, group=g)
    # bit-equal to the fused-multiply-add oracle; the path's stated tolerance is rtol 1e-3 / atol 1e-2
    assert np.array_equal(host(d).view(np.uint16), ref.view(np.uint16))


def test_rejected_wrapper_call_reports_and_leaves_outputs(capfd):
    """A call the library rejects (here: a group size it does not have) prints the reason and writes nothing."""
    x = torch.zeros(4, 48, dtype=torch.float16, device="cuda")
    q = torch.full((4, 24), 0x5A, dtype=torch.uint8, device="cuda")
    s = torch.full((4,), 3.0, dtype=torch.float16, device="cuda")
    run(entry("had_and_quant_host_gs", True), 48, x.data_ptr(), q.data_ptr(), s.data_ptr(), 4)
    err = capfd.readouterr().err
    assert "had_and_quant_host_gs failed" in err
    assert bool((q == 0x5A).all()) and bool((s == 3.0).all())
