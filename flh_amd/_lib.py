"""ctypes binding of libflh_hip.so (the C ABI declared in include/flh_hip.h).

The library is looked up next to this package.  There is no fallback: if it is missing
the import of any op fails with an explicit error telling how to build it.
"""
import ctypes
import os
import pathlib

_HERE = pathlib.Path(__file__).resolve().parent
# FLH_HIP_LIBRARY may name another build of the same library (e.g. an experimental one)
LIB_PATH = pathlib.Path(os.environ.get("FLH_HIP_LIBRARY") or (_HERE / "libflh_hip.so"))

_lib = None

_c = ctypes
_PTR = _c.c_void_p
_SIG = {
    "flh_abi_version": (_c.c_int, []),
    "flh_last_error": (_c.c_char_p, []),
    "flh_init": (_c.c_int, []),
    "flh_gemm_i4_o16": (_c.c_int, [_PTR, _PTR, _PTR, _PTR, _PTR, _c.c_size_t, _c.c_size_t, _c.c_size_t,
                                   _c.c_int, _c.c_int, _c.c_int, _PTR]),
    "flh_gemm_i4_add_o16": (_c.c_int, [_PTR, _PTR, _PTR, _PTR, _PTR, _PTR, _c.c_size_t, _c.c_size_t, _c.c_size_t,
                                       _c.c_int, _c.c_int, _c.c_int, _PTR]),
    "flh_gemm_f6_add_o16": (_c.c_int, [_PTR, _PTR, _PTR, _PTR, _PTR, _PTR, _c.c_size_t, _c.c_size_t, _c.c_size_t,
                                       _c.c_int, _c.c_int, _PTR]),
    "flh_gemm_i4_qkv_rope_o16": (_c.c_int, [_PTR, _PTR, _PTR, _PTR, _PTR, _PTR, _PTR, _PTR, _PTR, _PTR, _c.c_uint32,
                                            _c.c_uint32, _c.c_uint32, _c.c_uint32, _c.c_uint32, _c.c_size_t, _c.c_int,
                                            _c.c_int, _c.c_int, _PTR]),
    "flh_prefill_attention_f16": (_c.c_int, [_PTR, _PTR, _PTR, _PTR, _c.c_uint32, _c.c_uint32, _c.c_uint32, _c.c_uint32,
                                             _c.c_uint32, _c.c_uint32, _c.c_uint32, _c.c_float, _PTR]),
    "flh_gemm_f6_qkv_rope_o16": (_c.c_int, [_PTR, _PTR, _PTR, _PTR, _PTR, _PTR, _PTR, _PTR, _PTR, _PTR, _c.c_uint32,
                                            _c.c_uint32, _c.c_uint32, _c.c_uint32, _c.c_uint32, _c.c_size_t, _c.c_int,
                                            _c.c_int, _PTR]),
    "flh_gemm_i4_swiglu_o16": (_c.c_int, [_PTR, _PTR, _PTR, _PTR, _PTR, _PTR, _PTR, _c.c_size_t, _c.c_size_t, _c.c_size_t,
                                          _c.c_int, _c.c_int, _c.c_int, _PTR]),
    "flh_gemm_f6_swiglu_o16": (_c.c_int, [_PTR, _PTR, _PTR, _PTR, _PTR, _PTR, _PTR, _c.c_size_t, _c.c_size_t, _c.c_size_t,
                                          _c.c_int, _c.c_int, _PTR]),
    "flh_gemm_i4_o16_multi": (_c.c_int, [_PTR, _PTR, _c.c_int, _PTR, _PTR, _PTR, _PTR, _c.c_size_t, _c.c_size_t,
                                         _c.c_int, _c.c_int, _c.c_int, _PTR]),
    "flh_rotate_quant_gemm_i4_o16_multi": (_c.c_int, [_PTR, _c.c_int, _PTR, _PTR, _PTR, _PTR, _c.c_size_t, _c.c_size_t,
                                                      _c.c_int, _PTR]),
    "flh_rmsnorm_rotate_quant_gemm_i4_o16_multi": (_c.c_int, [_PTR, _PTR, _PTR, _PTR, _c.c_float, _c.c_int, _PTR, _PTR, _PTR,
                                                              _PTR, _c.c_size_t, _c.c_size_t, _c.c_int, _PTR]),
    "flh_gemm_i4_i32": (_c.c_int, [_PTR, _PTR, _PTR, _c.c_size_t, _c.c_size_t, _c.c_size_t, _PTR]),
    "flh_gemm_f6_o16_multi": (_c.c_int, [_PTR, _PTR, _c.c_int, _PTR, _PTR, _PTR, _PTR, _c.c_size_t, _c.c_size_t,
                                         _c.c_int, _c.c_int, _PTR]),
    "flh_gemm_set_tuning": (_c.c_int, [_c.c_int, _c.c_int]),
    "flh_rotate_quant_gemm_i4_o16": (_c.c_int, [_PTR, _PTR, _PTR, _PTR, _c.c_size_t, _c.c_size_t, _c.c_size_t,
                                                _c.c_int, _PTR]),
    "flh_encode_f6": (_c.c_int, [_PTR, _PTR, _c.c_size_t, _c.c_size_t, _PTR]),
    "flh_gemm_f6_o16": (_c.c_int, [_PTR, _PTR, _PTR, _PTR, _PTR, _c.c_size_t, _c.c_size_t, _c.c_size_t, _PTR]),
    "flh_group_quant_f6": (_c.c_int, [_PTR, _PTR, _PTR, _c.c_uint32, _c.c_uint32, _c.c_int, _c.c_float, _PTR]),
    "flh_gemm_f6_o16_gs": (_c.c_int, [_PTR, _PTR, _PTR, _PTR, _PTR, _c.c_size_t, _c.c_size_t, _c.c_size_t, _c.c_int,
                                      _c.c_int, _PTR]),
    "flh_gemm_f6_i32": (_c.c_int, [_PTR, _PTR, _PTR, _c.c_size_t, _c.c_size_t, _c.c_size_t, _PTR]),
    "flhDenseLayerGEMM_i4_o16": (None, [_PTR, _PTR, _PTR, _PTR, _PTR, _c.c_size_t, _c.c_size_t, _c.c_size_t]),
    "flhDenseLayerGEMM_i4_o16_gs": (None, [_c.c_int, _PTR, _PTR, _PTR, _c.c_size_t, _c.c_size_t, _c.c_size_t,
                                           _PTR, _PTR]),
    "flh_group_quant_i4": (_c.c_int, [_PTR, _PTR, _PTR, _c.c_uint32, _c.c_int, _c.c_int, _c.c_float, _PTR]),
    "flh_silu_mul_group_quant_i4": (_c.c_int, [_PTR, _PTR, _PTR, _PTR, _c.c_uint32, _c.c_int, _c.c_int, _c.c_float,
                                               _PTR]),
    "flh_rmsnorm_group_quant_i4": (_c.c_int, [_PTR, _PTR, _PTR, _PTR, _c.c_uint32, _c.c_uint32, _c.c_float, _c.c_int,
                                              _c.c_int, _c.c_float, _PTR]),
    "flh_rmsnorm_rotate_quant_i4": (_c.c_int, [_PTR, _PTR, _c.c_float, _PTR, _PTR, _PTR, _c.c_uint32, _c.c_uint32,
                                               _c.c_int, _c.c_float, _PTR]),
    "had_and_quant_host": (None, [_PTR, _PTR, _PTR, _c.c_uint32]),
    "quant_and_pack_host": (None, [_PTR, _PTR, _PTR, _c.c_uint32]),
    "had_and_quant_host_gs": (None, [_c.c_int, _PTR, _PTR, _PTR, _c.c_uint32]),
    "quant_and_pack_host_gs": (None, [_c.c_int, _PTR, _PTR, _PTR, _c.c_uint32]),
    "flh_rope_kv_cache_f16": (_c.c_int, [_PTR, _PTR, _PTR, _PTR, _PTR, _PTR, _PTR, _PTR, _c.c_uint32, _c.c_uint32,
                                         _c.c_uint32, _c.c_uint32, _c.c_uint32, _c.c_uint32, _PTR]),
    "flh_decode_attention_workspace_bytes": (_c.c_size_t, [_c.c_uint32, _c.c_uint32, _c.c_uint32, _c.c_uint32]),
    "flh_decode_attention_f16": (_c.c_int, [_PTR, _PTR, _PTR, _PTR, _c.c_uint32, _c.c_uint32, _c.c_uint32, _c.c_uint32,
                                            _c.c_uint32, _c.c_uint32, _c.c_float, _PTR, _c.c_size_t, _PTR]),
    "flh_decode_attention_rope_f16": (_c.c_int, [_PTR] * 9 + [_c.c_uint32] * 6 + [_c.c_float, _PTR, _c.c_size_t, _PTR]),
    "flh_decode_attention_static_scratch_bytes": (_c.c_size_t, []),
    "flh_decode_attention_f16_static": (_c.c_int, [_PTR, _PTR, _PTR, _PTR, _c.c_uint32, _c.c_uint32, _c.c_uint32,
                                                   _c.c_uint32, _c.c_uint32, _c.c_uint32, _c.c_float, _PTR]),
    "flh_add_rmsnorm_rotate_quant_i4": (_c.c_int, [_PTR, _PTR, _PTR, _PTR, _c.c_float, _PTR, _PTR, _c.c_uint32, _c.c_uint32,
                                                  _c.c_int, _c.c_float, _PTR]),
    "flh_rotate_quant_f6": (_c.c_int, [_PTR, _PTR, _PTR, _c.c_int, _PTR, _c.c_float, _PTR, _PTR, _c.c_uint32, _c.c_uint32,
                                      _c.c_int, _c.c_float, _PTR]),
    "flh_silu_mul_f16": (_c.c_int, [_PTR, _PTR, _PTR, _c.c_uint64, _PTR]),
    "flh_add_rmsnorm_f16": (_c.c_int, [_PTR, _PTR, _PTR, _c.c_float, _PTR, _PTR, _c.c_uint32, _c.c_uint32, _PTR]),
    "flh_silu_mul_rotate_quant_i4": (_c.c_int, [_PTR, _PTR, _PTR, _PTR, _c.c_uint32, _c.c_uint32, _PTR]),
    "flh_fwht_f16_inplace": (_c.c_int, [_PTR, _c.c_uint32, _c.c_int, _PTR]),
    "flh_rotate_quant_i4": (_c.c_int, [_PTR, _PTR, _PTR, _PTR, _c.c_uint32, _c.c_uint32, _c.c_int, _c.c_int,
                                       _c.c_int, _c.c_float, _PTR]),
}
EXPORTS = tuple(_SIG)

# The reference's C++-linkage declarations (include/flh_reference_native.h), by their Itanium-mangled names over
# `__half`: what a binding file compiled for HIP links against.  Same argument lists as the C-linkage twins above.
_SIG_CXX = {
    "flhDenseLayerGEMM_i4_o16_gs": "_Z27flhDenseLayerGEMM_i4_o16_gsiPKhS0_P6__halfmmmPKS1_S4_",
    "had_and_quant_host": "_Z18had_and_quant_hostPK6__halfPhPS_j",
    "quant_and_pack_host": "_Z19quant_and_pack_hostPK6__halfPhPS_j",
    "had_and_quant_host_gs": "_Z21had_and_quant_host_gsiPK6__halfPhPS_j",
    "quant_and_pack_host_gs": "_Z22quant_and_pack_host_gsiPK6__halfPhPS_j",
}
EXPORTS_CXX = tuple(_SIG_CXX.values())


class FLHLibraryError(RuntimeError):
    pass


def load():
    """Load (once) and return the ctypes handle; raises FLHLibraryError when the HIP
    library has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise FLHLibraryError(
            f"{LIB_PATH} is missing: build the HIP kernels first (python -m flh_amd.csrc.build). "
            "There is no CPU or torch fallback for these ops.")
    lib = ctypes.CDLL(str(LIB_PATH))
    for name, (res, args) in _SIG.items():
        fn = getattr(lib, name)  # AttributeError if the library does not export it
        fn.restype = res
        fn.argtypes = args
    for plain, mangled in _SIG_CXX.items():
        fn = getattr(lib, mangled)
        fn.restype, fn.argtypes = _SIG[plain]
    if lib.flh_abi_version() != 1:
        raise FLHLibraryError("libflh_hip.so has an unexpected ABI version; rebuild it")
    _lib = lib
    return lib


def check(rc):
    if rc != 0:
        msg = load().flh_last_error().decode(errors="replace")
        raise RuntimeError(f"libflh_hip: {msg} (code {rc})")
