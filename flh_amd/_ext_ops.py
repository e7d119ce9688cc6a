"""The op module backed by the PyTorch-ROCm C++ extension (flh_amd/_flh_torch.so, source csrc/torch_ext.cpp): what
``flh_amd._CUDA`` resolves to when that extension has been built.  The hot ops -- the reference's nine op names
(flh/cuda/flh_cuda_bindings.cpp:301-313) and this library's additions on the prefill / decode path -- are the C++
functions themselves (tensor checks, current stream and allocation in C++; about a third of the host time of the
ctypes route at decode sizes); everything else falls through to the ctypes ops of ``_ops``.  Both routes end in the
same C ABI of libflh_hip.so."""
import importlib

from . import _lib
from . import _ops

_lib.load()                                   # libflh_hip.so first: fails loudly with build instructions when missing
_ext = importlib.import_module("flh_amd._flh_torch")

FLH_HAD_NONE, FLH_HAD_F32, FLH_HAD_MFMA = _ops.FLH_HAD_NONE, _ops.FLH_HAD_F32, _ops.FLH_HAD_MFMA

gemm_i4_dequant = _ext.gemm_i4_dequant
gemm_i4_dequant_o16 = _ext.gemm_i4_dequant_o16
gemm_i4_dequant_o16_gs = _ext.gemm_i4_dequant_o16_gs
gemm_i4_dequant_multi = _ext.gemm_i4_dequant_multi
gemm_i4_swiglu = _ext.gemm_i4_swiglu
gemm_i4_dequant_add = _ext.gemm_i4_dequant_add
prefill_attention = _ext.prefill_attention
rope_kv_cache_ = _ext.rope_kv_cache_
rotate_quantize_gemm_i4 = _ext.rotate_quantize_gemm_i4
rotate_quantize_gemm_i4_multi = _ext.rotate_quantize_gemm_i4_multi
hadamard_transform_half = _ext.hadamard_transform_half
hadamard_transform_128_half = _ext.hadamard_transform_128_half
hadamard_transform_64_half = _ext.hadamard_transform_64_half
hadamard_transform_32_half = _ext.hadamard_transform_32_half
hadamard_and_quantize_i4 = _ext.hadamard_and_quantize_i4
quant_and_pack_i4 = _ext.quant_and_pack_i4
hadamard_and_quantize_i4_gs = _ext.hadamard_and_quantize_i4_gs
quant_and_pack_i4_gs = _ext.quant_and_pack_i4_gs
silu_mul_and_quantize_i4_gs = _ext.silu_mul_and_quantize_i4_gs
rmsnorm_and_quantize_i4_gs = _ext.rmsnorm_and_quantize_i4_gs

_MODES = {False: FLH_HAD_NONE, None: FLH_HAD_NONE, "exact": FLH_HAD_F32, "fast": FLH_HAD_MFMA}


def rotate_and_quantize_i4(x, hadamard=True, had_group=0, scale_group=0, clip_ratio=1.0, return_rotated=False):
    """As _ops.rotate_and_quantize_i4 (hadamard: False / "exact" / "fast" / True = "exact" for power-of-two K and
    "fast" for K = 11008 / 14336)."""
    if hadamard is True:
        hadamard = "fast" if x.size(-1) in (11008, 14336) else "exact"
    return tuple(_ext.rotate_and_quantize_i4_mode(x, _MODES[hadamard], int(had_group or 0), int(scale_group or 0),
                                                  clip_ratio, return_rotated))


def rmsnorm_rotate_and_quantize_i4(x, weight, eps, hadamard=True, clip_ratio=1.0, return_rotated=False):
    return tuple(_ext.rmsnorm_rotate_and_quantize_i4_mode(x, weight, eps, _ops._whole_row_mode(hadamard), clip_ratio,
                                                          return_rotated))


def __getattr__(name):        # ops the extension does not wrap (6-bit path, int32 output, tuning hook, ...)
    return getattr(_ops, name)
