"""Python-side guards around the raw ops, as in the reference's flh/cuda/*.py: they
validate their input and raise ValueError before anything reaches the device."""
import torch

from .. import _lib


def load_flh_cuda_ext():
    """Reference: flh/cuda/load_ext.py:11-47 (JIT-builds and returns the extension).
    Here the kernels are prebuilt into libflh_hip.so; this returns the op module (the same
    object as flh._CUDA) and raises when there is no GPU or no library."""
    if not torch.cuda.is_available():
        raise RuntimeError("CUDA not available")
    _lib.load()
    import flh_amd
    return flh_amd._CUDA


def _require(x, width=None):
    if not x.is_cuda:
        raise ValueError("Input tensor must be on CUDA")
    if x.dtype != torch.float16:
        raise ValueError("Input tensor must be float16 (half)")
    if x.dim() != 2:
        raise ValueError("Input tensor must be 2D")
    if width is not None and x.shape[-1] != width:
        raise ValueError(f"Last dimension must be {width}")


def hadamard_transform_half(x):
    """In-place unnormalised FWHT of an (M, 128) half matrix (flh/cuda/hadamard.py:4-35)."""
    _require(x, 128)
    return load_flh_cuda_ext().hadamard_transform_128_half(x)


def hadamard_transform_64_half(x):
    _require(x, 64)
    return load_flh_cuda_ext().hadamard_transform_64_half(x)


def hadamard_transform_32_half(x):
    _require(x, 32)
    return load_flh_cuda_ext().hadamard_transform_32_half(x)


def hadamard_transform(x, scale=1.0):
    """flh/cuda/hadamard.py:106-133: the kernel for (M, 128) half tensors on the GPU,
    otherwise the torch butterfly (which here is a correct transform)."""
    if x.is_cuda and x.dtype == torch.float16 and x.dim() == 2 and x.shape[-1] == 128:
        return hadamard_transform_half(x.clone()) * scale
    from ..functional.hadamard import hadamard_transform as torch_fwht
    return torch_fwht(x, scale=scale)


def hadamard_transform_n(x, n=128, scale=1.0):
    """flh/cuda/hadamard.py:136-175."""
    if n is None:
        n = x.shape[-1]
    if n not in (128, 64, 32):
        raise ValueError(f"n must be 128, 64, or 32, got {n}")
    if x.shape[-1] != n:
        raise ValueError(f"Last dimension must be {n}, got {x.shape[-1]}")
    _require(x)
    fn = {128: hadamard_transform_half, 64: hadamard_transform_64_half, 32: hadamard_transform_32_half}[n]
    return fn(x) * scale


def hadamard_and_quantize_i4(x):
    """flh/cuda/had_and_quant.py:4-28: (M, 128) fp16 -> (q [M, 64] u8, scales [M] fp16)."""
    _require(x, 128)
    q, s = load_flh_cuda_ext().hadamard_and_quantize_i4(x.contiguous())
    return q, s


def quant_and_pack_i4(x):
    """flh/cuda/quant_and_pack.py:4-28."""
    _require(x, 128)
    q, s = load_flh_cuda_ext().quant_and_pack_i4(x.contiguous())
    return q, s
