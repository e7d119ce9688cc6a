"""The op module that takes the place of the reference's ``flh._CUDA`` extension
(flh/cuda/flh_cuda_bindings.cpp:301-313): same function names, argument order, checks
and return values, implemented by hand-written HIP kernels for gfx950 reached through
the C ABI in include/flh_hip.h.  torch is used only for device memory and the current
stream.  Beyond the nine reference ops it exports the whole-row rotate+quantise op and
the generalised GEMM (per-token x per-channel scales, int32 output).
"""
import torch

from . import _lib

FLH_HAD_NONE = 0
FLH_HAD_F32 = 1
FLH_HAD_MFMA = 2


def _check(cond, msg):
    if not cond:
        raise RuntimeError(msg)  # TORCH_CHECK of the reference surfaces as RuntimeError


# the raw handle of torch's current stream without building a Stream object (a third of an op's host time at decode
# sizes went into that object and into the device context manager below)
_raw_stream = getattr(torch._C, "_cuda_getCurrentRawStream", None)


def _stream(t):
    if _raw_stream is not None:
        return _raw_stream(t.device.index)
    return torch.cuda.current_stream(t.device).cuda_stream


_initialised = set()   # devices on which flh_init has run


def _run(name, dev, *args):
    lib = _lib.load()
    if dev.index == torch.cuda.current_device() and dev.index in _initialised:
        rc = getattr(lib, name)(*args)        # the usual case: nothing to switch, nothing to set up
    else:
        with torch.cuda.device(dev):
            if dev.index not in _initialised:
                _lib.check(lib.flh_init())    # device check + constant tables, once
                _initialised.add(dev.index)
            rc = getattr(lib, name)(*args)
    if rc is not None:
        _lib.check(rc)


def _check_gemm_inputs(A, B, A_scale, B_scale):
    _check(A.is_cuda and B.is_cuda and A_scale.is_cuda and B_scale.is_cuda, "tensors must be CUDA")
    _check(A.dtype == torch.uint8, "A must be uint8 packed int4")
    _check(B.dtype == torch.uint8, "B must be uint8 packed int4")
    _check(A_scale.dtype == torch.float16, "A_scale must be float16")
    _check(B_scale.dtype == torch.float16, "B_scale must be float16")
    _check(A.is_contiguous() and B.is_contiguous() and A_scale.is_contiguous() and B_scale.is_contiguous(),
           "tensors must be contiguous")
    _check(A.dim() == 2 and B.dim() == 2, "A/B must be 2D")
    _check(B.size(1) == A.size(1), "B.shape[1] must equal A.shape[1]")
    _check(B.device == A.device and A_scale.device == A.device and B_scale.device == A.device,
           "tensors must be on one device")


def gemm_i4_dequant(A, B, A_scale, B_scale, group_size=128):
    """Generalised int4 GEMM + dequant: scales [M, 1 | K/g] and [N, 1 | K/g] -> fp16 [M, N]."""
    _check_gemm_inputs(A, B, A_scale, B_scale)
    return _gemm_i4_dequant_checked(A, B, A_scale, B_scale, group_size)


def _gemm_i4_dequant_checked(A, B, A_scale, B_scale, group_size):
    """gemm_i4_dequant behind a caller that has run _check_gemm_inputs already (the checks are a measurable part of an
    op's host time at decode sizes, so they run once)."""
    M, Kp = A.shape
    N, K = B.size(0), Kp * 2
    _check(A_scale.dim() == 2 and B_scale.dim() == 2, "scale must be 2D")
    _check(A_scale.size(0) == M, "A_scale.shape[0] must equal M")
    _check(B_scale.size(0) == N, "B_scale.shape[0] must equal N")
    _check(K % 128 == 0, "K must be a multiple of 128")
    D = torch.empty((M, N), dtype=torch.float16, device=A.device)
    if M == 0 or N == 0:
        return D
    _run("flh_gemm_i4_o16", A.device, A.data_ptr(), B.data_ptr(), A_scale.data_ptr(), B_scale.data_ptr(),
         D.data_ptr(), M, N, K, A_scale.size(1), B_scale.size(1), int(group_size), _stream(A))
    return D


def _check_residual(residual, M, N, device, out):
    _check(residual.is_cuda and residual.dtype == torch.float16 and residual.is_contiguous() and residual.device == device,
           "the residual must be a contiguous float16 CUDA tensor on the operands' device")
    _check(residual.numel() == M * N and residual.size(-1) == N, "the residual must have the shape of the output")
    if out is not None:
        _check(out.is_cuda and out.dtype == torch.float16 and out.is_contiguous() and out.device == device and
               out.numel() == M * N and out.size(-1) == N, "out must be a contiguous float16 CUDA tensor of the output's shape")


def gemm_i4_dequant_add(A, B, A_scale, B_scale, residual, group_size=128, out=None):
    """fp16(residual + gemm_i4_dequant(A, B, A_scale, B_scale, group_size)) in one launch: the residual addition of a
    decoder layer in the GEMM's epilogue (the GEMM's own fp16 rounding, then one fp16 addition -- the bits of the two
    separate operations).  residual [M, N] (or [..., N] with M rows) fp16; `out` may be the residual itself (in-place
    update of the residual stream) -> fp16 [M, N] (or `out`)."""
    _check_gemm_inputs(A, B, A_scale, B_scale)
    M, Kp = A.shape
    N, K = B.size(0), Kp * 2
    _check(A_scale.dim() == 2 and B_scale.dim() == 2, "scale must be 2D")
    _check(A_scale.size(0) == M, "A_scale.shape[0] must equal M")
    _check(B_scale.size(0) == N, "B_scale.shape[0] must equal N")
    _check(K % 128 == 0, "K must be a multiple of 128")
    _check_residual(residual, M, N, A.device, out)
    D = out if out is not None else torch.empty((M, N), dtype=torch.float16, device=A.device)
    if M and N:
        _run("flh_gemm_i4_add_o16", A.device, A.data_ptr(), B.data_ptr(), A_scale.data_ptr(), B_scale.data_ptr(),
             residual.data_ptr(), D.data_ptr(), M, N, K, A_scale.size(1), B_scale.size(1), int(group_size), _stream(A))
    return D


def gemm_i4_dequant_multi(A, Bs, A_scale, B_scales, group_size=128):
    """gemm_i4_dequant of the same activations against several weight matrices (q / k / v, gate / up) in one
    launch: Bs, B_scales are lists of up to four [N_s, K/2] / [N_s, 1 | K/g] tensors -> list of fp16 [M, N_s],
    each bit-identical to its own gemm_i4_dequant call."""
    import ctypes
    _check(len(Bs) == len(B_scales) and 1 <= len(Bs) <= 4, "one to four weight matrices, one scale tensor each")
    for B, B_scale in zip(Bs, B_scales):
        _check_gemm_inputs(A, B, A_scale, B_scale)
        _check(A_scale.dim() == 2 and B_scale.dim() == 2, "scale must be 2D")
        _check(B_scale.size(0) == B.size(0) and B_scale.size(1) == B_scales[0].size(1), "B_scale shapes")
        _check(B.device == A.device and B_scale.device == A.device, "tensors must be on one device")
    M, Kp = A.shape
    K = Kp * 2
    _check(K % 128 == 0, "K must be a multiple of 128")
    _check(A_scale.size(0) == M, "A_scale.shape[0] must equal M")
    Ds = [torch.empty((M, B.size(0)), dtype=torch.float16, device=A.device) for B in Bs]
    if M == 0 or any(B.size(0) == 0 for B in Bs):
        return [gemm_i4_dequant(A, B, A_scale, S, group_size) for B, S in zip(Bs, B_scales)]
    n = len(Bs)
    ptrs = lambda ts: (ctypes.c_void_p * n)(*[t.data_ptr() for t in ts])
    sizes = (ctypes.c_size_t * n)(*[B.size(0) for B in Bs])
    _run("flh_gemm_i4_o16_multi", A.device, A.data_ptr(), A_scale.data_ptr(), n, ptrs(Bs), ptrs(B_scales), ptrs(Ds),
         sizes, M, K, A_scale.size(1), B_scales[0].size(1), int(group_size), _stream(A))
    return Ds


def _check_rope_cache(M, batch, Bs, cos, sin, positions, k_cache, v_cache, device):
    _check(batch > 0 and M % batch == 0, "the rows of A must be batch * T tokens")
    T = M // batch
    _check(Bs[0].size(0) % 128 == 0 and Bs[1].size(0) % 128 == 0 and Bs[1].size(0) == Bs[2].size(0),
           "q / k / v must have whole heads of 128 channels, k and v the same number")
    Hq, Hkv = Bs[0].size(0) // 128, Bs[1].size(0) // 128
    for c in (cos, sin):
        _check(c.is_cuda and c.dtype == torch.float16 and c.is_contiguous() and tuple(c.shape) == (T, 128) and c.device == device,
               "cos / sin must be contiguous float16 CUDA tensors [T, 128]")
    _check(positions.is_cuda and positions.dtype == torch.int64 and positions.is_contiguous() and positions.numel() == T
           and positions.device == device, "positions must be a contiguous int64 CUDA tensor [T]")
    for c in (k_cache, v_cache):
        _check(c.is_cuda and c.dtype == torch.float16 and c.is_contiguous() and c.dim() == 4 and c.device == device and
               c.size(0) == batch and c.size(1) == Hkv and c.size(3) == 128 and c.shape == k_cache.shape,
               "the caches must be contiguous float16 CUDA tensors [batch, kv_heads, max_len, 128]")
    return T, Hq, Hkv, k_cache.size(2)


def gemm_i4_qkv_rope(A, A_scale, Bs, B_scales, cos, sin, positions, k_cache, v_cache, batch, group_size=128):
    """The q / k / v projections with the rotary embedding and the cache write in the GEMM's epilogue: what
    gemm_i4_dequant_multi(A, Bs, ...) followed by rope_kv_cache_ computes, same bits, in one launch.  A [batch * T, K/2]
    packed codes, Bs = [q, k, v] weights with heads of 128 channels, cos / sin [T, 128], positions [T] int64 (cache slots),
    k_cache / v_cache [batch, kv_heads, max_len, 128] (written in place) -> rotated queries [batch, T, heads, 128]."""
    import ctypes
    _check(len(Bs) == 3 and len(B_scales) == 3, "three weight matrices (q, k, v), one scale tensor each")
    for B, B_scale in zip(Bs, B_scales):
        _check_gemm_inputs(A, B, A_scale, B_scale)
        _check(A_scale.dim() == 2 and B_scale.dim() == 2, "scale must be 2D")
        _check(B_scale.size(0) == B.size(0) and B_scale.size(1) == B_scales[0].size(1), "B_scale shapes")
        _check(B.device == A.device and B_scale.device == A.device, "tensors must be on one device")
    M, Kp = A.shape
    K = Kp * 2
    _check(K % 128 == 0, "K must be a multiple of 128")
    _check(A_scale.size(0) == M, "A_scale.shape[0] must equal M")
    T, Hq, Hkv, max_len = _check_rope_cache(M, batch, Bs, cos, sin, positions, k_cache, v_cache, A.device)
    q_out = torch.empty((batch, T, Hq, 128), dtype=torch.float16, device=A.device)
    if M:
        ptrs = lambda ts: (ctypes.c_void_p * 3)(*[t.data_ptr() for t in ts])
        _run("flh_gemm_i4_qkv_rope_o16", A.device, A.data_ptr(), A_scale.data_ptr(), ptrs(Bs), ptrs(B_scales), cos.data_ptr(),
             sin.data_ptr(), positions.data_ptr(), q_out.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), batch, T, Hq, Hkv,
             max_len, K, A_scale.size(1), B_scales[0].size(1), int(group_size), _stream(A))
    return q_out


def gemm_i4_swiglu(A, B_gate, B_up, A_scale, gate_scale, up_scale, group_size=128):
    """fp16(fp16(silu(gate)) * up) with gate / up = gemm_i4_dequant(A, B_gate / B_up, A_scale, gate_scale / up_scale),
    in one launch that never stores gate and up: A [M, K/2], B_gate / B_up [N, K/2], scales as gemm_i4_dequant
    (group-scaled operands: groups of 128) -> fp16 [M, N]."""
    _check_gemm_inputs(A, B_gate, A_scale, gate_scale)
    _check_gemm_inputs(A, B_up, A_scale, up_scale)
    _check(B_up.shape == B_gate.shape and up_scale.shape == gate_scale.shape, "gate and up must have the same shapes")
    M, Kp = A.shape
    N, K = B_gate.size(0), Kp * 2
    _check(A_scale.dim() == 2 and gate_scale.dim() == 2, "scale must be 2D")
    _check(A_scale.size(0) == M and gate_scale.size(0) == N, "scale rows must match M / N")
    _check(K % 128 == 0, "K must be a multiple of 128")
    D = torch.empty((M, N), dtype=torch.float16, device=A.device)
    if M and N:
        _run("flh_gemm_i4_swiglu_o16", A.device, A.data_ptr(), B_gate.data_ptr(), B_up.data_ptr(), A_scale.data_ptr(),
             gate_scale.data_ptr(), up_scale.data_ptr(), D.data_ptr(), M, N, K, A_scale.size(1), gate_scale.size(1),
             int(group_size), _stream(A))
    return D


def gemm_i4_dequant_o16(A, B, A_scale, B_scale):
    """flh_cuda_bindings.cpp:75-113.  Scales are [M, K/128] and [N, K/128]; as an
    extension a width of 1 means one scale per row."""
    _check_gemm_inputs(A, B, A_scale, B_scale)
    _check(A_scale.dim() == 2 and B_scale.dim() == 2, "scale must be 2D")
    _check(A_scale.size(0) == A.size(0), "A_scale.shape[0] must equal M")
    _check(B_scale.size(0) == B.size(0), "B_scale.shape[0] must equal N")
    ng = A.size(1) * 2 // 128
    _check(A_scale.size(1) in (1, ng) and B_scale.size(1) in (1, ng), "scale.shape[1] must be K/128 (or 1)")
    return _gemm_i4_dequant_checked(A, B, A_scale, B_scale, 128)


def gemm_i4_dequant_o16_gs(A, B, A_scale, B_scale, group_size):
    """flh_cuda_bindings.cpp:254-299."""
    _check_gemm_inputs(A, B, A_scale, B_scale)
    _check(group_size in (32, 64, 128), "group_size must be 32, 64, or 128")
    K = A.size(1) * 2
    _check(K % group_size == 0, "K must be divisible by group_size")
    ng = K // group_size
    _check(A_scale.dim() == 2 and A_scale.size(0) == A.size(0), "A_scale.shape[0] must equal M")
    _check(A_scale.size(1) == ng, "A_scale.shape[1] must equal K/group_size")
    _check(B_scale.dim() == 2 and B_scale.size(0) == B.size(0), "B_scale.shape[0] must equal N")
    _check(B_scale.size(1) == ng, "B_scale.shape[1] must equal K/group_size")
    return _gemm_i4_dequant_checked(A, B, A_scale, B_scale, group_size)


def gemm_i4_int32(A, B):
    """Raw int32 accumulators sum_k A[m,k] * B[n,k]."""
    _check(A.is_cuda and B.is_cuda, "tensors must be CUDA")
    _check(A.dtype == torch.uint8 and B.dtype == torch.uint8, "A/B must be uint8 packed int4")
    _check(A.is_contiguous() and B.is_contiguous(), "tensors must be contiguous")
    _check(A.dim() == 2 and B.dim() == 2 and A.size(1) == B.size(1), "A/B must be 2D with equal K")
    M, N, K = A.size(0), B.size(0), A.size(1) * 2
    C = torch.empty((M, N), dtype=torch.int32, device=A.device)
    if M == 0 or N == 0:
        return C
    _run("flh_gemm_i4_i32", A.device, A.data_ptr(), B.data_ptr(), C.data_ptr(), M, N, K, _stream(A))
    return C


ROTATE_GEMM_MAX_TOKENS = 4
ROTATE_GEMM_WIDTHS = (4096,)


def rotate_quantize_gemm_i4(x, B, B_scale):
    """Decode: rotate_and_quantize_i4(x, "exact") followed by gemm_i4_dequant_o16 in one launch, same bits.
    x [M, 4096] fp16 with M <= 4; B [N, 2048] u8; B_scale [N, 1] or [N, 32] -> [M, N] fp16.  Worth it for one or
    two tokens (every workgroup repeats the rotation)."""
    _check(x.is_cuda and B.is_cuda and B_scale.is_cuda, "tensors must be CUDA")
    _check(x.dtype == torch.float16 and x.dim() == 2 and x.is_contiguous(), "x must be a contiguous 2D float16 tensor")
    _check(B.dtype == torch.uint8 and B.dim() == 2 and B.is_contiguous(), "B must be a contiguous 2D uint8 tensor")
    M, K = x.shape
    _check(B.size(1) * 2 == K, "x and B must have equal K")
    _check(M <= ROTATE_GEMM_MAX_TOKENS, "at most 4 tokens")
    _check(K in ROTATE_GEMM_WIDTHS, "K must be 4096")
    N = B.size(0)
    _check(B_scale.dtype == torch.float16 and B_scale.is_contiguous() and B_scale.dim() == 2 and B_scale.size(0) == N
           and B_scale.size(1) in (1, K // 128), "B_scale must be a contiguous float16 [N, 1] or [N, K/128] tensor")
    D = torch.empty((M, N), dtype=torch.float16, device=x.device)
    if M and N:
        _run("flh_rotate_quant_gemm_i4_o16", x.device, x.data_ptr(), B.data_ptr(), B_scale.data_ptr(), D.data_ptr(),
             M, N, K, B_scale.size(1), _stream(x))
    return D


def rotate_quantize_gemm_i4_multi(x, Bs, B_scales):
    """rotate_quantize_gemm_i4 for up to four weight matrices that share the tokens, in one launch:
    -> list of fp16 [M, N_s], each bit-identical to its own call."""
    import ctypes
    _check(len(Bs) == len(B_scales) and 1 <= len(Bs) <= 4, "one to four weight matrices, one scale tensor each")
    _check(x.is_cuda and x.dtype == torch.float16 and x.dim() == 2 and x.is_contiguous(),
           "x must be a contiguous 2D float16 CUDA tensor")
    M, K = x.shape
    _check(M <= ROTATE_GEMM_MAX_TOKENS, "at most 4 tokens")
    _check(K in ROTATE_GEMM_WIDTHS, "K must be 4096")
    for B, S in zip(Bs, B_scales):
        _check(B.is_cuda and S.is_cuda and B.device == x.device and S.device == x.device, "tensors must be on one device")
        _check(B.dtype == torch.uint8 and B.dim() == 2 and B.is_contiguous() and B.size(1) * 2 == K,
               "B must be a contiguous uint8 [N, K/2] tensor")
        _check(S.dtype == torch.float16 and S.is_contiguous() and S.dim() == 2 and S.size(0) == B.size(0)
               and S.size(1) in (1, K // 128) and S.size(1) == B_scales[0].size(1),
               "B_scale must be a contiguous float16 [N, 1] or [N, K/128] tensor, the same width for every matrix")
    Ds = [torch.empty((M, B.size(0)), dtype=torch.float16, device=x.device) for B in Bs]
    live = [i for i, B in enumerate(Bs) if B.size(0)]
    if M and live:
        n = len(live)
        ptrs = lambda ts: (ctypes.c_void_p * n)(*[ts[i].data_ptr() for i in live])
        sizes = (ctypes.c_size_t * n)(*[Bs[i].size(0) for i in live])
        _run("flh_rotate_quant_gemm_i4_o16_multi", x.device, x.data_ptr(), n, ptrs(Bs), ptrs(B_scales), ptrs(Ds), sizes,
             M, K, B_scales[0].size(1), _stream(x))
    return Ds


def rmsnorm_rotate_quantize_gemm_i4_multi(x, add, weight, eps, Bs, B_scales):
    """rotate_quantize_gemm_i4_multi on RMSNorm(x [+ add]) in one launch: x (and add, or None) [M, 4096] fp16 with M <= 4,
    weight [4096] fp16 or None -> (x + add [M, 4096] fp16 or None, [fp16 [M, N_s] ...]); the outputs are those of
    [add_]rmsnorm_rotate_and_quantize_i4 followed by gemm_i4_dequant_multi, bit for bit."""
    import ctypes
    _check(len(Bs) == len(B_scales) and 1 <= len(Bs) <= 4, "one to four weight matrices, one scale tensor each")
    _check(x.is_cuda and x.dtype == torch.float16 and x.dim() == 2 and x.is_contiguous(),
           "x must be a contiguous 2D float16 CUDA tensor")
    M, K = x.shape
    _check(M <= ROTATE_GEMM_MAX_TOKENS, "at most 4 tokens")
    _check(K in ROTATE_GEMM_WIDTHS, "K must be 4096")
    if add is not None:
        _check(add.is_cuda and add.dtype == torch.float16 and add.shape == x.shape and add.is_contiguous()
               and add.device == x.device, "add must be a contiguous float16 CUDA tensor of x's shape")
    if weight is not None:
        _check(weight.is_cuda and weight.dtype == torch.float16 and weight.is_contiguous() and weight.numel() == K
               and weight.device == x.device, "weight must be a contiguous float16 CUDA tensor of K values")
    for B, S in zip(Bs, B_scales):
        _check(B.is_cuda and S.is_cuda and B.device == x.device and S.device == x.device, "tensors must be on one device")
        _check(B.dtype == torch.uint8 and B.dim() == 2 and B.is_contiguous() and B.size(1) * 2 == K,
               "B must be a contiguous uint8 [N, K/2] tensor")
        _check(S.dtype == torch.float16 and S.is_contiguous() and S.dim() == 2 and S.size(0) == B.size(0)
               and S.size(1) in (1, K // 128) and S.size(1) == B_scales[0].size(1),
               "B_scale must be a contiguous float16 [N, 1] or [N, K/128] tensor, the same width for every matrix")
        _check(B.size(0) > 0, "empty weight matrix")
    total = torch.empty_like(x) if add is not None else None
    Ds = [torch.empty((M, B.size(0)), dtype=torch.float16, device=x.device) for B in Bs]
    if M:
        n = len(Bs)
        ptrs = lambda ts: (ctypes.c_void_p * n)(*[t.data_ptr() for t in ts])
        sizes = (ctypes.c_size_t * n)(*[B.size(0) for B in Bs])
        _run("flh_rmsnorm_rotate_quant_gemm_i4_o16_multi", x.device, x.data_ptr(),
             add.data_ptr() if add is not None else None, total.data_ptr() if total is not None else None,
             weight.data_ptr() if weight is not None else None, float(eps), n, ptrs(Bs), ptrs(B_scales), ptrs(Ds), sizes,
             M, K, B_scales[0].size(1), _stream(x))
    return total, Ds


def gemm_set_tuning(tile=0, k_split=0):
    """Test / tuning hook: force the GEMM tile (64, 128, 256) and in-workgroup K split (1, 2, 4); 0 = automatic."""
    _lib.check(_lib.load().flh_gemm_set_tuning(int(tile), int(k_split)))


def encode_f6(packed):
    """Re-encode packed int4 codes [R, K/2] u8 (K a multiple of 128) at 6 bits per code for the
    matrix instruction of gemm_f6_dequant_o16: -> [R, K/128 * 96] u8."""
    _check(packed.is_cuda and packed.dtype == torch.uint8 and packed.dim() == 2 and packed.is_contiguous(),
           "packed codes must be a contiguous 2D uint8 CUDA tensor")
    R, K = packed.size(0), packed.size(1) * 2
    _check(K % 128 == 0, "K must be a multiple of 128")
    out = torch.empty((R, K // 128 * 96), dtype=torch.uint8, device=packed.device)
    if R:
        _run("flh_encode_f6", packed.device, packed.data_ptr(), out.data_ptr(), R, K, _stream(packed))
    return out


def group_quantize_f6(x, hadamard=True, *, scale_mul=1.0):
    """hadamard_and_quantize_i4 / quant_and_pack_i4 over groups of 128 of x [M, K] fp16, with the codes
    written in the format of encode_f6: -> [q6 [M, K/128 * 96] u8, scales [M, K/128] fp16]."""
    _check(x.is_cuda and x.dtype == torch.float16 and x.dim() == 2 and x.is_contiguous(),
           "Input tensor must be a contiguous 2D float16 CUDA tensor")
    M, K = x.shape
    _check(K % 128 == 0 and K > 0, "Last dimension must be a multiple of 128")
    q6 = torch.empty((M, K // 128 * 96), dtype=torch.uint8, device=x.device)
    s = torch.empty((M, K // 128), dtype=torch.float16, device=x.device)
    if M:
        _run("flh_group_quant_f6", x.device, x.data_ptr(), q6.data_ptr(), s.data_ptr(), M, K, int(bool(hadamard)),
             float(scale_mul), _stream(x))
    return [q6, s]


def _check_f6(A6, B6):
    _check(A6.is_cuda and B6.is_cuda, "tensors must be CUDA")
    _check(A6.dtype == torch.uint8 and B6.dtype == torch.uint8, "encoded operands must be uint8")
    _check(A6.is_contiguous() and B6.is_contiguous(), "tensors must be contiguous")
    _check(A6.dim() == 2 and B6.dim() == 2 and A6.size(1) == B6.size(1) and A6.size(1) % 96 == 0,
           "encoded operands must be 2D with equal K")
    _check(A6.device == B6.device, "tensors must be on one device")
    return A6.size(0), B6.size(0), A6.size(1) // 96 * 128


def gemm_f6_dequant_o16(A6, B6, A_scale, B_scale):
    """gemm_i4_dequant_o16 with one scale per row on operands encoded by encode_f6 (same bits out)."""
    M, N, K = _check_f6(A6, B6)
    _check(A_scale.is_cuda and B_scale.is_cuda and A_scale.dtype == torch.float16 and B_scale.dtype == torch.float16,
           "scales must be float16 CUDA tensors")
    _check(A_scale.is_contiguous() and B_scale.is_contiguous() and A_scale.numel() == M and B_scale.numel() == N,
           "one scale per row of A and of B expected")
    _check(A_scale.device == A6.device and B_scale.device == A6.device, "tensors must be on one device")
    D = torch.empty((M, N), dtype=torch.float16, device=A6.device)
    if M and N:
        _run("flh_gemm_f6_o16", A6.device, A6.data_ptr(), B6.data_ptr(), A_scale.data_ptr(), B_scale.data_ptr(),
             D.data_ptr(), M, N, K, _stream(A6))
    return D


def gemm_f6_dequant_o16_gs(A6, B6, A_scale, B_scale):
    """gemm_i4_dequant_o16_gs with group_size 128 (A_scale [M, K/128], or [M, 1] for one scale per token;
    B_scale [N, K/128]) on operands encoded by encode_f6 (same bits out)."""
    M, N, K = _check_f6(A6, B6)
    ng = K // 128
    _check(A_scale.is_cuda and B_scale.is_cuda and A_scale.dtype == torch.float16 and B_scale.dtype == torch.float16,
           "scales must be float16 CUDA tensors")
    _check(A_scale.is_contiguous() and B_scale.is_contiguous() and A_scale.dim() == 2 and B_scale.dim() == 2,
           "scales must be contiguous and 2D")
    _check(A_scale.size(0) == M and A_scale.size(1) in (1, ng), "A_scale must be [M, K/128] or [M, 1]")
    _check(B_scale.size(0) == N and B_scale.size(1) == ng, "B_scale must be [N, K/128]")
    _check(A_scale.device == A6.device and B_scale.device == A6.device, "tensors must be on one device")
    D = torch.empty((M, N), dtype=torch.float16, device=A6.device)
    if M and N:
        _run("flh_gemm_f6_o16_gs", A6.device, A6.data_ptr(), B6.data_ptr(), A_scale.data_ptr(), B_scale.data_ptr(),
             D.data_ptr(), M, N, K, A_scale.size(1), ng, _stream(A6))
    return D


def gemm_f6_dequant_add(A6, B6, A_scale, B_scale, residual, out=None):
    """gemm_i4_dequant_add on operands encoded by encode_f6 (or written by rotate_and_quantize_f6): scales all one column, or
    weight scales [N, K/128] with A_scale [M, 1] or [M, K/128].  Same bits."""
    M, N, K = _check_f6(A6, B6)
    ng = K // 128
    _check(A_scale.is_cuda and B_scale.is_cuda and A_scale.dtype == torch.float16 and B_scale.dtype == torch.float16,
           "scales must be float16 CUDA tensors")
    _check(A_scale.is_contiguous() and B_scale.is_contiguous() and A_scale.dim() == 2 and B_scale.dim() == 2,
           "scales must be contiguous and 2D")
    _check(A_scale.size(0) == M and B_scale.size(0) == N, "one row of scales per row of A and of B expected")
    _check((A_scale.size(1), B_scale.size(1)) in ((1, 1), (1, ng), (ng, ng)),
           "scale columns must be (1, 1), (1, K/128) or (K/128, K/128)")
    _check(A_scale.device == A6.device and B_scale.device == A6.device, "tensors must be on one device")
    _check_residual(residual, M, N, A6.device, out)
    D = out if out is not None else torch.empty((M, N), dtype=torch.float16, device=A6.device)
    if M and N:
        _run("flh_gemm_f6_add_o16", A6.device, A6.data_ptr(), B6.data_ptr(), A_scale.data_ptr(), B_scale.data_ptr(),
             residual.data_ptr(), D.data_ptr(), M, N, K, A_scale.size(1), B_scale.size(1), _stream(A6))
    return D


def gemm_f6_qkv_rope(A6, A_scale, B6s, B_scales, cos, sin, positions, k_cache, v_cache, batch):
    """gemm_i4_qkv_rope on operands encoded by encode_f6 (or written by rotate_and_quantize_f6): scales all one column, or
    weight scales [N, K/128] with A_scale [M, 1] or [M, K/128].  Same bits."""
    import ctypes
    _check(len(B6s) == 3 and len(B_scales) == 3, "three weight matrices (q, k, v), one scale tensor each")
    M = K = None
    for B6, S in zip(B6s, B_scales):
        m, n, k = _check_f6(A6, B6)
        M, K = m, k
        _check(S.is_cuda and S.dtype == torch.float16 and S.is_contiguous() and S.dim() == 2 and S.size(0) == n
               and S.size(1) == B_scales[0].size(1) and S.device == A6.device, "B_scale shapes")
    ng = K // 128
    _check(A_scale.is_cuda and A_scale.dtype == torch.float16 and A_scale.is_contiguous() and A_scale.dim() == 2
           and A_scale.size(0) == M and A_scale.device == A6.device, "A_scale must be a contiguous float16 CUDA tensor [M, .]")
    _check((A_scale.size(1), B_scales[0].size(1)) in ((1, 1), (1, ng), (ng, ng)),
           "scale columns must be (1, 1), (1, K/128) or (K/128, K/128)")
    T, Hq, Hkv, max_len = _check_rope_cache(M, batch, B6s, cos, sin, positions, k_cache, v_cache, A6.device)
    q_out = torch.empty((batch, T, Hq, 128), dtype=torch.float16, device=A6.device)
    if M:
        ptrs = lambda ts: (ctypes.c_void_p * 3)(*[t.data_ptr() for t in ts])
        _run("flh_gemm_f6_qkv_rope_o16", A6.device, A6.data_ptr(), A_scale.data_ptr(), ptrs(B6s), ptrs(B_scales),
             cos.data_ptr(), sin.data_ptr(), positions.data_ptr(), q_out.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(),
             batch, T, Hq, Hkv, max_len, K, A_scale.size(1), B_scales[0].size(1), _stream(A6))
    return q_out


def gemm_f6_swiglu(A6, B6_gate, B6_up, A_scale, gate_scale, up_scale):
    """gemm_i4_swiglu on operands encoded by encode_f6 (or written by rotate_and_quantize_f6): fp16(fp16(silu(gate)) * up)
    in one launch, gate / up = gemm_f6_dequant_o16[_gs](A6, B6_gate / B6_up, ...); scales all one column, or weight scales
    [N, K/128] with A_scale [M, 1] or [M, K/128].  Same bits as gemm_i4_swiglu."""
    M, N, K = _check_f6(A6, B6_gate)
    _check(_check_f6(A6, B6_up) == (M, N, K), "gate and up must have the same shapes")
    ng = K // 128
    for t_ in (A_scale, gate_scale, up_scale):
        _check(t_.is_cuda and t_.dtype == torch.float16 and t_.is_contiguous() and t_.dim() == 2 and t_.device == A6.device,
               "scales must be contiguous 2D float16 CUDA tensors on the operands' device")
    _check(up_scale.shape == gate_scale.shape and gate_scale.size(0) == N and gate_scale.size(1) in (1, ng),
           "weight scales must be [N, 1] or [N, K/128], the same for gate and up")
    _check(A_scale.size(0) == M and A_scale.size(1) in (1, ng) and (A_scale.size(1) == 1 or gate_scale.size(1) == ng),
           "A_scale must be [M, 1], or [M, K/128] with group-scaled weights")
    D = torch.empty((M, N), dtype=torch.float16, device=A6.device)
    if M and N:
        _run("flh_gemm_f6_swiglu_o16", A6.device, A6.data_ptr(), B6_gate.data_ptr(), B6_up.data_ptr(), A_scale.data_ptr(),
             gate_scale.data_ptr(), up_scale.data_ptr(), D.data_ptr(), M, N, K, A_scale.size(1), gate_scale.size(1),
             _stream(A6))
    return D


def gemm_f6_dequant_multi(A6, B6s, A_scale, B_scales):
    """gemm_f6_dequant_o16 (all scales one column) resp. gemm_f6_dequant_o16_gs for up to four encoded weight
    matrices that share the encoded activations, in one launch -> list of fp16 [M, N_s], same bits as the single calls."""
    import ctypes
    _check(len(B6s) == len(B_scales) and 1 <= len(B6s) <= 4, "one to four weight matrices, one scale tensor each")
    M = K = None
    for B6, S in zip(B6s, B_scales):
        M, N, K = _check_f6(A6, B6)
        _check(S.is_cuda and S.dtype == torch.float16 and S.is_contiguous() and S.dim() == 2 and S.size(0) == N
               and S.size(1) == B_scales[0].size(1) and S.device == A6.device, "B_scale must be contiguous float16 [N, cols]")
    ng = K // 128
    _check(A_scale.is_cuda and A_scale.dtype == torch.float16 and A_scale.is_contiguous() and A_scale.dim() == 2
           and A_scale.size(0) == M, "A_scale must be a contiguous float16 [M, cols] tensor")
    a_cols, b_cols = A_scale.size(1), B_scales[0].size(1)
    _check((a_cols == 1 and b_cols == 1) or (b_cols == ng and a_cols in (1, ng)),
           "scale widths must be (1, 1) or (1 | K/128, K/128)")
    if M == 0 or any(B.size(0) == 0 for B in B6s):
        single = gemm_f6_dequant_o16 if (a_cols == 1 and b_cols == 1) else gemm_f6_dequant_o16_gs
        return [single(A6, B, A_scale, S) for B, S in zip(B6s, B_scales)]
    Ds = [torch.empty((M, B.size(0)), dtype=torch.float16, device=A6.device) for B in B6s]
    n = len(B6s)
    ptrs = lambda ts: (ctypes.c_void_p * n)(*[t.data_ptr() for t in ts])
    sizes = (ctypes.c_size_t * n)(*[B.size(0) for B in B6s])
    _run("flh_gemm_f6_o16_multi", A6.device, A6.data_ptr(), A_scale.data_ptr(), n, ptrs(B6s), ptrs(B_scales), ptrs(Ds),
         sizes, M, K, a_cols, b_cols, _stream(A6))
    return Ds


def gemm_f6_int32(A6, B6):
    """Raw int32 sums on operands encoded by encode_f6."""
    M, N, K = _check_f6(A6, B6)
    C = torch.empty((M, N), dtype=torch.int32, device=A6.device)
    if M and N:
        _run("flh_gemm_f6_i32", A6.device, A6.data_ptr(), B6.data_ptr(), C.data_ptr(), M, N, K, _stream(A6))
    return C


def rope_kv_cache_(q, k, v, cos, sin, positions, k_cache, v_cache):
    """Rotary embedding of q (in place) and k, and the new keys / values written into their cache slots, one launch:
    q [B, T, Hq, d], k / v [B, T, Hkv, d] fp16 contiguous; cos / sin [T, d] fp16; positions [T] int64 on the device;
    k_cache / v_cache [B, Hkv, max_len, d] fp16 contiguous.  The arithmetic of q * cos + rotate_half(q) * sin evaluated
    operation by operation in fp16.  Returns q."""
    for t_ in (q, k, v, cos, sin, k_cache, v_cache):
        _check(t_.is_cuda and t_.dtype == torch.float16 and t_.is_contiguous() and t_.device == q.device,
               "tensors must be contiguous float16 CUDA tensors on one device")
    _check(q.dim() == 4 and k.dim() == 4 and v.shape == k.shape and k.shape[:2] == q.shape[:2] and k.size(3) == q.size(3),
           "q [B, T, Hq, d] and k, v [B, T, Hkv, d] expected")
    B, T, Hq, d = q.shape
    Hkv = k.size(2)
    _check(cos.shape == (T, d) and sin.shape == (T, d), "cos / sin must be [T, d]")
    _check(positions.is_cuda and positions.dtype == torch.int64 and positions.is_contiguous() and positions.numel() == T
           and positions.device == q.device, "positions must be a contiguous int64 CUDA tensor of T entries")
    _check(k_cache.dim() == 4 and k_cache.shape == v_cache.shape and k_cache.size(0) == B and k_cache.size(1) == Hkv
           and k_cache.size(3) == d, "caches must be [B, Hkv, max_len, d]")
    _check(d % 16 == 0, "head_dim must be a multiple of 16")
    if q.numel():
        _run("flh_rope_kv_cache_f16", q.device, q.data_ptr(), k.data_ptr(), v.data_ptr(), cos.data_ptr(), sin.data_ptr(),
             positions.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), B, T, Hq, Hkv, d, k_cache.size(2), _stream(q))
    return q


_attention_workspaces = {}      # (device index, stream handle) -> uint8 tensor: launches of one stream run in order


def prefill_attention(q, k_cache, v_cache, past, scale=None):
    """Causal attention of a block of T new tokens over a cache: q [B, T, Hq, 128] fp16 (token-major), k_cache / v_cache
    [B, Hkv, max_len, 128] fp16 whose slots past .. past + T - 1 hold the block's own keys / values; query t sees the
    slots 0 .. past + t.  -> [B, T, Hq * 128] fp16 = softmax(q K^T * scale) V, float32 softmax and accumulation,
    probabilities rounded to fp16; grouped queries (Hq a multiple of Hkv)."""
    for t_ in (q, k_cache, v_cache):
        _check(t_.is_cuda and t_.dtype == torch.float16 and t_.is_contiguous() and t_.device == q.device,
               "tensors must be contiguous float16 CUDA tensors on one device")
    _check(q.dim() == 4 and k_cache.dim() == 4 and k_cache.shape == v_cache.shape and k_cache.size(0) == q.size(0)
           and k_cache.size(3) == q.size(3), "q [B, T, Hq, d] and caches [B, Hkv, max_len, d] expected")
    B, T, Hq, d = q.shape
    Hkv, max_len = k_cache.size(1), k_cache.size(2)
    _check(d == 128, "head_dim must be 128")
    _check(Hkv > 0 and Hq % Hkv == 0, "Hq must be a multiple of Hkv")
    past = int(past)
    _check(past >= 0 and past + T <= max_len, "past + T must fit the cache")
    out = torch.empty((B, T, Hq * d), dtype=torch.float16, device=q.device)
    if B and T:
        _run("flh_prefill_attention_f16", q.device, q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), out.data_ptr(), B, T,
             Hq, Hkv, d, past, max_len, float(scale if scale is not None else d ** -0.5), _stream(q))
    return out


def _default_attention_workspace(q, need):
    """The workspace kept per (device, stream) for calls that bring none.  A captured graph keeps the pointer it was
    recorded with, while this one may be replaced by a larger one later (and a stream handle may be reused by another
    stream): under capture the caller has to pass a workspace it owns for as long as the graph lives."""
    _check(not torch.cuda.is_current_stream_capturing(),
           "decode_attention: pass `workspace` (a tensor that outlives the graph) when capturing")
    key = (q.device.index, _stream(q))
    workspace = _attention_workspaces.get(key)
    if workspace is None or workspace.numel() < need:
        workspace = torch.empty(max(need, 1 << 20), dtype=torch.uint8, device=q.device)
        _attention_workspaces[key] = workspace
    return workspace


def decode_attention(q, k_cache, v_cache, kv_len, scale=None, workspace=None):
    """One new token per sequence against the first `kv_len` slots of a preallocated cache: q [B, Hq, d] fp16,
    k_cache / v_cache [B, Hkv, max_len, d] fp16 -> [B, Hq, d] fp16 = softmax(q K^T * scale) V with float32 scores,
    grouped queries (Hq / Hkv in {1, 2, 4, 8}), d in {64, 128}.  `workspace`: a uint8 CUDA tensor for the chunks' partial
    results; by default one per (device, stream) is kept and grown as needed (not under graph capture: pass one then)."""
    for t_ in (q, k_cache, v_cache):
        _check(t_.is_cuda and t_.dtype == torch.float16 and t_.is_contiguous() and t_.device == q.device,
               "tensors must be contiguous float16 CUDA tensors on one device")
    _check(q.dim() == 3 and k_cache.dim() == 4 and k_cache.shape == v_cache.shape and k_cache.size(0) == q.size(0)
           and k_cache.size(3) == q.size(2), "q [B, Hq, d] and caches [B, Hkv, max_len, d] expected")
    B, Hq, d = q.shape
    Hkv, max_len = k_cache.size(1), k_cache.size(2)
    _check(d in (64, 128), "head_dim must be 64 or 128")
    _check(Hkv > 0 and Hq % Hkv == 0 and Hq // Hkv in (1, 2, 4, 8), "Hq / Hkv must be 1, 2, 4 or 8")
    _check(0 < kv_len <= max_len, "kv_len must be in 1 .. max_len")
    out = torch.empty_like(q)
    if B == 0:
        return out
    need = int(_lib.load().flh_decode_attention_workspace_bytes(B, Hq, d, int(kv_len)))
    if workspace is None:
        workspace = _default_attention_workspace(q, need)
    else:
        _check(workspace.is_cuda and workspace.dtype == torch.uint8 and workspace.is_contiguous()
               and workspace.device == q.device and workspace.numel() >= need, f"workspace: {need} bytes of uint8 needed")
    _run("flh_decode_attention_f16", q.device, q.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), out.data_ptr(), B, Hq,
         Hkv, d, int(kv_len), max_len, float(scale if scale is not None else d ** -0.5), workspace.data_ptr(),
         workspace.numel(), _stream(q))
    return out


def decode_attention_rope(q, k_new, v_new, cos, sin, positions, k_cache, v_cache, kv_len, scale=None, workspace=None):
    """decode_attention with the rotary embedding and the cache write of the new token inside: q [B, Hq, d], k_new /
    v_new [B, Hkv, d] fp16 as projected (not rotated), cos / sin [1, d] or [d] fp16 of the new position, positions (int64
    CUDA tensor, first element = the cache slot of the new token, < kv_len) -> [B, Hq, d] fp16.  k_cache / v_cache receive
    the rotated key and the value at that slot (the bytes rope_kv_cache_ would write); q is not modified."""
    for t_ in (q, k_new, v_new, cos, sin, k_cache, v_cache):
        _check(t_.is_cuda and t_.dtype == torch.float16 and t_.is_contiguous() and t_.device == q.device,
               "tensors must be contiguous float16 CUDA tensors on one device")
    _check(q.dim() == 3 and k_cache.dim() == 4 and k_cache.shape == v_cache.shape and k_cache.size(0) == q.size(0)
           and k_cache.size(3) == q.size(2), "q [B, Hq, d] and caches [B, Hkv, max_len, d] expected")
    B, Hq, d = q.shape
    Hkv, max_len = k_cache.size(1), k_cache.size(2)
    _check(k_new.shape == (B, Hkv, d) and v_new.shape == (B, Hkv, d), "k_new / v_new [B, Hkv, d] expected")
    _check(cos.numel() == d and sin.numel() == d, "cos / sin of one position (d values each) expected")
    _check(positions.is_cuda and positions.dtype == torch.int64 and positions.numel() >= 1 and positions.device == q.device,
           "positions must be an int64 CUDA tensor")
    _check(d in (64, 128), "head_dim must be 64 or 128")
    _check(Hkv > 0 and Hq % Hkv == 0 and Hq // Hkv in (1, 2, 4, 8), "Hq / Hkv must be 1, 2, 4 or 8")
    _check(0 < kv_len <= max_len, "kv_len must be in 1 .. max_len")
    out = torch.empty_like(q)
    if B == 0:
        return out
    need = int(_lib.load().flh_decode_attention_workspace_bytes(B, Hq, d, int(kv_len)))
    if workspace is None:
        workspace = _default_attention_workspace(q, need)
    else:
        _check(workspace.is_cuda and workspace.dtype == torch.uint8 and workspace.is_contiguous()
               and workspace.device == q.device and workspace.numel() >= need, f"workspace: {need} bytes of uint8 needed")
    _run("flh_decode_attention_rope_f16", q.device, q.data_ptr(), k_new.data_ptr(), v_new.data_ptr(), cos.data_ptr(),
         sin.data_ptr(), positions.data_ptr(), k_cache.data_ptr(), v_cache.data_ptr(), out.data_ptr(), B, Hq, Hkv, d,
         int(kv_len), max_len, float(scale if scale is not None else d ** -0.5), workspace.data_ptr(), workspace.numel(),
         _stream(q))
    return out


def _check_rows(x, width):
    _check(x.is_cuda, "Input tensor must be on CUDA")
    _check(x.dtype == torch.float16, "Input tensor must be float16 (half)")
    _check(x.dim() == 2, "Input tensor must be 2D")
    _check(x.size(1) == width, f"Last dimension must be {width}")


def _fwht_inplace(x, width):
    _check_rows(x, width)
    _check(x.is_contiguous(), "Input tensor must be contiguous")
    if x.size(0) == 0:
        return x
    _run("flh_fwht_f16_inplace", x.device, x.data_ptr(), x.size(0), width, _stream(x))
    return x


def hadamard_transform_half(x):
    """In-place unnormalised FWHT-128 of each row (flh_cuda_bindings.cpp:115-126)."""
    return _fwht_inplace(x, 128)


hadamard_transform_128_half = hadamard_transform_half  # name used by flh/cuda/hadamard.py:35


def hadamard_transform_64_half(x):
    return _fwht_inplace(x, 64)


def hadamard_transform_32_half(x):
    return _fwht_inplace(x, 32)


def _group_quant(x, group, hadamard, scale_mul=1.0):
    _check_rows(x, group)
    _check(x.is_contiguous(), "Input tensor must be contiguous")
    R = x.size(0)
    q = torch.empty((R, group // 2), dtype=torch.uint8, device=x.device)
    s = torch.empty((R,), dtype=torch.float16, device=x.device)
    if R == 0:
        return [q, s]
    _run("flh_group_quant_i4", x.device, x.data_ptr(), q.data_ptr(), s.data_ptr(), R, group, int(hadamard),
         float(scale_mul), _stream(x))
    return [q, s]


def hadamard_and_quantize_i4(x, *, scale_mul=1.0):
    """flh_cuda_bindings.cpp:154-175: x [M, 128] fp16 -> [q [M, 64] u8, scales [M] fp16].
    scale_mul (extension): constant factor on the stored scales, fp16(float(s) * scale_mul)."""
    return _group_quant(x, 128, True, scale_mul)


def quant_and_pack_i4(x):
    """flh_cuda_bindings.cpp:177-198."""
    return _group_quant(x, 128, False)


def hadamard_and_quantize_i4_gs(x, group_size, *, scale_mul=1.0):
    """flh_cuda_bindings.cpp:202-226."""
    _check(group_size in (32, 64, 128), "group_size must be 32, 64, or 128")
    _check(x.dim() == 2 and x.size(1) == group_size, "Last dimension must equal group_size")
    return _group_quant(x, group_size, True, scale_mul)


def quant_and_pack_i4_gs(x, group_size, *, scale_mul=1.0):
    """flh_cuda_bindings.cpp:228-252."""
    _check(group_size in (32, 64, 128), "group_size must be 32, 64, or 128")
    _check(x.dim() == 2 and x.size(1) == group_size, "Last dimension must equal group_size")
    return _group_quant(x, group_size, False, scale_mul)


def silu_mul_and_quantize_i4_gs(gate, up, group_size, hadamard=False, *, scale_mul=1.0):
    """SwiGLU product + group quantiser in one launch (no reference op; the reference runs
    act_fn(gate) * up in torch and hands the result to ActQuantizer,
    flh/quantized_model/modeling_llama.py:522-526): gate, up [..., I] fp16 ->
    [q [..., I/2] u8, scales [..., I/group_size] fp16] of fp16(fp16(silu(gate)) * up)."""
    _check(group_size in (32, 64, 128), "group_size must be 32, 64, or 128")
    _check(gate.is_cuda and up.is_cuda, "Input tensors must be on CUDA")
    _check(gate.dtype == torch.float16 and up.dtype == torch.float16, "Input tensors must be float16 (half)")
    _check(gate.shape == up.shape, "gate and up must have the same shape")
    _check(gate.is_contiguous() and up.is_contiguous(), "Input tensors must be contiguous")
    _check(gate.dim() >= 1 and gate.size(-1) % group_size == 0, "Last dimension must be divisible by group_size")
    lead, width = gate.shape[:-1], gate.size(-1)
    q = torch.empty(lead + (width // 2,), dtype=torch.uint8, device=gate.device)
    s = torch.empty(lead + (width // group_size,), dtype=torch.float16, device=gate.device)
    rows = s.numel()
    if rows:
        _run("flh_silu_mul_group_quant_i4", gate.device, gate.data_ptr(), up.data_ptr(), q.data_ptr(), s.data_ptr(),
             rows, int(group_size), int(bool(hadamard)), float(scale_mul), _stream(gate))
    return [q, s]


SILU_ROTATE_MAX_ROWS = 256


def silu_mul(gate, up):
    """fp16(fp16(silu(gate)) * up) elementwise in one launch (fp16 tensors of one shape, element count a multiple of 8)."""
    _check(gate.is_cuda and up.is_cuda and gate.device == up.device, "Input tensors must be on CUDA")
    _check(gate.dtype == torch.float16 and up.dtype == torch.float16, "Input tensors must be float16 (half)")
    _check(gate.shape == up.shape and gate.is_contiguous() and up.is_contiguous(),
           "gate and up must be contiguous tensors of one shape")
    _check(gate.numel() % 8 == 0, "element count must be a multiple of 8")
    out = torch.empty_like(gate)
    if gate.numel():
        _run("flh_silu_mul_f16", gate.device, gate.data_ptr(), up.data_ptr(), out.data_ptr(), gate.numel(), _stream(gate))
    return out


def add_rmsnorm(x, weight=None, eps=1e-5, add=None, return_sum=False):
    """RMSNorm on its own, in one launch, optionally behind the residual addition: x [..., K] fp16 (`add` of the same
    shape or None; the row is then fp16(x + add)), weight [K] fp16 or None -> fp16 tensor of x's shape, statistics in
    float32 (flh/nn/normalization.py:12-20); with return_sum also the stored sum x + add, first."""
    _check(x.is_cuda and x.dtype == torch.float16 and x.dim() >= 1 and x.is_contiguous(),
           "Input tensor must be a contiguous float16 CUDA tensor")
    K = x.size(-1)
    _check(K % 8 == 0 and 0 < K <= 16384, "Last dimension must be a multiple of 8, at most 16384")
    if add is not None:
        _check(add.is_cuda and add.dtype == torch.float16 and add.shape == x.shape and add.is_contiguous()
               and add.device == x.device, "add must be a contiguous float16 CUDA tensor of x's shape")
    _check(not return_sum or add is not None, "return_sum needs add")
    if weight is not None:
        _check(weight.is_cuda and weight.dtype == torch.float16 and weight.is_contiguous() and weight.numel() == K
               and weight.device == x.device, "weight must be a contiguous float16 CUDA tensor of K values")
    out = torch.empty_like(x)
    total = torch.empty_like(x) if return_sum else None
    M = x.numel() // K
    if M:
        _run("flh_add_rmsnorm_f16", x.device, x.data_ptr(), add.data_ptr() if add is not None else None,
             weight.data_ptr() if weight is not None else None, float(eps), out.data_ptr(),
             total.data_ptr() if total is not None else None, M, K, _stream(x))
    return (total, out) if return_sum else out


def silu_mul_rotate_and_quantize_i4(gate, up):
    """Decode-sized batches: rotate_and_quantize_i4(silu(gate) * up, hadamard="fast") in one launch that never stores the
    product: gate, up [M, K] fp16 with K = 11008 or 14336, M <= 256 -> (q [M, K/2] u8, scales [M, 1] fp16)."""
    _check(gate.is_cuda and up.is_cuda and gate.device == up.device, "Input tensors must be on CUDA")
    _check(gate.dtype == torch.float16 and up.dtype == torch.float16, "Input tensors must be float16 (half)")
    _check(gate.dim() == 2 and gate.shape == up.shape and gate.is_contiguous() and up.is_contiguous(),
           "gate and up must be contiguous 2D tensors of one shape")
    M, K = gate.shape
    _check(K in (11008, 14336), "Last dimension must be 11008 or 14336")
    _check(M <= SILU_ROTATE_MAX_ROWS, "at most 256 rows")
    q = torch.empty((M, K // 2), dtype=torch.uint8, device=gate.device)
    s = torch.empty((M, 1), dtype=torch.float16, device=gate.device)
    if M:
        _run("flh_silu_mul_rotate_quant_i4", gate.device, gate.data_ptr(), up.data_ptr(), q.data_ptr(), s.data_ptr(), M, K,
             _stream(gate))
    return q, s


def rmsnorm_and_quantize_i4_gs(x, weight, eps, group_size, hadamard=False, *, scale_mul=1.0):
    """RMSNorm (flh/nn/normalization.py:12-20) + group quantiser in one launch: x [..., K] fp16,
    weight [K] fp16 or None -> [q [..., K/2] u8, scales [..., K/group_size] fp16]."""
    _check(group_size in (32, 64, 128), "group_size must be 32, 64, or 128")
    _check(x.is_cuda, "Input tensor must be on CUDA")
    _check(x.dtype == torch.float16, "Input tensor must be float16 (half)")
    _check(x.is_contiguous() and x.dim() >= 1, "Input tensor must be contiguous")
    K = x.size(-1)
    _check(K % group_size == 0 and 0 < K <= 16384, "Last dimension must be divisible by group_size and at most 16384")
    if weight is not None:
        _check(weight.is_cuda and weight.dtype == torch.float16 and weight.is_contiguous() and weight.numel() == K,
               "weight must be a contiguous float16 CUDA tensor of K values")
    lead = x.shape[:-1]
    q = torch.empty(lead + (K // 2,), dtype=torch.uint8, device=x.device)
    s = torch.empty(lead + (K // group_size,), dtype=torch.float16, device=x.device)
    M = x.numel() // K
    if M:
        _run("flh_rmsnorm_group_quant_i4", x.device, x.data_ptr(), weight.data_ptr() if weight is not None else None,
             q.data_ptr(), s.data_ptr(), M, K, float(eps), int(group_size), int(bool(hadamard)), float(scale_mul),
             _stream(x))
    return [q, s]


def _whole_row_mode(hadamard):
    """hadamard argument of the power-of-two whole-row ops -> mode of the C ABI: False / None, True = "exact" (float32
    butterflies), "fast" (matrix cores where a kernel exists: K = 4096; else the butterflies)."""
    _check(hadamard in (True, False, None, "exact", "fast"), "hadamard must be True / 'exact', 'fast' or False")
    return {True: FLH_HAD_F32, "exact": FLH_HAD_F32, "fast": FLH_HAD_MFMA, False: FLH_HAD_NONE, None: FLH_HAD_NONE}[hadamard]


def rmsnorm_rotate_and_quantize_i4(x, weight, eps, hadamard=True, clip_ratio=1.0, return_rotated=False):
    """RMSNorm (flh/nn/normalization.py:12-20) + whole-row rotation + per-token quantiser in one launch:
    x [M, K] fp16, K in {512, ..., 8192}, weight [K] fp16 or None -> (q [M, K/2] u8, scales [M, 1] fp16
    [, y [M, K] fp16]) of rotate_and_quantize_i4(rmsnorm(x), hadamard="exact" / False)."""
    _check(x.is_cuda, "Input tensor must be on CUDA")
    _check(x.dtype == torch.float16, "Input tensor must be float16 (half)")
    _check(x.dim() == 2 and x.is_contiguous(), "Input tensor must be 2D and contiguous")
    M, K = x.shape
    _check(K in (512, 1024, 2048, 4096, 8192), "Last dimension must be 512, 1024, 2048, 4096 or 8192")
    if weight is not None:
        _check(weight.is_cuda and weight.dtype == torch.float16 and weight.is_contiguous() and weight.numel() == K,
               "weight must be a contiguous float16 CUDA tensor of K values")
    q = torch.empty((M, K // 2), dtype=torch.uint8, device=x.device)
    s = torch.empty((M, 1), dtype=torch.float16, device=x.device)
    y = torch.empty_like(x) if return_rotated else None
    if M:
        _run("flh_rmsnorm_rotate_quant_i4", x.device, x.data_ptr(), weight.data_ptr() if weight is not None else None,
             float(eps), q.data_ptr(), s.data_ptr(), y.data_ptr() if y is not None else None, M, K,
             _whole_row_mode(hadamard), float(clip_ratio), _stream(x))
    return (q, s, y) if return_rotated else (q, s)


def add_rmsnorm_rotate_and_quantize_i4(x, add, weight, eps, hadamard=True, clip_ratio=1.0):
    """The residual addition in front of rmsnorm_rotate_and_quantize_i4, in the same launch: x, add [M, K] fp16 ->
    (x + add [M, K] fp16, q [M, K/2] u8, scales [M, 1] fp16), q and scales those of
    rmsnorm_rotate_and_quantize_i4(x + add, weight, eps, hadamard, clip_ratio)."""
    _check(x.is_cuda and add.is_cuda and x.device == add.device, "Input tensors must be on CUDA")
    _check(x.dtype == torch.float16 and add.dtype == torch.float16, "Input tensors must be float16 (half)")
    _check(x.dim() == 2 and x.shape == add.shape and x.is_contiguous() and add.is_contiguous(),
           "x and add must be contiguous 2D tensors of one shape")
    M, K = x.shape
    _check(K in (512, 1024, 2048, 4096, 8192), "Last dimension must be 512, 1024, 2048, 4096 or 8192")
    if weight is not None:
        _check(weight.is_cuda and weight.dtype == torch.float16 and weight.is_contiguous() and weight.numel() == K,
               "weight must be a contiguous float16 CUDA tensor of K values")
    total = torch.empty_like(x)
    q = torch.empty((M, K // 2), dtype=torch.uint8, device=x.device)
    s = torch.empty((M, 1), dtype=torch.float16, device=x.device)
    if M:
        _run("flh_add_rmsnorm_rotate_quant_i4", x.device, x.data_ptr(), add.data_ptr(), total.data_ptr(),
             weight.data_ptr() if weight is not None else None, float(eps), q.data_ptr(), s.data_ptr(), M, K,
             _whole_row_mode(hadamard), float(clip_ratio), _stream(x))
    return total, q, s


def rotate_and_quantize_f6(x, hadamard=True, clip_ratio=1.0, norm_weight=None, eps=None, add=None):
    """rotate_and_quantize_i4 (one scale per token) with the codes written in the 6-bit operand format of gemm_f6_*
    directly: x [M, K] fp16 -> (encoded [M, K / 128 * 96] u8, scales [M, 1] fp16), the bytes of encode_f6(q).
    K = 512 .. 8192 a power of two (float32 butterflies, `hadamard` True / "exact" / False) -- optionally behind RMSNorm
    (`eps` given; `norm_weight` [K] fp16 or None) and a residual addition (`add` [M, K]: the sum is returned first) --
    or K = 11008 / 14336 on the matrix cores (`hadamard` True / "fast")."""
    _check(x.is_cuda and x.dtype == torch.float16 and x.dim() == 2 and x.is_contiguous(),
           "Input tensor must be a contiguous 2D float16 CUDA tensor")
    M, K = x.shape
    dense = K in (11008, 14336)
    _check(dense or K in (512, 1024, 2048, 4096, 8192), "Last dimension must be a power of two in 512 .. 8192, 11008 or 14336")
    if dense:
        _check(hadamard in (True, "fast") and eps is None and add is None, "K = 11008 / 14336: matrix-core rotation, no prologue")
        mode = FLH_HAD_MFMA
    else:
        _check(hadamard != "fast" or K == 4096, "power-of-two K: the matrix-core rotation ('fast') exists for K = 4096")
        mode = _whole_row_mode(hadamard)
    _check(add is None or eps is not None, "the residual addition comes with the RMSNorm prologue (eps)")
    if add is not None:
        _check(add.is_cuda and add.dtype == torch.float16 and add.shape == x.shape and add.is_contiguous()
               and add.device == x.device, "add must be a contiguous float16 CUDA tensor of x's shape")
    if norm_weight is not None:
        _check(eps is not None and norm_weight.is_cuda and norm_weight.dtype == torch.float16 and norm_weight.is_contiguous()
               and norm_weight.numel() == K and norm_weight.device == x.device,
               "norm_weight must be a contiguous float16 CUDA tensor of K values (with eps)")
    enc = torch.empty((M, K // 128 * 96), dtype=torch.uint8, device=x.device)
    s = torch.empty((M, 1), dtype=torch.float16, device=x.device)
    total = torch.empty_like(x) if add is not None else None
    if M:
        _run("flh_rotate_quant_f6", x.device, x.data_ptr(), add.data_ptr() if add is not None else None,
             total.data_ptr() if total is not None else None, 1 if eps is not None else 0,
             norm_weight.data_ptr() if norm_weight is not None else None, float(eps or 0.0), enc.data_ptr(), s.data_ptr(), M, K,
             mode, float(clip_ratio), _stream(x))
    return (total, enc, s) if add is not None else (enc, s)


def rotate_and_quantize_i4(x, hadamard=True, had_group=0, scale_group=0, clip_ratio=1.0, return_rotated=False):
    """Whole-row online rotation + symmetric int4 quantise + pack: x [M, K] fp16 ->
    (q [M, K/2] u8, scales [M, 1 or K/scale_group] fp16 [, y [M, K] fp16]).
    K = 2^m, 28 * 2^m or 172 * 2^m (any literal size of the reference's get_hadK) when
    `hadamard`; had_group > 0 rotates each contiguous group independently.
    hadamard: False / "exact" (float32 butterflies: the bit-exact mode for power-of-two K) / "fast"
    (matrix cores; not bit-exact: K = 4096 differs from the exact transform in fewer than 1e-5 of the
    codes, K = 11008 / 14336 in about 4e-4 of them by one step) / True = "exact" for power-of-two K and
    "fast" for K = 11008 / 14336, where no summation order of the dense factor is defined by the
    reference and the float32 kernel is ten times slower at the same accuracy."""
    if hadamard is True:
        hadamard = "fast" if x.size(-1) in (11008, 14336) else "exact"
    mode = {False: FLH_HAD_NONE, "exact": FLH_HAD_F32, "fast": FLH_HAD_MFMA, None: FLH_HAD_NONE}[hadamard]
    _check(x.is_cuda, "Input tensor must be on CUDA")
    _check(x.dtype == torch.float16, "Input tensor must be float16 (half)")
    _check(x.dim() == 2 and x.is_contiguous(), "Input tensor must be 2D and contiguous")
    M, K = x.shape
    ns = K // scale_group if scale_group and scale_group > 0 else 1
    q = torch.empty((M, K // 2), dtype=torch.uint8, device=x.device)
    s = torch.empty((M, ns), dtype=torch.float16, device=x.device)
    y = torch.empty_like(x) if return_rotated else None
    if M == 0:
        return (q, s, y) if return_rotated else (q, s)
    _run("flh_rotate_quant_i4", x.device, x.data_ptr(), q.data_ptr(), s.data_ptr(), y.data_ptr() if y is not None else None,
         M, K, mode, int(had_group or 0), int(scale_group or 0),
         float(clip_ratio), _stream(x))
    return (q, s, y) if return_rotated else (q, s)
