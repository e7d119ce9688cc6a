"""CPU oracle for the W4A4 linear hot path -- TEST INFRASTRUCTURE ONLY.

This package restates, in plain numpy, the arithmetic that the reference's own torch
code and CUDA kernels define for the hot path (pack/unpack of int4 nibbles, fast
Walsh-Hadamard rotation, symmetric int4 activation / weight quantisation, int4 x int4
GEMM with int32 accumulation and the fp16 dequantising epilogue).  It exists so that
the HIP kernels can be checked against something that follows the reference line by
line.  Nothing in the product (``flh_amd``) may import it: only ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` do.

Every function cites the reference file:line it follows.  Pinning status (what other
than "retyping the formula" fixes each function) is listed per module; the summary:

* ``pack``      -- pinned exhaustively (all 256 bytes) and by the byte formula that the
                   reference repeats in four places.
* ``hadamard``  -- power-of-two transforms pinned against the dense Sylvester matrix,
                   the involution H(H x) = n x, unit vectors, integer inputs (all
                   float widths must agree bit for bit) ; K x 2^m transforms pinned
                   against the dense Kronecker product built from the reference's
                   literal matrices (sha256 of the bit-packed literals is checked).
* ``quant``     -- pinned on closed-form rows (max = 7 * 2^e gives scale 2^e and
                   codes rint(y / 2^e) with visible half-to-even ties), against an
                   independent exact-rational evaluation, and against golden vectors
                   written from the reference's own torch code where that import was
                   possible (see tests/golden).
* ``prologue``  -- SwiGLU product and RMSNorm in front of the quantiser: pinned against
                   float64 evaluations over every fp16 input (silu) and on closed-form
                   rows (rmsnorm); device comparison by mismatch rate (exp / rsqrt and
                   summation order are the device's in the reference too).
* ``gemm``      -- int32 accumulators pinned against numpy int64 matmul (exact);
                   per-token x per-channel epilogue is a closed form (one fp32
                   rounding, one fp16 rounding); group epilogue follows the reference
                   kernel's ascending-group fp32 accumulation with fused multiply-add.
* ``layer``     -- a decoder layer / decode step composed of the pieces above with float64 rotary embedding and
                   attention, pinned by special cases (tests/test_oracle_layer.py).
* ``gptq``      -- GPTQ in the rotated basis in its elimination form, pinned by closed forms and properties and by
                   the reference's own output on eight seeded cases (tests/golden/gptq_vectors.npz, written from
                   flh/nn/gptq.py on the CPU by tests/golden/make_gptq_vectors.py; tests/test_oracle_gptq.py).

Parity unpinned (no vector of the reference can exist here, and no closed form decides the open choice):
``gemm.gemm_i4_dequant`` with group scales beyond rtol 1e-3 / atol 1e-2 (whether the reference's compiler fuses the
multiply-add of the fold cannot be observed); ``quant.kernel_had_and_quant`` on random data (CUDA-only arithmetic:
fp16 butterflies and the ``s <= 1e-6`` rule are restated from the kernel's text, pinned on integer and closed-form rows
only).
"""
from . import pack, hadamard, quant, gemm, linear  # noqa: F401
