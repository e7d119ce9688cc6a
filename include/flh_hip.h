/*
 * libflh_hip -- C ABI of the MI355X (gfx950) implementation of FLH's W4A4 linear-layer
 * hot path: fast Walsh-Hadamard rotation, symmetric int4 quantise-and-pack of fp16
 * activations, and int4 x int4 GEMM with int32 accumulation and fp16 dequant epilogue.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer on the current HIP device; buffers are borrowed
 *     for the duration of the (asynchronous) launch only; nothing is allocated or freed;
 *   - fp16 values travel as uint16_t bit patterns (IEEE binary16);
 *   - packed int4: byte j of a row holds element 2j in bits 0-3 and element 2j+1 in
 *     bits 4-7, two's complement codes in [-8, 7]
 *     (reference: flh/functional/quantization.py:43-49, flh/kernels/had_and_quant.cu:142-147);
 *   - `stream` is a hipStream_t passed as void* (NULL = the legacy default stream);
 *   - functions returning int return FLH_OK (0) or a negative FLH_E* code and leave a
 *     message retrievable with flh_last_error() (thread local).  The `void` functions
 *     carry the reference's own native signatures and launch on the default stream.
 */
#ifndef FLH_HIP_H
#define FLH_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define FLH_OK 0
#define FLH_EINVAL (-1)   /* bad shape / argument                      */
#define FLH_ELAUNCH (-2)  /* HIP reported an error at launch           */
#define FLH_EDEVICE (-3)  /* the current device is not a gfx950 device */

typedef uint16_t flh_half; /* IEEE binary16 bit pattern */

/* version of this ABI (bumped on any incompatible change) */
int flh_abi_version(void);
/* message of the last failing call on this thread ("" if none) */
const char* flh_last_error(void);
/* set-up of the current device, once per device: checks the device and builds the constant tables of the
 * matrix-core rotation (a short kernel on the default stream, waited for).  Optional -- first use on a device does
 * the same -- but call it before capturing a stream into a graph, since that first use synchronises. */
int flh_init(void);

/* ---------------------------------------------------------------------------------
 * int4 x int4 GEMM + dequant:  D[m,n] = fp16( sum_g float(acc_g[m,n]) * (As[m,g] * Bs[n,g]) )
 *   A [M, K/2] u8, B [N, K/2] u8 (both K-contiguous), D [M, N] fp16, K % 128 == 0.
 *   a_scale [M, a_cols], b_scale [N, b_cols] fp16 with *_cols == 1 (one scale per row,
 *   i.e. per token / per output channel) or K / group (group in {32, 64, 128}).
 *   a_cols == b_cols == 1 gives fp16(float(acc) * (a * b)) -- one rounding to fp32, one to fp16.
 *   a_cols == 1 < b_cols (one scale per token, group-scaled weights; not offered by the reference kernel):
 *   the token scale is applied once, after the groups -- fp16( (sum_g float(acc_g) * Bs[n,g]) * As[m] ).
 *   The group sum is accumulated in float32 in ascending g with one fused multiply-add per group.
 *   M <= 64 (M <= 16 with scale groups of 128) runs a weight-streaming decode kernel, larger M the tiled one;
 *   both give the same bits.
 * Replaces flh._CUDA.gemm_i4_dequant_o16 / _gs (flh/cuda/flh_cuda_bindings.cpp:75-113,
 * 254-299) -> flhDenseLayerGEMM_i4_o16 (flh/kernels/gemm_and_dequant_i4.cu:471-508) and
 * the per-token x per-channel epilogue of benchmark/nn/benchmark_linear_flh.py:74-86.
 * Unlike the reference kernel, N and M need not be multiples of the tile.
 * --------------------------------------------------------------------------------- */
int flh_gemm_i4_o16(const uint8_t* A, const uint8_t* B, const flh_half* a_scale, const flh_half* b_scale,
                    flh_half* D, size_t M, size_t N, size_t K, int a_cols, int b_cols, int group,
                    void* stream);

/* flh_gemm_i4_o16 with the residual addition of a decoder layer in its epilogue: D = fp16(residual + fp16(result)), the
 * bits of the GEMM's own fp16 output followed by an fp16 addition (hidden = residual + o_proj(...) resp. + down_proj(...),
 * flh/quantized_model/modeling_llama.py:600-618).  residual [M, N] fp16, 16-byte aligned; it may be D (in-place update of
 * the residual stream).  No native counterpart in the reference, which adds in torch. */
int flh_gemm_i4_add_o16(const uint8_t* A, const uint8_t* B, const flh_half* a_scale, const flh_half* b_scale,
                        const flh_half* residual, flh_half* D, size_t M, size_t N, size_t K, int a_cols, int b_cols,
                        int group, void* stream);

/* flh_gemm_i4_o16 for several weight matrices that share the activations -- q / k / v, gate / up -- in ONE launch:
 * D[s] [M, N[s]] = the result of flh_gemm_i4_o16(A, B[s], a_scale, b_scale[s], ...) for s < count <= 4, same bits.
 * B, b_scale, D and N are host arrays of `count` entries (device pointers resp. sizes); a_cols, b_cols and group
 * hold for every matrix.  The launch tiles the concatenated output columns, so the compute units see one large
 * problem instead of several short ones (the tail of one GEMM no longer idles next to the head of the next).
 * No counterpart in the reference, which calls its GEMM once per linear with the same quantised activations
 * (flh/quantized_model/modeling_llama.py:389-401). */
int flh_gemm_i4_o16_multi(const uint8_t* A, const flh_half* a_scale, int count, const uint8_t* const* B,
                          const flh_half* const* b_scale, flh_half* const* D, const size_t* N, size_t M, size_t K,
                          int a_cols, int b_cols, int group, void* stream);

/* The q / k / v projections of an attention block in one launch whose epilogue applies the rotary embedding and writes the
 * key / value cache: flh_gemm_i4_o16_multi (three weight matrices B[0..2] = q, k, v with Hq, Hkv, Hkv heads of 128 channels,
 * scales b_scale[0..2]) followed by flh_rope_kv_cache_f16, same bits, without the pass over q, k and v in between
 * (flh/quantized_model/modeling_llama.py:386-424 computes the three projections, transformers' apply_rotary_pos_emb and the
 * cache update as separate tensor operations).  Rows of A are tokens b * T + t; cos, sin [T, 128] and positions [T] (int64,
 * on the device) as in flh_rope_kv_cache_f16; q_out [batch, T, Hq, 128] receives the rotated queries, k_cache / v_cache
 * [batch, Hkv, max_len, 128] the rotated keys resp. the values at slot positions[t] (a position outside the cache writes
 * nothing).  Scales as in flh_gemm_i4_o16 (groups of 128 only). */
int flh_gemm_i4_qkv_rope_o16(const uint8_t* A, const flh_half* a_scale, const uint8_t* const* B,
                             const flh_half* const* b_scale, const flh_half* cos, const flh_half* sin,
                             const int64_t* positions, flh_half* q_out, flh_half* k_cache, flh_half* v_cache,
                             uint32_t batch, uint32_t T, uint32_t Hq, uint32_t Hkv, uint32_t max_len, size_t K,
                             int a_cols, int b_cols, int group, void* stream);

/* The gate and up projections of a SwiGLU MLP in one launch that stores only their combination:
 *   D[m, c] = fp16( float(fp16(silu(gate[m, c]))) * float(up[m, c]) ),  silu(g) = g / (1 + exp(-g)) in float32,
 * where gate = flh_gemm_i4_o16(A, B_gate, a_scale, gate_scale, ...) and up = the same with B_up / up_scale, both
 * [M, N] and rounded to fp16 exactly as those calls would store them -- D is what the reference's MLP computes with
 * two GEMM calls and two torch kernels, act_fn(gate_proj(x)) * up_proj(x) (flh/quantized_model/modeling_llama.py:522-526),
 * before it quantises the product for down_proj.  A workgroup computes the same output channels of both matrices, so
 * the two fp16 [M, N] intermediates never go to memory.  Scale layouts as flh_gemm_i4_o16 (group-scaled operands:
 * groups of 128 only).  The exponential and the reciprocal are the device's: against a float64 evaluation the fp16
 * result differs in its last bit in fewer than 2e-3 of the values. */
int flh_gemm_i4_swiglu_o16(const uint8_t* A, const uint8_t* B_gate, const uint8_t* B_up, const flh_half* a_scale,
                           const flh_half* gate_scale, const flh_half* up_scale, flh_half* D, size_t M, size_t N,
                           size_t K, int a_cols, int b_cols, int group, void* stream);

/* Decode: flh_rotate_quant_i4 (float32 butterflies, one scale per token) and flh_gemm_i4_o16 in ONE launch, for one
 * to four tokens: x [M, 4096] fp16 (M <= 4), B [N, 2048], b_scale [N, b_cols] with b_cols = 1 or 32 -> D [M, N] fp16.
 * Every workgroup rotates and quantises the tokens itself (the additions of the stand-alone kernel in the same
 * order, hence the same codes and scales) while its weights arrive, so the outputs are bit-identical to the two
 * calls and a decode step loses one launch per GEMM.  It pays for one or two tokens (about a microsecond of repeated
 * work per token and workgroup against a launch of 4-5 us).  No native counterpart in the reference, whose
 * quantised model quantises in its own launch (flh/quantized_model/modeling_llama.py:389-393) and whose GEMM
 * always computes a full 128-row tile (flh/kernels/gemm_and_dequant_i4.cu:471-508). */
int flh_rotate_quant_gemm_i4_o16(const flh_half* x, const uint8_t* B, const flh_half* b_scale, flh_half* D, size_t M,
                                 size_t N, size_t K, int b_cols, void* stream);
/* ... and for several weight matrices that share the tokens (arrays as in flh_gemm_i4_o16_multi, count <= 4). */
int flh_rotate_quant_gemm_i4_o16_multi(const flh_half* x, int count, const uint8_t* const* B,
                                       const flh_half* const* b_scale, flh_half* const* D, const size_t* N, size_t M,
                                       size_t K, int b_cols, void* stream);

/* flh_rotate_quant_gemm_i4_o16_multi with the prologues of flh_rmsnorm_rotate_quant_i4 / flh_add_rmsnorm_rotate_quant_i4 in
 * front of the rotation, still one launch: the tokens are RMS-normalised (weight [K] fp16 or null, eps), after the
 * residual addition fp16(x + add) when add / sum_out [M, K] are given (both or neither; sum_out receives the sum and
 * overlaps neither input).  M <= 4, K = 4096.  A decode step's "residual + attention output -> norm -> quantiser ->
 * q / k / v" (flh/quantized_model/modeling_llama.py:389-393, 600-618) as one launch; same bits as the separate launches. */
int flh_rmsnorm_rotate_quant_gemm_i4_o16_multi(const flh_half* x, const flh_half* add, flh_half* sum_out,
                                               const flh_half* weight, float eps, int count, const uint8_t* const* B,
                                               const flh_half* const* b_scale, flh_half* const* D, const size_t* N, size_t M,
                                               size_t K, int b_cols, void* stream);

/* The raw int32 accumulators C[m,n] = sum_k A[m,k] * B[n,k] (for parity checks of the
 * contraction itself; the reference keeps them in registers,
 * flh/kernels/gemm_and_dequant_i4.cu:384-453). */
int flh_gemm_i4_i32(const uint8_t* A, const uint8_t* B, int32_t* C, size_t M, size_t N, size_t K,
                    void* stream);

/* Reference-native signatures (flh/cuda/flh_cuda_bindings.cpp:12-23 and
 * flh/kernels/gemm_and_dequant_i4_gs.h:20-30): scales are [M, K/128] / [N, K/128]
 * (resp. K/group_size), default stream. */
void flhDenseLayerGEMM_i4_o16(const uint8_t* A, const uint8_t* B, const flh_half* A_scale,
                              const flh_half* B_scale, flh_half* D, size_t M, size_t N, size_t K);
void flhDenseLayerGEMM_i4_o16_gs(int group_size, const uint8_t* A, const uint8_t* B, flh_half* D,
                                 size_t M, size_t N, size_t K, const flh_half* A_scale,
                                 const flh_half* B_scale);

/* ---------------------------------------------------------------------------------
 * Group kernels with the arithmetic of the reference's CUDA kernels: x [R, G] fp16,
 * G in {32, 64, 128}; optional unnormalised FWHT-G with every butterfly rounded to fp16;
 * s = fp16(max|y| / 7), s <= fp16(1e-6) -> 1; q = clamp(rint(fp16(y / s)), -8, 7);
 * q_packed [R, G/2] u8, scales [R] fp16.  scale_mul (> 0, normally 1) is a constant factor on the STORED scales
 * only, fp16(float(s) * scale_mul): with 1 / sqrt(G) it folds the rescaling that ActQuantizer.forward applies
 * after the unnormalised transform (flh/nn/quantization.py:159) into the same launch.
 * Replaces had_and_quant_host[_gs] (flh/kernels/had_and_quant.cu:158-176,
 * had_and_quant_gs.cu:256-275) and quant_and_pack_host[_gs] (quant_and_pack.cu:99-117,
 * quant_and_pack_gs.cu:187-206).
 * --------------------------------------------------------------------------------- */
int flh_group_quant_i4(const flh_half* x, uint8_t* q_packed, flh_half* scales, uint32_t R, int group,
                       int hadamard, float scale_mul, void* stream);
void had_and_quant_host(const flh_half* data, uint8_t* quantized, flh_half* scales, uint32_t M);
void quant_and_pack_host(const flh_half* data, uint8_t* quantized, flh_half* scales, uint32_t M);
void had_and_quant_host_gs(int group_size, const flh_half* data, uint8_t* quantized, flh_half* scales,
                           uint32_t M);
void quant_and_pack_host_gs(int group_size, const flh_half* data, uint8_t* quantized, flh_half* scales,
                            uint32_t M);

/* -------------------------------------------------------------------------------------
 * The same GEMM on the 6-bit floating-point matrix instruction (no counterpart in the reference; for callers that
 * can keep a second encoding of their operands: twice the matrix rate of the int8 path, bit-identical results).
 * Every int4 code is exactly representable in e3m2, products and partial sums are integers below 2^24, so the
 * float32 accumulator holds the exact integer sum.  Operands are re-encoded once at 6 bits per code:
 *   flh_encode_f6:  packed_i4 [rows, K/2] u8  ->  encoded [rows, K/128 * 96] u8   (K a multiple of 128)
 * weights when they are loaded, activations after the quantiser.  Then
 *   flh_gemm_f6_o16:  D[m, n] = fp16( float(sum_k A[m,k] * B[n,k]) * (a_scale[m] * b_scale[n]) )
 * with a_scale [M], b_scale [N] (the result of flh_gemm_i4_o16 with a_cols = b_cols = 1 on the same codes), and
 *   flh_gemm_f6_i32:  the int32 sums.
 * Layout of one 96-byte block (128 codes of one row): code k = 64 m + 32 h + pos is the 6-bit field at bit 6 pos of
 * the 24 bytes at offset 48 h + 24 m; a code c is stored as sign << 5 | {0, 12, 16, 18, 20, 21, 22, 23, 24}[|c|].
 * --------------------------------------------------------------------------------- */
int flh_encode_f6(const uint8_t* packed_i4, uint8_t* encoded, size_t rows, size_t K, void* stream);
int flh_gemm_f6_o16(const uint8_t* A6, const uint8_t* B6, const flh_half* a_scale, const flh_half* b_scale,
                    flh_half* D, size_t M, size_t N, size_t K, void* stream);
int flh_gemm_f6_i32(const uint8_t* A6, const uint8_t* B6, int32_t* C, size_t M, size_t N, size_t K, void* stream);
/* The group quantiser of flh_group_quant_i4 with groups of 128, writing its codes in that format directly
 * (x [M, K] fp16 -> encoded [M, K/128 * 96], scales [M, K/128]); same codes and scales, no separate encoding pass. */
int flh_group_quant_f6(const flh_half* x, uint8_t* encoded, flh_half* scales, uint32_t M, uint32_t K, int hadamard,
                       float scale_mul, void* stream);

/* The whole-row rotation + per-token quantiser writing the 6-bit operand format directly (no flh_encode_f6 pass):
 * encoded [M rows, K / 128 * 96 bytes] as flh_encode_f6 lays it out, scales [M].  hadamard FLH_HAD_NONE / FLH_HAD_F32 with
 * K = 512 .. 8192 a power of two, optionally with the prologues of flh_rmsnorm_rotate_quant_i4 (rmsnorm != 0; weight [K]
 * or null, eps) and flh_add_rmsnorm_rotate_quant_i4 (add / sum_out [M, K], both or neither, only with rmsnorm);
 * FLH_HAD_MFMA with K = 4096 (any prologue) or K = 11008 / 14336 (no prologue).  The bytes equal flh_encode_f6 of the nibble output of the
 * corresponding flh_*rotate_quant_i4 call, the scales are the same.  No counterpart in the reference. */
int flh_rotate_quant_f6(const flh_half* x, const flh_half* add, flh_half* sum_out, int rmsnorm, const flh_half* weight,
                        float eps, uint8_t* encoded, flh_half* scales, uint32_t M, uint32_t K, int hadamard, float clip_ratio,
                        void* stream);
/* Group scales of 128 codes on the same instruction: b_scale [N, K/128], a_scale [M, K/128] (a_cols = K/128) or
 * [M] (a_cols = 1: one scale per token, applied after the groups).  The float32 accumulator makes the fold per
 * group one FMA per output; same bits as flh_gemm_i4_o16 with group = 128 on the same codes and scales. */
int flh_gemm_f6_o16_gs(const uint8_t* A6, const uint8_t* B6, const flh_half* a_scale, const flh_half* b_scale,
                       flh_half* D, size_t M, size_t N, size_t K, int a_cols, int b_cols, void* stream);
/* flh_gemm_f6_o16 (a_cols = b_cols = 1) resp. flh_gemm_f6_o16_gs for several encoded weight matrices that share the
 * encoded activations, in one launch (arrays as in flh_gemm_i4_o16_multi, count <= 4); same bits as the single calls. */
int flh_gemm_f6_o16_multi(const uint8_t* A6, const flh_half* a_scale, int count, const uint8_t* const* B6,
                          const flh_half* const* b_scale, flh_half* const* D, const size_t* N, size_t M, size_t K,
                          int a_cols, int b_cols, void* stream);

/* flh_gemm_i4_add_o16 on 6-bit operands (a_cols = b_cols = 1, or groups of 128 as in flh_gemm_f6_o16_gs); same bits. */
int flh_gemm_f6_add_o16(const uint8_t* A6, const uint8_t* B6, const flh_half* a_scale, const flh_half* b_scale,
                        const flh_half* residual, flh_half* D, size_t M, size_t N, size_t K, int a_cols, int b_cols,
                        void* stream);

/* flh_gemm_i4_qkv_rope_o16 on 6-bit operands (a_cols = b_cols = 1, or groups of 128 as in flh_gemm_f6_o16_gs); same bits. */
int flh_gemm_f6_qkv_rope_o16(const uint8_t* A6, const flh_half* a_scale, const uint8_t* const* B6,
                             const flh_half* const* b_scale, const flh_half* cos, const flh_half* sin,
                             const int64_t* positions, flh_half* q_out, flh_half* k_cache, flh_half* v_cache,
                             uint32_t batch, uint32_t T, uint32_t Hq, uint32_t Hkv, uint32_t max_len, size_t K,
                             int a_cols, int b_cols, void* stream);

/* flh_gemm_i4_swiglu_o16 on 6-bit operands: gate = A . Bg^T and up = A . Bu^T in one launch that stores only
 * D[m, n] = fp16(fp16(silu(gate)) * up), [M, N] with N the width of one of the two encoded weight matrices.  a_cols = b_cols
 * = 1: one scale per row / channel; b_cols = K / 128 with a_cols 1 or K / 128: groups of 128.  Same bits as
 * flh_gemm_i4_swiglu_o16 on the nibble operands. */
int flh_gemm_f6_swiglu_o16(const uint8_t* A6, const uint8_t* B6_gate, const uint8_t* B6_up, const flh_half* a_scale,
                           const flh_half* gate_scale, const flh_half* up_scale, flh_half* D, size_t M, size_t N, size_t K,
                           int a_cols, int b_cols, void* stream);

/* -------------------------------------------------------------------------------------
 * The two elementwise producers of quantised activations in a Llama block, fused into the group quantiser so
 * that the fp16 intermediate never goes to memory.  Neither has a native counterpart in the reference, which
 * runs them as separate torch kernels in front of ActQuantizer; the outputs are q_packed / scales exactly as
 * flh_group_quant_i4 would give on the fp16 intermediate defined below.
 *
 * flh_silu_mul_group_quant_i4: gate, up [R, G] fp16 (a [M, I] pair viewed as rows of G);
 *   x = fp16( float(fp16(silu(float(gate)))) * float(up) ), silu(g) = g / (1 + exp(-g)) in float32
 *   (the product the reference's MLP hands to its second quantiser, flh/quantized_model/modeling_llama.py:522-526).
 * flh_rmsnorm_group_quant_i4: x [M, K] fp16, weight [K] fp16 or NULL (= ones), K a multiple of `group`, K <= 16384;
 *   y = fp16( float(x) * rsqrt(sum_k x^2 / K + eps) [* float(weight)] ), statistics and products in float32
 *   (flh/nn/normalization.py:12-20); scales [M, K / group].
 * Both: float32 summation order and the rounding of exp, reciprocal and square root are the device's, so agreement with a CPU evaluation is
 * to the last bit of the fp16 intermediate in all but a few values per million, not bit-exact.
 * --------------------------------------------------------------------------------- */
int flh_silu_mul_group_quant_i4(const flh_half* gate, const flh_half* up, uint8_t* q_packed, flh_half* scales,
                                uint32_t R, int group, int hadamard, float scale_mul, void* stream);
int flh_rmsnorm_group_quant_i4(const flh_half* x, const flh_half* weight, uint8_t* q_packed, flh_half* scales,
                               uint32_t M, uint32_t K, float eps, int group, int hadamard, float scale_mul,
                               void* stream);

/* RMSNorm in front of the whole-row rotate + quantise (no native counterpart in the reference, which runs
 * RMSNorm.forward in torch, flh/nn/normalization.py:12-20, before its quantiser): x [M, K] fp16, weight [K] fp16 or
 * NULL, K in {512, 1024, 2048, 4096, 8192}; the fp16 row y = fp16(float(x) * rsqrt(sum x^2 / K + eps) [* weight]) is
 * then treated exactly as flh_rotate_quant_i4 treats its input (hadamard FLH_HAD_NONE or FLH_HAD_F32, one scale per
 * row, optional clip, optional y_out = the rotated row).  The float32 summation order is the device's.
 * hadamard FLH_HAD_MFMA: K = 4096 without y_out rotates on the matrix cores (not bit-exact, as for flh_rotate_quant_i4;
 * other shapes take FLH_HAD_F32); the same holds for flh_add_rmsnorm_rotate_quant_i4 and flh_rotate_quant_f6. */
int flh_rmsnorm_rotate_quant_i4(const flh_half* x, const flh_half* weight, float eps, uint8_t* q_packed,
                                flh_half* scales, flh_half* y_out, uint32_t M, uint32_t K, int hadamard,
                                float clip_ratio, void* stream);

/* In-place unnormalised fp16 FWHT of each row of x [R, G], G in {32, 64, 128}
 * (had_trans_half_cuda / _64_ / _32_, flh/kernels/cuda_had_kernel.cu:295-354). */
int flh_fwht_f16_inplace(flh_half* x, uint32_t R, int group, void* stream);

/* ---------------------------------------------------------------------------------
 * Online rotation + quantisation of whole activation rows (the QuaRot-style path the
 * reference defines only in torch): x [M, K] fp16 ->
 *   y = fp16( H_K x / sqrt(K) )       K = 2^m, or Kd * 2^m with Kd one of the literal orders 12 ... 172 (matmul_hadU,
 *                                     flh/functional/hadamard.py:92-113), or y = x; K a multiple of 16
 *   optional clip to +-fp16(max|y| * clip_ratio)              (flh/nn/quantization.py:173-178)
 *   per scale group (scale_group == 0: the whole row, else contiguous groups):
 *   s = fp16(max|y| / 7), s == 0 -> 1; q = clamp(rint(fp16(y / s)), -8, 7)  (:181-234)
 *   q_packed [M, K/2] u8, scales [M, K/scale_group or 1] fp16.
 * hadamard: FLH_HAD_NONE; FLH_HAD_F32 (butterflies in float32 in ascending stride order:
 * bit-exact with the float32 restatement of had_transform for power-of-two K; had_group > 0
 * rotates each contiguous group of that size independently); FLH_HAD_MFMA (the same
 * rotation evaluated on the matrix cores as M . X . H64 -- not bit-exact: for K = 4096 codes
 * differ from the exactly rounded transform at a rate below 1e-5; for K = 11008 / 14336 about
 * 4e-4 of the codes differ by one step and a scale may differ by one fp16 ulp; whole rows with
 * one scale per row only, K in {4096, 11008, 14336}; other shapes fall back to FLH_HAD_F32).
 * y_out (optional, may be NULL) receives the rotated fp16 rows (FLH_HAD_F32 / NONE only).
 * --------------------------------------------------------------------------------- */
#define FLH_HAD_NONE 0
#define FLH_HAD_F32 1
#define FLH_HAD_MFMA 2
int flh_rotate_quant_i4(const flh_half* x, uint8_t* q_packed, flh_half* scales, flh_half* y_out,
                        uint32_t M, uint32_t K, int hadamard, int had_group, int scale_group,
                        float clip_ratio, void* stream);

/* The residual addition in front of flh_rmsnorm_rotate_quant_i4: sum_out = fp16(x + add) row by row (one rounding per
 * value, torch's fp16 addition), then exactly flh_rmsnorm_rotate_quant_i4(sum_out, ...) -- x, add, sum_out [M, K] fp16 (sum_out
 * overlaps neither input), K = 512 .. 8192 a power of two, hadamard FLH_HAD_NONE or FLH_HAD_F32.  A decoder layer's
 * "hidden = residual + attn; residual = hidden; hidden = norm(hidden)" followed by the quantiser of the next linears
 * (flh/quantized_model/modeling_llama.py:600-618) in one launch instead of three.  Same bytes as the separate launches. */
int flh_add_rmsnorm_rotate_quant_i4(const flh_half* x, const flh_half* add, flh_half* sum_out, const flh_half* weight,
                                    float eps, uint8_t* q_packed, flh_half* scales, uint32_t M, uint32_t K, int hadamard,
                                    float clip_ratio, void* stream);

/* The SwiGLU product in front of the online rotation of down_proj, for decode-sized batches (M <= 256; prefill takes
 * flh_gemm_i4_swiglu_o16): x = fp16(fp16(silu(gate)) * up) row by row, then exactly flh_rotate_quant_i4(x, ..., FLH_HAD_MFMA,
 * one scale per row) -- gate, up [M, K] fp16 with K = 11008 (172 x 64) or 14336 (28 x 512); q_packed [M, K/2], scales [M].
 * The product is formed in LDS and never stored.  The reference runs act_fn(gate) * up as torch kernels in front of its
 * quantiser (flh/quantized_model/modeling_llama.py:522-526) and the online rotation of down_proj in front of that
 * (fake_quant/main.py:30-35).  Same codes and scales as the separate launches on the same fp16 product. */
int flh_silu_mul_rotate_quant_i4(const flh_half* gate, const flh_half* up, uint8_t* q_packed, flh_half* scales,
                                 uint32_t M, uint32_t K, void* stream);

/* RMSNorm on its own, optionally behind the residual addition -- a model's final norm in front of its fp16 head
 * (flh/nn/normalization.py:12-20 after the last residual addition of flh/quantized_model/modeling_llama.py:600-618):
 * s = add ? fp16(x + add) : x;  out = fp16( fl32(fl32(s) * rsqrt(sum(s^2) / K + eps)) * fl32(weight) ), statistics in
 * float32.  x, add (or NULL), out, sum_out (or NULL; receives s, needs add) [M, K] fp16; weight [K] fp16 or NULL (ones);
 * K a multiple of 8, at most 16384.  One launch for torch's addition and the eight kernels of the norm's expression. */
int flh_add_rmsnorm_f16(const flh_half* x, const flh_half* add, const flh_half* weight, float eps, flh_half* out,
                        flh_half* sum_out, uint32_t M, uint32_t K, void* stream);

/* The same product on its own: out[i] = fp16(fp16(silu(gate[i])) * up[i]) for n fp16 values (n a multiple of 8; out may
 * be gate or up).  One launch for the two torch kernels of modeling_llama.py:522-526 where no quantiser follows directly. */
int flh_silu_mul_f16(const flh_half* gate, const flh_half* up, flh_half* out, uint64_t n, void* stream);

/* ---------------------------------------------------------------------------------
 * Between the q / k / v GEMM and attention of a decode (or prefill) step: rotary position embedding of the query and
 * key heads and the write of the new keys / values into a preallocated cache, one launch.  No native counterpart in the
 * reference, whose attention calls transformers' apply_rotary_pos_emb and cache update as separate tensor operations
 * (flh/quantized_model/modeling_llama.py:403-424).
 *   q [B, T, Hq, d] fp16, rotated in place;  k, v [B, T, Hkv, d] fp16 (read only);
 *   cos, sin [T, d] fp16 (the tables of the T new positions);  positions [T] int64 ON THE DEVICE (the cache slots of
 *   the new tokens: a captured graph is replayed for other positions by overwriting this tensor);
 *   k_cache, v_cache [B, Hkv, max_len, d] fp16: slot positions[t] receives the rotated key resp. the value of token t
 *   (a position outside [0, max_len) writes nothing).
 * y = fp16( fp16(x * cos) + fp16(rotate_half(x) * sin) ), rotate_half((x1, x2)) = (-x2, x1) over the two halves of a
 * head -- the roundings of the tensor expression evaluated operation by operation in fp16.  d a multiple of 16.
 * --------------------------------------------------------------------------------- */
int flh_rope_kv_cache_f16(flh_half* q, const flh_half* k, const flh_half* v, const flh_half* cos, const flh_half* sin,
                          const int64_t* positions, flh_half* k_cache, flh_half* v_cache, uint32_t B, uint32_t T,
                          uint32_t Hq, uint32_t Hkv, uint32_t head_dim, uint32_t max_len, void* stream);

/* Causal attention of a block of T new tokens per sequence over the cache (prefill): query t sees the slots 0 .. past + t of
 * its sequence's keys / values (the block's own keys / values sit in slots past .. past + T - 1, where flh_rope_kv_cache_f16
 * or flh_gemm_i4_qkv_rope_o16 put them).  Stands where the reference calls flash-attn on the rotated projections
 * (flh/quantized_model/modeling_llama.py:426-460).  q [B, T, Hq, 128] fp16 (token-major, as those launches write it),
 * k_cache / v_cache [B, Hkv, max_len, 128], out [B, T, Hq * 128] fp16; head_dim must be 128, Hq a multiple of Hkv;
 * softmax(scale * q . k) in float32, probabilities rounded to fp16 for the second product, float32 accumulation. */
int flh_prefill_attention_f16(const flh_half* q, const flh_half* k_cache, const flh_half* v_cache, flh_half* out, uint32_t B,
                              uint32_t T, uint32_t Hq, uint32_t Hkv, uint32_t head_dim, uint32_t past, uint32_t max_len,
                              float scale, void* stream);

/* Attention of ONE new token per sequence over the cache that flh_rope_kv_cache_f16 fills (the decode step), grouped
 * queries included:  out[b, h] = softmax(q[b, h] . K[b, h / rep]^T * scale) V[b, h / rep]  over cache slots [0, kv_len),
 * rep = Hq / Hkv in {1, 2, 4, 8}, head_dim 64 or 128; scores, probabilities and sums in float32, fp16 in and out.
 *   q, out [B, Hq, d];  k_cache, v_cache [B, Hkv, max_len, d].
 * Stands where the reference's attention calls the flash-attn package on the cached keys / values
 * (flh/quantized_model/modeling_llama.py:449-460).  The cached positions are split into chunks of 64 that run in
 * parallel; their partial results meet in `workspace` (device memory, 16-byte aligned, at least
 * flh_decode_attention_workspace_bytes(B, Hq, d, kv_len) bytes, contents irrelevant before and after; launches that
 * share a workspace must not overlap, i.e. one workspace per stream).  Two launches on `stream`. */
size_t flh_decode_attention_workspace_bytes(uint32_t B, uint32_t Hq, uint32_t head_dim, uint32_t kv_len);
int flh_decode_attention_f16(const flh_half* q, const flh_half* k_cache, const flh_half* v_cache, flh_half* out,
                             uint32_t B, uint32_t Hq, uint32_t Hkv, uint32_t head_dim, uint32_t kv_len, uint32_t max_len,
                             float scale, void* workspace, size_t workspace_bytes, void* stream);

/* flh_decode_attention_f16 with the rotary embedding and the cache update of the step's new token inside, replacing
 * flh_rope_kv_cache_f16 (T = 1) + flh_decode_attention_f16 by one pair of launches: q [B, Hq, d], k_new / v_new [B, Hkv, d]
 * as the q / k / v GEMM wrote them (not rotated), cos / sin [d] of the new position, positions[0] (device int64) the
 * cache slot the new token takes in every sequence (< kv_len, else the new token is ignored).  The rotated key and the
 * value are written into k_cache / v_cache [B, Hkv, max_len, d] at that slot -- the same bytes flh_rope_kv_cache_f16 writes
 * -- and attention runs over the first kv_len slots including it; q is left as it came.  Reference: apply_rotary_pos_emb +
 * cache update + attention, flh/quantized_model/modeling_llama.py:403-460. */
int flh_decode_attention_rope_f16(const flh_half* q, const flh_half* k_new, const flh_half* v_new, const flh_half* cos,
                                  const flh_half* sin, const int64_t* positions, flh_half* k_cache, flh_half* v_cache,
                                  flh_half* out, uint32_t B, uint32_t Hq, uint32_t Hkv, uint32_t head_dim, uint32_t kv_len,
                                  uint32_t max_len, float scale, void* workspace, size_t workspace_bytes, void* stream);

/* flh_decode_attention_f16 for callers that cannot allocate device memory and have no workspace to hand over -- code
 * under stream capture, tight serving loops, harnesses that forbid allocation.  No counterpart in the reference.  It
 * allocates nothing: the partial results go to a static device array of flh_decode_attention_static_scratch_bytes()
 * (16 MiB) that every device the library runs on holds until the process ends.  A call that needs more
 * (B * Hq * ceil(kv_len / 64) * (head_dim + 2) * 4 bytes) is rejected with FLH_EINVAL.  All calls on one device share the
 * array: calls that overlap in time (different streams) race; calls on one stream do not.  Same results, bit for bit,
 * as flh_decode_attention_f16. */
size_t flh_decode_attention_static_scratch_bytes(void);
int flh_decode_attention_f16_static(const flh_half* q, const flh_half* k_cache, const flh_half* v_cache, flh_half* out,
                                    uint32_t B, uint32_t Hq, uint32_t Hkv, uint32_t head_dim, uint32_t kv_len,
                                    uint32_t max_len, float scale, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* FLH_HIP_H */
