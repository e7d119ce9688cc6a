/*
 * The reference's native function declarations, for a C++ binding file that is compiled for HIP and linked against
 * libflh_hip.so unchanged (C++ only: these have C++ linkage and `half` = `__half` parameters, as in the reference).
 *
 *   flhDenseLayerGEMM_i4_o16_gs   flh/cuda/flh_cuda_bindings.cpp:26-36, flh/kernels/gemm_and_dequant_i4_gs.h:20-30
 *   had_and_quant_host            flh_cuda_bindings.cpp:60-65, flh/kernels/had_and_quant.h:19-24
 *   quant_and_pack_host           flh_cuda_bindings.cpp:68-73, flh/kernels/quant_and_pack.h:19-24
 *   had_and_quant_host_gs         flh_cuda_bindings.cpp:38-44, flh/kernels/had_and_quant_gs.h
 *   quant_and_pack_host_gs        flh_cuda_bindings.cpp:46-52, flh/kernels/quant_and_pack_gs.h
 *
 * flhDenseLayerGEMM_i4_o16 has C linkage in the reference (flh_cuda_bindings.cpp:12-23) and is declared in flh_hip.h,
 * which also declares C-linkage twins of the five functions below (fp16 as uint16_t) for C callers.
 * Scales are [M, K/group_size] and [N, K/group_size] (group 128 for the functions without the parameter); group rows
 * are [M, group_size] fp16 -> [M, group_size/2] packed codes + [M] scales.  Default stream, no return value; a rejected
 * call prints the reason to stderr.
 */
#ifndef FLH_REFERENCE_NATIVE_H
#define FLH_REFERENCE_NATIVE_H
#ifdef __cplusplus

#include <hip/hip_fp16.h>
#include <stddef.h>
#include <stdint.h>

using Int4Storage = uint8_t;

void flhDenseLayerGEMM_i4_o16_gs(int group_size, const uint8_t* A, const uint8_t* B, __half* D, size_t M_GLOBAL,
                                 size_t N_GLOBAL, size_t K_GLOBAL, const __half* A_scale, const __half* B_scale);
void had_and_quant_host(const __half* data, Int4Storage* quantized_data, __half* scales, uint32_t M);
void quant_and_pack_host(const __half* data, Int4Storage* quantized_data, __half* scales, uint32_t M);
void had_and_quant_host_gs(int group_size, const __half* data, Int4Storage* quantized_data, __half* scales, uint32_t M);
void quant_and_pack_host_gs(int group_size, const __half* data, Int4Storage* quantized_data, __half* scales, uint32_t M);

#endif /* __cplusplus */
#endif /* FLH_REFERENCE_NATIVE_H */
