// The reference's own native entry points, by name and argument list, on top of this library's C ABI.
//
// The reference's torch binding (flh/cuda/flh_cuda_bindings.cpp:12-73) declares one function with C linkage,
//   flhDenseLayerGEMM_i4_o16                                         (:12-23, defined gemm_and_dequant_i4.cu:471)
// and five with C++ linkage and `half*` parameters,
//   flhDenseLayerGEMM_i4_o16_gs   (:26-36, flh/kernels/gemm_and_dequant_i4_gs.h:20-30)
//   had_and_quant_host_gs         (:38-44, had_and_quant_gs.h)     quant_and_pack_host_gs  (:46-52, quant_and_pack_gs.h)
//   had_and_quant_host            (:60-65, had_and_quant.h:19-24)  quant_and_pack_host     (:68-73, quant_and_pack.h:19-24)
// A binding file compiled for HIP (where `half` is `__half`) looks for exactly those symbols: the C one unmangled, the
// others mangled over `__half`.  Both sets are defined here, plus C-linkage twins of the five (fp16 as uint16_t bit
// patterns) for callers without a C++ compiler.  All launch on the legacy default stream and return nothing, as the
// reference's do; a call that this library rejects (bad K, group size, alignment) prints the reason to stderr instead
// of leaving the outputs silently untouched.
#include <cstdio>

#include "common.h"
#include "../../include/flh_reference_native.h"

namespace {

void report(const char* who, int rc) {
  if (rc != FLH_OK) fprintf(stderr, "libflh_hip: %s failed (code %d): %s\n", who, rc, flh_last_error());
}

void gemm_gs(const char* who, int group_size, const uint8_t* A, const uint8_t* B, flh_half* D, size_t M, size_t N, size_t K,
             const flh_half* A_scale, const flh_half* B_scale) {
  const int ng = group_size > 0 ? (int)(K / group_size) : 0;
  report(who, flh_gemm_i4_o16(A, B, A_scale, B_scale, D, M, N, K, ng, ng, group_size, nullptr));
}

void group_quant(const char* who, int group_size, int hadamard, const flh_half* data, uint8_t* quantized, flh_half* scales,
                 uint32_t M) {
  report(who, flh_group_quant_i4(data, quantized, scales, M, group_size, hadamard, 1.0f, nullptr));
}

}  // namespace

// ---- C linkage ----------------------------------------------------------------------------------------------
extern "C" void flhDenseLayerGEMM_i4_o16(const uint8_t* A, const uint8_t* B, const flh_half* A_scale,
                                         const flh_half* B_scale, flh_half* D, size_t M, size_t N, size_t K) {
  gemm_gs("flhDenseLayerGEMM_i4_o16", 128, A, B, D, M, N, K, A_scale, B_scale);
}
extern "C" void flhDenseLayerGEMM_i4_o16_gs(int group_size, const uint8_t* A, const uint8_t* B, flh_half* D, size_t M,
                                            size_t N, size_t K, const flh_half* A_scale, const flh_half* B_scale) {
  gemm_gs("flhDenseLayerGEMM_i4_o16_gs", group_size, A, B, D, M, N, K, A_scale, B_scale);
}
extern "C" void had_and_quant_host(const flh_half* data, uint8_t* quantized, flh_half* scales, uint32_t M) {
  group_quant("had_and_quant_host", 128, 1, data, quantized, scales, M);
}
extern "C" void quant_and_pack_host(const flh_half* data, uint8_t* quantized, flh_half* scales, uint32_t M) {
  group_quant("quant_and_pack_host", 128, 0, data, quantized, scales, M);
}
extern "C" void had_and_quant_host_gs(int group_size, const flh_half* data, uint8_t* quantized, flh_half* scales,
                                      uint32_t M) {
  group_quant("had_and_quant_host_gs", group_size, 1, data, quantized, scales, M);
}
extern "C" void quant_and_pack_host_gs(int group_size, const flh_half* data, uint8_t* quantized, flh_half* scales,
                                       uint32_t M) {
  group_quant("quant_and_pack_host_gs", group_size, 0, data, quantized, scales, M);
}

// ---- C++ linkage, the reference's declarations verbatim (half = __half) ------------------------------------------
void flhDenseLayerGEMM_i4_o16_gs(int group_size, const uint8_t* A, const uint8_t* B, __half* D, size_t M_GLOBAL,
                                 size_t N_GLOBAL, size_t K_GLOBAL, const __half* A_scale, const __half* B_scale) {
  gemm_gs("flhDenseLayerGEMM_i4_o16_gs", group_size, A, B, (flh_half*)D, M_GLOBAL, N_GLOBAL, K_GLOBAL,
          (const flh_half*)A_scale, (const flh_half*)B_scale);
}
void had_and_quant_host(const __half* data, Int4Storage* quantized_data, __half* scales, uint32_t M) {
  group_quant("had_and_quant_host", 128, 1, (const flh_half*)data, quantized_data, (flh_half*)scales, M);
}
void quant_and_pack_host(const __half* data, Int4Storage* quantized_data, __half* scales, uint32_t M) {
  group_quant("quant_and_pack_host", 128, 0, (const flh_half*)data, quantized_data, (flh_half*)scales, M);
}
void had_and_quant_host_gs(int group_size, const __half* data, Int4Storage* quantized_data, __half* scales, uint32_t M) {
  group_quant("had_and_quant_host_gs", group_size, 1, (const flh_half*)data, quantized_data, (flh_half*)scales, M);
}
void quant_and_pack_host_gs(int group_size, const __half* data, Int4Storage* quantized_data, __half* scales, uint32_t M) {
  group_quant("quant_and_pack_host_gs", group_size, 0, (const flh_half*)data, quantized_data, (flh_half*)scales, M);
}
