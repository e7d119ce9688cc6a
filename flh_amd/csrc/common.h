// Shared helpers of libflh_hip (gfx950 only).
#pragma once
#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>

#include <atomic>
#include <type_traits>

#include "../../include/flh_hip.h"
#include "../../include/flh_hip_testing.h"

namespace flh {

// record a message for flh_last_error() and return `code`
int fail(int code, const char* fmt, ...);
// check for a launch error on the current device
int check_launch(const char* what);

// Set-up that a process repeats on every device it drives (a kernel's LDS reservation, a constant table, the address of
// a __device__ array) is kept per device index.
constexpr int kMaxDevices = 64;
// the current device's index in [0, kMaxDevices) into *dev, or an error recorded for `what`
int current_device(int* dev, const char* what);
// the dynamic LDS a kernel has been granted on each device; one object with static storage (all zero) per kernel
struct LdsGrant {
  std::atomic<size_t> bytes[kMaxDevices];
};
// make `bytes` of dynamic LDS available to `kernel` on the current device unless that much already is
int reserve_lds(const void* kernel, size_t bytes, LdsGrant& grant, const char* what);

// true when any of the pointers is not a multiple of 16 bytes: rows are moved in 16-byte pieces (vector loads,
// direct-to-LDS loads, vector stores), and every row is a whole number of such pieces from an aligned base only
template <typename... P>
inline bool misaligned16(P... p) { return (((uintptr_t)p | ...) & 15) != 0; }

typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v2f __attribute__((ext_vector_type(2)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef _Float16 h2 __attribute__((ext_vector_type(2)));
typedef _Float16 h8 __attribute__((ext_vector_type(8)));
typedef _Float16 h4 __attribute__((ext_vector_type(4)));

// Keep a float32 value as computed: without this the compiler may merge a float32
// multiply (or multiply-add) with a following conversion to fp16 into one mixed-precision
// instruction that rounds once, where the arithmetic being reproduced rounds twice.
__device__ __forceinline__ float round_here(float v) {
  asm("" : "+v"(v));  // not volatile: free to be scheduled, but opaque to instruction fusion
  return v;
}

// eight fp16 additions (four packed pairs), each rounded once
__device__ __forceinline__ v4i add_h8(v4i a, v4i b) {
  v4i r;
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    const unsigned ua = (unsigned)a[d], ub = (unsigned)b[d];   // (scalar copies: a bit cast of a vector element miscompiles)
    const h2 s2 = __builtin_bit_cast(h2, ua) + __builtin_bit_cast(h2, ub);
    r[d] = (int)__builtin_bit_cast(unsigned, s2);
  }
  return r;
}

// fp16( float(fp16(silu(gate))) * float(up) ): the two roundings of torch's fp16 silu followed by its fp16 multiply
// (the product the reference's MLP hands to the quantiser of down_proj, flh/quantized_model/modeling_llama.py:522-526);
// silu in float32 as g * rcp(1 + exp(-g)) on the hardware exponential and reciprocal
__device__ __forceinline__ _Float16 silu_mul_f16(_Float16 gate, _Float16 up) {
  const float g = (float)gate;
  const _Float16 act = (_Float16)round_here(g * __builtin_amdgcn_rcpf(1.0f + __expf(-g)));
  return (_Float16)round_here((float)act * (float)up);
}

// 16 bytes per lane from global memory straight into LDS: lane i of the wave writes
// lds_base + 16 * i (lds_base wave-uniform).  Counted by vmcnt; the compiler does not know
// about it, so every wait for these loads is written out by hand below.
__device__ __forceinline__ void load_to_lds16(const void* gptr, unsigned lds_base) {
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, off" ::"s"(lds_base), "v"(gptr) : "memory", "m0");
}

// the same with a wave-uniform base address in scalar registers plus a 32-bit per-lane offset
__device__ __forceinline__ void load_to_lds16(const void* sbase, unsigned voffset, unsigned lds_base) {
  asm volatile("s_mov_b32 m0, %0\n\tglobal_load_lds_dwordx4 %1, %2" ::"s"(lds_base), "v"(voffset), "s"(sbase) : "memory", "m0");
}

// Workgroup barrier without the memory fence of __syncthreads(): the fence makes every wave wait for ALL of
// its outstanding LDS reads and global loads, which drains a software pipeline at every use.  For callers
// that order their own memory traffic with explicit waits; the "memory" clobber keeps the compiler from
// moving memory operations across it.
__device__ __forceinline__ void barrier_no_fence() { asm volatile("s_barrier" ::: "memory"); }

// every LDS (and scalar memory) operation of this wave has completed
__device__ __forceinline__ void wait_lgkmcnt0() { __builtin_amdgcn_s_waitcnt(0xC07F); }

template <int N>
__device__ __forceinline__ void wait_vmcnt() {
  static_assert(N >= 0 && N < 64, "vmcnt range");
  // s_waitcnt simm16: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt[5:4] << 14
  __builtin_amdgcn_s_waitcnt((N & 0xF) | ((N >> 4) << 14) | 0x0F70);
}

// f(integral_constant<int, 0>{}), ..., f(integral_constant<int, N - 1>{}): a loop whose index is a constant expression
// inside the body, so that it can select among register-resident objects (an index that is merely unrolled later sends
// a local array to scratch memory)
template <int N, int I = 0, typename F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    static_for<N, I + 1>(f);
  }
}

constexpr int kNumXCD = 8;  // MI355X: 8 accelerator dies, workgroup i is dispatched to die i % 8

// Map the hardware workgroup index to a logical one so that each die works on a
// contiguous range of logical indices (its own L2 then sees a compact set of tiles).
__device__ __forceinline__ unsigned xcd_contiguous(unsigned wg, unsigned total) {
  const unsigned per = total / kNumXCD, rem = total % kNumXCD;
  const unsigned xcd = wg % kNumXCD, slot = wg / kNumXCD;
  // dies [0, rem) own per+1 indices, the others per
  const unsigned base = xcd * per + (xcd < rem ? xcd : rem);
  return base + slot;
}

}  // namespace flh
