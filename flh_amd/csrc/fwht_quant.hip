// Walsh-Hadamard rotation, symmetric int4 quantisation and nibble packing of fp16 rows.
//
// Three families of kernels live here:
//
//  1. group kernels (rows of G = 32 / 64 / 128 fp16) with the arithmetic of the
//     reference's CUDA kernels: every butterfly rounded to fp16, s = fp16(max / 7),
//     s <= fp16(1e-6) -> 1, q = clamp(rint(fp16(y / s)), -8, 7)
//     (flh/kernels/had_and_quant.cu:13-155, quant_and_pack.cu:8-97, cuda_had_kernel.cu:190-354);
//  2. the wave-per-row kernel for whole rows of K = 512 * J fp16 (J = 1 .. 16): butterflies
//     in float32 in ascending stride order, so that the fp16 result equals the float32
//     restatement of had_transform (flh/nn/quantization.py:42-74) bit for bit; strides
//     1, 2, 4 and >= 512 are register-to-register, strides 8 .. 256 cross lanes with DPP
//     (quad permutes, row mirrors) and v_permlane16/32_swap -- no LDS, no barrier;
//  3. a generic workgroup-per-row kernel (any K = Kd * 2^m, Kd one of the literal
//     Hadamard sizes, grouped rotation, grouped scales), staged in LDS.
//
// Quantisation (all kernels): the fp16 quotient y / s is needed only through
// rint(fp16(y / s)).  For every pair of fp16 values the code obtained from
// fp16(float(y) * r), r = the float32 reciprocal of s (even when r is off by one ulp),
// equals the code from the correctly rounded fp16 quotient -- verified exhaustively over
// all 6.3e8 (y, s) pairs with |y / s| <= 20 on the host (tests/native/divcheck.c).
#include <atomic>
#include <cstdlib>
#include <type_traits>
#include "lane_ops.h"
#include "quant_pack.h"
#include "f6_codes.h"
#include "rotate_row.h"

namespace flh {
namespace {

#include "hadk_tables.inc"

__device__ __forceinline__ const uint8_t* hadk_bits(int kd) {
  switch (kd) {
    case 12: return kHad12Bits;
    case 20: return kHad20Bits;
    case 28: return kHad28Bits;
    case 36: return kHad36Bits;
    case 40: return kHad40Bits;
    case 52: return kHad52Bits;
    case 60: return kHad60Bits;
    case 108: return kHad108Bits;
    case 140: return kHad140Bits;
    case 156: return kHad156Bits;
    case 172: return kHad172Bits;
    default: return nullptr;
  }
}

// code in [-8, 7] of an fp16 value y for reciprocal scale r, as a nibble
__device__ __forceinline__ unsigned quant_nibble(_Float16 y, float r) {
  const _Float16 h = (_Float16)((float)y * r);
  float c = __builtin_rintf((float)h);
  c = fminf(fmaxf(c, -8.f), 7.f);
  return (unsigned)(int)c & 0xFu;
}

// ------------------------------------------------------------------------------------
// 1. group kernels, fp16 butterflies.  One lane owns 8 consecutive values (16 bytes), G/8
//    adjacent lanes own a row.  Which chunk of the row a lane owns is a relabelling of its
//    position, chosen so that every cross-lane stride is ONE DPP pattern: chunk bits b1, b2
//    flip with quad xor 1 / 2, b3 with the mirror inside 8 lanes, b4 with the mirror inside 16:
//    position = b1*0001 ^ b2*0010 ^ b3*0111 ^ b4*1111.
// ------------------------------------------------------------------------------------
template <int LPR>
__device__ __forceinline__ int group_chunk(int pos) {
  if constexpr (LPR <= 4) return pos;
  const int b1 = (pos ^ (pos >> 2)) & 1, b2 = ((pos >> 1) ^ (pos >> 2)) & 1;
  if constexpr (LPR == 8) return b1 | (b2 << 1) | (pos & 4);
  const int b3 = ((pos >> 2) ^ (pos >> 3)) & 1;
  return b1 | (b2 << 1) | (b3 << 2) | (pos & 8);
}

// butterfly with the partner lane of pattern CTRL: lower lane v + o, upper lane o - v, both as one
// packed fused multiply-add v * (+-1) + o (the product is exact, so the rounding is that of the sum)
template <int CTRL>
__device__ __forceinline__ void group_cross(h2 (&v)[4], bool upper) {
  const _Float16 sg = upper ? (_Float16)-1.0f : (_Float16)1.0f;
  const h2 sgn = {sg, sg};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const h2 o = __builtin_bit_cast(h2, dpp_i<CTRL>(__builtin_bit_cast(int, v[i])));
    v[i] = __builtin_elementwise_fma(v[i], sgn, o);
  }
}

template <int G>
__device__ __forceinline__ void fwht_group_f16(h2 (&v)[4], int chunk) {
#pragma unroll
  for (int i = 0; i < 4; ++i) v[i] = h2{(_Float16)(v[i].x + v[i].y), (_Float16)(v[i].x - v[i].y)};
#pragma unroll
  for (int i = 0; i < 4; i += 2) {
    const h2 a = v[i], b = v[i + 1];
    v[i] = a + b;
    v[i + 1] = a - b;
  }
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const h2 a = v[i], b = v[i + 2];
    v[i] = a + b;
    v[i + 2] = a - b;
  }
  group_cross<kDppQuadXor1>(v, chunk & 1);
  group_cross<kDppQuadXor2>(v, chunk & 2);
  if constexpr (G >= 64) group_cross<kDppRowHalfMirror>(v, chunk & 4);
  if constexpr (G >= 128) group_cross<kDppRowMirror>(v, chunk & 8);
}

// max |v| over a lane's eight halves, as float: sign bits masked, three packed maxima, one across the pair
// (written out so that no canonicalising copies are added; NaNs are ignored as fmaxf ignores them)
__device__ __forceinline__ float lane_abs_max(const h2 (&v)[4]) {
  unsigned a[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) a[i] = __builtin_bit_cast(unsigned, v[i]) & 0x7FFF7FFFu;
  unsigned m01, m23, m;
  asm("v_pk_max_f16 %0, %1, %2" : "=v"(m01) : "v"(a[0]), "v"(a[1]));
  asm("v_pk_max_f16 %0, %1, %2" : "=v"(m23) : "v"(a[2]), "v"(a[3]));
  asm("v_pk_max_f16 %0, %1, %2" : "=v"(m) : "v"(m01), "v"(m23));
  const h2 p = __builtin_bit_cast(h2, m);
  float lo = (float)p.x, hi = (float)p.y, r;
  asm("v_max_f32 %0, %1, %2" : "=v"(r) : "v"(lo), "v"(hi));
  return r;
}

// max(m, m of the partner lane) in one instruction (the DPP operand feeds the maximum directly; the two wait
// states a DPP read needs after the write of its source are spelled out, the assembler does not add them here)
template <int CTRL>
__device__ __forceinline__ float max_across(float m) {
  float r;
  if constexpr (CTRL == kDppQuadXor1)
    asm volatile("s_nop 1\n\tv_max_f32_dpp %0, %1, %1 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf" : "=v"(r) : "v"(m));
  else if constexpr (CTRL == kDppQuadXor2)
    asm volatile("s_nop 1\n\tv_max_f32_dpp %0, %1, %1 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf" : "=v"(r) : "v"(m));
  else if constexpr (CTRL == kDppRowHalfMirror)
    asm volatile("s_nop 1\n\tv_max_f32_dpp %0, %1, %1 row_half_mirror row_mask:0xf bank_mask:0xf" : "=v"(r) : "v"(m));
  else
    asm volatile("s_nop 1\n\tv_max_f32_dpp %0, %1, %1 row_mirror row_mask:0xf bank_mask:0xf" : "=v"(r) : "v"(m));
  return r;
}

// scale, codes and stores of one row of G values held by LPR = G / 8 adjacent lanes (this lane: chunk `lir`)
//
// F6 (G = 128 only): the codes leave in the operand format of the 6-bit matrix instruction instead -- 6 bits per
// code, the 96-byte block of this group at ((row % groups_per_token) * tokens + row / groups_per_token) * 96
// (K-slab-major, see gemm_f6.hip).  A lane's eight codes are 48 bits; the four lanes of a quad own one 24-byte
// piece of the block (chunks 4 p .. 4 p + 3, in an order that depends on the quad), and three of them store eight
// bytes each after fetching their successor's bits from the lane whose chunk index is one higher (chunk index
// and quad position differ by a constant XOR inside a quad, so that lane is the xor-1 resp. xor-3 partner).
template <int G, bool F6 = false, bool OFF32 = false>
__device__ __forceinline__ void group_finish(const h2 (&v)[4], int lir, bool valid, uint32_t row, uint8_t* __restrict__ q,
                                             __half* __restrict__ scales, float scale_mul, uint32_t tokens = 0,
                                             uint32_t groups_per_token = 1) {
  static_assert(!F6 || G == 128, "one 6-bit block is 128 codes");
  constexpr int LPR = G / 8;
  float m = lane_abs_max(v);
  m = max_across<kDppQuadXor1>(m);
  m = max_across<kDppQuadXor2>(m);
  if constexpr (LPR >= 8) m = max_across<kDppRowHalfMirror>(m);
  if constexpr (LPR >= 16) m = max_across<kDppRowMirror>(m);
  // no division sequences (see scale_of_max): a lane has only eight values to spread them over
  _Float16 s = scale_of_max(m);
  if (s <= (_Float16)1e-6f) s = (_Float16)1.0f;
  const float r = reciprocal_of_scale(s);
  // |y / s| <= 7.004 unless the scale is subnormal: only then (any row of this wave) clamp the quotients
  const bool careful = __builtin_amdgcn_ballot_w64((float)s < 6.2e-5f) != 0;
  const h2 hb = {(_Float16)65504.0f, (_Float16)65504.0f};   // no clipping in the group kernels
  const unsigned y01 = __builtin_bit_cast(unsigned, v[0]), y23 = __builtin_bit_cast(unsigned, v[1]),
                 y45 = __builtin_bit_cast(unsigned, v[2]), y67 = __builtin_bit_cast(unsigned, v[3]);
  const unsigned w = careful ? nibbles8<true>(y01, y23, y45, y67, r, hb) : nibbles8<false>(y01, y23, y45, y67, r, hb);
  if constexpr (F6) {
    const size_t block = (size_t)(row % groups_per_token) * tokens + row / groups_per_token;
    f6_store_chunk(w, lir, q + block * kF6BlockBytes, valid);
  }
  if (valid) {
    using offset_t = std::conditional_t<OFF32, uint32_t, size_t>;
    if constexpr (!F6) *(unsigned*)(q + ((offset_t)row * (LPR * 4) + (offset_t)lir * 4)) = w;
    // the stored scale may carry a constant factor (the reference divides its scales by sqrt(G) in a
    // second kernel after the unnormalised transform): float32 product, then fp16; the codes above use s
    if (lir == 0) *(__half*)((char*)scales + (offset_t)row * 2) = scale_mul == 1.0f ? __builtin_bit_cast(__half, s) : __float2half(round_here((float)s * scale_mul));
  }
}

// OFF32: every byte offset of the launch fits 32 bits, so that the addresses are a scalar base plus a 32-bit lane
// offset (the instruction count of these kernels is what bounds them: eight values per lane, ~170 instructions).
template <int G, bool HAD, bool QUANT, bool F6 = false, bool OFF32 = false>
__global__ __launch_bounds__(256) void group_kernel(const __half* __restrict__ x, uint8_t* __restrict__ q,
                                                    __half* __restrict__ scales, __half* __restrict__ y_inplace,
                                                    uint32_t R, float scale_mul, uint32_t tokens = 0,
                                                    uint32_t groups_per_token = 1) {
  constexpr int LPR = G / 8;
  using offset_t = std::conditional_t<OFF32, uint32_t, size_t>;
  const uint32_t gl = blockIdx.x * 256u + threadIdx.x;
  const uint32_t row = gl / LPR;
  const int lir = group_chunk<LPR>(gl % LPR);         // the chunk of the row this lane owns
  const bool valid = row < R;
  const uint32_t rr = valid ? row : R - 1;
  const __half* src = QUANT ? x : y_inplace;
  const h8 raw = *(const h8*)((const char*)src + ((offset_t)rr * (G * 2) + (offset_t)lir * 16));
  h2 v[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) v[i] = h2{raw[2 * i], raw[2 * i + 1]};
  if constexpr (HAD) fwht_group_f16<G>(v, lir);
  if constexpr (!QUANT) {
    h8 o;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      o[2 * i] = v[i].x;
      o[2 * i + 1] = v[i].y;
    }
    if (valid) *(h8*)((char*)y_inplace + ((offset_t)row * (G * 2) + (offset_t)lir * 16)) = o;
  } else {
    group_finish<G, F6, OFF32>(v, lir, valid, row, q, scales, scale_mul, tokens, groups_per_token);
  }
}

// SwiGLU in front of the group kernel: x = fp16( float(fp16(silu(gate))) * float(up) ) -- the two roundings
// of torch's fp16 silu and fp16 multiply (flh/quantized_model/modeling_llama.py:522-526 feeds exactly this
// product to the quantiser of down_proj) -- then transform + quantise as group_kernel<G, HAD, true>.
template <int G, bool HAD>
__global__ __launch_bounds__(256) void silu_mul_group_kernel(const __half* __restrict__ gate,
                                                             const __half* __restrict__ up, uint8_t* __restrict__ q,
                                                             __half* __restrict__ scales, uint32_t R, float scale_mul) {
  constexpr int LPR = G / 8;
  const uint32_t gl = blockIdx.x * 256u + threadIdx.x;
  const uint32_t row = gl / LPR;
  const int lir = group_chunk<LPR>(gl % LPR);
  const bool valid = row < R;
  const uint32_t rr = valid ? row : R - 1;
  const h8 g8 = *(const h8*)(gate + (size_t)rr * G + lir * 8);
  const h8 u8 = *(const h8*)(up + (size_t)rr * G + lir * 8);
  h2 v[4];
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const _Float16 prod = silu_mul_f16(g8[i], u8[i]);
    if (i & 1) v[i >> 1].y = prod;
    else v[i >> 1].x = prod;
  }
  if constexpr (HAD) fwht_group_f16<G>(v, lir);
  group_finish<G>(v, lir, valid, row, q, scales, scale_mul);
}

// the SwiGLU product alone, eight values per thread
__global__ __launch_bounds__(256) void silu_mul_kernel(const __half* __restrict__ gate, const __half* __restrict__ up,
                                                       __half* __restrict__ out, uint64_t chunks) {
  const uint64_t i = (uint64_t)blockIdx.x * 256u + threadIdx.x;
  if (i >= chunks) return;
  const h8 g = *(const h8*)(gate + i * 8), u = *(const h8*)(up + i * 8);
  h8 o;
#pragma unroll
  for (int e = 0; e < 8; ++e) o[e] = silu_mul_f16(g[e], u[e]);
  *(h8*)(out + i * 8) = o;
}

// RMSNorm in front of the group kernel, one workgroup per token row of K = 8 * chunks values (K <= 16384):
// y = fp16( float(x) * rsqrt(sum(x^2) / K + eps) [* float(weight)] ) with the statistics in float32
// (flh/nn/normalization.py:12-20), then transform + quantise per group of G as group_kernel<G, HAD, true>.
template <int G, bool HAD>
__global__ __launch_bounds__(256) void rmsnorm_group_kernel(const __half* __restrict__ x,
                                                            const __half* __restrict__ weight, uint8_t* __restrict__ q,
                                                            __half* __restrict__ scales, uint32_t K, float eps,
                                                            float scale_mul) {
  constexpr int LPR = G / 8, MAXC = 8;
  __shared__ float part[4];
  const int tid = threadIdx.x;
  const uint32_t token = blockIdx.x, chunks = K / 8;
  const int lir = group_chunk<LPR>(tid % LPR);
  const uint32_t c0 = (tid / LPR) * LPR + lir;        // chunk of pass 0; pass i adds 256 i
  const __half* xr = x + (size_t)token * K;
  h8 raw[MAXC];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < MAXC; ++i) {
    const uint32_t c = c0 + 256u * i;
    if (c < chunks) {
      raw[i] = *(const h8*)(xr + (size_t)c * 8);
#pragma unroll
      for (int e = 0; e < 8; ++e) ss = __builtin_fmaf((float)raw[i][e], (float)raw[i][e], ss);
    }
  }
  // workgroup sum: across the wave with DPP / swaps, across the four waves through LDS
  ss += dpp_f<kDppQuadXor1>(ss);
  ss += dpp_f<kDppQuadXor2>(ss);
  ss += dpp_f<kDppRowHalfMirror>(ss);
  ss += dpp_f<kDppRowMirror>(ss);
  ss += lane_xor_f<16>(ss);
  ss += lane_xor_f<32>(ss);
  if ((tid & 63) == 0) part[tid >> 6] = ss;
  __syncthreads();
  const float total = (part[0] + part[1]) + (part[2] + part[3]);
  const float inv = 1.0f / __builtin_sqrtf(total / (float)K + eps);
#pragma unroll
  for (int i = 0; i < MAXC; ++i) {
    const uint32_t c = c0 + 256u * i;
    if (c < chunks) {                                 // whole groups of LPR lanes take this branch together
      h8 w8;
      if (weight) w8 = *(const h8*)(weight + (size_t)c * 8);
      h2 v[4];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        float t = round_here((float)raw[i][e] * inv);
        if (weight) t = round_here(t * (float)w8[e]);
        if (e & 1) v[e >> 1].y = (_Float16)t;
        else v[e >> 1].x = (_Float16)t;
      }
      if constexpr (HAD) fwht_group_f16<G>(v, lir);
      const uint32_t row = token * (K / G) + c / LPR;
      group_finish<G>(v, lir, true, row, q, scales, scale_mul);
    }
  }
}

// RMSNorm on its own (a model's final norm, in front of an fp16 head), optionally behind the residual addition: one
// workgroup per row of K = 8 * chunks values (K <= 16384), the statistics and roundings of rmsnorm_group_kernel;
// with `add` the row is fp16(x + add), one rounding per value, stored to sum_out as well when that is given.
__global__ __launch_bounds__(256) void add_rmsnorm_kernel(const __half* __restrict__ x, const __half* __restrict__ add,
                                                          const __half* __restrict__ weight, __half* __restrict__ out,
                                                          __half* __restrict__ sum_out, uint32_t K, float eps) {
  constexpr int MAXC = 8;
  __shared__ float part[4];
  const int tid = threadIdx.x;
  const uint32_t chunks = K / 8;
  const size_t row = (size_t)blockIdx.x * K;
  h8 raw[MAXC];
  float ss = 0.f;
#pragma unroll
  for (int i = 0; i < MAXC; ++i) {
    const uint32_t c = tid + 256u * i;
    if (c < chunks) {
      raw[i] = *(const h8*)(x + row + (size_t)c * 8);
      if (add) {
        raw[i] = __builtin_bit_cast(h8, add_h8(__builtin_bit_cast(v4i, raw[i]), *(const v4i*)(add + row + (size_t)c * 8)));
        if (sum_out) *(h8*)(sum_out + row + (size_t)c * 8) = raw[i];
      }
#pragma unroll
      for (int e = 0; e < 8; ++e) ss = __builtin_fmaf((float)raw[i][e], (float)raw[i][e], ss);
    }
  }
  ss += dpp_f<kDppQuadXor1>(ss);
  ss += dpp_f<kDppQuadXor2>(ss);
  ss += dpp_f<kDppRowHalfMirror>(ss);
  ss += dpp_f<kDppRowMirror>(ss);
  ss += lane_xor_f<16>(ss);
  ss += lane_xor_f<32>(ss);
  if ((tid & 63) == 0) part[tid >> 6] = ss;
  __syncthreads();
  const float total = (part[0] + part[1]) + (part[2] + part[3]);
  const float inv = 1.0f / __builtin_sqrtf(total / (float)K + eps);
#pragma unroll
  for (int i = 0; i < MAXC; ++i) {
    const uint32_t c = tid + 256u * i;
    if (c < chunks) {
      h8 w8, y;
      if (weight) w8 = *(const h8*)(weight + (size_t)c * 8);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        float t = round_here((float)raw[i][e] * inv);
        if (weight) t = round_here(t * (float)w8[e]);
        y[e] = (_Float16)t;
      }
      *(h8*)(out + row + (size_t)c * 8) = y;
    }
  }
}

// ------------------------------------------------------------------------------------
// 2. wave-per-row kernel, float32 butterflies, K = 512 * J: four rows per workgroup, rotate_quant_row (rotate_row.h)
// ------------------------------------------------------------------------------------
template <int J, bool HAD, bool EXACT_NORM, bool RMS = false>
__global__ __launch_bounds__(256) void rotate_quant_wave_kernel(const __half* __restrict__ x, uint8_t* __restrict__ q,
                                                                __half* __restrict__ scales,
                                                                __half* __restrict__ y_out, uint32_t M, float norm,
                                                                float clip, const __half* __restrict__ rms_weight = nullptr,
                                                                float rms_eps = 0.f, const __half* add = nullptr,
                                                                __half* sum_out = nullptr, uint32_t f6 = 0) {
  constexpr int K = 512 * J;
  const uint32_t row = blockIdx.x * 4u + (threadIdx.x >> 6);
  if (row >= M) return;  // wave-uniform
  // f6: q is the encoded matrix of M rows in the 6-bit operand format instead of [M, K / 2] nibbles
  rotate_quant_row<J, HAD, EXACT_NORM, RMS>(x + (size_t)row * K, f6 ? q : q + (size_t)row * (K / 2), scales + row,
                                            y_out ? y_out + (size_t)row * K : nullptr, norm, clip, rms_weight, rms_eps,
                                            add ? add + (size_t)row * K : nullptr,
                                            add ? sum_out + (size_t)row * K : nullptr, f6 ? M : 0u, row);
}

constexpr int kGenericThreads = 1024;      // one workgroup per compute unit (LDS): two waves per SIMD hide latencies

// 2^LOGR-point butterflies (strides 2^shift .. 2^(shift + LOGR - 1), ascending) over a row of K floats in LDS
template <int LOGR>
__device__ __forceinline__ void fwht_pass(float* a, uint32_t K, int shift, int tid) {
  constexpr int R = 1 << LOGR;
  for (uint32_t p = tid; p < K / R; p += kGenericThreads) {
    const uint32_t base = ((p >> shift) << (shift + LOGR)) | (p & ((1u << shift) - 1));
    float v[R];
#pragma unroll
    for (int r = 0; r < R; ++r) v[r] = a[base + ((uint32_t)r << shift)];
#pragma unroll
    for (int h = 1; h < R; h <<= 1)
#pragma unroll
      for (int r = 0; r < R; ++r)
        if (!(r & h)) {
          const float u = v[r], w = v[r + h];
          v[r] = u + w;
          v[r + h] = u - w;
        }
#pragma unroll
    for (int r = 0; r < R; ++r) a[base + ((uint32_t)r << shift)] = v[r];
  }
  __syncthreads();
}

// ------------------------------------------------------------------------------------
// 3. generic kernel: one workgroup per row, data in LDS as float32.
//    K = Kd * P: float32 butterflies over each contiguous block of P (ascending strides),
//    then (Kd > 1) out[j][t] = sum_j' H[j][j'] * a[j'][t] with the +/-1 literal matrix
//    (matmul_hadU, flh/functional/hadamard.py:92-113), then / norm.
//    had_width == 0: no rotation.  Scales per contiguous scale_group (0 = whole row).
// ------------------------------------------------------------------------------------
__global__ __launch_bounds__(kGenericThreads) void rotate_quant_generic_kernel(const __half* __restrict__ x, uint8_t* __restrict__ q,
                                                                   __half* __restrict__ scales,
                                                                   __half* __restrict__ y_out, uint32_t K, int P,
                                                                   int Kd, float norm, int scale_group, float clip) {
  extern __shared__ __align__(16) float smem[];
  float* a = smem;
  float* b = smem + K;                       // used only when Kd > 1
  __shared__ float red[kGenericThreads / 64];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const size_t row = blockIdx.x;
  const __half* xr = x + row * K;
  if (K % 8 == 0 && reinterpret_cast<uintptr_t>(x) % 16 == 0) {
    // 16-byte loads, four in flight per lane: a workgroup owns a whole compute unit's LDS here, so nothing
    // else hides the latency of this read
    const uint4* xv = reinterpret_cast<const uint4*>(xr);
    const uint32_t n = K / 8;
    for (uint32_t i0 = tid; i0 < n; i0 += 4 * kGenericThreads) {
      uint4 w[4];
#pragma unroll
      for (int u = 0; u < 4; ++u)
        if (i0 + kGenericThreads * u < n) w[u] = xv[i0 + kGenericThreads * u];
#pragma unroll
      for (int u = 0; u < 4; ++u)
        if (i0 + kGenericThreads * u < n) {
          const __half2* h = reinterpret_cast<const __half2*>(&w[u]);
          const float2 f0 = __half22float2(h[0]), f1 = __half22float2(h[1]), f2 = __half22float2(h[2]),
                       f3 = __half22float2(h[3]);
          float4* dst = reinterpret_cast<float4*>(a + 8 * (size_t)(i0 + kGenericThreads * u));
          dst[0] = make_float4(f0.x, f0.y, f1.x, f1.y);
          dst[1] = make_float4(f2.x, f2.y, f3.x, f3.y);
        }
    }
  } else {
    for (uint32_t i = tid; i < K / 2; i += kGenericThreads) {       // K is even (two codes per output byte)
      const float2 v = __half22float2(reinterpret_cast<const __half2*>(xr)[i]);
      a[2 * i] = v.x;
      a[2 * i + 1] = v.y;
    }
  }
  __syncthreads();
  if (P > 1) {
    // three butterfly stages per pass over LDS (then what is left), each thread holding the 2^LOGR values that
    // those stages couple; every value still goes through the same additions in ascending stride order
    int shift = 0, stages = 0;
    while ((1 << stages) < P) ++stages;
    for (; shift + 3 <= stages; shift += 3) fwht_pass<3>(a, K, shift, tid);
    if (stages - shift == 2) fwht_pass<2>(a, K, shift, tid);
    if (stages - shift == 1) fwht_pass<1>(a, K, shift, tid);
    if (Kd > 1) {
      const uint8_t* bits = hadk_bits(Kd);
      if (P >= 16) {
        // Lanes hold 64 output blocks j, registers 16 positions t: a[jj * P + t] is then one address for the
        // whole wave (an LDS broadcast) and the sign of (j, jj) one value per lane, so that an accumulation is
        // a single FMA, acc = fma(+-1, a, acc) -- the same sum, in the same order, as the loop below.
        uint8_t* sign_bits = reinterpret_cast<uint8_t*>(smem + 2 * (size_t)K);
        for (int i = tid; i < (Kd * Kd + 7) >> 3; i += kGenericThreads) sign_bits[i] = bits[i];
        __syncthreads();
        const int jblocks = (Kd + 63) >> 6, units = jblocks * (P >> 4);
        for (int u = wave; u < units; u += kGenericThreads / 64) {
          const int j = (u % jblocks) * 64 + lane, t0 = (u / jblocks) << 4;
          // the signs of row j are Kd consecutive bits (most significant first) from bit j * Kd of the table:
          // a 16-bit window over two bytes covers the 8 columns of a chunk whatever the row's bit offset
          const uint32_t jbit = (uint32_t)(j < Kd ? j : Kd - 1) * Kd;
          const uint8_t* sb = sign_bits + (jbit >> 3);
          const uint32_t align = 16 + (jbit & 7);
          float acc[16] = {};
          auto four = [&](int jj, uint32_t minus, int e0) {     // columns jj .. jj + 3 are bits 31 - e0 .. of ~window
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const float sgn = __uint_as_float(((minus << (e0 + e)) & 0x80000000u) | 0x3f800000u);
              const float4* av = reinterpret_cast<const float4*>(a + (jj + e) * P + t0);
#pragma unroll
              for (int i = 0; i < 4; ++i) {
                const float4 v = av[i];
                acc[4 * i + 0] = fmaf(sgn, v.x, acc[4 * i + 0]);
                acc[4 * i + 1] = fmaf(sgn, v.y, acc[4 * i + 1]);
                acc[4 * i + 2] = fmaf(sgn, v.z, acc[4 * i + 2]);
                acc[4 * i + 3] = fmaf(sgn, v.w, acc[4 * i + 3]);
              }
            }
          };
          uint32_t cur = sb[0];
          for (int jj = 0; jj < Kd; jj += 8) {                  // every literal size is a multiple of 4
            const uint32_t next = sb[(jj >> 3) + 1];
            const uint32_t minus = ~(((cur << 8) | next) << align);
            cur = next;
            four(jj, minus, 0);
            if (jj + 4 < Kd) four(jj + 4, minus, 4);
          }
          if (j < Kd) {
            float4* bv = reinterpret_cast<float4*>(b + j * P + t0);
#pragma unroll
            for (int i = 0; i < 4; ++i) bv[i] = make_float4(acc[4 * i], acc[4 * i + 1], acc[4 * i + 2], acc[4 * i + 3]);
          }
        }
      } else {
        for (uint32_t o = tid; o < K; o += kGenericThreads) {
          const int j = o / P, t = o % P;
          float acc = 0.f;
          for (int jj = 0; jj < Kd; ++jj) {
            const int bit = j * Kd + jj;
            const bool plus = (bits[bit >> 3] >> (7 - (bit & 7))) & 1;
            const float val = a[jj * P + t];
            acc += plus ? val : -val;
          }
          b[o] = acc;
        }
      }
      __syncthreads();
      a = b;
    }
  }
  // normalise (norm = 1 without rotation), round to fp16 (kept as float in LDS), optional copy out, row maximum
  float m = 0.f;
  for (uint32_t i = tid; i < K / 2; i += kGenericThreads) {
    const __half2 h = __floats2half2_rn(a[2 * i] / norm, a[2 * i + 1] / norm);
    const float2 f = __half22float2(h);
    a[2 * i] = f.x;
    a[2 * i + 1] = f.y;
    m = fmaxf(m, fmaxf(fabsf(f.x), fabsf(f.y)));
    if (y_out) reinterpret_cast<__half2*>(y_out + row * K)[i] = h;
  }
  m = wave_max(m);
  if (lane == 0) red[wave] = m;
  __syncthreads();
  m = red[0];
#pragma unroll
  for (int w = 1; w < kGenericThreads / 64; ++w) m = fmaxf(m, red[w]);
  if (clip < 1.0f) {
    const float bound = __half2float(__float2half(round_here(m * clip)));
    for (uint32_t i = tid; i < K; i += kGenericThreads) a[i] = fminf(fmaxf(a[i], -bound), bound);
    m = fminf(m, bound);
    __syncthreads();
  }
  const uint32_t G = scale_group > 0 ? (uint32_t)scale_group : K;
  const uint32_t ng = K / G;
  if (ng == 1) {                               // one scale for the row: the whole workgroup quantises it
    _Float16 s = (_Float16)(m / 7.0f);
    if (s == (_Float16)0.0f) s = (_Float16)1.0f;
    const float r = 1.0f / (float)s;
    uint8_t* qg = q + row * (K / 2);
    for (uint32_t i = tid; i < K / 2; i += kGenericThreads)
      qg[i] = (uint8_t)(quant_nibble((_Float16)a[2 * i], r) | (quant_nibble((_Float16)a[2 * i + 1], r) << 4));
    if (tid == 0) scales[row] = __builtin_bit_cast(__half, s);
    return;
  }
  // one wave per scale group at a time
  for (uint32_t g = wave; g < ng; g += kGenericThreads / 64) {
    const float* ag = a + g * G;
    float mg = 0.f;
    for (uint32_t i = lane; i < G; i += 64) mg = fmaxf(mg, fabsf(ag[i]));
    mg = wave_max(mg);
    _Float16 s = (_Float16)(mg / 7.0f);
    if (s == (_Float16)0.0f) s = (_Float16)1.0f;
    const float r = 1.0f / (float)s;
    uint8_t* qg = q + row * (K / 2) + g * (G / 2);
    for (uint32_t i = lane; i < G / 2; i += 64)
      qg[i] = (uint8_t)(quant_nibble((_Float16)ag[2 * i], r) | (quant_nibble((_Float16)ag[2 * i + 1], r) << 4));
    if (lane == 0) scales[row * ng + g] = __builtin_bit_cast(__half, s);
  }
}

bool is_pow2(uint32_t n) { return n && !(n & (n - 1)); }

// K = Kd * P with the reference's divisor order (flh/functional/hadamard.py:41-84)
bool factor_hadamard(uint32_t K, int* Kd, int* P) {
  static const int order[] = {172, 156, 140, 108, 60, 52, 36, 28, 40, 20, 12};
  for (int k : order)
    if (K % k == 0) {
      if (!is_pow2(K / k)) return false;
      *Kd = k;
      *P = (int)(K / k);
      return true;
    }
  if (!is_pow2(K)) return false;
  *Kd = 1;
  *P = (int)K;
  return true;
}

template <int J>
int launch_wave(const __half* x, uint8_t* q, __half* s, __half* y, uint32_t M, bool had, float clip,
                hipStream_t stream, uint32_t f6 = 0) {
  constexpr int K = 512 * J;
  int lg = 0;
  while ((1 << lg) < K) ++lg;
  const bool even = (lg % 2) == 0;
  const dim3 grid((M + 3) / 4), block(256);
  if (!had)
    hipLaunchKernelGGL((rotate_quant_wave_kernel<J, false, true>), grid, block, 0, stream, x, q, s, y, M, 1.0f, clip,
                       (const __half*)nullptr, 0.f, (const __half*)nullptr, (__half*)nullptr, f6);
  else if (even)
    hipLaunchKernelGGL((rotate_quant_wave_kernel<J, true, true>), grid, block, 0, stream, x, q, s, y, M,
                       1.0f / (float)(1 << (lg / 2)), clip, (const __half*)nullptr, 0.f, (const __half*)nullptr,
                       (__half*)nullptr, f6);
  else
    hipLaunchKernelGGL((rotate_quant_wave_kernel<J, true, false>), grid, block, 0, stream, x, q, s, y, M,
                       sqrtf((float)K), clip, (const __half*)nullptr, 0.f, (const __half*)nullptr, (__half*)nullptr, f6);
  return check_launch("rotate_quant_wave");
}

// A few rows of 4096: one workgroup of eight waves per row (rotate_quant_row_8waves: the same additions in the same
// order as the wave-per-row kernel, hence the same bytes), so that a decode-sized batch waits for an eighth of a
// row's arithmetic instead of a whole row's on a single wave.
__global__ __launch_bounds__(512) void rotate_quant_row8_kernel(const __half* __restrict__ x, uint8_t* __restrict__ q,
                                                                __half* __restrict__ scales, float norm) {
  __shared__ float stage[8 * 8 * 64];
  __shared__ float wave_max8[8];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const size_t row = blockIdx.x;
  rotate_quant_row_8waves(x + row * 4096, stage, wave_max8, q + row * 2048, scales + row, norm, wave);
}
// ... and with RMSNorm in front (flh_rmsnorm_rotate_quant_i4), the same bytes as rotate_quant_wave_kernel<8, ..., RMS>
__global__ __launch_bounds__(512) void rmsnorm_rotate_quant_row8_kernel(const __half* __restrict__ x,
                                                                        const __half* __restrict__ weight, float eps,
                                                                        uint8_t* __restrict__ q,
                                                                        __half* __restrict__ scales, float norm) {
  __shared__ float stage[8 * 8 * 64];
  __shared__ float wave_max8[8];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const size_t row = blockIdx.x;
  rotate_quant_row_8waves<true>(x + row * 4096, stage, wave_max8, q + row * 2048, scales + row, norm, wave, weight, eps);
}
// ... and with the residual addition in front of that (flh_add_rmsnorm_rotate_quant_i4)
__global__ __launch_bounds__(512) void add_rmsnorm_rotate_quant_row8_kernel(const __half* __restrict__ x,
                                                                            const __half* __restrict__ add,
                                                                            __half* __restrict__ sum_out,
                                                                            const __half* __restrict__ weight, float eps,
                                                                            uint8_t* __restrict__ q,
                                                                            __half* __restrict__ scales, float norm) {
  __shared__ float stage[8 * 8 * 64];
  __shared__ float wave_max8[8];
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const size_t row = blockIdx.x;
  rotate_quant_row_8waves<true, true>(x + row * 4096, stage, wave_max8, q + row * 2048, scales + row, norm, wave, weight,
                                      eps, add + row * 4096, sum_out + row * 4096);
}
// measured per launch inside a replayed graph: 2.7 against 4.4 us for one row, 3.2 against 4.9 us for 256 rows,
// 3.9 against 5.0 us for 512; from 1024 rows on the wave-per-row kernel is the faster one
constexpr uint32_t kRow8MaxRows = 512;

template <int J>
int launch_wave_rms(const __half* x, const __half* w, float eps, uint8_t* q, __half* s, __half* y, uint32_t M, bool had,
                    float clip, hipStream_t stream, const __half* add = nullptr, __half* sum_out = nullptr,
                    uint32_t f6 = 0) {
  constexpr int K = 512 * J;
  int lg = 0;
  while ((1 << lg) < K) ++lg;
  const dim3 grid((M + 3) / 4), block(256);
  if (!had)
    hipLaunchKernelGGL((rotate_quant_wave_kernel<J, false, true, true>), grid, block, 0, stream, x, q, s, y, M, 1.0f,
                       clip, w, eps, add, sum_out, f6);
  else if (lg % 2 == 0)
    hipLaunchKernelGGL((rotate_quant_wave_kernel<J, true, true, true>), grid, block, 0, stream, x, q, s, y, M,
                       1.0f / (float)(1 << (lg / 2)), clip, w, eps, add, sum_out, f6);
  else
    hipLaunchKernelGGL((rotate_quant_wave_kernel<J, true, false, true>), grid, block, 0, stream, x, q, s, y, M,
                       sqrtf((float)K), clip, w, eps, add, sum_out, f6);
  return check_launch("rmsnorm_rotate_quant_wave");
}

template <int G>
int launch_group(const __half* x, uint8_t* q, __half* s, __half* y, uint32_t R, bool had, bool quant,
                 float scale_mul, hipStream_t stream) {
  constexpr int LPR = G / 8;
  const dim3 grid((unsigned)(((uint64_t)R * LPR + 255) / 256)), block(256);
  auto go = [&](auto off32_tag) {
    constexpr bool OFF32 = decltype(off32_tag)::value;
    if (!quant)
      hipLaunchKernelGGL((group_kernel<G, true, false, false, OFF32>), grid, block, 0, stream, x, q, s, y, R, scale_mul, 0u, 1u);
    else if (had)
      hipLaunchKernelGGL((group_kernel<G, true, true, false, OFF32>), grid, block, 0, stream, x, q, s, y, R, scale_mul, 0u, 1u);
    else
      hipLaunchKernelGGL((group_kernel<G, false, true, false, OFF32>), grid, block, 0, stream, x, q, s, y, R, scale_mul, 0u, 1u);
  };
  if ((uint64_t)R * G * 2 <= 0xFFFFFFFFull) go(std::true_type{});   // the largest array of the launch: the fp16 rows
  else go(std::false_type{});
  return check_launch("group_kernel");
}

int group_dispatch(const __half* x, uint8_t* q, __half* s, __half* y, uint32_t R, int group, bool had, bool quant,
                   float scale_mul, hipStream_t stream) {
  if (R == 0) return FLH_OK;
  switch (group) {
    case 32: return launch_group<32>(x, q, s, y, R, had, quant, scale_mul, stream);
    case 64: return launch_group<64>(x, q, s, y, R, had, quant, scale_mul, stream);
    case 128: return launch_group<128>(x, q, s, y, R, had, quant, scale_mul, stream);
    default: return fail(FLH_EINVAL, "group size must be 32, 64 or 128 (got %d)", group);
  }
}

template <int G>
int launch_silu_mul(const __half* gate, const __half* up, uint8_t* q, __half* s, uint32_t R, bool had, float scale_mul,
                    hipStream_t stream) {
  const dim3 grid((unsigned)(((uint64_t)R * (G / 8) + 255) / 256)), block(256);
  if (had)
    hipLaunchKernelGGL((silu_mul_group_kernel<G, true>), grid, block, 0, stream, gate, up, q, s, R, scale_mul);
  else
    hipLaunchKernelGGL((silu_mul_group_kernel<G, false>), grid, block, 0, stream, gate, up, q, s, R, scale_mul);
  return check_launch("silu_mul_group_kernel");
}

template <int G>
int launch_rmsnorm(const __half* x, const __half* w, uint8_t* q, __half* s, uint32_t M, uint32_t K, float eps, bool had,
                   float scale_mul, hipStream_t stream) {
  if (had)
    hipLaunchKernelGGL((rmsnorm_group_kernel<G, true>), dim3(M), dim3(256), 0, stream, x, w, q, s, K, eps, scale_mul);
  else
    hipLaunchKernelGGL((rmsnorm_group_kernel<G, false>), dim3(M), dim3(256), 0, stream, x, w, q, s, K, eps, scale_mul);
  return check_launch("rmsnorm_group_kernel");
}

}  // namespace

// matrix-core variant (fwht_mfma.hip)
int launch_rotate_quant_mfma(const __half* x, uint8_t* q, __half* scales, uint32_t M, uint32_t K, float clip,
                             hipStream_t stream);
bool rotate_quant_mfma_supports(uint32_t K);
int launch_silu_mul_rotate_quant_mfma(const __half* gate, const __half* up, uint8_t* q, __half* scales, uint32_t M,
                                      uint32_t K, hipStream_t stream);
int launch_rotate_quant_mfma4096(const __half* x, const __half* add, __half* sum_out, bool rms, const __half* weight,
                                 float eps, uint8_t* q, __half* scales, uint32_t M, float clip, bool f6,
                                 hipStream_t stream);
int launch_rotate_quant_mfma_f6(const __half* x, uint8_t* encoded, __half* scales, uint32_t M, uint32_t K, float clip,
                                hipStream_t stream);

}  // namespace flh

using namespace flh;

extern "C" int flh_group_quant_i4(const flh_half* x, uint8_t* q_packed, flh_half* scales, uint32_t R, int group,
                                  int hadamard, float scale_mul, void* stream) {
  if (!x || !q_packed || !scales) return fail(FLH_EINVAL, "group_quant: null pointer");
  if (misaligned16(x, q_packed)) return fail(FLH_EINVAL, "group_quant: x and q_packed must be 16-byte aligned");
  if (!(scale_mul > 0.f)) return fail(FLH_EINVAL, "group_quant: scale_mul must be positive");
  return group_dispatch((const __half*)x, q_packed, (__half*)scales, nullptr, R, group, hadamard != 0, true, scale_mul,
                        (hipStream_t)stream);
}

extern "C" int flh_silu_mul_group_quant_i4(const flh_half* gate, const flh_half* up, uint8_t* q_packed, flh_half* scales,
                                           uint32_t R, int group, int hadamard, float scale_mul, void* stream) {
  if (!gate || !up || !q_packed || !scales) return fail(FLH_EINVAL, "silu_mul_group_quant: null pointer");
  if (misaligned16(gate, up, q_packed)) return fail(FLH_EINVAL, "silu_mul_group_quant: gate, up and q_packed must be 16-byte aligned");
  if (!(scale_mul > 0.f)) return fail(FLH_EINVAL, "silu_mul_group_quant: scale_mul must be positive");
  if (R == 0) return FLH_OK;
  const __half *g = (const __half*)gate, *u = (const __half*)up;
  switch (group) {
    case 32: return launch_silu_mul<32>(g, u, q_packed, (__half*)scales, R, hadamard != 0, scale_mul, (hipStream_t)stream);
    case 64: return launch_silu_mul<64>(g, u, q_packed, (__half*)scales, R, hadamard != 0, scale_mul, (hipStream_t)stream);
    case 128: return launch_silu_mul<128>(g, u, q_packed, (__half*)scales, R, hadamard != 0, scale_mul, (hipStream_t)stream);
    default: return fail(FLH_EINVAL, "group size must be 32, 64 or 128 (got %d)", group);
  }
}

extern "C" int flh_rmsnorm_group_quant_i4(const flh_half* x, const flh_half* weight, uint8_t* q_packed, flh_half* scales,
                                          uint32_t M, uint32_t K, float eps, int group, int hadamard, float scale_mul,
                                          void* stream) {
  if (!x || !q_packed || !scales) return fail(FLH_EINVAL, "rmsnorm_group_quant: null pointer");
  if (misaligned16(x, q_packed)) return fail(FLH_EINVAL, "rmsnorm_group_quant: x and q_packed must be 16-byte aligned");
  if (!(scale_mul > 0.f)) return fail(FLH_EINVAL, "rmsnorm_group_quant: scale_mul must be positive");
  if (!(eps >= 0.f)) return fail(FLH_EINVAL, "rmsnorm_group_quant: eps must not be negative");
  if (group != 32 && group != 64 && group != 128)
    return fail(FLH_EINVAL, "group size must be 32, 64 or 128 (got %d)", group);
  if (K == 0 || K % (uint32_t)group || K > 16384u)
    return fail(FLH_EINVAL, "rmsnorm_group_quant: K (%u) must be a multiple of the group size, at most 16384", K);
  if (M == 0) return FLH_OK;
  const __half *xh = (const __half*)x, *wh = (const __half*)weight;
  switch (group) {
    case 32: return launch_rmsnorm<32>(xh, wh, q_packed, (__half*)scales, M, K, eps, hadamard != 0, scale_mul, (hipStream_t)stream);
    case 64: return launch_rmsnorm<64>(xh, wh, q_packed, (__half*)scales, M, K, eps, hadamard != 0, scale_mul, (hipStream_t)stream);
    default: return launch_rmsnorm<128>(xh, wh, q_packed, (__half*)scales, M, K, eps, hadamard != 0, scale_mul, (hipStream_t)stream);
  }
}

extern "C" int flh_rmsnorm_rotate_quant_i4(const flh_half* x, const flh_half* weight, float eps, uint8_t* q_packed,
                                           flh_half* scales, flh_half* y_out, uint32_t M, uint32_t K, int hadamard,
                                           float clip_ratio, void* stream) {
  if (!x || !q_packed || !scales) return fail(FLH_EINVAL, "rmsnorm_rotate_quant: null pointer");
  if (misaligned16(x, q_packed)) return fail(FLH_EINVAL, "rmsnorm_rotate_quant: x and q_packed must be 16-byte aligned");
  if (!(clip_ratio > 0.f)) return fail(FLH_EINVAL, "rmsnorm_rotate_quant: clip_ratio must be positive");
  if (!(eps >= 0.f)) return fail(FLH_EINVAL, "rmsnorm_rotate_quant: eps must not be negative");
  if (hadamard != FLH_HAD_NONE && hadamard != FLH_HAD_F32 && hadamard != FLH_HAD_MFMA)
    return fail(FLH_EINVAL, "rmsnorm_rotate_quant: unknown hadamard mode %d", hadamard);
  if (K % 512 || !is_pow2(K / 512) || K > 8192)
    return fail(FLH_EINVAL, "rmsnorm_rotate_quant: K (%u) must be 512, 1024, 2048, 4096 or 8192", K);
  if (M == 0) return FLH_OK;
  const __half *xh = (const __half*)x, *wh = (const __half*)weight;
  __half *sh = (__half*)scales, *yh = (__half*)y_out;
  if (hadamard == FLH_HAD_MFMA) {                      // matrix cores: K = 4096 without y_out, else the float32 butterflies
    if (K == 4096 && !yh && (!wh || !misaligned16(wh)))
      return launch_rotate_quant_mfma4096(xh, nullptr, nullptr, true, wh, eps, q_packed, sh, M, clip_ratio, false,
                                          (hipStream_t)stream);
    hadamard = FLH_HAD_F32;
  }
  const bool had = hadamard != FLH_HAD_NONE;
  hipStream_t st = (hipStream_t)stream;
  if (had && K == 4096 && !yh && clip_ratio >= 1.0f && M <= kRow8MaxRows && (!wh || !misaligned16(wh))) {
    hipLaunchKernelGGL(rmsnorm_rotate_quant_row8_kernel, dim3(M), dim3(512), 0, st, xh, wh, eps, q_packed, sh, 1.0f / 64.0f);
    return check_launch("rmsnorm_rotate_quant_row8");
  }
  switch (K / 512) {
    case 1: return launch_wave_rms<1>(xh, wh, eps, q_packed, sh, yh, M, had, clip_ratio, st);
    case 2: return launch_wave_rms<2>(xh, wh, eps, q_packed, sh, yh, M, had, clip_ratio, st);
    case 4: return launch_wave_rms<4>(xh, wh, eps, q_packed, sh, yh, M, had, clip_ratio, st);
    case 8: return launch_wave_rms<8>(xh, wh, eps, q_packed, sh, yh, M, had, clip_ratio, st);
    default: return launch_wave_rms<16>(xh, wh, eps, q_packed, sh, yh, M, had, clip_ratio, st);
  }
}

extern "C" int flh_add_rmsnorm_rotate_quant_i4(const flh_half* x, const flh_half* add, flh_half* sum_out,
                                               const flh_half* weight, float eps, uint8_t* q_packed, flh_half* scales,
                                               uint32_t M, uint32_t K, int hadamard, float clip_ratio, void* stream) {
  if (!x || !add || !sum_out || !q_packed || !scales) return fail(FLH_EINVAL, "add_rmsnorm_rotate_quant: null pointer");
  if (misaligned16(x, add, sum_out) || misaligned16(q_packed))
    return fail(FLH_EINVAL, "add_rmsnorm_rotate_quant: x, add, sum_out and q_packed must be 16-byte aligned");
  if (weight && misaligned16(weight)) return fail(FLH_EINVAL, "add_rmsnorm_rotate_quant: weight must be 16-byte aligned");
  if (!(clip_ratio > 0.f)) return fail(FLH_EINVAL, "add_rmsnorm_rotate_quant: clip_ratio must be positive");
  if (!(eps >= 0.f)) return fail(FLH_EINVAL, "add_rmsnorm_rotate_quant: eps must not be negative");
  if (hadamard != FLH_HAD_NONE && hadamard != FLH_HAD_F32 && hadamard != FLH_HAD_MFMA)
    return fail(FLH_EINVAL, "add_rmsnorm_rotate_quant: unknown hadamard mode %d", hadamard);
  if (K % 512 || !is_pow2(K / 512) || K > 8192)
    return fail(FLH_EINVAL, "add_rmsnorm_rotate_quant: K (%u) must be 512, 1024, 2048, 4096 or 8192", K);
  if (M == 0) return FLH_OK;
  const __half *xh = (const __half*)x, *ah = (const __half*)add, *wh = (const __half*)weight;
  __half *sh = (__half*)scales, *oh = (__half*)sum_out;
  hipStream_t st = (hipStream_t)stream;
  // (the eight-waves-per-row kernel lets other waves read x and add after one has stored its part of the sum)
  if ((const void*)sum_out == (const void*)x || (const void*)sum_out == (const void*)add)
    return fail(FLH_EINVAL, "add_rmsnorm_rotate_quant: sum_out must not be x or add");
  if (hadamard == FLH_HAD_MFMA) {                      // matrix cores: K = 4096, else the float32 butterflies
    if (K == 4096) return launch_rotate_quant_mfma4096(xh, ah, oh, true, wh, eps, q_packed, sh, M, clip_ratio, false, st);
    hadamard = FLH_HAD_F32;
  }
  const bool had = hadamard != FLH_HAD_NONE;
  if (had && K == 4096 && clip_ratio >= 1.0f && M <= kRow8MaxRows) {
    hipLaunchKernelGGL(add_rmsnorm_rotate_quant_row8_kernel, dim3(M), dim3(512), 0, st, xh, ah, oh, wh, eps, q_packed, sh,
                       1.0f / 64.0f);
    return check_launch("add_rmsnorm_rotate_quant_row8");
  }
  switch (K / 512) {
    case 1: return launch_wave_rms<1>(xh, wh, eps, q_packed, sh, nullptr, M, had, clip_ratio, st, ah, oh);
    case 2: return launch_wave_rms<2>(xh, wh, eps, q_packed, sh, nullptr, M, had, clip_ratio, st, ah, oh);
    case 4: return launch_wave_rms<4>(xh, wh, eps, q_packed, sh, nullptr, M, had, clip_ratio, st, ah, oh);
    case 8: return launch_wave_rms<8>(xh, wh, eps, q_packed, sh, nullptr, M, had, clip_ratio, st, ah, oh);
    default: return launch_wave_rms<16>(xh, wh, eps, q_packed, sh, nullptr, M, had, clip_ratio, st, ah, oh);
  }
}

extern "C" int flh_rotate_quant_f6(const flh_half* x, const flh_half* add, flh_half* sum_out, int rmsnorm,
                                   const flh_half* weight, float eps, uint8_t* encoded, flh_half* scales, uint32_t M,
                                   uint32_t K, int hadamard, float clip_ratio, void* stream) {
  const char* who = "rotate_quant_f6";
  if (!x || !encoded || !scales) return fail(FLH_EINVAL, "%s: null pointer", who);
  if (misaligned16(x, encoded)) return fail(FLH_EINVAL, "%s: x and encoded must be 16-byte aligned", who);
  if ((add == nullptr) != (sum_out == nullptr)) return fail(FLH_EINVAL, "%s: add and sum_out come together or not at all", who);
  if (add && !rmsnorm) return fail(FLH_EINVAL, "%s: the residual addition comes with the RMSNorm prologue", who);
  if (add && misaligned16(add, sum_out)) return fail(FLH_EINVAL, "%s: add and sum_out must be 16-byte aligned", who);
  if (sum_out && ((const void*)sum_out == (const void*)x || (const void*)sum_out == (const void*)add))
    return fail(FLH_EINVAL, "%s: sum_out must not be x or add", who);
  if (weight && (!rmsnorm || misaligned16(weight))) return fail(FLH_EINVAL, "%s: weight needs rmsnorm != 0 and 16-byte alignment", who);
  if (!(clip_ratio > 0.f)) return fail(FLH_EINVAL, "%s: clip_ratio must be positive", who);
  if (!(eps >= 0.f)) return fail(FLH_EINVAL, "%s: eps must not be negative", who);
  if (M == 0) return FLH_OK;
  const __half *xh = (const __half*)x, *ah = (const __half*)add, *wh = (const __half*)weight;
  __half *sh = (__half*)scales, *oh = (__half*)sum_out;
  hipStream_t st = (hipStream_t)stream;
  if (hadamard == FLH_HAD_MFMA) {
    if (K == 4096) return launch_rotate_quant_mfma4096(xh, ah, oh, rmsnorm != 0, wh, eps, encoded, sh, M, clip_ratio, true, st);
    if (rmsnorm) return fail(FLH_EINVAL, "%s: the matrix-core rotation has an RMSNorm prologue for K = 4096 only", who);
    if (K != 11008 && K != 14336)
      return fail(FLH_EINVAL, "%s: matrix-core rotation with 6-bit output: K (%u) must be 4096, 11008 or 14336", who, K);
    return launch_rotate_quant_mfma_f6(xh, encoded, sh, M, K, clip_ratio, st);
  }
  if (hadamard != FLH_HAD_NONE && hadamard != FLH_HAD_F32) return fail(FLH_EINVAL, "%s: unknown hadamard mode %d", who, hadamard);
  if (K % 512 || !is_pow2(K / 512) || K > 8192)
    return fail(FLH_EINVAL, "%s: K (%u) must be 512, 1024, 2048, 4096 or 8192 (or 11008 / 14336 on the matrix cores)", who, K);
  const bool had = hadamard != FLH_HAD_NONE;
  if (rmsnorm) {
    switch (K / 512) {
      case 1: return launch_wave_rms<1>(xh, wh, eps, encoded, sh, nullptr, M, had, clip_ratio, st, ah, oh, 1);
      case 2: return launch_wave_rms<2>(xh, wh, eps, encoded, sh, nullptr, M, had, clip_ratio, st, ah, oh, 1);
      case 4: return launch_wave_rms<4>(xh, wh, eps, encoded, sh, nullptr, M, had, clip_ratio, st, ah, oh, 1);
      case 8: return launch_wave_rms<8>(xh, wh, eps, encoded, sh, nullptr, M, had, clip_ratio, st, ah, oh, 1);
      default: return launch_wave_rms<16>(xh, wh, eps, encoded, sh, nullptr, M, had, clip_ratio, st, ah, oh, 1);
    }
  }
  switch (K / 512) {
    case 1: return launch_wave<1>(xh, encoded, sh, nullptr, M, had, clip_ratio, st, 1);
    case 2: return launch_wave<2>(xh, encoded, sh, nullptr, M, had, clip_ratio, st, 1);
    case 4: return launch_wave<4>(xh, encoded, sh, nullptr, M, had, clip_ratio, st, 1);
    case 8: return launch_wave<8>(xh, encoded, sh, nullptr, M, had, clip_ratio, st, 1);
    default: return launch_wave<16>(xh, encoded, sh, nullptr, M, had, clip_ratio, st, 1);
  }
}

extern "C" int flh_silu_mul_f16(const flh_half* gate, const flh_half* up, flh_half* out, uint64_t n, void* stream) {
  if (!gate || !up || !out) return fail(FLH_EINVAL, "silu_mul: null pointer");
  if (misaligned16(gate, up, out)) return fail(FLH_EINVAL, "silu_mul: gate, up and out must be 16-byte aligned");
  if (n % 8) return fail(FLH_EINVAL, "silu_mul: the element count (%llu) must be a multiple of 8", (unsigned long long)n);
  if (n / 8 > 0x7fffffffull * 256) return fail(FLH_EINVAL, "silu_mul: too many elements");
  if (n == 0) return FLH_OK;
  hipLaunchKernelGGL(silu_mul_kernel, dim3((unsigned)((n / 8 + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                     (const __half*)gate, (const __half*)up, (__half*)out, n / 8);
  return check_launch("silu_mul_kernel");
}

extern "C" int flh_add_rmsnorm_f16(const flh_half* x, const flh_half* add, const flh_half* weight, float eps, flh_half* out,
                                   flh_half* sum_out, uint32_t M, uint32_t K, void* stream) {
  if (!x || !out) return fail(FLH_EINVAL, "add_rmsnorm: null pointer");
  if (sum_out && !add) return fail(FLH_EINVAL, "add_rmsnorm: sum_out is the stored sum x + add and needs add");
  if (misaligned16(x, add, weight, out, sum_out)) return fail(FLH_EINVAL, "add_rmsnorm: tensors must be 16-byte aligned");
  if (K == 0 || K % 8 || K > 16384) return fail(FLH_EINVAL, "add_rmsnorm: K (%u) must be a multiple of 8, at most 16384", K);
  if (!(eps >= 0.f)) return fail(FLH_EINVAL, "add_rmsnorm: eps must not be negative");
  if (M == 0) return FLH_OK;
  hipLaunchKernelGGL(add_rmsnorm_kernel, dim3(M), dim3(256), 0, (hipStream_t)stream, (const __half*)x, (const __half*)add,
                     (const __half*)weight, (__half*)out, (__half*)sum_out, K, eps);
  return check_launch("add_rmsnorm_kernel");
}

extern "C" int flh_silu_mul_rotate_quant_i4(const flh_half* gate, const flh_half* up, uint8_t* q_packed, flh_half* scales,
                                            uint32_t M, uint32_t K, void* stream) {
  if (!gate || !up || !q_packed || !scales) return fail(FLH_EINVAL, "silu_mul_rotate_quant: null pointer");
  if (misaligned16(gate, up, q_packed)) return fail(FLH_EINVAL, "silu_mul_rotate_quant: gate, up and q_packed must be 16-byte aligned");
  if (K != 11008 && K != 14336) return fail(FLH_EINVAL, "silu_mul_rotate_quant: K (%u) must be 11008 or 14336", K);
  if (M > 256) return fail(FLH_EINVAL, "silu_mul_rotate_quant: at most 256 rows (%u given); longer batches take the gate / up GEMM that stores the product", M);
  if (M == 0) return FLH_OK;
  return launch_silu_mul_rotate_quant_mfma((const __half*)gate, (const __half*)up, q_packed, (__half*)scales, M, K,
                                           (hipStream_t)stream);
}

extern "C" int flh_group_quant_f6(const flh_half* x, uint8_t* encoded, flh_half* scales, uint32_t M, uint32_t K,
                                  int hadamard, float scale_mul, void* stream) {
  if (!x || !encoded || !scales) return fail(FLH_EINVAL, "group_quant_f6: null pointer");
  if (misaligned16(x, encoded)) return fail(FLH_EINVAL, "group_quant_f6: x and encoded must be 16-byte aligned");
  if (!(scale_mul > 0.f)) return fail(FLH_EINVAL, "group_quant_f6: scale_mul must be positive");
  if (K == 0 || K % 128) return fail(FLH_EINVAL, "group_quant_f6: K (%u) must be a positive multiple of 128", K);
  if ((uint64_t)M * (K / 128) > 0xFFFFFFFFull) return fail(FLH_EINVAL, "group_quant_f6: too many groups");
  if (M == 0) return FLH_OK;
  const uint32_t R = M * (K / 128);
  const dim3 grid((unsigned)(((uint64_t)R * 16 + 255) / 256)), block(256);
  const __half* xh = (const __half*)x;
  if (hadamard)
    hipLaunchKernelGGL((group_kernel<128, true, true, true>), grid, block, 0, (hipStream_t)stream, xh, encoded,
                       (__half*)scales, nullptr, R, scale_mul, M, K / 128);
  else
    hipLaunchKernelGGL((group_kernel<128, false, true, true>), grid, block, 0, (hipStream_t)stream, xh, encoded,
                       (__half*)scales, nullptr, R, scale_mul, M, K / 128);
  return check_launch("group_kernel (6-bit output)");
}

extern "C" int flh_fwht_f16_inplace(flh_half* x, uint32_t R, int group, void* stream) {
  if (!x) return fail(FLH_EINVAL, "fwht: null pointer");
  if (misaligned16(x)) return fail(FLH_EINVAL, "fwht: x must be 16-byte aligned");
  return group_dispatch(nullptr, nullptr, nullptr, (__half*)x, R, group, true, false, 1.0f, (hipStream_t)stream);
}

extern "C" int flh_rotate_quant_i4(const flh_half* x, uint8_t* q_packed, flh_half* scales, flh_half* y_out, uint32_t M,
                                   uint32_t K, int hadamard, int had_group, int scale_group, float clip_ratio,
                                   void* stream) {
  if (!x || !q_packed || !scales) return fail(FLH_EINVAL, "rotate_quant: null pointer");
  if (misaligned16(x, q_packed, y_out)) return fail(FLH_EINVAL, "rotate_quant: x, q_packed and y_out must be 16-byte aligned");
  if (K == 0 || K % 16) return fail(FLH_EINVAL, "rotate_quant: K (%u) must be a positive multiple of 16", K);
  if (!(clip_ratio > 0.f)) return fail(FLH_EINVAL, "rotate_quant: clip_ratio must be positive");
  if (scale_group < 0) scale_group = 0;
  if (scale_group > 0 && (K % scale_group || scale_group % 2))
    return fail(FLH_EINVAL, "rotate_quant: scale group %d must be even and divide K = %u", scale_group, K);
  if (M == 0) return FLH_OK;
  hipStream_t st = (hipStream_t)stream;
  const __half* xh = (const __half*)x;
  __half* sh = (__half*)scales;
  __half* yh = (__half*)y_out;

  if (hadamard == FLH_HAD_MFMA) {
    if (had_group <= 0 && scale_group == 0 && !y_out && rotate_quant_mfma_supports(K))
      return launch_rotate_quant_mfma(xh, q_packed, sh, M, K, clip_ratio, st);
    hadamard = FLH_HAD_F32;  // shapes / options the matrix-core kernels do not cover
  }
  int Kd = 1, P = 1;
  float norm = 1.f;
  if (hadamard == FLH_HAD_F32) {
    if (had_group > 0 && (uint32_t)had_group != K) {
      if (!is_pow2(had_group) || K % had_group)
        return fail(FLH_EINVAL, "rotate_quant: hadamard group %d must be a power of two dividing K = %u", had_group, K);
      P = had_group;
      norm = sqrtf((float)had_group);
    } else {
      if (!factor_hadamard(K, &Kd, &P))
        return fail(FLH_EINVAL, "rotate_quant: no Hadamard factorisation for K = %u", K);
      norm = sqrtf((float)K);
    }
  } else if (hadamard != FLH_HAD_NONE) {
    return fail(FLH_EINVAL, "rotate_quant: unknown hadamard mode %d", hadamard);
  }

  const bool whole_row_pow2 = (hadamard == FLH_HAD_NONE || (Kd == 1 && (uint32_t)P == K));
  if (whole_row_pow2 && scale_group == 0 && K % 512 == 0 && is_pow2(K / 512) && K <= 8192) {
    const bool had = hadamard != FLH_HAD_NONE;
    if (had && K == 4096 && !yh && clip_ratio >= 1.0f && M <= kRow8MaxRows) {
      hipLaunchKernelGGL(rotate_quant_row8_kernel, dim3(M), dim3(512), 0, st, xh, q_packed, sh, 1.0f / 64.0f);
      return check_launch("rotate_quant_row8");
    }
    switch (K / 512) {
      case 1: return launch_wave<1>(xh, q_packed, sh, yh, M, had, clip_ratio, st);
      case 2: return launch_wave<2>(xh, q_packed, sh, yh, M, had, clip_ratio, st);
      case 4: return launch_wave<4>(xh, q_packed, sh, yh, M, had, clip_ratio, st);
      case 8: return launch_wave<8>(xh, q_packed, sh, yh, M, had, clip_ratio, st);
      case 16: return launch_wave<16>(xh, q_packed, sh, yh, M, had, clip_ratio, st);
    }
  }
  // the row in float32, a second copy for the dense factor's output and that factor's sign bits
  const size_t smem = (size_t)K * sizeof(float) * (Kd > 1 ? 2 : 1) + (Kd > 1 ? (((size_t)Kd * Kd + 7) / 8 / 16 + 2) * 16 : 0);   // + the byte after the last row's window
  if (smem > 160 * 1024 - 64) return fail(FLH_EINVAL, "rotate_quant: K = %u does not fit the LDS staging", K);
  static LdsGrant grant;                               // grows to the largest row asked for
  if (int rc = reserve_lds((const void*)rotate_quant_generic_kernel, smem, grant, "rotate_quant")) return rc;
  hipLaunchKernelGGL(rotate_quant_generic_kernel, dim3(M), dim3(kGenericThreads), smem, st, xh, q_packed, sh, yh, K,
                     hadamard == FLH_HAD_NONE ? 0 : P, Kd, norm, scale_group, clip_ratio);
  return check_launch("rotate_quant_generic");
}
