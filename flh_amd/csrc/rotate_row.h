// One wave rotates, quantises and packs one row of K = 512 * J fp16 values entirely in registers (float32
// butterflies in ascending stride order: bit-equal to the float32 restatement of had_transform,
// flh/nn/quantization.py:42-74).  Shared by the wave-per-row kernel and by the decode GEMM that quantises its own
// activations.
#pragma once
#include "lane_ops.h"
#include "quant_pack.h"
#include "f6_codes.h"

namespace flh {
namespace {

// ------------------------------------------------------------------------------------
// Wave-per-row layout, float32 butterflies, K = 512 * J.
//
// Element index i = j*512 + c*8 + e: e in registers, j in registers, c = the 16-byte chunk
// this lane loads.  Lanes are labelled so that the four DPP distances that exist as one
// instruction (quad xor 1, quad xor 2, mirror of 8, mirror of 16) flip exactly one label
// bit each: lane = b1*0001 ^ b2*0010 ^ b3*0111 ^ b4*1111 (bits 0-3), b5 = lane bit 4,
// b6 = lane bit 5, and c = b1 + 2 b2 + 4 b3 + 8 b4 + 16 b5 + 32 b6.  A wave still reads
// whole 1 KiB segments; only the order of chunks inside each 256 bytes differs.
// ------------------------------------------------------------------------------------
__device__ __forceinline__ int lane_chunk(int lane) {
  const int b1 = (lane ^ (lane >> 2)) & 1;
  const int b2 = ((lane >> 1) ^ (lane >> 2)) & 1;
  const int b3 = ((lane >> 2) ^ (lane >> 3)) & 1;
  return b1 | (b2 << 1) | (b3 << 2) | (lane & 0x38);
}

// One butterfly stage across a lane-label bit, in one instruction per value:
//     v <- v + sgn * v[partner lane]        (v_fmac_f32 with the DPP operand as the multiplicand)
// with sgn = +1 in the lower lane of each pair and -1 in the upper one.  The lower lane gets the
// sum.  The upper lane gets own - partner, the NEGATIVE of the butterfly's difference: every such
// stage flips the sign of what the upper lanes store (rounding is symmetric, so the magnitudes are
// those of the plain butterfly).  A pair's two lanes agree in all earlier stages' label bits, hence
// in their accumulated sign, so the stage stays correct on sign-flipped data; the caller folds the
// final sign (-1)^(number of upper stages of the lane) into the normalisation constant.
// Written as volatile asm so that the stage order is kept: the hardware needs two instructions
// between a write of a register and a DPP read of it, which the 8 J - 1 other values of a stage
// provide (the caller pads the ends with s_nop).
template <int CTRL, int N>
__device__ __forceinline__ void stage_fmac(float (&v)[N], float sgn) {
#pragma unroll
  for (int i = 0; i < N; ++i) {
    if constexpr (CTRL == kDppQuadXor1)
      asm volatile("v_fmac_f32_dpp %0, %0, %1 quad_perm:[1,0,3,2] row_mask:0xf bank_mask:0xf" : "+v"(v[i]) : "v"(sgn));
    else if constexpr (CTRL == kDppQuadXor2)
      asm volatile("v_fmac_f32_dpp %0, %0, %1 quad_perm:[2,3,0,1] row_mask:0xf bank_mask:0xf" : "+v"(v[i]) : "v"(sgn));
    else if constexpr (CTRL == kDppRowHalfMirror)
      asm volatile("v_fmac_f32_dpp %0, %0, %1 row_half_mirror row_mask:0xf bank_mask:0xf" : "+v"(v[i]) : "v"(sgn));
    else
      asm volatile("v_fmac_f32_dpp %0, %0, %1 row_mirror row_mask:0xf bank_mask:0xf" : "+v"(v[i]) : "v"(sgn));
  }
}

// butterfly across lane bit 4 (WIDE = false) or 5 (WIDE = true): swap halves of a register
// pair so that both operands of each butterfly sit in one lane, combine, swap back.
template <bool WIDE, int N>
__device__ __forceinline__ void stage_swap(float (&v)[N]) {
#pragma unroll
  for (int i = 0; i < N; i += 2) {
    unsigned x = __float_as_uint(v[i]), y = __float_as_uint(v[i + 1]);
    auto r = WIDE ? __builtin_amdgcn_permlane32_swap(x, y, false, false)
                  : __builtin_amdgcn_permlane16_swap(x, y, false, false);
    const float a = __uint_as_float(r[0]), b = __uint_as_float(r[1]);
    const float s = a + b, d = a - b;
    auto r2 = WIDE ? __builtin_amdgcn_permlane32_swap(__float_as_uint(s), __float_as_uint(d), false, false)
                   : __builtin_amdgcn_permlane16_swap(__float_as_uint(s), __float_as_uint(d), false, false);
    v[i] = __uint_as_float(r2[0]);
    v[i + 1] = __uint_as_float(r2[1]);
  }
}

// RMS: the row is first normalised as flh/nn/normalization.py:12-20 does -- float32 sum of squares / K,
// x * (1 / sqrt(. + eps)) [* weight] with every product rounded to float32, then fp16 -- and that fp16 row is
// what the rotation and the quantiser see.
//
// add_row / sum_row (both or neither): the row is x + add in fp16 (one rounding per value, torch's fp16 addition), and
// that sum is also stored to sum_row -- the residual stream of a decoder layer (modeling_llama.py:600-618:
// hidden = residual + attention output; residual = hidden; hidden = norm(hidden)) without a launch of its own.
// sum_row overlaps neither input.
//
// f6_rows > 0: the codes leave in the operand format of the 6-bit matrix instruction (gemm_f6.hip: K-slab-major blocks
// of 96 bytes per 128 codes and row) -- q_row is then the BASE of the encoded matrix, f6_rows its row count and f6_row
// this row's index.
template <int J, bool HAD, bool EXACT_NORM, bool RMS = false>
__device__ __forceinline__ void rotate_quant_row(const __half* __restrict__ x_row, uint8_t* q_row, __half* scale_dst,
                                                 __half* y_row, float norm, float clip,
                                                 const __half* __restrict__ rms_weight = nullptr, float rms_eps = 0.f,
                                                 const __half* add_row = nullptr, __half* sum_row = nullptr,
                                                 uint32_t f6_rows = 0, uint32_t f6_row = 0) {
  constexpr int K = 512 * J, N = 8 * J;
  const int lane = threadIdx.x & 63;
  const int c = lane_chunk(lane);
  const __half* xr = x_row + c * 8;

  v4i raw[J];
#pragma unroll
  for (int j = 0; j < J; ++j) raw[j] = *(const v4i*)(xr + j * 512);
  if (add_row) {                                       // wave-uniform
#pragma unroll
    for (int j = 0; j < J; ++j) raw[j] = add_h8(raw[j], *(const v4i*)(add_row + c * 8 + j * 512));
#pragma unroll
    for (int j = 0; j < J; ++j) *(v4i*)(sum_row + c * 8 + j * 512) = raw[j];
  }

  if constexpr (RMS) {
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < J; ++j)
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        const unsigned w = (unsigned)raw[j][d];
        const h2 t = __builtin_bit_cast(h2, w);
        ss = __builtin_fmaf((float)t[0], (float)t[0], ss);
        ss = __builtin_fmaf((float)t[1], (float)t[1], ss);
      }
    ss = wave_sum(ss);
    const float inv = 1.0f / __builtin_sqrtf(ss / (float)K + rms_eps);
#pragma unroll
    for (int j = 0; j < J; ++j) {
      v4i wv = {0, 0, 0, 0};
      if (rms_weight) wv = *(const v4i*)(rms_weight + j * 512 + c * 8);
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        const unsigned w = (unsigned)raw[j][d], ww = (unsigned)wv[d];
        const h2 t = __builtin_bit_cast(h2, w), g = __builtin_bit_cast(h2, ww);
        float a = round_here((float)t[0] * inv), b = round_here((float)t[1] * inv);
        if (rms_weight) {
          a = round_here(a * (float)g[0]);
          b = round_here(b * (float)g[1]);
        }
        raw[j][d] = (int)pack_f16(a, b);
      }
    }
  }

  unsigned yp[N / 2];                                  // the rotated row as packed fp16 pairs
  float mx = 0.f;                                      // row maximum of |y|, exactly representable in fp16
  if constexpr (HAD) {
    float v[N];
    // stride 1 straight from the packed halves: lo + hi and lo - hi are exact float32 sums of fp16 values
#pragma unroll
    for (int j = 0; j < J; ++j)
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        const int w = raw[j][d];
        asm("v_fma_mix_f32 %0, %1, 1.0, %1 op_sel:[0,0,1] op_sel_hi:[1,0,1]" : "=v"(v[j * 8 + 2 * d]) : "v"(w));
        asm("v_fma_mix_f32 %0, %1, -1.0, %1 op_sel:[1,0,0] op_sel_hi:[1,0,1]" : "=v"(v[j * 8 + 2 * d + 1]) : "v"(w));
      }
#pragma unroll
    for (int s = 2; s < 8; s <<= 1)
#pragma unroll
      for (int i = 0; i < N; ++i)
        if ((i & s) == 0) {
          const float a = v[i], b = v[i + s];
          v[i] = a + b;
          v[i + s] = a - b;
        }
    const float sg1 = (c & 1) ? -1.f : 1.f, sg2 = (c & 2) ? -1.f : 1.f, sg3 = (c & 4) ? -1.f : 1.f,
                sg4 = (c & 8) ? -1.f : 1.f;
    asm volatile("s_nop 1" : "+v"(v[0]), "+v"(v[1]));   // the first DPP reads must not follow their writes directly
    stage_fmac<kDppQuadXor1>(v, sg1);
    stage_fmac<kDppQuadXor2>(v, sg2);
    stage_fmac<kDppRowHalfMirror>(v, sg3);
    stage_fmac<kDppRowMirror>(v, sg4);
    asm volatile("s_nop 1" : "+v"(v[N - 1]), "+v"(v[N - 2]));
    stage_swap<false>(v);
    stage_swap<true>(v);
#pragma unroll
    for (int s = 8; s < N; s <<= 1)
#pragma unroll
      for (int i = 0; i < N; ++i)
        if ((i & s) == 0) {
          const float a = v[i], b = v[i + s];
          v[i] = a + b;
          v[i + s] = a - b;
        }
    // this lane's values carry the sign (-1)^(upper stages); it rides on the normalisation
    const bool flipped = __builtin_popcount(c & 15) & 1;
    float m32 = 0.f;
#pragma unroll
    for (int i = 0; i < N; i += 2) m32 = __builtin_fmaxf(__builtin_fmaxf(__builtin_fabsf(v[i]), __builtin_fabsf(v[i + 1])), m32);
    if constexpr (EXACT_NORM) {
      // norm = 1 / sqrt(K) is a power of two: the product is exact, one rounding to fp16
      const float nf = flipped ? -norm : norm;
#pragma unroll
      for (int i = 0; i < N; i += 2) yp[i / 2] = scale_pack_f16(v[i], v[i + 1], nf);
      mx = (float)__builtin_bit_cast(h2, scale_pack_f16(m32, 0.f, norm))[0];
    } else {
      // sqrt(K) is not a power of two: float32 quotient, then fp16, as the float32 restatement does
      const unsigned flip = flipped ? 0x80008000u : 0u;
#pragma unroll
      for (int i = 0; i < N; i += 2) yp[i / 2] = pack_f16(round_here(v[i] / norm), round_here(v[i + 1] / norm)) ^ flip;
      mx = (float)(_Float16)round_here(m32 / norm);
    }
  } else {
#pragma unroll
    for (int j = 0; j < J; ++j)
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        const unsigned w = (unsigned)raw[j][d];        // (a bit_cast of the vector element itself miscompiles)
        yp[j * 4 + d] = w;
        const h2 t = __builtin_bit_cast(h2, w);
        mx = __builtin_fmaxf(__builtin_fmaxf(__builtin_fabsf((float)t[0]), __builtin_fabsf((float)t[1])), mx);
      }
  }
  mx = wave_max(mx);
  if (y_row) {
    // zeros leave the sign-carrying lanes as -0; adding +0 turns them into the +0 the plain butterfly
    // gives (x + 0 = x for every other value).  Codes and scales do not depend on the sign of zero.
    const h2 zero2 = {(_Float16)0.0f, (_Float16)0.0f};
#pragma unroll
    for (int j = 0; j < J; ++j) {
      v4i t;
#pragma unroll
      for (int d = 0; d < 4; ++d) t[d] = __builtin_bit_cast(int, __builtin_bit_cast(h2, yp[4 * j + d]) + zero2);
      *(v4i*)(y_row + j * 512 + c * 8) = t;
    }
  }
  if (clip < 1.0f) mx = (float)(_Float16)round_here(mx * clip);   // clip bound; values are clamped below
  _Float16 s = scale_of_max(mx);
  if (s == (_Float16)0.0f) s = (_Float16)1.0f;
  const float r = reciprocal_of_scale(s);
  // |y / s| <= 7.004 unless the scale is subnormal (its rounding error is then unbounded) or the row
  // was clipped: only then are the clamps needed
  const bool careful = __builtin_amdgcn_readfirstlane((float)s < 6.2e-5f || clip < 1.0f);
  const h2 hb = {(_Float16)mx, (_Float16)mx};
  unsigned* qr = (unsigned*)q_row + c;
#pragma unroll
  for (int j = 0; j < J; ++j) {
    const unsigned w = careful ? nibbles8<true>(yp[4 * j], yp[4 * j + 1], yp[4 * j + 2], yp[4 * j + 3], r, hb)
                               : nibbles8<false>(yp[4 * j], yp[4 * j + 1], yp[4 * j + 2], yp[4 * j + 3], r, hb);
    if (f6_rows) {                                     // wave-uniform; chunk c of segment j sits in 128-code block 4 j + c / 16
      const size_t block = (size_t)(4 * j + (c >> 4)) * f6_rows + f6_row;
      f6_store_chunk(w, c & 15, q_row + block * kF6BlockBytes, true);
    } else {
      qr[j * 64] = w;
    }
  }
  if (lane == 0) *scale_dst = __builtin_bit_cast(__half, s);
}

// One row of 4096 values by the eight waves of a workgroup, for callers where a single row's latency matters:
// wave w takes the 512 values from 512 w -- strides 1 .. 256 in registers and across lanes as above -- and the
// strides 512, 1024, 2048 run across the waves through LDS (stage: 8 x 8 x 64 floats, wave_max: 8 floats).
// The same additions in the same order as rotate_quant_row<8>, hence the same codes and scale.  Every wave of the
// workgroup must call it (four barriers).
// RMS: the row is normalised first, as rotate_quant_row<8, ..., RMS> does it.  Every wave reads the whole row once
// more (it is in the compute unit's cache by then) and sums the squares in exactly that routine's order -- per lane
// over the eight 512-value segments, then the fixed tree over the lanes -- so that the statistics, the normalised
// fp16 row and therefore the codes are bit-identical to the wave-per-row kernel's, without a pass over the waves.
// ADD: the row is x + add_row (fp16), stored to sum_row as well, as in rotate_quant_row.  Every wave forms the whole sum
// for the statistics and stores only its own segment (the other waves still read x_row and add_row meanwhile).
template <bool RMS = false, bool ADD = false>
__device__ __forceinline__ void rotate_quant_row_8waves(const __half* __restrict__ x_row, float* stage, float* wave_max8,
                                                        uint8_t* q_row, __half* scale_dst, float norm, int wave,
                                                        const __half* __restrict__ rms_weight = nullptr,
                                                        float rms_eps = 0.f, const __half* __restrict__ add_row = nullptr,
                                                        __half* __restrict__ sum_row = nullptr) {
  const int lane = threadIdx.x & 63;
  const int c = lane_chunk(lane);
  v4i raw = *(const v4i*)(x_row + wave * 512 + c * 8);
  if constexpr (ADD) {
    raw = add_h8(raw, *(const v4i*)(add_row + wave * 512 + c * 8));
    if (sum_row) *(v4i*)(sum_row + wave * 512 + c * 8) = raw;    // (null: another workgroup stores the same sum)
  }
  if constexpr (RMS) {
    float ss = 0.f;
#pragma unroll
    for (int j = 0; j < 8; ++j) {
      v4i seg = *(const v4i*)(x_row + j * 512 + c * 8);
      if constexpr (ADD) seg = add_h8(seg, *(const v4i*)(add_row + j * 512 + c * 8));
#pragma unroll
      for (int d = 0; d < 4; ++d) {
        const unsigned w = (unsigned)seg[d];
        const h2 t = __builtin_bit_cast(h2, w);
        ss = __builtin_fmaf((float)t[0], (float)t[0], ss);
        ss = __builtin_fmaf((float)t[1], (float)t[1], ss);
      }
    }
    ss = wave_sum(ss);
    const float inv = 1.0f / __builtin_sqrtf(ss / 4096.0f + rms_eps);
    v4i wv = {0, 0, 0, 0};
    if (rms_weight) wv = *(const v4i*)(rms_weight + wave * 512 + c * 8);
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const unsigned w = (unsigned)raw[d], ww = (unsigned)wv[d];
      const h2 t = __builtin_bit_cast(h2, w), g = __builtin_bit_cast(h2, ww);
      float a = round_here((float)t[0] * inv), b = round_here((float)t[1] * inv);
      if (rms_weight) {
        a = round_here(a * (float)g[0]);
        b = round_here(b * (float)g[1]);
      }
      raw[d] = (int)pack_f16(a, b);
    }
  }
  float v[8];
#pragma unroll
  for (int d = 0; d < 4; ++d) {
    const int w = raw[d];
    asm("v_fma_mix_f32 %0, %1, 1.0, %1 op_sel:[0,0,1] op_sel_hi:[1,0,1]" : "=v"(v[2 * d]) : "v"(w));
    asm("v_fma_mix_f32 %0, %1, -1.0, %1 op_sel:[1,0,0] op_sel_hi:[1,0,1]" : "=v"(v[2 * d + 1]) : "v"(w));
  }
#pragma unroll
  for (int s = 2; s < 8; s <<= 1)
#pragma unroll
    for (int i = 0; i < 8; ++i)
      if ((i & s) == 0) {
        const float a = v[i], b = v[i + s];
        v[i] = a + b;
        v[i + s] = a - b;
      }
  const float sg1 = (c & 1) ? -1.f : 1.f, sg2 = (c & 2) ? -1.f : 1.f, sg3 = (c & 4) ? -1.f : 1.f,
              sg4 = (c & 8) ? -1.f : 1.f;
  asm volatile("s_nop 1" : "+v"(v[0]), "+v"(v[1]));
  stage_fmac<kDppQuadXor1>(v, sg1);
  stage_fmac<kDppQuadXor2>(v, sg2);
  stage_fmac<kDppRowHalfMirror>(v, sg3);
  stage_fmac<kDppRowMirror>(v, sg4);
  asm volatile("s_nop 1" : "+v"(v[7]), "+v"(v[6]));
  stage_swap<false>(v);
  stage_swap<true>(v);
  // across the waves: value e of every lane goes to wave e, which combines the eight waves' copies
#pragma unroll
  for (int e = 0; e < 8; ++e) stage[(e * 8 + wave) * 64 + lane] = v[e];
  __syncthreads();
  float u[8];
#pragma unroll
  for (int w2 = 0; w2 < 8; ++w2) u[w2] = stage[(wave * 8 + w2) * 64 + lane];
#pragma unroll
  for (int s = 1; s < 8; s <<= 1)
#pragma unroll
    for (int i = 0; i < 8; ++i)
      if ((i & s) == 0) {
        const float a = u[i], b = u[i + s];
        u[i] = a + b;
        u[i + s] = a - b;
      }
  __syncthreads();
#pragma unroll
  for (int w2 = 0; w2 < 8; ++w2) stage[(wave * 8 + w2) * 64 + lane] = u[w2];
  __syncthreads();
#pragma unroll
  for (int e = 0; e < 8; ++e) v[e] = stage[(e * 8 + wave) * 64 + lane];
  // from here on as rotate_quant_row: sign of the lane folded into the power-of-two normalisation
  const bool flipped = __builtin_popcount(c & 15) & 1;
  float m32 = 0.f;
#pragma unroll
  for (int i = 0; i < 8; i += 2) m32 = __builtin_fmaxf(__builtin_fmaxf(__builtin_fabsf(v[i]), __builtin_fabsf(v[i + 1])), m32);
  const float nf = flipped ? -norm : norm;
  unsigned yp[4];
#pragma unroll
  for (int i = 0; i < 8; i += 2) yp[i / 2] = scale_pack_f16(v[i], v[i + 1], nf);
  float mx = (float)__builtin_bit_cast(h2, scale_pack_f16(m32, 0.f, norm))[0];
  mx = wave_max(mx);
  if (lane == 0) wave_max8[wave] = mx;
  __syncthreads();
#pragma unroll
  for (int w2 = 0; w2 < 8; ++w2) mx = __builtin_fmaxf(mx, wave_max8[w2]);
  _Float16 s = scale_of_max(mx);
  if (s == (_Float16)0.0f) s = (_Float16)1.0f;
  const float r = reciprocal_of_scale(s);
  const bool careful = __builtin_amdgcn_readfirstlane((float)s < 6.2e-5f);
  const h2 hb = {(_Float16)mx, (_Float16)mx};
  ((unsigned*)q_row)[wave * 64 + c] = careful ? nibbles8<true>(yp[0], yp[1], yp[2], yp[3], r, hb)
                                              : nibbles8<false>(yp[0], yp[1], yp[2], yp[3], r, hb);
  if (wave == 0 && lane == 0) *scale_dst = __builtin_bit_cast(__half, s);
}

}  // namespace
}  // namespace flh
