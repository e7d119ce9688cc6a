// Matrix-core version of the whole-row Hadamard rotation + int4 quantisation.
//
// A row of K = D * 64 values is the D x 64 matrix X[j][t] (t contiguous); the rotation is
//        Y = M . X . H64 / sqrt(K)
// with H64 the 64-point Sylvester matrix and M the D x D factor across blocks: H64 again
// for K = 4096, the reference's literal had172 for K = 11008 = 172 * 64, and
// had28 (x) H8 (224 x 224) for K = 14336 = 28 * 512 (flh/functional/hadamard.py:92-113).
// Both factors are +/-1 matrices, exact in fp16, so each product is one pass over
// v_mfma_f32_32x32x16_f16 with fp32 accumulation:
//
//   level 1   Z[j][t'] = sum_t X[j][t] H64[t][t']      A = X straight from global memory
//   level 2   W[t'][j'] = sum_j Z[j][t'] M[j'][j]       A = Z as it sits in the level-1
//                                                       accumulators (lane = t', regs = j)
//
// The level-1 accumulators feed level 2 without leaving the registers; the output lane
// holds one block j' and 4 consecutive t' per register quad, which packs into 16-byte
// stores of 32 consecutive nibbles per lane.  Level 2 needs Z in fp16: it is split into
// hi + lo halves (two MFMAs) so that about 22 bits of each intermediate survive.
//
// This path does not reproduce the float32 butterfly order bit for bit (the matrix core
// sums in its own order).  The K = 4096 kernel splits Z into hi + lo halves and its codes
// differ from the exactly rounded transform at a rate below 1e-5; the dense-factor kernels
// keep one fp16 half of Z: about 4e-4 of their codes differ by one step and a row scale
// may differ by one fp16 ulp.  The tests measure these rates; the VALU kernels in
// fwht_quant.hip remain the bit-exact mode.
#include <atomic>
#include <mutex>
#include <type_traits>

#include "lane_ops.h"
#include "quant_pack.h"
#include "f6_codes.h"

namespace flh {
namespace {

// Quantise one block column (32 j' x 64 t' of a row, this lane: block j', 32 codes) and store
// its 16 bytes.  y[mt][2 g + u]: packed fp16 pairs, t' = 32 mt + 8 g + 4 h + 2 u (+1).
// CAREFUL also clamps the values to +-bound and the quotients to [-8, 7]; it is needed only
// for clipping (clip_ratio < 1) or a subnormal scale, chosen once per row.
template <bool CAREFUL>
__device__ __forceinline__ v4i quantise_block(const unsigned (&y0)[8], const unsigned (&y1)[8], float rinv, h2 hb) {
  unsigned pair[4];
#pragma unroll
  for (int p = 0; p < 4; ++p) {
    unsigned t[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int gp = 2 * p + u, g = gp & 3;
      unsigned y01 = gp < 4 ? y0[2 * g] : y1[2 * g], y23 = gp < 4 ? y0[2 * g + 1] : y1[2 * g + 1];
      if constexpr (CAREFUL) {
        y01 = __builtin_bit_cast(unsigned, __builtin_elementwise_min(__builtin_elementwise_max(__builtin_bit_cast(h2, y01), -hb), hb));
        y23 = __builtin_bit_cast(unsigned, __builtin_elementwise_min(__builtin_elementwise_max(__builtin_bit_cast(h2, y23), -hb), hb));
      }
      unsigned h01 = mul_halves(y01, rinv), h23 = mul_halves(y23, rinv);
      if constexpr (CAREFUL) {
        const h2 lo8 = {(_Float16)-8.0f, (_Float16)-8.0f}, hi7 = {(_Float16)7.0f, (_Float16)7.0f};
        h01 = __builtin_bit_cast(unsigned, __builtin_elementwise_min(__builtin_elementwise_max(__builtin_bit_cast(h2, h01), lo8), hi7));
        h23 = __builtin_bit_cast(unsigned, __builtin_elementwise_min(__builtin_elementwise_max(__builtin_bit_cast(h2, h23), lo8), hi7));
      }
      t[u] = quad_nibbles(h01, h23);
    }
    pair[p] = ((t[1] << 16) + t[0] - kPairBias) ^ 0x88888888u;
  }
  // pair[p]: halfwords of g' = 2 p, 2 p + 1 (g' = 4 mt + g).  The lower half-wave keeps dwords
  // g' = 0..3 of the block and needs the partner's halfwords for them, the upper one keeps 4..7.
  v4i out;
#pragma unroll
  for (int p = 0; p < 2; ++p) {
    auto sw = __builtin_amdgcn_permlane32_swap(pair[p], pair[p + 2], false, false);
    // sw[0] = {own pair[p] | lower lanes' pair[p+2]},  sw[1] = {upper lanes' pair[p] | own pair[p+2]}:
    // in both halves bytes 0-1 of a dword come from sw[0] and bytes 2-3 from sw[1]
    out[2 * p] = (int)__builtin_amdgcn_perm(sw[1], sw[0], 0x05040100u);
    out[2 * p + 1] = (int)__builtin_amdgcn_perm(sw[1], sw[0], 0x07060302u);
  }
  return out;
}

// K = 4096: one wave per row (rows strided over the waves), both factors H64, the constant
// fragments live in registers.  Level-1 slot map: fragment (s, h, i) holds t = 16 s + 8 h + i
// (s = k-step, h = lane / 32).  Level-2 slot map: (jb, s, h, i) holds
// j = 32 jb + 16 s + 8 (i / 4) + 4 h + i % 4, which is where registers 8 s .. 8 s + 7 of the
// level-1 accumulator tile jb sit.  The level-2 constants carry the 1/64 normalisation.
//
// Prologues and output format of the float32-butterfly kernels, on this rotation:
//   ADD   the row is x + add in fp16 (one rounding per value), stored to sum_out as well (the residual stream);
//   RMS   RMSNorm in front of the rotation (flh/nn/normalization.py:12-20): float32 sum of squares / K,
//         x * (1 / sqrt(. + eps)) * weight with every product rounded to float32, then fp16 (the order of the
//         additions of the sum of squares differs from the float32-butterfly kernel's, which can move 1 / sqrt by a
//         float32 ulp); the weight row sits in LDS (ones when the norm has none);
//   F6    the codes leave in the operand format of the 6-bit matrix instruction (gemm_f6.hip) -- q is then the encoded
//         matrix of M rows, K-slab-major blocks of 96 bytes per 128 codes and row: a lane's 32 codes are one 24-byte piece.
template <bool SPLIT, bool RMS = false, bool ADD = false, bool F6 = false>
__global__ __launch_bounds__(256, 2) void rotate_quant_mfma4096_kernel(const __half* __restrict__ x,
                                                                    uint8_t* __restrict__ q,
                                                                    __half* __restrict__ scales, uint32_t M,
                                                                    float clip, const __half* __restrict__ add,
                                                                    __half* __restrict__ sum_out,
                                                                    const __half* __restrict__ weight, float eps) {
  const int lane = threadIdx.x & 63, col = lane & 31, h = lane >> 5;
  const uint32_t wave0 = blockIdx.x * 4u + (threadIdx.x >> 6), nwaves = gridDim.x * 4u;
  __shared__ h8 wlds[RMS ? 512 : 1];                   // the norm weight, 16-byte chunk c = channels 8 c .. 8 c + 7
  if constexpr (RMS) {
    const h8 ones = {1, 1, 1, 1, 1, 1, 1, 1};
    for (int i = threadIdx.x; i < 512; i += 256) wlds[i] = weight ? *(const h8*)(weight + 8 * i) : ones;
    __syncthreads();
  }

  // sign of H64[a][b] = parity(a & b).  Within a fragment only the low slot bits vary:
  // pattern over i times a per-fragment sign.
  auto par = [](int v) { return __builtin_popcount(v) & 1; };
  h8 b1[4][2], b2[2][2][2];
#pragma unroll
  for (int nt = 0; nt < 2; ++nt) {
    const int tp = 32 * nt + col;
    h8 pat1, pat2;
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      pat1[i] = par(i & tp) ? (_Float16)-1.0f : (_Float16)1.0f;
      pat2[i] = par((8 * (i >> 2) + (i & 3)) & tp) ? (_Float16)-0.015625f : (_Float16)0.015625f;
    }
#pragma unroll
    for (int s = 0; s < 4; ++s) b1[s][nt] = par((16 * s + 8 * h) & tp) ? -pat1 : pat1;
#pragma unroll
    for (int jb = 0; jb < 2; ++jb)
#pragma unroll
      for (int s = 0; s < 2; ++s) b2[jb][s][nt] = par((32 * jb + 16 * s + 4 * h) & tp) ? -pat2 : pat2;
  }

  // The next row of this wave is requested before the current one is worked on: with two or three waves on a
  // SIMD nothing else would cover the two microseconds a row takes to arrive.
  h8 xa[2][4], xn[2][4], an[ADD ? 2 : 1][ADD ? 4 : 1];
  auto request = [&](const __half* base, uint32_t row, auto& dst) {
    const __half* xr = base + (size_t)row * 4096;
#pragma unroll
    for (int jb = 0; jb < 2; ++jb)
#pragma unroll
      for (int s = 0; s < 4; ++s) dst[jb][s] = *(const h8*)(xr + (32 * jb + col) * 64 + 16 * s + 8 * h);
  };
  if (wave0 < M) {
    request(x, wave0, xn);
    if constexpr (ADD) request(add, wave0, an);
  }
  for (uint32_t row = wave0; row < M; row += nwaves) {
#pragma unroll
    for (int jb = 0; jb < 2; ++jb)
#pragma unroll
      for (int s = 0; s < 4; ++s) {
        xa[jb][s] = xn[jb][s];
        if constexpr (ADD) {
          xa[jb][s] = __builtin_bit_cast(h8, add_h8(__builtin_bit_cast(v4i, xn[jb][s]), __builtin_bit_cast(v4i, an[jb][s])));
          *(h8*)(sum_out + (size_t)row * 4096 + (32 * jb + col) * 64 + 16 * s + 8 * h) = xa[jb][s];
        }
      }
    if (row + nwaves < M) {
      request(x, row + nwaves, xn);
      if constexpr (ADD) request(add, row + nwaves, an);
    }
    if constexpr (RMS) {
      float ss = 0.f;
#pragma unroll
      for (int jb = 0; jb < 2; ++jb)
#pragma unroll
        for (int s = 0; s < 4; ++s)
#pragma unroll
          for (int i = 0; i < 8; ++i) ss = __builtin_fmaf((float)xa[jb][s][i], (float)xa[jb][s][i], ss);
      ss = wave_sum(ss);
      const float inv = 1.0f / __builtin_sqrtf(ss / 4096.0f + eps);
#pragma unroll
      for (int jb = 0; jb < 2; ++jb)
#pragma unroll
        for (int s = 0; s < 4; ++s) {
          const h8 g = wlds[(32 * jb + col) * 8 + 2 * s + h];
          h8 y;
#pragma unroll
          for (int i = 0; i < 8; ++i)
            y[i] = (_Float16)round_here(round_here((float)xa[jb][s][i] * inv) * (float)g[i]);
          xa[jb][s] = y;
        }
    }

    v16f w[2][2];  // level-2 accumulators [t' tile][j' tile]
#pragma unroll
    for (int a = 0; a < 2; ++a)
#pragma unroll
      for (int b = 0; b < 2; ++b)
#pragma unroll
        for (int r = 0; r < 16; ++r) w[a][b][r] = 0.f;

#pragma unroll
    for (int jb = 0; jb < 2; ++jb) {
      v16f z[2];  // level 1 for blocks j = 32 jb .. 32 jb + 31
#pragma unroll
      for (int nt = 0; nt < 2; ++nt) {
#pragma unroll
        for (int r = 0; r < 16; ++r) z[nt][r] = 0.f;
#pragma unroll
        for (int s = 0; s < 4; ++s)
          z[nt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(xa[jb][s], b1[s][nt], z[nt], 0, 0, 0);
      }
      // level 2: the Z tile (lane = t', registers = j) is the A operand, rows t' = 32 mt + lane % 32
#pragma unroll
      for (int mt = 0; mt < 2; ++mt)
#pragma unroll
        for (int s = 0; s < 2; ++s) {
          v4i hi, lo;
#pragma unroll
          for (int u = 0; u < 4; ++u) {
            const float v0 = z[mt][8 * s + 2 * u], v1 = z[mt][8 * s + 2 * u + 1];
            const unsigned ph = pack_f16(v0, v1);
            hi[u] = (int)ph;
            if constexpr (SPLIT) lo[u] = (int)pack_f16(sub_half<0>(v0, ph), sub_half<1>(v1, ph));
          }
#pragma unroll
          for (int nt = 0; nt < 2; ++nt) {
            w[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(h8, hi), b2[jb][s][nt], w[mt][nt], 0, 0, 0);
            if constexpr (SPLIT)
              w[mt][nt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(h8, lo), b2[jb][s][nt], w[mt][nt], 0, 0, 0);
          }
        }
    }

    // w[mt][nt][4 g + e]: t' = 32 mt + 8 g + 4 h + e,  j' = 32 nt + col.  Round to fp16, row maximum.
    unsigned y[2][2][8];
    float mx = 0.f;
#pragma unroll
    for (int mt = 0; mt < 2; ++mt)
#pragma unroll
      for (int nt = 0; nt < 2; ++nt)
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          const float a = w[mt][nt][2 * u], b = w[mt][nt][2 * u + 1];
          y[mt][nt][u] = pack_f16(a, b);
          mx = __builtin_fmaxf(__builtin_fmaxf(__builtin_fabsf(a), __builtin_fabsf(b)), mx);
        }
    mx = (float)(_Float16)wave_max(mx);      // max |fp16(w)| = fp16(max |w|): rounding is monotonic
    if (clip < 1.0f) mx = (float)(_Float16)round_here(mx * clip);   // clip bound; values are clamped in quantise_block
    _Float16 s16 = scale_of_max(mx);
    if (s16 == (_Float16)0.0f) s16 = (_Float16)1.0f;
    const float rinv = reciprocal_of_scale(s16);
    // |y / s| <= 7.004 unless the scale is subnormal (its rounding error is then unbounded) or the
    // row was clipped: only then are the clamps needed
    const bool careful = __builtin_amdgcn_readfirstlane((float)s16 < 6.2e-5f || clip < 1.0f);
    const h2 hb = {(_Float16)mx, (_Float16)mx};
    uint8_t* qr = q + (size_t)row * 2048;
#pragma unroll
    for (int nt = 0; nt < 2; ++nt) {
      const v4i out = careful ? quantise_block<true>(y[0][nt], y[1][nt], rinv, hb)
                              : quantise_block<false>(y[0][nt], y[1][nt], rinv, hb);
      if constexpr (F6) {
        // this lane: codes 32 h .. 32 h + 31 of block j' = 32 nt + col = the piece (h, j' % 2) of 128-code block j' / 2
        const int jp = 32 * nt + col;
        const unsigned long long c0 = bf6_of_nibbles((unsigned)out[0]), c1 = bf6_of_nibbles((unsigned)out[1]),
                                 c2 = bf6_of_nibbles((unsigned)out[2]), c3 = bf6_of_nibbles((unsigned)out[3]);
        v2i* dst = (v2i*)(q + ((size_t)(jp >> 1) * M + row) * kF6BlockBytes + 48 * h + 24 * (jp & 1));
        dst[0] = v2i{(int)(unsigned)c0, (int)((unsigned)(c0 >> 32) | ((unsigned)c1 << 16))};
        dst[1] = v2i{(int)(unsigned)(c1 >> 16), (int)(unsigned)c2};
        dst[2] = v2i{(int)((unsigned)(c2 >> 32) | ((unsigned)c3 << 16)), (int)(unsigned)(c3 >> 16)};
      } else {
        *(v4i*)(qr + (32 * nt + col) * 32 + 16 * h) = out;
      }
    }
    if (lane == 0) scales[row] = __builtin_bit_cast(__half, s16);
  }
}

// -------------------------------------------------------------------------------------
// K = D * 64 with a dense +/-1 factor M across the D blocks (D = 172: had172, K = 11008;
// D = 224: had28 (x) H8, K = 14336).  D is padded to DP = 32 * DT.  The level-2 B fragments
// (M^T in MFMA register order, 1 KiB each) are built once per device into a global table and
// copied into LDS by every workgroup; workgroups are persistent, two waves per row (see the kernel).
// Level 2 takes Z rounded to fp16 (one MFMA per fragment): for these sizes the reference's own
// summation order is undefined, and the codes differ from the exactly rounded transform at a
// rate of a few 1e-4 (measured by the tests).
// -------------------------------------------------------------------------------------
#include "hadk_tables.inc"

template <int DT>
struct DenseFactor;
template <>
struct DenseFactor<6> {
  static constexpr int D = 172;
  __device__ static bool plus(int r, int c) {   // M[r][c] = had172[r][c]
    const int bit = r * 172 + c;
    return (kHad172Bits[bit >> 3] >> (7 - (bit & 7))) & 1;
  }
};
template <>
struct DenseFactor<7> {
  static constexpr int D = 224;
  __device__ static bool plus(int r, int c) {   // M = had28 (x) H8, block index = 8 a + b
    const int bit = (r >> 3) * 28 + (c >> 3);
    const bool p28 = (kHad28Bits[bit >> 3] >> (7 - (bit & 7))) & 1;
    return p28 != (bool)(__builtin_popcount((r & 7) & (c & 7)) & 1);
  }
};

// fragment (kb, s, nt), lane (col, h), slot i  ->  M[j' = 32 nt + col][j = 32 kb + 16 s + 8 (i/4) + 4 h + i%4]
template <int DT>
__global__ void build_dense_fragments(h8* table) {
  const int frag = blockIdx.x, lane = threadIdx.x, col = lane & 31, h = lane >> 5;
  const int nt = frag % DT, s = (frag / DT) & 1, kb = frag / (2 * DT);
  h8 v;
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int jp = 32 * nt + col, j = 32 * kb + 16 * s + 8 * (i >> 2) + 4 * h + (i & 3);
    constexpr int D = DenseFactor<DT>::D;
    v[i] = (jp < D && j < D) ? (DenseFactor<DT>::plus(jp, j) ? (_Float16)1.0f : (_Float16)-1.0f) : (_Float16)0.0f;
  }
  table[frag * 64 + lane] = v;
}

static __device__ h8 g_frag172[2 * 6 * 6 * 64];
static __device__ h8 g_frag224[2 * 7 * 7 * 64];

// Half of a block column: the 32 t' of one t' tile of block j' (16 codes per lane before the exchange).
// y[2 g + u]: packed fp16 pairs, t' = 8 g + 4 h + 2 u (+1) inside the tile.  Returns the 8 bytes this lane
// stores: lower half-wave t' 0..15, upper half-wave t' 16..31.
template <bool CAREFUL>
__device__ __forceinline__ v2i quantise_half_block(const unsigned (&y)[8], float rinv, h2 hb) {
  unsigned pr[2];
#pragma unroll
  for (int p = 0; p < 2; ++p) {
    unsigned t[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int g = 2 * p + u;
      unsigned y01 = y[2 * g], y23 = y[2 * g + 1];
      if constexpr (CAREFUL) {
        y01 = __builtin_bit_cast(unsigned, __builtin_elementwise_min(__builtin_elementwise_max(__builtin_bit_cast(h2, y01), -hb), hb));
        y23 = __builtin_bit_cast(unsigned, __builtin_elementwise_min(__builtin_elementwise_max(__builtin_bit_cast(h2, y23), -hb), hb));
      }
      unsigned h01 = mul_halves(y01, rinv), h23 = mul_halves(y23, rinv);
      if constexpr (CAREFUL) {
        const h2 lo8 = {(_Float16)-8.0f, (_Float16)-8.0f}, hi7 = {(_Float16)7.0f, (_Float16)7.0f};
        h01 = __builtin_bit_cast(unsigned, __builtin_elementwise_min(__builtin_elementwise_max(__builtin_bit_cast(h2, h01), lo8), hi7));
        h23 = __builtin_bit_cast(unsigned, __builtin_elementwise_min(__builtin_elementwise_max(__builtin_bit_cast(h2, h23), lo8), hi7));
      }
      t[u] = quad_nibbles(h01, h23);
    }
    pr[p] = ((t[1] << 16) + t[0] - kPairBias) ^ 0x88888888u;   // halfwords of g = 2 p, 2 p + 1
  }
  // lower lanes: sw[0] = own g 0,1 and sw[1] = the upper lanes' g 0,1; upper lanes: sw[0] = the lower lanes' g 2,3
  // and sw[1] = own g 2,3 -- in both halves a dword takes its low halfword from sw[0], its high one from sw[1]
  auto sw = __builtin_amdgcn_permlane32_swap(pr[0], pr[1], false, false);
  return v2i{(int)__builtin_amdgcn_perm(sw[1], sw[0], 0x05040100u), (int)__builtin_amdgcn_perm(sw[1], sw[0], 0x07060302u)};
}

// Two waves per row: wave 2 r + mt of a workgroup of eight works on row slot r and on the t' tile mt --
// its own half of level 1 (X is read by both waves of the pair), then all of level 2 for that tile
// (DT accumulator tiles, few enough registers for two waves per SIMD), then half of every block column
// of the epilogue.  The pair meets once per row to exchange its maxima through LDS.
//
// SPLIT (short batches, one row per workgroup): the four wave pairs share one row instead -- every pair runs
// level 1, but of level 2 and of the epilogue only the output tiles j' = slot, slot + 4, ...; the row maximum is
// the maximum over all eight waves.  Every output still accumulates its K blocks in the same order, so the
// codes are the ones the unsplit kernel produces; a batch of M rows then occupies M compute units instead of
// M / 4, each with a third to a half of the MFMA work per wave.  Here a row's latency is what counts, and all
// eight waves read the whole row: it is staged in LDS once, requested together with the factor table (direct-to-LDS
// loads, 16-byte chunks XOR-swizzled by the row so that the tile reads are free of bank conflicts), instead of
// every wave waiting for its X tiles from memory three at a time (in-kernel timestamps for one row of 14336: the
// main loop took 13 k clocks of a 23 k clock kernel, almost all of it waiting for those tiles).
//
// SILU (short batches only): the row is the SwiGLU product fp16(fp16(silu(gate)) * up) of two input rows, x = gate and
// x2 = up -- what the reference's MLP hands to the quantiser of down_proj (flh/quantized_model/modeling_llama.py:522-526).
// Both rows are staged in LDS the same way and combined in place before the first tile is read, so the product never
// goes to memory.
//
// F6 (long batches only): the codes leave in the operand format of the 6-bit matrix instruction (gemm_f6.hip) -- q is
// then the encoded matrix of M rows, K-slab-major blocks of 96 bytes per 128 codes and row.
template <int DT, bool SPLIT, bool SILU = false, bool F6 = false>
__global__ __launch_bounds__(512) void rotate_quant_mfma_dense_kernel(const __half* __restrict__ x,
                                                                       uint8_t* __restrict__ q,
                                                                       __half* __restrict__ scales,
                                                                       const h8* __restrict__ table, uint32_t M,
                                                                       float inv_norm, float clip,
                                                                       const __half* __restrict__ x2 = nullptr) {
  static_assert(!SILU || SPLIT, "the SwiGLU prologue works on the row staged in LDS");
  static_assert(!F6 || !SPLIT, "6-bit output is a prefill format");
  constexpr int D = DenseFactor<DT>::D, K = D * 64, NFRAG = 2 * DT * DT;
  extern __shared__ __align__(1024) h8 mfrag[];        // [kb][s][nt][lane], then the maxima
  float* red = (float*)(mfrag + NFRAG * 64);           // [parity][row slot][mt]
  const uint8_t* xs = (const uint8_t*)(red + 16);      // SPLIT: the row, DT * 32 rows of 128 bytes, chunk c of row j at c ^ (j & 7)
  const int lane = threadIdx.x & 63, col = lane & 31, h = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int slot = wave >> 1, mt = wave & 1;
  auto par = [](int v) { return __builtin_popcount(v) & 1; };
  // level-1 constants H64[t][t'] / 8 for t = 16 s + 8 h + i and t' = 32 mt + col
  const int tp = 32 * mt + col;
  h8 pat;
  unsigned flip[4];
#pragma unroll
  for (int i = 0; i < 8; ++i) pat[i] = par(i & tp) ? (_Float16)-0.125f : (_Float16)0.125f;
#pragma unroll
  for (int s = 0; s < 4; ++s) flip[s] = par((16 * s + 8 * h) & tp) ? 0x80008000u : 0u;
  auto b1 = [&](int s) {
    v4i v = __builtin_bit_cast(v4i, pat);
#pragma unroll
    for (int u = 0; u < 4; ++u) v[u] ^= (int)flip[s];
    return __builtin_bit_cast(h8, v);
  };
  const float c = inv_norm * 8.0f;

  constexpr int NB = 3;                                // X tiles in flight
  h8 xa[NB][4];
  auto load_tile = [&](const __half* xr, int kb, int buf) {
    const int j = 32 * kb + col;
    if constexpr (SPLIT) {
      const uint8_t* src = xs + j * 128;               // (rows past D hold a copy of the last row, zeroed below)
#pragma unroll
      for (int s = 0; s < 4; ++s) xa[buf][s] = *(const h8*)(src + (((2 * s + h) ^ (j & 7)) << 4));
    } else {
      const __half* src = xr + (j < D ? j : D - 1) * 64 + 8 * h;   // padded rows: any valid address, zeroed below
#pragma unroll
      for (int s = 0; s < 4; ++s) xa[buf][s] = *(const h8*)(src + 16 * s);
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  auto finish_tile = [&](int kb, int buf) {
    if (32 * kb + col >= D) {
#pragma unroll
      for (int s = 0; s < 4; ++s) xa[buf][s] = h8{0, 0, 0, 0, 0, 0, 0, 0};
    }
  };
  auto row_ptr = [&](uint32_t base) {
    const uint32_t r = SPLIT ? base : base + slot;
    return x + (size_t)(r < M ? r : M - 1) * K;        // rows past the end repeat the last one and store nothing
  };
  constexpr uint32_t RPW = SPLIT ? 1u : 4u;            // rows per workgroup and iteration
  const uint32_t base0 = blockIdx.x * RPW, stride = gridDim.x * RPW;
  // the first row's first tiles are requested before the factor table, so that both travel together
  if constexpr (SPLIT) {
    // the whole row into LDS: one instruction moves eight rows of X (64 chunks of 16 bytes), lane p of it the chunk
    // that belongs at slot p
    const __half* xr = row_ptr(base0);
    const unsigned xs0 = (unsigned)(size_t)xs;
    for (int i = wave; i < DT * 4; i += 8) {
      const int j = 8 * i + (lane >> 3), c = (lane & 7) ^ (j & 7);
      load_to_lds16(xr + (j < D ? j : D - 1) * 64 + c * 8, xs0 + i * 1024);
      if constexpr (SILU)                              // the up row behind the gate row, same slot order
        load_to_lds16(x2 + (xr - x) + (j < D ? j : D - 1) * 64 + c * 8, xs0 + DT * 4096 + i * 1024);
    }
  } else if (base0 < M) {
#pragma unroll
    for (int t = 0; t < NB - 1; ++t) load_tile(row_ptr(base0), t, t);
  }
  {
    const unsigned lds0 = (unsigned)(size_t)mfrag;
    const int first = (blockIdx.x * 5) % NFRAG;        // workgroups start at different fragments (L2 hot spots)
    for (int i = wave; i < NFRAG; i += 8) {
      const int f = (i + first) % NFRAG;
      load_to_lds16(table + f * 64 + lane, lds0 + f * 1024);
    }
    wait_vmcnt<0>();
    __syncthreads();
  }
  if constexpr (SILU) {
    h8* g8 = (h8*)xs;
    const h8* u8 = (const h8*)(xs + DT * 4096);
    for (int i = threadIdx.x; i < DT * 256; i += 512) {
      const h8 g = g8[i], u = u8[i];
      h8 o;
#pragma unroll
      for (int e = 0; e < 8; ++e) o[e] = silu_mul_f16(g[e], u[e]);
      g8[i] = o;
    }
    __syncthreads();
  }
  if constexpr (SPLIT) {
#pragma unroll
    for (int t = 0; t < NB - 1; ++t) load_tile(nullptr, t, t);
  }

  // The wave pairs of row slots 2 and 3 run one phase behind those of slots 0 and 1: every iteration has two
  // workgroup barriers (after the MFMA phase, where a pair exchanges its maxima, and after the quantising
  // phase), and the late pairs pass one extra barrier before the loop, the early pairs one after it.  While
  // one half of the waves issues MFMAs the other half quantises and stores; each SIMD hosts one wave of each
  // half (waves w and w + 4), so the matrix pipe and the vector ALU of a SIMD are busy at the same time.
  const bool late = !SPLIT && slot >= 2;
  if (late) barrier_no_fence();
  int parity = 0;
  for (uint32_t base = base0; base < M; base += stride, parity ^= 1) {
    const uint32_t row = SPLIT ? base : base + slot;
    const bool valid = row < M;
    const __half* xr = row_ptr(base);
    v16f w[DT];                                        // level-2 accumulators of this t' tile, [j' tile]
#pragma unroll
    for (int b = 0; b < DT; ++b)
#pragma unroll
      for (int r = 0; r < 16; ++r) w[b][r] = 0.f;
    constexpr int AHEAD = DT <= 6 ? 7 : 3, RING = AHEAD + 1;   // factor fragments travel a few fragments ahead
    h8 fr[RING];
    auto fetch = [&](int f) { fr[f % RING] = mfrag[f * 64 + lane]; };
#pragma unroll
    for (int f = 0; f < AHEAD; ++f) fetch(f);
#pragma unroll
    for (int kb = 0; kb < DT; ++kb) {
      if (kb + NB - 1 < DT) load_tile(xr, kb + NB - 1, (kb + NB - 1) % NB);
      finish_tile(kb, kb % NB);
      v16f z;
#pragma unroll
      for (int r = 0; r < 16; ++r) z[r] = 0.f;
#pragma unroll
      for (int s = 0; s < 4; ++s) z = __builtin_amdgcn_mfma_f32_32x32x16_f16(xa[kb % NB][s], b1(s), z, 0, 0, 0);
      v4i a[2];
#pragma unroll
      for (int s = 0; s < 2; ++s)
#pragma unroll
        for (int u = 0; u < 4; ++u) a[s][u] = (int)pack_f16(z[8 * s + 2 * u], z[8 * s + 2 * u + 1]);
#pragma unroll
      for (int s = 0; s < 2; ++s)
#pragma unroll
        for (int nt = 0; nt < DT; ++nt) {
          const int f = (kb * 2 + s) * DT + nt;
          if (f + AHEAD < NFRAG) fetch(f + AHEAD);
          if (!SPLIT || (nt & 3) == slot)
            w[nt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(h8, a[s]), fr[f % RING], w[nt], 0, 0, 0);
        }
    }
    if constexpr (!SPLIT) {
      if (base + stride < M) {                         // the next row's first tiles travel during the epilogue
#pragma unroll
        for (int t = 0; t < NB - 1; ++t) load_tile(row_ptr(base + stride), t, t);
      }
    }

    // w[nt][4 g + e]: t' = 32 mt + 8 g + 4 h + e,  j' = 32 nt + col
    float mx = 0.f;
#pragma unroll
    for (int nt = 0; nt < DT; ++nt)
#pragma unroll
      for (int u = 0; u < 8; ++u)
        mx = __builtin_fmaxf(__builtin_fmaxf(__builtin_fabsf(w[nt][2 * u]), __builtin_fabsf(w[nt][2 * u + 1])), mx);
    mx = wave_max(mx);
    if (lane == 0) red[(parity * 4 + slot) * 2 + mt] = mx;
    __syncthreads();                                   // the pair's maxima (slots alternate between rows)
    if constexpr (SPLIT) {
      mx = 0.f;
#pragma unroll
      for (int i = 0; i < 8; ++i) mx = __builtin_fmaxf(mx, red[parity * 8 + i]);
    } else {
      mx = __builtin_fmaxf(red[(parity * 4 + slot) * 2], red[(parity * 4 + slot) * 2 + 1]);
    }
    // max |fp16(w c)| = fp16(max|w| c): the product and its single rounding are monotonic
    mx = (float)__builtin_bit_cast(h2, scale_pack_f16(mx, 0.f, c))[0];
    if (clip < 1.0f) mx = (float)(_Float16)round_here(mx * clip);   // clip bound; values are clamped below
    _Float16 s16 = scale_of_max(mx);
    if (s16 == (_Float16)0.0f) s16 = (_Float16)1.0f;
    const float rinv = reciprocal_of_scale(s16);
    const bool careful = __builtin_amdgcn_readfirstlane((float)s16 < 6.2e-5f || clip < 1.0f);
    const h2 hb = {(_Float16)mx, (_Float16)mx};

    // A row slot past the end works on a copy of the last row and stores the same bytes as that row's
    // own pair: no predicate, so that all block columns form one straight run of code to schedule.
    uint8_t* qr = q + (size_t)(valid ? row : M - 1) * (K / 2) + mt * 16 + h * 8;
    auto emit = [&](auto careful_tag) {
#pragma unroll
      for (int nt = 0; nt < DT; ++nt) {
        if (SPLIT && (nt & 3) != slot) continue;
        unsigned y[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) y[u] = scale_pack_f16(w[nt][2 * u], w[nt][2 * u + 1], c);
        const v2i out = quantise_half_block<decltype(careful_tag)::value>(y, rinv, hb);
        if constexpr (F6) {
          // this lane: codes 32 mt + 16 h + 0 .. 15 of block j' = 32 nt + col, i.e. 12 bytes at byte 12 h of the piece
          // (half mt, sub-block j' % 2) of 128-code block j' / 2
          const int jp = 32 * nt + col;
          const unsigned long long lo = bf6_of_nibbles((unsigned)out[0]), hi = bf6_of_nibbles((unsigned)out[1]);
          unsigned* dst = (unsigned*)(q + ((size_t)(jp >> 1) * M + (valid ? row : M - 1)) * kF6BlockBytes + 48 * mt +
                                      24 * (jp & 1) + 12 * h);
          if (32 * nt + 31 < D || jp < D) {
            dst[0] = (unsigned)lo;
            dst[1] = (unsigned)(lo >> 32) | ((unsigned)hi << 16);
            dst[2] = (unsigned)(hi >> 16);
          }
        } else {
          if (32 * nt + 31 < D || 32 * nt + col < D) *(v2i*)(qr + (32 * nt + col) * 32) = out;
        }
      }
    };
    if (careful) emit(std::true_type{});
    else emit(std::false_type{});
    if (valid && lane == 0 && mt == 0 && (!SPLIT || slot == 0)) scales[row] = __builtin_bit_cast(__half, s16);
    barrier_no_fence();                                // end of the quantising phase (see above the loop)
    if constexpr (SPLIT) break;                        // one row per workgroup: only that row was staged
  }
  if (!late) barrier_no_fence();
}

// The factor table of one size: built on first use on a device (or by flh_init with that device current) on the
// legacy default stream and waited for, so that later launches on any stream find it complete.  Every device holds
// its own copy of the array at its own address.  Not to be first reached under stream capture -- call flh_init()
// before capturing.
template <int DT>
int dense_table(const h8** out) {
  static std::atomic<const h8*> table[kMaxDevices];
  int dev = 0;
  if (int rc = current_device(&dev, "rotate_quant")) return rc;
  const h8* t = table[dev].load(std::memory_order_acquire);
  if (!t) {
    static std::mutex once;
    std::lock_guard<std::mutex> lock(once);
    t = table[dev].load(std::memory_order_relaxed);
    if (!t) {
      constexpr int NFRAG = 2 * DT * DT;
      void* sym = nullptr;
      const hipError_t e = DT == 6 ? hipGetSymbolAddress(&sym, HIP_SYMBOL(g_frag172)) : hipGetSymbolAddress(&sym, HIP_SYMBOL(g_frag224));
      if (e != hipSuccess) return fail(FLH_ELAUNCH, "rotate_quant: cannot locate the factor table: %s", hipGetErrorString(e));
      hipLaunchKernelGGL((build_dense_fragments<DT>), dim3(NFRAG), dim3(64), 0, nullptr, (h8*)sym);
      if (int rc = check_launch("build_dense_fragments")) return rc;
      if (hipStreamSynchronize(nullptr) != hipSuccess) return fail(FLH_ELAUNCH, "rotate_quant: building the factor table failed");
      t = (const h8*)sym;
      table[dev].store(t, std::memory_order_release);
    }
  }
  *out = t;
  return FLH_OK;
}

// the SwiGLU product of two rows in front of the rotation (short batches: one row per workgroup)
template <int DT>
int launch_dense_silu(const __half* gate, const __half* up, uint8_t* q, __half* scales, uint32_t M, hipStream_t stream) {
  constexpr int NFRAG = 2 * DT * DT;
  constexpr int K = DenseFactor<DT>::D * 64;
  const h8* table = nullptr;
  if (int rc = dense_table<DT>(&table)) return rc;
  const size_t smem = (size_t)NFRAG * 1024 + 64 + 2 * (size_t)DT * 4096;   // factor fragments, maxima, gate row, up row
  auto kern = rotate_quant_mfma_dense_kernel<DT, true, true>;
  static LdsGrant grant;
  if (int rc = reserve_lds((const void*)kern, smem, grant, "silu_mul_rotate_quant")) return rc;
  hipLaunchKernelGGL(kern, dim3(M), dim3(512), smem, stream, gate, q, scales, table, M, 1.0f / sqrtf((float)K), 1.0f, up);
  return check_launch("silu_mul_rotate_quant");
}

template <int DT>
int launch_dense(const __half* x, uint8_t* q, __half* scales, uint32_t M, float clip, hipStream_t stream, bool f6 = false) {
  constexpr int NFRAG = 2 * DT * DT;
  constexpr int K = DenseFactor<DT>::D * 64;
  const h8* table = nullptr;
  if (int rc = dense_table<DT>(&table)) return rc;
  // short batches take one row per workgroup (SPLIT: exactly one -- the grid is M -- with the row staged in LDS),
  // long ones four; 6-bit output (a prefill format) always takes the long-batch kernel
  const bool split = M <= 256 && !f6;
  const size_t smem = (size_t)NFRAG * 1024 + 64 + (split ? (size_t)DT * 4096 : 0);   // factor fragments, the pairs' maxima, the row
  auto kern = f6 ? rotate_quant_mfma_dense_kernel<DT, false, false, true>
                 : split ? rotate_quant_mfma_dense_kernel<DT, true> : rotate_quant_mfma_dense_kernel<DT, false>;
  constexpr int kThreadsDense = 512;
  static LdsGrant grants[3];                           // one per kernel variant
  if (int rc = reserve_lds((const void*)kern, smem, grants[f6 ? 2 : split], "rotate_quant")) return rc;
  const unsigned blocks = split ? M : ((M + 3) / 4 < 256u ? (M + 3) / 4 : 256u);
  hipLaunchKernelGGL(kern, dim3(blocks), dim3(kThreadsDense), smem, stream, x, q, scales, table, M,
                     1.0f / sqrtf((float)K), clip, (const __half*)nullptr);
  return check_launch("rotate_quant_mfma_dense");
}

}  // namespace

bool rotate_quant_mfma_supports(uint32_t K) { return K == 4096 || K == 11008 || K == 14336; }

// one-time set-up of the matrix-core kernels (called by flh_init)
int rotate_quant_mfma_init() {
  const h8* t = nullptr;
  if (int rc = dense_table<6>(&t)) return rc;
  return dense_table<7>(&t);
}

// launcher used by flh_silu_mul_rotate_quant_i4 (fwht_quant.hip): K = 11008 / 14336, at most kSiluRotateMaxRows rows
int launch_silu_mul_rotate_quant_mfma(const __half* gate, const __half* up, uint8_t* q, __half* scales, uint32_t M,
                                      uint32_t K, hipStream_t stream) {
  if (K == 11008) return launch_dense_silu<6>(gate, up, q, scales, M, stream);
  if (K == 14336) return launch_dense_silu<7>(gate, up, q, scales, M, stream);
  return fail(FLH_EINVAL, "silu_mul_rotate_quant: K = %u is not supported (11008 or 14336)", K);
}

// launcher used by flh_rotate_quant_f6 (fwht_quant.hip): the dense-factor sizes with 6-bit output
int launch_rotate_quant_mfma_f6(const __half* x, uint8_t* encoded, __half* scales, uint32_t M, uint32_t K, float clip,
                                hipStream_t stream) {
  if (K == 11008) return launch_dense<6>(x, encoded, scales, M, clip, stream, true);
  if (K == 14336) return launch_dense<7>(x, encoded, scales, M, clip, stream, true);
  return fail(FLH_EINVAL, "rotate_quant_f6 (matrix-core mode): K = %u is not supported", K);
}

int launch_rotate_quant_mfma4096(const __half* x, const __half* add, __half* sum_out, bool rms, const __half* weight,
                                 float eps, uint8_t* q, __half* scales, uint32_t M, float clip, bool f6,
                                 hipStream_t stream);

// launcher used by flh_rotate_quant_i4 (fwht_quant.hip)
int launch_rotate_quant_mfma(const __half* x, uint8_t* q, __half* scales, uint32_t M, uint32_t K, float clip,
                             hipStream_t stream) {
  if (K == 11008) return launch_dense<6>(x, q, scales, M, clip, stream);
  if (K == 14336) return launch_dense<7>(x, q, scales, M, clip, stream);
  if (K != 4096) return fail(FLH_EINVAL, "rotate_quant (matrix-core mode): K = %u is not supported", K);
  // persistent waves (two workgroups of four per compute unit are resident): rows beyond the first are prefetched
  return launch_rotate_quant_mfma4096(x, nullptr, nullptr, false, nullptr, 0.f, q, scales, M, clip, false, stream);
}

// K = 4096 on the matrix cores with the prologues / output format of the float32-butterfly kernels (used by the
// entry points of fwht_quant.hip for FLH_HAD_MFMA): residual addition (add, sum_out: both or neither; with rms only),
// RMSNorm (weight may be null), 6-bit operand output
int launch_rotate_quant_mfma4096(const __half* x, const __half* add, __half* sum_out, bool rms, const __half* weight,
                                 float eps, uint8_t* q, __half* scales, uint32_t M, float clip, bool f6,
                                 hipStream_t stream) {
  const unsigned blocks = (M + 3) / 4 < 512u ? (M + 3) / 4 : 512u;
  auto go = [&](auto kern) {
    hipLaunchKernelGGL(kern, dim3(blocks), dim3(256), 0, stream, x, q, scales, M, clip, add, sum_out, weight, eps);
    return check_launch("rotate_quant_mfma");
  };
  if (add && !rms) return fail(FLH_EINVAL, "rotate_quant (matrix-core mode): the residual addition comes with RMSNorm");
  if (!rms) return f6 ? go(rotate_quant_mfma4096_kernel<true, false, false, true>) : go(rotate_quant_mfma4096_kernel<true>);
  if (!add) return f6 ? go(rotate_quant_mfma4096_kernel<true, true, false, true>) : go(rotate_quant_mfma4096_kernel<true, true>);
  return f6 ? go(rotate_quant_mfma4096_kernel<true, true, true, true>) : go(rotate_quant_mfma4096_kernel<true, true, true>);
}

}  // namespace flh
