// int4 x int4 GEMM + dequant for a handful of tokens (decode, M <= 64): the weights are
// streamed from HBM exactly once and the contraction is split over K inside a workgroup.
//
// Same arithmetic as gemm_i4.hip (codes x 16 as int8 on the matrix cores, exact int32 sums,
// identical epilogue roundings); reference: flh/kernels/gemm_and_dequant_i4.cu:315-508.
//
// One workgroup of 8 waves owns 16 output channels and every token.  A wave takes every 8th
// "double step" of K (256 codes = one 128-byte line of each of the 16 weight rows): lane l
// loads 2 x 16 packed bytes of weight row l % 16 at chunk l / 16, the same of the activation
// row l % 16 of each 16-token tile, and issues v_mfma_i32_16x16x64_i8 on the low and the high
// nibbles.  With 256 workgroups x 8 waves x two double steps in flight the whole of a
// 4096 x 4096 weight matrix is requested at once, which is what a latency-bound stream needs.
// Partial sums meet in LDS:
//   * one scale per row: the eight waves' int32 tiles are added and dequantised;
//   * scale groups of 128: every group's int32 tile is kept in LDS and the fp32 result is built
//     by one fused multiply-add per group in ascending order, exactly as the prefill kernel does.
#include <atomic>
#include "gemm_i4.h"
#include "rotate_row.h"

namespace flh {
namespace {

constexpr int kWaves = 8;
constexpr int kRotateGemmMaxTokens = 4;    // tokens of the GEMM that quantises its own activations
constexpr int kGroupMaxKT = 128;   // groups of 128 codes that fit the LDS tile store (K <= 16384)

__device__ __forceinline__ void unpack_lo_hi(const v4i w, v4i& lo, v4i& hi) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    lo[i] = (w[i] << 4) & (int)0xF0F0F0F0;
    hi[i] = w[i] & (int)0xF0F0F0F0;
  }
}

// The weight matrix a workgroup's block of 16 output channels belongs to (several may share the activations in
// one launch; segment starts are counted in blocks of 16 here) and the block's first channel inside it.
struct DecodeWeights {
  const uint8_t* B;
  const __half* Bs;
  void* D;
  int N, n0;
};
__device__ __forceinline__ DecodeWeights decode_weights(const GemmArgs& p, int block) {
  DecodeWeights w{p.B, p.Bs, p.D, p.N, block * 16};
  for (int s = 1; s < p.n_seg; ++s)
    if (block >= p.seg_tile0[s]) w = DecodeWeights{p.seg_B[s], p.seg_Bs[s], p.seg_D[s], p.seg_N[s], (block - p.seg_tile0[s]) * 16};
  return w;
}
// host side: segment starts in blocks of 16 channels; returns the number of blocks of the launch
int decode_blocks(GemmArgs& a) {
  int blocks = (a.N + 15) / 16;
  for (int s = 1; s < a.n_seg; ++s) {
    a.seg_tile0[s] = blocks;
    blocks += (a.seg_N[s] + 15) / 16;
  }
  return blocks;
}

// one fp16 output; with a residual (single weight matrix) the stored value is fp16(R + value)
__device__ __forceinline__ void store_f16(const GemmArgs& p, const DecodeWeights& w, int gm, int gn, _Float16 v) {
  const size_t at = (size_t)gm * w.N + gn;
  if (p.R) v = v + ((const _Float16*)p.R)[at];
  ((_Float16*)w.D)[at] = v;
}

// Partial sums in LDS -> outputs.  Lane l of a tile holds token l % 16 and channels 4 (l / 16) + i, i = 0..3.
// a_scales: one scale per token (row-scale epilogue); sA / sB: the group tables (group epilogue).
template <int MT, int EPI>
__device__ __forceinline__ void decode_finish(const GemmArgs& p, const DecodeWeights& w, const int* red, const float* sA,
                                              const float* sB, const __half* a_scales, int tid) {
  const int KT = p.K >> 7;
  for (int idx = tid; idx < MT * 256; idx += kWaves * 64) {
    const int mt = idx >> 8, m = (idx >> 4) & 15, n = idx & 15;
    const int pos = (((n >> 2) * 16 + m) << 2) + (n & 3);
    const int gm = mt * 16 + m, gn = w.n0 + n;
    if (gm >= p.M || gn >= w.N) continue;
    if constexpr (EPI == kGroupScale) {
      float out = 0.f;
      if (p.a_cols == 1 && p.b_cols > 1) {           // one scale per token: applied once, after the groups
        for (int g = 0; g < KT; ++g)
          out = __builtin_fmaf((float)(red[(g * MT + mt) * 256 + pos] >> 8), sB[g * 16 + n], out);
        out = round_here(out) * sA[m];
      } else {
        for (int g = 0; g < KT; ++g)
          out = __builtin_fmaf((float)(red[(g * MT + mt) * 256 + pos] >> 8), sA[g * 16 + m] * sB[g * 16 + n], out);
      }
      store_f16(p, w, gm, gn, (_Float16)round_here(out));
    } else {
      int sum = 0;
#pragma unroll
      for (int w = 0; w < kWaves; ++w) sum += red[(w * MT + mt) * 256 + pos];
      if constexpr (EPI == kInt32) {
        ((int32_t*)w.D)[(size_t)gm * w.N + gn] = sum >> 8;
      } else {
        // sum = 256 * (exact contraction); the weight scale carries the matching exact 2^-8
        const float sa = __half2float(a_scales[gm]), sb = __half2float(w.Bs[gn]) * 0.00390625f;
        store_f16(p, w, gm, gn, (_Float16)round_here((float)sum * (sa * sb)));
      }
    }
  }
}

template <int MT, int EPI>
__global__ __launch_bounds__(kWaves * 64) void gemm_i4_decode_kernel(const GemmArgs p) {
  extern __shared__ __align__(16) int red[];   // int32 tiles: [wave | group][MT][64 lanes][4]; then the scale tables
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15, c = lane >> 4;
  const DecodeWeights w = decode_weights(p, blockIdx.x);
  const int n0 = w.n0;
  const int Kb = p.K >> 1, KT = p.K >> 7, ND = (KT + 1) >> 1;

  const uint8_t* bptr = w.B + (size_t)min(n0 + r, w.N - 1) * Kb + c * 16;
  const uint8_t* aptr[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) aptr[mt] = p.A + (size_t)min(mt * 16 + r, p.M - 1) * Kb + c * 16;

  float* sA = (float*)(red + KT * MT * 256);    // group mode: scales as float, [g][16]
  float* sB = sA + KT * 16;
  if constexpr (EPI == kGroupScale) {
    for (int i = tid; i < 16 * KT; i += kWaves * 64) {
      const int row = i / KT, g = i - row * KT;
      sA[g * 16 + row] = row < p.M ? __half2float(p.As[(size_t)row * p.a_cols + (p.a_cols > 1 ? g : 0)]) : 0.f;
      sB[g * 16 + row] = n0 + row < w.N ? __half2float(w.Bs[(size_t)(n0 + row) * p.b_cols + (p.b_cols > 1 ? g : 0)]) : 0.f;
    }
  }

  v4i acc[MT];
#pragma unroll
  for (int mt = 0; mt < MT; ++mt) acc[mt] = v4i{0, 0, 0, 0};

  auto load = [&](int ds, v4i (&b)[2], v4i (&a)[MT][2]) {
    const size_t off = (size_t)ds * 128;
    const bool second = 2 * ds + 1 < KT;           // K = 128 * odd: the last double step is half empty
    b[0] = *(const v4i*)(bptr + off);
    b[1] = second ? *(const v4i*)(bptr + off + 64) : v4i{0, 0, 0, 0};
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) {
      a[mt][0] = *(const v4i*)(aptr[mt] + off);
      a[mt][1] = second ? *(const v4i*)(aptr[mt] + off + 64) : v4i{0, 0, 0, 0};
    }
  };
  auto compute = [&](int ds, const v4i (&b)[2], const v4i (&a)[MT][2]) {
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      v4i blo, bhi;
      unpack_lo_hi(b[half], blo, bhi);
#pragma unroll
      for (int mt = 0; mt < MT; ++mt) {
        v4i alo, ahi;
        unpack_lo_hi(a[mt][half], alo, ahi);
        acc[mt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(blo, alo, acc[mt], 0, 0, 0);
        acc[mt] = __builtin_amdgcn_mfma_i32_16x16x64_i8(bhi, ahi, acc[mt], 0, 0, 0);
        if constexpr (EPI == kGroupScale) {
          const int g = 2 * ds + half;
          if (g < KT) *(v4i*)(red + ((g * MT + mt) * 64 + lane) * 4) = acc[mt];
          acc[mt] = v4i{0, 0, 0, 0};
        }
      }
    }
  };

  // two double steps in flight per wave
  v4i b0[2], b1[2], a0[MT][2], a1[MT][2];
  int ds = wave;
  if (ds < ND) load(ds, b0, a0);
  for (; ds < ND; ds += 2 * kWaves) {
    const bool more = ds + kWaves < ND;
    if (more) load(ds + kWaves, b1, a1);
    compute(ds, b0, a0);
    if (more) {
      if (ds + 2 * kWaves < ND) load(ds + 2 * kWaves, b0, a0);
      compute(ds + kWaves, b1, a1);
    }
  }
  if constexpr (EPI != kGroupScale) {
#pragma unroll
    for (int mt = 0; mt < MT; ++mt) *(v4i*)(red + ((wave * MT + mt) * 64 + lane) * 4) = acc[mt];
  }
  __syncthreads();

  decode_finish<MT, EPI>(p, w, red, sA, sB, p.As, tid);
}

template <int MT, int EPI>
int launch_decode(const GemmArgs& a, hipStream_t stream) {
  const int KT = a.K >> 7;
  const size_t smem = EPI == kGroupScale ? (size_t)KT * MT * 1024 + (size_t)KT * 128 : (size_t)kWaves * MT * 1024;
  auto kern = gemm_i4_decode_kernel<MT, EPI>;
  if constexpr (EPI == kGroupScale) {
    static LdsGrant grant;                             // per instantiation; sized for the longest rows it takes
    if (int rc = reserve_lds((const void*)kern, (size_t)kGroupMaxKT * MT * 1024 + (size_t)kGroupMaxKT * 128, grant, "gemm (decode)"))
      return rc;
  }
  GemmArgs g = a;
  const int blocks = decode_blocks(g);
  hipLaunchKernelGGL(kern, dim3(blocks), dim3(kWaves * 64), smem, stream, g);
  return check_launch("gemm_i4_decode");
}

// The decode GEMM with the activation quantiser inside, for one to four tokens of K = 4096: every workgroup
// requests its share of the weights, then rotates, quantises and packs the tokens into LDS itself -- all eight
// waves on each row, rotate_quant_row_8waves: the additions of the stand-alone kernel in the same order, so the
// codes and scales are the same bits -- while the weights are still on their way from HBM.  The rotation is
// repeated by every workgroup (about a microsecond per token); what it saves is a whole launch in front of the
// GEMM, which is worth more than that for one or two tokens and outputs up to about 12 K channels.
//
// NORM / ADD: the tokens are RMS-normalised first (NORM), after a residual addition x + add (ADD) -- the prologues of
// flh_rmsnorm_rotate_quant_i4 / flh_add_rmsnorm_rotate_quant_i4 with the same roundings, so again the same bits as the
// separate launches.  Every workgroup forms the sum for itself; workgroup 0 stores it (the new residual stream).
struct DecodePrologue {
  const __half* rms_weight;   // NORM: null = no weight
  float eps;
  const __half* add;          // ADD
  __half* sum_out;            // ADD
};

template <int EPI, bool NORM = false, bool ADD = false>
__global__ __launch_bounds__(kWaves * 64) void rotate_gemm_i4_decode_kernel(const __half* __restrict__ x,
                                                                            const GemmArgs p, float norm,
                                                                            const DecodePrologue pro) {
  constexpr int K = 4096, Kb = K / 2, KT = K / 128, ND = KT / 2, NDW = ND / kWaves;
  constexpr int ROW = Kb + 16;                 // code rows 16 bytes apart in the banks
  constexpr int TILES = EPI == kGroupScale ? KT : 2 * kWaves;   // at least the 16 KB the rotation stages in
  extern __shared__ __align__(16) int red[];   // int32 tiles [wave | group][64 lanes][4], sB [KT][16], sA [16], codes, scales
  float* sB = (float*)(red + TILES * 256);
  float* sA = sB + KT * 16;
  uint8_t* codes = (uint8_t*)(sA + 16);
  __half* tok = (__half*)(codes + kRotateGemmMaxTokens * ROW);
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int r = lane & 15, c = lane >> 4;
  const DecodeWeights w = decode_weights(p, blockIdx.x);
  const int n0 = w.n0;

  // this wave's weights first: all of them are in flight while the tokens are rotated
  const uint8_t* bptr = w.B + (size_t)min(n0 + r, w.N - 1) * Kb + c * 16;
  v4i b[NDW][2];
#pragma unroll
  for (int i = 0; i < NDW; ++i) {
    const int ds = wave + i * kWaves;
    b[i][0] = *(const v4i*)(bptr + (size_t)ds * 128);
    b[i][1] = *(const v4i*)(bptr + (size_t)ds * 128 + 64);
  }
  if constexpr (EPI == kGroupScale) {
    for (int i = tid; i < 16 * KT; i += kWaves * 64) {
      const int row = i / KT, g = i - row * KT;
      sB[g * 16 + row] = n0 + row < w.N ? __half2float(w.Bs[(size_t)(n0 + row) * KT + g]) : 0.f;
    }
  }
  for (int row = 0; row < p.M; ++row) {
    if constexpr (NORM || ADD)
      rotate_quant_row_8waves<NORM, ADD>(x + (size_t)row * K, (float*)red, sA, codes + row * ROW, tok + row, norm, wave,
                                         pro.rms_weight, pro.eps, ADD ? pro.add + (size_t)row * K : nullptr,
                                         ADD && blockIdx.x == 0 ? pro.sum_out + (size_t)row * K : nullptr);
    else
      rotate_quant_row_8waves(x + (size_t)row * K, (float*)red, sA, codes + row * ROW, tok + row, norm, wave);
  }
  __syncthreads();
  if (tid < 16) sA[tid] = tid < p.M ? __half2float(tok[tid]) : 0.f;

  v4i acc = {0, 0, 0, 0};
  const uint8_t* arow = codes + min(r, p.M - 1) * ROW + c * 16;
#pragma unroll
  for (int i = 0; i < NDW; ++i) {
    const int ds = wave + i * kWaves;
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      v4i blo, bhi, alo, ahi;
      unpack_lo_hi(b[i][half], blo, bhi);
      unpack_lo_hi(*(const v4i*)(arow + ds * 128 + half * 64), alo, ahi);
      acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(blo, alo, acc, 0, 0, 0);
      acc = __builtin_amdgcn_mfma_i32_16x16x64_i8(bhi, ahi, acc, 0, 0, 0);
      if constexpr (EPI == kGroupScale) {
        *(v4i*)(red + ((2 * ds + half) * 64 + lane) * 4) = acc;
        acc = v4i{0, 0, 0, 0};
      }
    }
  }
  if constexpr (EPI != kGroupScale) *(v4i*)(red + (wave * 64 + lane) * 4) = acc;
  __syncthreads();
  decode_finish<1, EPI>(p, w, red, sA, sB, tok, tid);
}

template <int EPI>
int launch_rotate_decode(const __half* x, const GemmArgs& a, hipStream_t stream, const DecodePrologue* pro = nullptr) {
  constexpr int K = 4096, KT = K / 128;
  constexpr size_t smem = (size_t)(EPI == kGroupScale ? KT : 2 * kWaves) * 1024 + KT * 64 + 64 +
                          kRotateGemmMaxTokens * (K / 2 + 16) + 32;
  static_assert(smem <= 64 * 1024, "fits the default dynamic LDS limit");
  GemmArgs g = a;
  const int blocks = decode_blocks(g);
  const dim3 grid(blocks), block(kWaves * 64);
  const DecodePrologue none{nullptr, 0.f, nullptr, nullptr};
  if (!pro)
    hipLaunchKernelGGL((rotate_gemm_i4_decode_kernel<EPI>), grid, block, smem, stream, x, g, 1.0f / 64.0f, none);
  else if (pro->add)
    hipLaunchKernelGGL((rotate_gemm_i4_decode_kernel<EPI, true, true>), grid, block, smem, stream, x, g, 1.0f / 64.0f, *pro);
  else
    hipLaunchKernelGGL((rotate_gemm_i4_decode_kernel<EPI, true, false>), grid, block, smem, stream, x, g, 1.0f / 64.0f, *pro);
  return check_launch("rotate_gemm_i4_decode");
}

}  // namespace

bool gemm_decode_supports(const GemmArgs& a, int epi, int group) {
  if (a.M <= 0 || a.M > kDecodeMaxM) return false;
  if (epi == kGroupScale) return group == 128 && a.M <= 16 && (a.K >> 7) <= kGroupMaxKT;
  return true;
}

int gemm_decode_dispatch(const GemmArgs& a, int epi, hipStream_t stream) {
  const int mt = (a.M + 15) / 16;
  if (epi == kGroupScale) return launch_decode<1, kGroupScale>(a, stream);
  if (epi == kInt32) {
    if (mt == 1) return launch_decode<1, kInt32>(a, stream);
    if (mt == 2) return launch_decode<2, kInt32>(a, stream);
    return launch_decode<4, kInt32>(a, stream);
  }
  if (mt == 1) return launch_decode<1, kRowScale>(a, stream);
  if (mt == 2) return launch_decode<2, kRowScale>(a, stream);
  return launch_decode<4, kRowScale>(a, stream);
}

}  // namespace flh

namespace {
int rotate_gemm_checked(const char* who, const flh_half* x, const flh::DecodePrologue* pro, int count,
                        const uint8_t* const* B, const flh_half* const* b_scale, flh_half* const* D, const size_t* N,
                        size_t M, size_t K, int b_cols, void* stream) {
  using namespace flh;
  if (count < 1 || count > kMaxGemmSegments)
    return fail(FLH_EINVAL, "%s: count = %d, must be 1 .. %d", who, count, kMaxGemmSegments);
  if (!B || !b_scale || !D || !N) return fail(FLH_EINVAL, "%s: null array", who);
  if (M == 0) return FLH_OK;
  if (!x) return fail(FLH_EINVAL, "%s: null pointer", who);
  if (misaligned16(x)) return fail(FLH_EINVAL, "%s: x must be 16-byte aligned", who);
  if (M > (size_t)kRotateGemmMaxTokens)
    return fail(FLH_EINVAL, "%s: M = %zu, at most %d tokens (more tokens quantise once, in their own launch)", who, M,
                kRotateGemmMaxTokens);
  if (K != 4096) return fail(FLH_EINVAL, "%s: K = %zu is not supported (4096)", who, K);
  if (b_cols != 1 && (size_t)b_cols != K / 128)
    return fail(FLH_EINVAL, "%s: weight scale columns (%d) must be 1 or K / 128 = %zu", who, b_cols, K / 128);
  size_t n_all = 0;
  for (int s = 0; s < count; ++s) {
    if (N[s] == 0) return fail(FLH_EINVAL, "%s: N[%d] = 0", who, s);
    if (!B[s] || !b_scale[s] || !D[s]) return fail(FLH_EINVAL, "%s: null pointer", who);
    if (misaligned16(B[s], D[s])) return fail(FLH_EINVAL, "%s: B and D must be 16-byte aligned", who);
    n_all += N[s];
  }
  if (n_all > (1u << 30)) return fail(FLH_EINVAL, "%s: N too large", who);
  GemmArgs g{nullptr, B[0], nullptr, (const __half*)b_scale[0], D[0], (int)M, (int)N[0], (int)K, 1, b_cols, 0, 0, 0};
  g.n_seg = count;
  for (int s = 1; s < count; ++s) {
    g.seg_B[s] = B[s];
    g.seg_Bs[s] = (const __half*)b_scale[s];
    g.seg_D[s] = D[s];
    g.seg_N[s] = (int)N[s];
  }
  return b_cols == 1 ? launch_rotate_decode<kRowScale>((const __half*)x, g, (hipStream_t)stream, pro)
                     : launch_rotate_decode<kGroupScale>((const __half*)x, g, (hipStream_t)stream, pro);
}
}  // namespace

extern "C" int flh_rotate_quant_gemm_i4_o16_multi(const flh_half* x, int count, const uint8_t* const* B,
                                                  const flh_half* const* b_scale, flh_half* const* D, const size_t* N,
                                                  size_t M, size_t K, int b_cols, void* stream) {
  return rotate_gemm_checked("rotate_quant_gemm", x, nullptr, count, B, b_scale, D, N, M, K, b_cols, stream);
}

extern "C" int flh_rmsnorm_rotate_quant_gemm_i4_o16_multi(const flh_half* x, const flh_half* add, flh_half* sum_out,
                                                          const flh_half* weight, float eps, int count,
                                                          const uint8_t* const* B, const flh_half* const* b_scale,
                                                          flh_half* const* D, const size_t* N, size_t M, size_t K,
                                                          int b_cols, void* stream) {
  using namespace flh;
  const char* who = "rmsnorm_rotate_quant_gemm";
  if (!(eps >= 0.f)) return fail(FLH_EINVAL, "%s: eps must not be negative", who);
  if ((add == nullptr) != (sum_out == nullptr)) return fail(FLH_EINVAL, "%s: add and sum_out come together or not at all", who);
  if (add && (misaligned16(add, sum_out))) return fail(FLH_EINVAL, "%s: add and sum_out must be 16-byte aligned", who);
  if (weight && misaligned16(weight)) return fail(FLH_EINVAL, "%s: weight must be 16-byte aligned", who);
  if (sum_out && ((const void*)sum_out == (const void*)x || (const void*)sum_out == (const void*)add))
    return fail(FLH_EINVAL, "%s: sum_out must not be x or add", who);
  const DecodePrologue pro{(const __half*)weight, eps, (const __half*)add, (__half*)sum_out};
  return rotate_gemm_checked(who, x, &pro, count, B, b_scale, D, N, M, K, b_cols, stream);
}

extern "C" int flh_rotate_quant_gemm_i4_o16(const flh_half* x, const uint8_t* B, const flh_half* b_scale, flh_half* D,
                                            size_t M, size_t N, size_t K, int b_cols, void* stream) {
  if (N == 0) return FLH_OK;
  return flh_rotate_quant_gemm_i4_o16_multi(x, 1, &B, &b_scale, &D, &N, M, K, b_cols, stream);
}
