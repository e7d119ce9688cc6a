// The int4 x int4 GEMM on the CDNA4 6-bit floating-point matrix instruction.
//
// Every int4 code -8 .. 7 is exactly representable in the 6-bit format e3m2 ("bf6": sign, 3 exponent bits with
// bias 3, 2 mantissa bits; 1 = 0b001100, 3 = 0b010010, 7 = 0b010111, 8 = 0b011000), every product of two codes
// is an integer of magnitude <= 64, and every partial sum over K <= 131072 codes stays below 2^24 in magnitude, so
// the float32 accumulator of v_mfma_f32_32x32x64_f8f6f4 holds the exact integer sum whatever the order of its
// additions: the result is the int32 accumulator of the integer GEMM, bit for bit.  The instruction retires 64
// codes of K per 32 x 32 tile in the time the int8 instruction needs for 32, and its operands need no unpacking
// in the loop: both are re-encoded once (flh_encode_f6; weights when they are loaded, activations after the
// quantiser) at 6 bits per code.
//
//   D[m, n] = fp16( float(sum_k A[m,k] * B[n,k]) * (As[m] * Bs[n]) )       (one scale per row / per channel)
//
// Same results as flh_gemm_i4_o16 with a_cols = b_cols = 1 (flhDenseLayerGEMM_i4_o16 of the reference with
// per-token x per-channel scales, benchmark/nn/benchmark_linear_flh.py:74-86), on operands in the encoded format.
//
// Encoded operand format.  An [R, K] matrix is K / 128 slabs of R blocks of 96 bytes: slab kt holds, row after row,
// the codes k = 128 kt .. 128 kt + 127 of every row, so that the rows a tile needs for one K step are one contiguous
// run of memory (whole cache lines per load instruction; with row-major operands every 128-byte line would be
// fetched in two different K steps).  Inside a block the code k = 128 kt + 64 m + 32 h + pos (m, h in {0, 1},
// pos in 0..31) is the 6-bit field at bit 6 pos of the 24-byte piece (h, m) at byte 48 h + 24 m: a lane of MFMA
// number m that sits in wave half h takes one piece as its operand, and the 48 bytes of a wave half are three
// 16-byte chunks.
//
// Tiling as the int8 kernel: workgroup = 4 waves (2 x 2), wave tile of 32 x 32 MFMA tiles, K advances by 128 codes
// (96 bytes per row) per stage, stages form a ring in LDS filled by direct-to-LDS loads.  Chunk c of tile row r
// sits in slot 6 r + (c ^ ((r >> 3) & 1)): sixteen consecutive rows read at one logical chunk touch sixteen
// different groups of four banks.  Fragment reads run half a stage ahead of the MFMAs that use them.
#include <atomic>

#include <type_traits>

#include "gemm_i4.h"
#include "f6_codes.h"

namespace flh {

namespace {

constexpr int kBlockBytes = 96;   // encoded bytes of K per row per stage (128 codes)
constexpr int kEpiPadF6 = 16;     // bytes of padding per row of the epilogue staging tile
constexpr int kBf6 = 3;           // format selector of the matrix instruction: e3m2

typedef int v8i __attribute__((ext_vector_type(8)));

//
// SWIGLU (as in the int8 kernel): the launch computes gate = A . Bg^T and up = A . Bu^T for the SAME output channels in one
// workgroup -- the tile's BN weight rows are BN / 2 rows of the gate matrix and the same BN / 2 rows of the up matrix, the
// two wave columns -- rounds both to fp16 as their own launches would store them, and stores only
// fp16(fp16(silu(gate)) * up): [M, N] with N the width of ONE of the matrices.
//
// ROPE (as in the int8 kernel): a q / k / v launch with heads of 128 channels = one tile column each, whose epilogue
// applies the rotary embedding to the query and key heads and writes keys and values into their cache slots.
template <int BM, int BN, int WM, int WN, int STAGES, int EPI, bool SWIGLU = false, bool ROPE = false>
__global__ __launch_bounds__(64 * (BM / WM) * (BN / WN), ((BM / WM) * (BN / WN) == 4 && WM * WN <= 64 * 64) ? 2 : 1)
void gemm_f6_kernel(const GemmArgs p) {
  constexpr int TM = WM / 32, TN = WN / 32;
  constexpr int WAVES_N = BN / WN;
  constexpr int WAVES = (BM / WM) * (BN / WN);        // 4, or 8 (two per SIMD from one workgroup)
  constexpr int T = 64 * WAVES;
  constexpr int STAGE = (BM + BN) * kBlockBytes;
  constexpr int TI = (BM + BN) * 6 / 64;              // 1 KiB load instructions per stage
  constexpr int NI_LO = TI / WAVES, NI_X = TI % WAVES; // the first NI_X waves issue one more than the others
  constexpr int NI = NI_LO + (NI_X ? 1 : 0);
  constexpr int EPI_PITCH = WN * 2 + kEpiPadF6;
  static_assert((WAVES == 4 || WAVES == 8) && BM % 64 == 0 && BN % 64 == 0, "tile shape");
  static_assert(!SWIGLU || (EPI != kInt32 && WAVES_N == 2), "gate | up halves are the two wave columns");
  static_assert(!ROPE || (EPI != kInt32 && BN == 128 && WN == 64 && !SWIGLU), "a tile column is one head of 128");
  constexpr int BNC = SWIGLU ? BN / 2 : BN;           // output channels per tile
  static_assert((BM + BN) * 6 % 64 == 0 && (BM * 6) % 64 == 0, "whole load instructions, none straddling A | B");
  static_assert(STAGES >= 3, "ring depth");
  static_assert(EPI == kInt32 || WAVES * WM * EPI_PITCH <= STAGES * STAGE, "epilogue staging must fit the ring");
  // group scales (one scale group = one 128-code stage): kGroupScale has one activation scale per token and
  // group, kTokenGroup one per token (applied after the groups); both have one weight scale per channel and group
  constexpr bool GROUPED = EPI == kGroupScale || EPI == kTokenGroup;
  constexpr bool token_scale = EPI == kTokenGroup;
  constexpr int SCROWS = BM + BN;
  static_assert(!GROUPED || (SCROWS <= T && STAGES == 3), "one thread per scale row; prefetch relies on the full wait");

  extern __shared__ __align__(1024) uint8_t lds[];    // [STAGES][STAGE], then the tile's scales

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const unsigned lds0 = (unsigned)(size_t)lds;
  const int wm = (wave / WAVES_N) * WM, wn = (wave % WAVES_N) * WN;

  const unsigned total = p.tiles_m * p.tiles_n;
  const unsigned L = xcd_contiguous(blockIdx.x, total);
  const unsigned band = p.group_m * p.tiles_n;
  const unsigned first_m = (L / band) * p.group_m;
  const unsigned gsz = min((unsigned)p.tiles_m - first_m, (unsigned)p.group_m);
  const int tile_m = first_m + (L % band) % gsz;
  const int tile_n = (L % band) / gsz;
  // the weight matrix this tile belongs to (several may share A in one launch)
  const uint8_t* wB = p.B;
  const __half* wBs = p.Bs;
  void* wD = p.D;
  int wN = p.N, seg_tile = tile_n, seg = 0;
  for (int s = 1; s < p.n_seg; ++s)
    if (tile_n >= p.seg_tile0[s]) {
      wB = p.seg_B[s];
      wBs = p.seg_Bs[s];
      wD = p.seg_D[s];
      wN = p.seg_N[s];
      seg_tile = tile_n - p.seg_tile0[s];
      seg = s;
    }
  const int m0 = tile_m * BM, n0 = seg_tile * BNC;

  // per-lane byte offsets of this wave's NI load instructions inside A resp. B (stage 0)
  const int my_ni = NI_LO + (wave < NI_X ? 1 : 0);     // wave-uniform
  const int first_i = wave * NI_LO + (wave < NI_X ? wave : NI_X);
  unsigned voff[NI];
  int src_of[NI];                                      // 0: activations, 1: weights, 2: the up matrix (SWIGLU)
  static_assert(!SWIGLU || (BNC * 6) % 64 == 0, "a load instruction never straddles gate | up");
#pragma unroll
  for (int i = 0; i < NI; ++i) {
    const int slot = (min(first_i + i, TI - 1)) * 64 + lane;
    const bool isA = __builtin_amdgcn_readfirstlane(slot < BM * 6);
    const int s = isA ? slot : slot - BM * 6;
    const int r = s / 6, c = (s % 6) ^ ((r >> 3) & 1);
    const bool second = SWIGLU && !isA && __builtin_amdgcn_readfirstlane(s >= BNC * 6);
    const int gr = isA ? min(m0 + r, p.M - 1) : min(n0 + (second ? r - BNC : r), wN - 1);
    voff[i] = (unsigned)gr * kBlockBytes + c * 16;
    src_of[i] = isA ? 0 : second ? 2 : 1;
  }
  const int KT = p.K / 128;
  auto issue_stage = [&](int stage, int kt) {
    const int k = kt < KT ? kt : KT - 1;              // past the end: harmless reload, keeps the wait counts fixed
    const unsigned base = lds0 + stage * STAGE + first_i * 1024;
    const uint8_t* ka = p.A + (size_t)k * p.M * kBlockBytes;   // slab k of either operand
    const uint8_t* kb = wB + (size_t)k * wN * kBlockBytes;
    const uint8_t* kb2 = SWIGLU ? p.B2 + (size_t)k * wN * kBlockBytes : kb;
#pragma unroll
    for (int i = 0; i < NI; ++i)
      if (i < NI_LO || i < my_ni)
        load_to_lds16(src_of[i] == 0 ? ka : src_of[i] == 1 ? kb : kb2, voff[i], base + i * 1024);
  };
  // wait until at most `stages` stages of this wave's loads are still in flight
  auto wait_stages = [&](auto stages_tag) {
    constexpr int S = decltype(stages_tag)::value;
    if constexpr (NI_X == 0) {
      wait_vmcnt<S * NI_LO>();
    } else {
      if (wave < NI_X) wait_vmcnt<S * (NI_LO + 1)>();
      else wait_vmcnt<S * NI_LO>();
    }
  };

  v16f acc[TM][TN];                                    // exact integer sums (grouped: the float32 result so far)
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.f;

  const int frag_row = lane & 31, frag_chunk = lane >> 5;
  const int sw = (frag_row >> 3) & 1;
  // byte offsets inside a tile row of the three chunks of this wave half
  const int c0 = ((3 * frag_chunk) ^ sw) * 16, c1 = ((3 * frag_chunk + 1) ^ sw) * 16, c2 = ((3 * frag_chunk + 2) ^ sw) * 16;
  const int a_base = (wm + frag_row) * kBlockBytes, b_base = (BM + wn + frag_row) * kBlockBytes;

  constexpr int NF = TM + TN;                          // fragments per stage (A first, then B)
  v4i fr[2][NF][3];                                    // [parity][fragment][chunk]: 48 bytes = the operands of two MFMAs
  auto read_stage = [&](int par, int stage) {
    const uint8_t* st = lds + stage * STAGE;
#pragma unroll
    for (int f = 0; f < NF; ++f) {
      const uint8_t* row = st + (f < TM ? a_base + f * 32 * kBlockBytes : b_base + (f - TM) * 32 * kBlockBytes);
      fr[par][f][0] = *(const v4i*)(row + c0);
      fr[par][f][1] = *(const v4i*)(row + c1);
      fr[par][f][2] = *(const v4i*)(row + c2);
    }
  };
  auto operand = [&](int par, int f, int m) {
    const v4i a = fr[par][f][0], b = fr[par][f][1], c = fr[par][f][2];
    return m == 0 ? v8i{a[0], a[1], a[2], a[3], b[0], b[1], 0, 0} : v8i{b[2], b[3], c[0], c[1], c[2], c[3], 0, 0};
  };
  auto mfma_stage = [&](int par) {
#pragma unroll
    for (int m = 0; m < 2; ++m)
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(operand(par, TM + j, m), operand(par, i, m),
                                                                     acc[i][j], kBf6, kBf6, 0, 0, 0, 0);
  };

  // ---- group scales travel through LDS (as in the int8 kernel): thread t owns row t of the tile's BM activation
  // rows and BN weight rows, fetches that row's next eight group scales one block ahead and stores them
  // transposed, sc[buffer][group & 7][row], where the fold reads four channels' scales as one 8-byte run
  __half* const sc = (__half*)(lds + STAGES * STAGE);  // [2][8][SCROWS]
  unsigned short sraw[8];
  const bool sc_thread = tid < SCROWS;
  const int sc_cols = tid < BM ? p.a_cols : p.b_cols;
  const int sc_brow = min(tid, SCROWS - 1) - BM;      // weight row of the tile this thread fetches scales for
  const bool sc_second = SWIGLU && sc_brow >= BNC;
  const __half* const sc_src = (tid < BM ? p.As + (size_t)min(m0 + tid, p.M - 1) * p.a_cols
                                         : (sc_second ? p.Bs2 : wBs) +
                                               (size_t)min(n0 + (sc_second ? sc_brow - BNC : sc_brow), wN - 1) * p.b_cols);
  auto sc_issue = [&](int blk) {
#pragma unroll
    for (int i = 0; i < 8; ++i) sraw[i] = ((const unsigned short*)sc_src)[min(blk * 8 + i, sc_cols - 1)];
  };
  auto sc_store = [&](int blk) {
    if (sc_thread) {
#pragma unroll
      for (int i = 0; i < 8; ++i) ((unsigned short*)sc)[((blk & 1) * 8 + i) * SCROWS + tid] = sraw[i];
    }
  };
  // One group: each 32 x 32 tile's two MFMAs start from zero, and the exact sums are folded into the float32
  // result at once -- out = fma(sum, a_g * b_g, out) (token scale: fma(sum, b_g, out)) in ascending g, which is
  // the int8 kernel's arithmetic without its int -> float conversion
  auto mfma_fold = [&](int par, int kt) {
    const __half* sg = sc + (((kt >> 3) & 1) * 8 + (kt & 7)) * SCROWS;
    const v16f zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    auto tile_sum = [&](int i, int j) {
      v16f t = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(operand(par, TM + j, 0), operand(par, i, 0), zero, kBf6,
                                                              kBf6, 0, 0, 0, 0);
      return __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(operand(par, TM + j, 1), operand(par, i, 1), t, kBf6, kBf6,
                                                             0, 0, 0, 0);
    };
    // this group's weight scales of the wave tile's columns, converted once for all row blocks
    float sbf[TN][16];
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const h4 b4 = *(const h4*)(sg + BM + wn + j * 32 + 8 * q + 4 * frag_chunk);
#pragma unroll
        for (int e = 0; e < 4; ++e) sbf[j][4 * q + e] = (float)b4[e];
      }
    auto fold = [&](int i, int j, const v16f& t) {
      const float sa = token_scale ? 1.f : __half2float(sg[wm + i * 32 + frag_row]);
#pragma unroll
      for (int r = 0; r < 16; ++r)
        acc[i][j][r] = __builtin_fmaf(t[r], token_scale ? sbf[j][r] : sa * sbf[j][r], acc[i][j][r]);
    };
    // the MFMAs of tile n + 1 are issued together with the fold of tile n; a scheduling barrier after each
    // such pair keeps at most two tiles of sums alive (more would not fit the register file)
    v16f prev = tile_sum(0, 0);
#pragma unroll
    for (int n = 1; n < TM * TN; ++n) {
      const v16f cur = tile_sum(n / TN, n % TN);
      fold((n - 1) / TN, (n - 1) % TN, prev);
      __builtin_amdgcn_sched_barrier(0);
      prev = cur;
    }
    fold(TM - 1, TN - 1, prev);
  };

  // One-scale-per-row epilogue: the tile's scales are fetched now and parked in LDS behind the ring
  __half* const lds_sa = (__half*)(lds + STAGES * STAGE);   // [BM] then [BN]
  __half scale_reg[(BM + BN + T - 1) / T];
  if constexpr (EPI == kRowScale) {
#pragma unroll
    for (int i = 0; i < (BM + BN + T - 1) / T; ++i) {
      const int e = tid + i * T;
      const bool second = SWIGLU && e - BM >= BNC;
      const int m = m0 + e, n = n0 + e - BM - (second ? BNC : 0);
      scale_reg[i] = e < BM ? (m < p.M ? p.As[m] : __float2half(1.f))
                            : (e < BM + BN && n < wN ? (second ? p.Bs2 : wBs)[n] : __float2half(1.f));
    }
  }
  if constexpr (GROUPED) sc_issue(0);
#pragma unroll
  for (int s = 0; s < STAGES - 1; ++s) issue_stage(s, s);
  wait_stages(std::integral_constant<int, STAGES - 2>{});   // stage 0 has landed (this wave's part)
  if constexpr (GROUPED) sc_store(0);
  if constexpr (EPI == kRowScale) {
#pragma unroll
    for (int i = 0; i < (BM + BN + T - 1) / T; ++i) {
      const int e = tid + i * T;
      if (e < BM + BN) lds_sa[e] = scale_reg[i];
    }
  }
  __syncthreads();
  if constexpr (!GROUPED) read_stage(0, 0);

  int stage = 0;
  // one K step; `par` (a compile-time constant) says which half of the fragment registers feeds the MFMAs
  auto k_step = [&](auto par_tag, int kt) {
    constexpr int par = decltype(par_tag)::value;
    const int nxt = stage + 1 == STAGES ? 0 : stage + 1;
    wait_stages(std::integral_constant<int, STAGES - 3>{});   // this wave's part of stage kt+1 has landed
    // ... everybody's has, and stage kt-1 is free: its fragment reads were consumed an iteration ago; the LDS
    // reads still in flight here belong to stage kt, which nobody overwrites before the next barrier
    barrier_no_fence();
    if constexpr (GROUPED) {
      // the next block of eight group scales, requested at the end of the previous iteration (everything
      // outstanding has been waited for above)
      if ((kt & 7) == 7) sc_store((kt >> 3) + 1);
    }
    {
      int fill = stage + STAGES - 1;
      if (fill >= STAGES) fill -= STAGES;
      issue_stage(fill, kt + STAGES - 1);
    }
    if constexpr (GROUPED) {
      // the float32 result doubles the accumulator registers, so the fragments are not double-buffered here: this
      // stage's are read now, and the other waves of the SIMD cover the LDS latency
      read_stage(0, stage);
      mfma_fold(0, kt);
    } else {
      // fragment reads run one stage ahead of the MFMAs that use them
      read_stage(par ^ 1, nxt);
      mfma_stage(par);
    }
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (GROUPED) {
      if (((kt + 1) & 7) == 7) sc_issue(((kt + 1) >> 3) + 1);
    }
    stage = nxt;
  };
  for (int kt = 0; kt < KT; kt += 2) {
    k_step(std::integral_constant<int, 0>{}, kt);
    if (kt + 1 < KT) k_step(std::integral_constant<int, 1>{}, kt + 1);
  }
  wait_vmcnt<0>();                                    // drain the trailing reloads
  __syncthreads();                                    // every wave is done with the ring

  if constexpr (EPI == kInt32) {
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      const int m = m0 + wm + i * 32 + frag_row;
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int n = n0 + wn + j * 32 + 8 * g + 4 * frag_chunk;
          int32_t* dst = (int32_t*)wD + (size_t)m * wN + n;
          if (m < p.M) {
            if (n + 4 <= wN && (wN & 3) == 0) {
              *(v4i*)dst = v4i{(int)acc[i][j][4 * g], (int)acc[i][j][4 * g + 1], (int)acc[i][j][4 * g + 2],
                               (int)acc[i][j][4 * g + 3]};
            } else {
#pragma unroll
              for (int e = 0; e < 4; ++e)
                if (n + e < wN) dst[e] = (int)acc[i][j][4 * g + e];
            }
          }
        }
    }
  } else {
    // dequantise into this wave's private [WM][WN] fp16 tile in LDS ...
    uint8_t* ep = lds + wave * (WM * EPI_PITCH);
    float sa[TM];
#pragma unroll
    for (int i = 0; i < TM; ++i) {
      if constexpr (EPI == kRowScale) {
        sa[i] = __half2float(lds_sa[wm + i * 32 + frag_row]);
      } else {
        const int m = m0 + wm + i * 32 + frag_row;
        sa[i] = token_scale && m < p.M ? __half2float(p.As[m]) : 1.f;
      }
    }
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int nl = j * 32 + 8 * g + 4 * frag_chunk;   // column inside the wave tile
        h4 t = {(_Float16)1.0f, (_Float16)1.0f, (_Float16)1.0f, (_Float16)1.0f};
        if constexpr (EPI == kRowScale) t = *(const h4*)(lds_sa + BM + wn + nl);
#pragma unroll
        for (int i = 0; i < TM; ++i) {
          h4 v;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            float f;
            // row scales: float(sum) * (a * b), the scale product is exact, the result rounded once
            if constexpr (EPI == kRowScale) f = acc[i][j][4 * g + e] * (sa[i] * (float)t[e]);
            else f = token_scale ? acc[i][j][4 * g + e] * sa[i] : acc[i][j][4 * g + e];
            v[e] = (_Float16)round_here(f);
          }
          *(h4*)(ep + (i * 32 + frag_row) * EPI_PITCH + nl * 2) = v;
        }
      }
    constexpr int CPR = WN / 8, RPI = 64 / CPR;
    const int crow = lane / CPR, cchunk = lane % CPR;
    const bool vec_ok = (wN & 7) == 0;
    if constexpr (SWIGLU) {
      // the gate tile (left wave column) and the up tile (right wave column) of this row band are both in LDS after
      // the barrier; each of the two waves combines half of the band's rows and stores 16-byte runs of the product
      __syncthreads();
      const int wcol = wave % WAVES_N;
      const uint8_t* gate_t = lds + (wave - wcol) * (WM * EPI_PITCH);
      const uint8_t* up_t = gate_t + WM * EPI_PITCH;
#pragma unroll
      for (int it = 0; it < WM / (2 * RPI); ++it) {
        const int row = wcol * (WM / 2) + it * RPI + crow;
        const int m = m0 + wm + row, n = n0 + cchunk * 8;
        const h8 g8 = *(const h8*)(gate_t + row * EPI_PITCH + cchunk * 16);
        const h8 u8 = *(const h8*)(up_t + row * EPI_PITCH + cchunk * 16);
        h8 o;
#pragma unroll
        for (int e = 0; e < 8; ++e) o[e] = silu_mul_f16(g8[e], u8[e]);
        if (m < p.M) {
          __half* dst = (__half*)wD + (size_t)m * wN + n;
          if (vec_ok && n + 8 <= wN) {
            *(h8*)dst = o;
          } else {
            const __half* hv = (const __half*)&o;
#pragma unroll
            for (int e = 0; e < 8; ++e)
              if (n + e < wN) dst[e] = hv[e];
          }
        }
      }
      return;
    }
    if constexpr (ROPE) {
      // the tile's 128 columns are one head: its first 64 channels sit in the left wave column's staging tile, the other
      // 64 in the right one's; each of the two waves finishes half of the band's rows, both halves of every row.  The
      // table entries and cache slots of all rows are requested before the barrier.
      constexpr int NIT = WM / (2 * RPI);
      const int wcol = wave % WAVES_N;
      const int head = seg_tile;
      h8 c1[NIT], c2[NIT], s1[NIT], s2[NIT];
      long long slot[NIT];
      int bi[NIT];
      {
        const int m_first = m0 + wm + wcol * (WM / 2) + crow;
        int b = m_first / p.rope_T, tt = m_first - b * p.rope_T;
#pragma unroll
        for (int it = 0; it < NIT; ++it) {
          const int m = m_first + it * RPI;
          const int tc = m < p.M ? tt : 0;               // rows past the end: any valid table row, nothing is stored
          bi[it] = b;
          slot[it] = seg == 0 ? 0 : p.rope_pos[tc];
          if (seg < 2) {
            const __half* ct = p.rope_cos + (size_t)tc * 128 + cchunk * 8;
            const __half* st = p.rope_sin + (size_t)tc * 128 + cchunk * 8;
            c1[it] = *(const h8*)ct, c2[it] = *(const h8*)(ct + 64), s1[it] = *(const h8*)st, s2[it] = *(const h8*)(st + 64);
          }
          tt += RPI;
          while (tt >= p.rope_T) tt -= p.rope_T, ++b;
        }
      }
      __syncthreads();
      const uint8_t* lo_t = lds + (wave - wcol) * (WM * EPI_PITCH);
      const uint8_t* hi_t = lo_t + WM * EPI_PITCH;
#pragma unroll
      for (int it = 0; it < NIT; ++it) {
        const int row = wcol * (WM / 2) + it * RPI + crow;
        const int m = m0 + wm + row;
        h8 x1 = *(const h8*)(lo_t + row * EPI_PITCH + cchunk * 16);
        h8 x2 = *(const h8*)(hi_t + row * EPI_PITCH + cchunk * 16);
        if (m < p.M) {
          bool in_range = true;
          __half* dst;
          if (seg == 0) {
            dst = (__half*)wD + (size_t)m * wN + head * 128;
          } else {
            in_range = slot[it] >= 0 && slot[it] < (long long)p.rope_max_len;
            dst = (__half*)wD +
                  (((size_t)bi[it] * p.rope_hkv + head) * p.rope_max_len + (size_t)(in_range ? slot[it] : 0)) * 128;
          }
          if (seg < 2) {                                 // queries and keys: fp16(fp16(x cos) + fp16(rotate_half(x) sin))
            h8 y1, y2;
#pragma unroll
            for (int e = 0; e < 8; ++e) {
              const _Float16 a1 = (_Float16)round_here((float)x1[e] * (float)c1[it][e]);
              const _Float16 r1 = (_Float16)round_here(-1.f * (float)x2[e] * (float)s1[it][e]);
              y1[e] = (_Float16)round_here((float)a1 + (float)r1);
              const _Float16 a2 = (_Float16)round_here((float)x2[e] * (float)c2[it][e]);
              const _Float16 r2 = (_Float16)round_here(1.f * (float)x1[e] * (float)s2[it][e]);
              y2[e] = (_Float16)round_here((float)a2 + (float)r2);
            }
            x1 = y1;
            x2 = y2;
          }
          if (in_range) {
            *(h8*)(dst + cchunk * 8) = x1;
            *(h8*)(dst + 64 + cchunk * 8) = x2;
          }
        }
      }
      return;
    }
    // ... and write it out as whole row segments (the tile is private to the wave: no barrier)
#pragma unroll
    for (int it = 0; it < WM / RPI; ++it) {
      const int row = it * RPI + crow;
      const int m = m0 + wm + row, n = n0 + wn + cchunk * 8;
      const v4i v = *(const v4i*)(ep + row * EPI_PITCH + cchunk * 16);
      if (m < p.M) {
        __half* dst = (__half*)wD + (size_t)m * wN + n;
        const __half* res = p.R ? p.R + (size_t)m * wN + n : nullptr;   // residual: read before the store (may be D)
        if (vec_ok && n + 8 <= wN) {
          *(v4i*)dst = res ? add_h8(v, *(const v4i*)res) : v;
        } else {
          const _Float16* hv = (const _Float16*)&v;
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (n + e < wN) ((_Float16*)dst)[e] = res ? hv[e] + ((const _Float16*)res)[e] : hv[e];
        }
      }
    }
  }
}

template <int BM, int BN, int WM, int WN, int STAGES, int EPI, bool SWIGLU = false, bool ROPE = false>
int launch_f6(GemmArgs a, hipStream_t stream) {
  constexpr int BNC = SWIGLU ? BN / 2 : BN;           // output channels per tile
  a.tiles_m = (a.M + BM - 1) / BM;
  a.tiles_n = (a.N + BNC - 1) / BNC;
  for (int s = 1; s < a.n_seg; ++s) {                 // further weight matrices: their tiles follow
    a.seg_tile0[s] = a.tiles_n;
    a.tiles_n += (a.seg_N[s] + BN - 1) / BN;
  }
  a.group_m = a.tiles_m < 4 ? a.tiles_m : 4;
  const size_t smem = (size_t)STAGES * (BM + BN) * kBlockBytes +
                      (EPI == kRowScale ? (BM + BN) * 2 : (EPI == kGroupScale || EPI == kTokenGroup) ? (BM + BN) * 32 : 0);
  auto kern = gemm_f6_kernel<BM, BN, WM, WN, STAGES, EPI, SWIGLU, ROPE>;
  static LdsGrant grant;                               // per instantiation
  if (int rc = reserve_lds((const void*)kern, smem, grant, "gemm_f6")) return rc;
  hipLaunchKernelGGL(kern, dim3(a.tiles_m * a.tiles_n), dim3(64 * (BM / WM) * (BN / WN)), smem, stream, a);
  return check_launch("gemm_f6");
}

// output columns of a launch over all its weight matrices
int total_n_f6(const GemmArgs& a) {
  int n = a.N;
  for (int s = 1; s < a.n_seg; ++s) n += a.seg_N[s];
  return n;
}

template <int EPI>
int launch_f6_grouped(const GemmArgs& a, hipStream_t stream) {
  const int n_all = total_n_f6(a);
  auto tiles = [&](int bm, int bn) { return (long)((a.M + bm - 1) / bm) * ((n_all + bn - 1) / bn); };
  int tile = tiles(128, 128) >= 200 ? 128 : 64;
  const int forced = g_tune_tile.load(std::memory_order_relaxed);
  if (forced == 128 || forced == 64) tile = forced;
  if (tile == 128) return launch_f6<128, 128, 64, 64, 3, EPI>(a, stream);
  return launch_f6<64, 64, 32, 32, 3, EPI>(a, stream);
}

// SwiGLU launches: tiles by the number of 64-channel output tiles (128 weight rows of [gate | up] each)
template <int EPI>
int launch_f6_swiglu(const GemmArgs& a, hipStream_t stream) {
  auto tiles = [&](int bm, int bnc) { return (long)((a.M + bm - 1) / bm) * ((a.N + bnc - 1) / bnc); };
  int tile = tiles(128, 64) >= 200 ? 128 : 64;
  const int forced = g_tune_tile.load(std::memory_order_relaxed);
  if (forced == 128 || forced == 64) tile = forced;
  if (tile == 128) return launch_f6<128, 128, 64, 64, 3, EPI, true>(a, stream);
  return launch_f6<64, 64, 32, 32, 3, EPI, true>(a, stream);
}

// flh_gemm_set_tuning overrides the tile choice (256 / 128 / 64; the hook through which the tests cover every variant)
template <int EPI>
int launch_f6_by_shape(const GemmArgs& a, hipStream_t stream) {
  const int env_tile = g_tune_tile.load(std::memory_order_relaxed);
  const int n_all = total_n_f6(a);
  auto tiles = [&](int bm, int bn) { return (long)((a.M + bm - 1) / bm) * ((n_all + bn - 1) / bn); };
  // measured at M = 2048 on the Llama shapes: two 128 x 128 workgroups per compute unit beat one 256 x 128
  // workgroup of eight waves by 2-10 %; the large tile is kept for the override
  int tile = tiles(128, 128) >= 256 ? 128 : 64;
  if (env_tile == 256 || env_tile == 128 || env_tile == 64) tile = env_tile;
  if (tile == 256) return launch_f6<256, 128, 64, 64, 4, EPI>(a, stream);
  if (tile == 128) return launch_f6<128, 128, 64, 64, 3, EPI>(a, stream);
  return launch_f6<64, 64, 32, 32, 3, EPI>(a, stream);
}

// one thread per (row, block, wave half): 2 x 16 bytes of nibbles in, 48 bytes of 6-bit codes out.  A workgroup
// takes 32 rows x 4 blocks, so that it reads 256 contiguous bytes per row and writes 3 KiB runs per slab.
__global__ __launch_bounds__(256) void encode_f6_kernel(const uint8_t* __restrict__ src, uint8_t* __restrict__ dst,
                                                        size_t rows, int blocks_per_row) {
  const int t = threadIdx.x, h = t & 1;
  const size_t kt = (size_t)blockIdx.y * 4 + ((t >> 1) & 3), row = (size_t)blockIdx.x * 32 + (t >> 3);
  if (row >= rows || kt >= (size_t)blocks_per_row) return;
  const uint8_t* in = src + (row * blocks_per_row + kt) * 64 + 16 * h;
  unsigned out[12];
#pragma unroll
  for (int m = 0; m < 2; ++m) {
    const v4i w = *(const v4i*)(in + 32 * m);
    const unsigned long long q0 = bf6_of_nibbles((unsigned)w[0]), q1 = bf6_of_nibbles((unsigned)w[1]),
                             q2 = bf6_of_nibbles((unsigned)w[2]), q3 = bf6_of_nibbles((unsigned)w[3]);
    out[6 * m + 0] = (unsigned)q0;
    out[6 * m + 1] = (unsigned)(q0 >> 32) | ((unsigned)q1 << 16);
    out[6 * m + 2] = (unsigned)(q1 >> 16);
    out[6 * m + 3] = (unsigned)q2;
    out[6 * m + 4] = (unsigned)(q2 >> 32) | ((unsigned)q3 << 16);
    out[6 * m + 5] = (unsigned)(q3 >> 16);
  }
  v4i* o = (v4i*)(dst + (kt * rows + row) * kBlockBytes + 48 * h);
#pragma unroll
  for (int i = 0; i < 3; ++i) o[i] = v4i{(int)out[4 * i], (int)out[4 * i + 1], (int)out[4 * i + 2], (int)out[4 * i + 3]};
}

int check_f6(const void* A, const void* B, const void* D, size_t M, size_t N, size_t K) {
  if ((M && N) && (!A || !B || !D)) return fail(FLH_EINVAL, "gemm_f6: null pointer");
  if (misaligned16(A, B, D)) return fail(FLH_EINVAL, "gemm_f6: A, B and D must be 16-byte aligned");
  if (K == 0 || K % 128) return fail(FLH_EINVAL, "gemm_f6: K (%zu) must be a positive multiple of 128", K);
  if (K > 131072) return fail(FLH_EINVAL, "gemm_f6: K (%zu) too large for an exact float32 accumulator", K);
  if (M > (1u << 30) || N > (1u << 30)) return fail(FLH_EINVAL, "gemm_f6: M/N too large");
  if (M * kBlockBytes > 0xFFFFFFFFull || N * kBlockBytes > 0xFFFFFFFFull)
    return fail(FLH_EINVAL, "gemm_f6: more than 2^32 / 96 rows are not supported");
  return FLH_OK;
}

}  // namespace

}  // namespace flh

using namespace flh;

extern "C" int flh_encode_f6(const uint8_t* packed_i4, uint8_t* encoded, size_t rows, size_t K, void* stream) {
  if (K == 0 || K % 128) return fail(FLH_EINVAL, "encode_f6: K (%zu) must be a positive multiple of 128", K);
  if (rows == 0) return FLH_OK;
  if (!packed_i4 || !encoded) return fail(FLH_EINVAL, "encode_f6: null pointer");
  if (misaligned16(packed_i4, encoded)) return fail(FLH_EINVAL, "encode_f6: packed_i4 and encoded must be 16-byte aligned");
  if ((rows + 31) / 32 > 0x7FFFFFFFull || (K / 128 + 3) / 4 > 65535) return fail(FLH_EINVAL, "encode_f6: matrix too large");
  hipLaunchKernelGGL(encode_f6_kernel, dim3((unsigned)((rows + 31) / 32), (unsigned)((K / 128 + 3) / 4)), dim3(256), 0,
                     (hipStream_t)stream, packed_i4, encoded, rows, (int)(K / 128));
  return check_launch("encode_f6");
}

extern "C" int flh_gemm_f6_o16(const uint8_t* A6, const uint8_t* B6, const flh_half* a_scale, const flh_half* b_scale,
                               flh_half* D, size_t M, size_t N, size_t K, void* stream) {
  if (int e = check_f6(A6, B6, D, M, N, K)) return e;
  if (M == 0 || N == 0) return FLH_OK;
  if (!a_scale || !b_scale) return fail(FLH_EINVAL, "gemm_f6: null scale pointer");
  GemmArgs g{A6, B6, (const __half*)a_scale, (const __half*)b_scale, D, (int)M, (int)N, (int)K, 1, 1, 0, 0, 0};
  return launch_f6_by_shape<kRowScale>(g, (hipStream_t)stream);
}

extern "C" int flh_gemm_f6_o16_gs(const uint8_t* A6, const uint8_t* B6, const flh_half* a_scale, const flh_half* b_scale,
                                  flh_half* D, size_t M, size_t N, size_t K, int a_cols, int b_cols, void* stream) {
  if (int e = check_f6(A6, B6, D, M, N, K)) return e;
  if (M == 0 || N == 0) return FLH_OK;
  if (!a_scale || !b_scale) return fail(FLH_EINVAL, "gemm_f6: null scale pointer");
  const int ng = (int)(K / 128);
  if (b_cols != ng || (a_cols != 1 && a_cols != ng))
    return fail(FLH_EINVAL, "gemm_f6: scale columns (%d, %d) must be (1 or K/128, K/128) with K/128 = %d", a_cols, b_cols, ng);
  GemmArgs g{A6, B6, (const __half*)a_scale, (const __half*)b_scale, D, (int)M, (int)N, (int)K, a_cols, b_cols, 0, 0, 0};
  if (a_cols == 1) return launch_f6_grouped<kTokenGroup>(g, (hipStream_t)stream);
  return launch_f6_grouped<kGroupScale>(g, (hipStream_t)stream);
}

extern "C" int flh_gemm_f6_add_o16(const uint8_t* A6, const uint8_t* B6, const flh_half* a_scale, const flh_half* b_scale,
                                   const flh_half* residual, flh_half* D, size_t M, size_t N, size_t K, int a_cols,
                                   int b_cols, void* stream) {
  if (int e = check_f6(A6, B6, D, M, N, K)) return e;
  if (M == 0 || N == 0) return FLH_OK;
  if (!a_scale || !b_scale) return fail(FLH_EINVAL, "gemm_f6: null scale pointer");
  if (!residual) return fail(FLH_EINVAL, "gemm_f6 (residual): null pointer");
  if (misaligned16(residual)) return fail(FLH_EINVAL, "gemm_f6 (residual): the residual must be 16-byte aligned");
  const int ng = (int)(K / 128);
  const bool rows_only = a_cols == 1 && b_cols == 1;
  if (!rows_only && (b_cols != ng || (a_cols != 1 && a_cols != ng)))
    return fail(FLH_EINVAL, "gemm_f6: scale columns (%d, %d) must be (1, 1) or (1 or K/128, K/128) with K/128 = %d", a_cols, b_cols, ng);
  GemmArgs g{A6, B6, (const __half*)a_scale, (const __half*)b_scale, D, (int)M, (int)N, (int)K, a_cols, b_cols, 0, 0, 0};
  g.R = (const __half*)residual;
  if (rows_only) return launch_f6_by_shape<kRowScale>(g, (hipStream_t)stream);
  if (a_cols == 1) return launch_f6_grouped<kTokenGroup>(g, (hipStream_t)stream);
  return launch_f6_grouped<kGroupScale>(g, (hipStream_t)stream);
}

extern "C" int flh_gemm_f6_swiglu_o16(const uint8_t* A6, const uint8_t* B6_gate, const uint8_t* B6_up, const flh_half* a_scale,
                                      const flh_half* gate_scale, const flh_half* up_scale, flh_half* D, size_t M, size_t N,
                                      size_t K, int a_cols, int b_cols, void* stream) {
  if (int e = check_f6(A6, B6_gate, D, M, N, K)) return e;
  if ((M && N) && !B6_up) return fail(FLH_EINVAL, "gemm_f6: null pointer");
  if (misaligned16(B6_up)) return fail(FLH_EINVAL, "gemm_f6: A, B and D must be 16-byte aligned");
  if (M == 0 || N == 0) return FLH_OK;
  if (!a_scale || !gate_scale || !up_scale) return fail(FLH_EINVAL, "gemm_f6: null scale pointer");
  const int ng = (int)(K / 128);
  const bool grouped = a_cols != 1 || b_cols != 1;
  if (grouped && (b_cols != ng || (a_cols != 1 && a_cols != ng)))
    return fail(FLH_EINVAL, "gemm_f6 (SwiGLU): scale columns (%d, %d): weights need 1 or K / 128 = %d, activations 1 or %d",
                a_cols, b_cols, ng, ng);
  GemmArgs g{A6, B6_gate, (const __half*)a_scale, (const __half*)gate_scale, D, (int)M, (int)N, (int)K, a_cols, b_cols, 0, 0, 0};
  g.B2 = B6_up;
  g.Bs2 = (const __half*)up_scale;
  if (!grouped) return launch_f6_swiglu<kRowScale>(g, (hipStream_t)stream);
  if (a_cols == 1) return launch_f6_swiglu<kTokenGroup>(g, (hipStream_t)stream);
  return launch_f6_swiglu<kGroupScale>(g, (hipStream_t)stream);
}

extern "C" int flh_gemm_f6_qkv_rope_o16(const uint8_t* A6, const flh_half* a_scale, const uint8_t* const* B6,
                                        const flh_half* const* b_scale, const flh_half* cos, const flh_half* sin,
                                        const int64_t* positions, flh_half* q_out, flh_half* k_cache, flh_half* v_cache,
                                        uint32_t batch, uint32_t T, uint32_t Hq, uint32_t Hkv, uint32_t max_len, size_t K,
                                        int a_cols, int b_cols, void* stream) {
  if (!B6 || !b_scale) return fail(FLH_EINVAL, "gemm_f6 (q/k/v + rotary): null array");
  if (Hq == 0 || Hkv == 0 || max_len == 0)
    return fail(FLH_EINVAL, "gemm_f6 (q/k/v + rotary): heads and cache length must be positive");
  const size_t M = (size_t)batch * T;
  const size_t N[3] = {(size_t)Hq * 128, (size_t)Hkv * 128, (size_t)Hkv * 128};
  flh_half* const D[3] = {q_out, k_cache, v_cache};
  for (int s = 0; s < 3; ++s) {
    if (int e = check_f6(A6, B6[s], D[s], M, N[s], K)) return e;
    if (!b_scale[s]) return fail(FLH_EINVAL, "gemm_f6: null scale pointer");
  }
  if (M == 0) return FLH_OK;
  if (!a_scale || !cos || !sin || !positions) return fail(FLH_EINVAL, "gemm_f6 (q/k/v + rotary): null pointer");
  if (misaligned16(cos, sin)) return fail(FLH_EINVAL, "gemm_f6 (q/k/v + rotary): cos and sin must be 16-byte aligned");
  if ((uint64_t)batch * Hkv * max_len > (1ull << 40) / 128) return fail(FLH_EINVAL, "gemm_f6 (q/k/v + rotary): cache too large");
  const int ng = (int)(K / 128);
  const bool rows_only = a_cols == 1 && b_cols == 1;
  if (!rows_only && (b_cols != ng || (a_cols != 1 && a_cols != ng)))
    return fail(FLH_EINVAL, "gemm_f6: scale columns (%d, %d) must be (1, 1) or (1 or K/128, K/128) with K/128 = %d", a_cols, b_cols, ng);
  GemmArgs g{A6, B6[0], (const __half*)a_scale, (const __half*)b_scale[0], q_out, (int)M, (int)N[0], (int)K, a_cols, b_cols, 0, 0, 0};
  g.n_seg = 3;
  for (int s = 1; s < 3; ++s) {
    g.seg_B[s] = B6[s];
    g.seg_Bs[s] = (const __half*)b_scale[s];
    g.seg_D[s] = D[s];
    g.seg_N[s] = (int)N[s];
  }
  g.rope_cos = (const __half*)cos;
  g.rope_sin = (const __half*)sin;
  g.rope_pos = (const long long*)positions;
  g.rope_T = (int)T;
  g.rope_max_len = (int)max_len;
  g.rope_hkv = (int)Hkv;
  // 128 x 128 tiles (a tile column = one head)
  if (rows_only) return launch_f6<128, 128, 64, 64, 3, kRowScale, false, true>(g, (hipStream_t)stream);
  if (a_cols == 1) return launch_f6<128, 128, 64, 64, 3, kTokenGroup, false, true>(g, (hipStream_t)stream);
  return launch_f6<128, 128, 64, 64, 3, kGroupScale, false, true>(g, (hipStream_t)stream);
}

extern "C" int flh_gemm_f6_o16_multi(const uint8_t* A6, const flh_half* a_scale, int count, const uint8_t* const* B6,
                                     const flh_half* const* b_scale, flh_half* const* D, const size_t* N, size_t M,
                                     size_t K, int a_cols, int b_cols, void* stream) {
  if (count < 1 || count > kMaxGemmSegments)
    return fail(FLH_EINVAL, "gemm_f6 (several weight matrices): count = %d, must be 1 .. %d", count, kMaxGemmSegments);
  if (!B6 || !b_scale || !D || !N) return fail(FLH_EINVAL, "gemm_f6 (several weight matrices): null array");
  size_t n_all = 0;
  for (int s = 0; s < count; ++s) {
    if (N[s] == 0) return fail(FLH_EINVAL, "gemm_f6 (several weight matrices): N[%d] = 0", s);
    if (int e = check_f6(A6, B6[s], D[s], M, N[s], K)) return e;
    if (!b_scale[s]) return fail(FLH_EINVAL, "gemm_f6: null scale pointer");
    n_all += N[s];
  }
  if (n_all > (1u << 30)) return fail(FLH_EINVAL, "gemm_f6: M/N too large");
  if (M == 0) return FLH_OK;
  if (!a_scale) return fail(FLH_EINVAL, "gemm_f6: null scale pointer");
  const int ng = (int)(K / 128);
  const bool rows_only = a_cols == 1 && b_cols == 1;
  if (!rows_only && (b_cols != ng || (a_cols != 1 && a_cols != ng)))
    return fail(FLH_EINVAL, "gemm_f6: scale columns (%d, %d) must be (1, 1) or (1 or K/128, K/128) with K/128 = %d", a_cols, b_cols, ng);
  GemmArgs g{A6, B6[0], (const __half*)a_scale, (const __half*)b_scale[0], D[0], (int)M, (int)N[0], (int)K, a_cols, b_cols, 0, 0, 0};
  g.n_seg = count;
  for (int s = 1; s < count; ++s) {
    g.seg_B[s] = B6[s];
    g.seg_Bs[s] = (const __half*)b_scale[s];
    g.seg_D[s] = D[s];
    g.seg_N[s] = (int)N[s];
  }
  if (rows_only) return launch_f6_by_shape<kRowScale>(g, (hipStream_t)stream);
  if (a_cols == 1) return launch_f6_grouped<kTokenGroup>(g, (hipStream_t)stream);
  return launch_f6_grouped<kGroupScale>(g, (hipStream_t)stream);
}

extern "C" int flh_gemm_f6_i32(const uint8_t* A6, const uint8_t* B6, int32_t* C, size_t M, size_t N, size_t K,
                               void* stream) {
  if (int e = check_f6(A6, B6, C, M, N, K)) return e;
  if (M == 0 || N == 0) return FLH_OK;
  GemmArgs g{A6, B6, nullptr, nullptr, C, (int)M, (int)N, (int)K, 1, 1, 0, 0, 0};
  return launch_f6_by_shape<kInt32>(g, (hipStream_t)stream);
}
