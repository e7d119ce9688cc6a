// int4 x int4 GEMM with int32 accumulation on the CDNA4 int8 matrix cores and a fused
// fp16 dequantising epilogue.
//
//   D[m, n] = fp16( sum_g float(sum_{k in g} A[m,k] * B[n,k]) * (As[m,g] * Bs[n,g]) )
//
// Replaces flhDenseLayerGEMM_i4_o16 / flh_gemm_i4_dequant_o16_kernel of the reference
// (flh/kernels/gemm_and_dequant_i4.cu:315-508; group epilogue :287-313) and the
// per-token x per-channel epilogue of benchmark/nn/benchmark_linear_flh.py:74-86.
//
// How the nibbles reach the matrix cores.  A 32-bit word w of a packed row holds the
// eight codes c0..c7 (c0 in bits 0-3).  (w << 4) & 0xF0F0F0F0 is, read as four int8,
// 16*c0, 16*c2, 16*c4, 16*c6 and w & 0xF0F0F0F0 is 16*c1, 16*c3, 16*c5, 16*c7: the
// two's-complement nibble lands in the high half of the byte, so no sign extension is
// needed.  Both operands are treated alike, so v_mfma_i32_32x32x32_i8 accumulates
// 256 * sum(a*b); |256 * 64 * K| < 2^31 for K <= 131071.  A dot product does not depend
// on the order of its terms, so "even codes then odd codes" is as good as natural order
// as long as A and B fragments come from the same load + unpack code.  acc >> 8 is the
// exact int32 accumulator.
//
// Tiling: workgroup = 4 waves (2 x 2), macro tile BM x BN, wave tile WM x WN made of
// 32 x 32 MFMA tiles; K advances by 128 codes (64 bytes per row) per stage.  Stages form a
// ring in LDS that is filled by direct-to-LDS global loads (no staging registers); the
// packed bytes sit in LDS in an XOR-swizzled chunk order so that fragment reads are free of
// bank conflicts.  One ds_read_b128 per lane feeds two MFMAs.  Fragment reads run one
// half-stage ahead of the MFMAs that consume them, so that with a single wave per SIMD
// the LDS latency and the per-stage barrier hide behind sixteen MFMAs.
// The weights are the MFMA's row operand: an output lane then holds one row m (lane % 32)
// and four consecutive columns n per register quad, which packs into 8-byte LDS writes for
// the epilogue; the tile leaves through LDS as full 128-byte row segments.
#include <atomic>

#include <type_traits>

#include "gemm_i4.h"

namespace flh {

// tile / K-split override of the shape heuristics (0 = automatic), set by flh_gemm_set_tuning
std::atomic<int> g_tune_tile{0}, g_tune_ks{0};

namespace {

#ifndef FLH_GEMM_OCC
#define FLH_GEMM_OCC 2
#endif
constexpr int kStageBytes = 64;   // packed bytes of K per row per stage (128 codes)
constexpr int kEpiPad = 16;       // bytes of padding per row of the epilogue staging tile


__device__ __forceinline__ void unpack8(const v4i w, v4i& lo, v4i& hi) {
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    lo[i] = (w[i] << 4) & 0xF0F0F0F0;
    hi[i] = w[i] & 0xF0F0F0F0;
  }
}

// Scheduling hint for one half-stage: NM MFMAs, NV VALU instructions and ND LDS reads, spread
// evenly as "1 MFMA, its share of VALU, its share of LDS reads", NM times.
template <int M, int NM, int NV, int ND>
__device__ __forceinline__ void interleave_hint() {
  if constexpr (M < NM) {
    constexpr int v = (NV * (M + 1)) / NM - (NV * M) / NM;
    constexpr int d = (ND * (M + 1)) / NM - (ND * M) / NM;
    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
    if constexpr (v > 0) __builtin_amdgcn_sched_group_barrier(0x002, v, 0);
    if constexpr (d > 0) __builtin_amdgcn_sched_group_barrier(0x100, d, 0);
    interleave_hint<M + 1, NM, NV, ND>();
  }
}

// LDS stage layout: row r of a tile is four 16-byte chunks; chunk c of row r lives in slot
// 4 r + (c ^ ((r >> 2) & 3)).  Sixteen consecutive rows read at the same logical chunk then
// touch sixteen different groups of four banks, and a wave's 64 lanes fill 64 consecutive
// slots when loading, which is what the direct-to-LDS load requires.
//
// GROUP is the scale group of the group-scale epilogue.  128 is one whole stage and runs the
// software-pipelined loop; 64 (half a stage: one lo/hi MFMA pair) and 32 (one 16-byte chunk:
// each lane half takes 8 bytes of it, low nibbles then high nibbles, so one MFMA covers
// exactly the group) read their fragments straight from the current stage and fold the
// accumulators into the fp32 result after every group.
//
// KS > 1 splits K inside the workgroup: KS groups of four waves ("quads") each run the loop
// above on their own LDS ring over a contiguous 1/KS of K, then add their int32 accumulators
// through LDS.  This doubles / quadruples the waves per SIMD when a problem has only about
// one tile per compute unit, so that one wave's unpack work overlaps another's MFMAs; integer
// addition keeps the result bit-identical.  With KS == 2 each quad finishes half of the rows.
//
// SWIGLU: the launch computes gate = A . Bg^T and up = A . Bu^T for the SAME output channels in one workgroup and stores
// fp16(fp16(silu(gate)) * up) only.  The tile's BN weight rows are BN/2 rows of the gate matrix followed by the same
// BN/2 rows of the up matrix, so the waves of the left half of the tile hold gate values and those of the right half
// the matching up values; both halves go through the epilogue's fp16 staging tiles in LDS (rounded to fp16 exactly as
// the two separate GEMMs would store them), where each wave then combines half of the rows.
//
// ROPE: a q / k / v launch (three weight matrices, heads of 128 channels = one tile column each) whose epilogue applies
// the rotary embedding to the query and key heads and writes keys and values into their cache slots -- the arithmetic of
// rope_kv_cache_kernel (rope_cache.hip) on the fp16 values the plain launch would have stored, so the same bits without
// the pass over q, k and v that follows the GEMM otherwise.  The two halves of a head are the two wave columns, paired
// through the staging tiles as for SWIGLU.
template <int BM, int BN, int WM, int WN, int STAGES, int EPI, int GROUP = 128, int KS = 1, bool SWIGLU = false,
          bool ROPE = false>
__global__ __launch_bounds__(64 * (BM / WM) * (BN / WN) * KS, (KS == 1 && WM * WN <= 128 * 64) ? FLH_GEMM_OCC : 1)
void gemm_i4_kernel(const GemmArgs p) {
  constexpr bool GROUPED = EPI == kGroupScale || EPI == kTokenGroup;
  constexpr bool token_scale = EPI == kTokenGroup;
  constexpr int TM = WM / 32, TN = WN / 32;          // MFMA tiles per wave
  constexpr int WAVES_N = BN / WN;
  constexpr int STAGE = (BM + BN) * kStageBytes;      // bytes per stage
  constexpr int WPQ = (BM / WM) * (BN / WN);          // waves that share one K slice ("quad": 4, or 2)
  constexpr int QT = 64 * WPQ;                        // threads of a quad
  constexpr int NI = (BM + BN) / (16 * WPQ);          // 1 KiB load instructions per wave per stage
  constexpr int EPI_PITCH = WN * 2 + kEpiPad;         // bytes per row of a wave's fp16 output tile
  static_assert(BM % 64 == 0 && BN % 64 == 0 && ((BM / WM) * (BN / WN) == 4 || (BM / WM) * (BN / WN) == 2), "tile shape");
  static_assert(STAGES >= 3, "ring depth");
  static_assert(EPI == kInt32 || (BM / WM) * (BN / WN) * WM * EPI_PITCH <= KS * STAGES * STAGE,
                "epilogue staging must fit the ring");
  static_assert(KS == 1 || (!GROUPED && (KS - 1) * BM * BN * 4 <= KS * STAGES * STAGE), "K split");
  static_assert(!SWIGLU || (KS == 1 && EPI != kInt32 && BN / WN == 2), "gate | up halves are the two wave columns");
  static_assert(!ROPE || (KS == 1 && EPI != kInt32 && BN == 128 && WN == 64 && !SWIGLU), "a tile column is one head of 128");
  constexpr int BNC = SWIGLU ? BN / 2 : BN;           // output channels per tile
  constexpr int ES = (KS == 2 && TM % 2 == 0) ? 2 : 1;   // quads that take part in the epilogue
  constexpr int TE = TM / ES;                            // 32-row blocks of a wave tile finished per quad

  extern __shared__ __align__(1024) uint8_t lds[];    // [KS][STAGES][STAGE]

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave_all = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int quad = KS == 1 ? 0 : wave_all / WPQ;      // which slice of K
  const int wave = wave_all % WPQ;                    // position in the grid of wave tiles
  uint8_t* const ring = lds + quad * (STAGES * STAGE);
  const unsigned lds0 = (unsigned)(size_t)ring;
  const int wm = (wave / WAVES_N) * WM, wn = (wave % WAVES_N) * WN;

  // workgroup -> tile: contiguous logical range per die, then bands of group_m tile rows
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
  const int Kb = p.K >> 1;                            // bytes per packed row

  // per-lane byte offsets of this wave's NI load instructions inside A resp. B (stage 0); rows past
  // the end of A / B are clamped to the last row (their results are never stored).  The loads take
  // a wave-uniform base (matrix + K position) in scalar registers plus this 32-bit offset, so a
  // stage costs no vector address arithmetic.
  unsigned voff[NI];
  int src_of[NI];                                      // 0: activations, 1: weights, 2: the up matrix (SWIGLU)
#pragma unroll
  for (int i = 0; i < NI; ++i) {
    const int slot = (wave * NI + i) * 64 + lane;
    const bool isA = __builtin_amdgcn_readfirstlane(slot < BM * 4);   // a 64-slot group (16 rows) never straddles A | B
    const int r = (isA ? slot : slot - BM * 4) >> 2;
    const int c = (slot & 3) ^ ((r >> 2) & 3);
    const bool second = SWIGLU && !isA && __builtin_amdgcn_readfirstlane(r >= BNC);   // ... nor gate | up
    const int gr = isA ? min(m0 + r, p.M - 1) : min(n0 + (second ? r - BNC : r), wN - 1);
    voff[i] = (unsigned)gr * (unsigned)Kb + c * 16;
    src_of[i] = isA ? 0 : second ? 2 : 1;
  }
  // stages of this quad: the K steps are dealt out as evenly as possible, the first quads take the remainder
  const int KTall = p.K / (2 * kStageBytes), kt_base = KTall / KS, kt_rem = KTall % KS;
  const int KT = kt_base + (quad < kt_rem ? 1 : 0);
  const int kt0 = quad * kt_base + min(quad, kt_rem);
  const int KTmax = kt_base + (kt_rem ? 1 : 0);       // iterations every quad runs (barriers are workgroup-wide)
  auto issue_stage = [&](int stage, int kt) {
    const int k = kt0 + (kt < KT ? kt : KT - 1);      // past the end: harmless reload, keeps the wait counts fixed
    const unsigned base = lds0 + stage * STAGE + wave * NI * 1024;
    const uint8_t* ka = p.A + (size_t)k * kStageBytes;
    const uint8_t* kb = wB + (size_t)k * kStageBytes;
    const uint8_t* kb2 = SWIGLU ? p.B2 + (size_t)k * kStageBytes : kb;
#pragma unroll
    for (int i = 0; i < NI; ++i) load_to_lds16(src_of[i] == 0 ? ka : src_of[i] == 1 ? kb : kb2, voff[i], base + i * 1024);
  };

  v16i acc[TM][TN];
  float out[GROUPED ? TM : 1][GROUPED ? TN : 1][16];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j) {
#pragma unroll
      for (int r = 0; r < 16; ++r) acc[i][j][r] = 0;
      if constexpr (GROUPED) {
#pragma unroll
        for (int r = 0; r < 16; ++r) out[i][j][r] = 0.f;
      }
    }

  const int frag_row = lane & 31, frag_chunk = lane >> 5;
  const int sw = (frag_row >> 2) & 3;
  // byte offsets of this lane's fragment chunk inside a tile, for the two 64-code halves of a stage
  const int off_k0 = frag_row * 64 + ((frag_chunk ^ sw) << 4);
  const int off_k1 = frag_row * 64 + (((frag_chunk ^ sw) ^ 2) << 4);
  const int a_base = wm * 64, b_base = BM * 64 + wn * 64;

  // Software pipeline over half-stages h (64 codes of K each):
  //     ds_read P(h+2)  ->  unpack U(h+1)  ->  MFMA on U(h)
  // all three act on different registers inside one half-stage, so the scheduler is free to
  // (and is told to) interleave one MFMA with four or five unpack instructions.
  constexpr int NF = TM + TN;                          // fragments per half-stage (A first, then B)
  v4i pk[NF];                                          // packed fragments, being read / unpacked
  v4i ulo[2][NF], uhi[2][NF];                          // unpacked fragments: [parity][fragment]
  auto frag_ptr = [&](int stage, int f, int off) -> const v4i* {
    const uint8_t* st = ring + stage * STAGE;
    return (const v4i*)(st + (f < TM ? a_base + f * 2048 : b_base + (f - TM) * 2048) + off);
  };
  const v16i zero16 = {0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0, 0};
  auto half_step = [&](auto fresh, int par, int read_stage, int read_off) {
    // MFMAs of this half on U[par] (starting from zero accumulators if `fresh`); unpack pk -> U[par ^ 1];
    // refill pk from LDS
#pragma unroll
    for (int f = 0; f < NF; ++f) {
      unpack8(pk[f], ulo[par ^ 1][f], uhi[par ^ 1][f]);
      pk[f] = *frag_ptr(read_stage, f, read_off);
    }
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(ulo[par][TM + j], ulo[par][i],
                                                          decltype(fresh)::value ? zero16 : acc[i][j], 0, 0, 0);
        acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(uhi[par][TM + j], uhi[par][i], acc[i][j], 0, 0, 0);
      }
    // desired issue order: MFMA, a handful of unpack VALU ops, now and then one LDS read
    interleave_hint<0, 2 * TM * TN, 12 * NF, NF>();
    // nothing moves across the end of a half-step: left alone, the scheduler sinks the LDS reads to just
    // before their first use and bunches the MFMAs
    __builtin_amdgcn_sched_barrier(0);
  };

  // ---- group scales travel through LDS --------------------------------------------------------
  // Thread t owns row t of the tile's BM activation rows and BN weight rows.  Every SPB stages it
  // fetches that row's next eight group scales (2-byte loads written out by hand, so that their
  // completion is covered by the stage loads' own wait counts) and stores them transposed,
  // sc[buffer][group & 7][row], where the fold reads them as 8-byte runs of four channels.
  constexpr int GPS = 128 / GROUP;                    // scale groups per stage
  constexpr int SPB = 8 / GPS;                        // stages per block of eight groups
  constexpr int SCROWS = BM + BN;
  static_assert(!GROUPED || SCROWS <= QT * KS, "one thread per scale row");
  __half* const sc = (__half*)(lds + KS * STAGES * STAGE);   // [2][8][SCROWS]
  unsigned short sraw[8];
  const bool sc_thread = tid < SCROWS;
  const int sc_cols = tid < BM ? p.a_cols : p.b_cols;
  const int sc_brow = min(tid, SCROWS - 1) - BM;      // weight row of the tile this thread fetches scales for
  const bool sc_second = SWIGLU && sc_brow >= BNC;
  const __half* const sc_src = (tid < BM ? p.As + (size_t)min(m0 + tid, p.M - 1) * p.a_cols
                                         : (sc_second ? p.Bs2 : wBs) +
                                               (size_t)min(n0 + (sc_second ? sc_brow - BNC : sc_brow), wN - 1) * p.b_cols);
  // Ordinary loads: the compiler's own wait for them is "everything outstanding", which is what the top
  // of the next iteration waits for anyway with a three-stage ring -- so they are requested in one iteration
  // (right behind its stage loads) and stored at the top of the next.
  static_assert(!GROUPED || STAGES == 3, "the scale prefetch relies on the full wait at the loop top");
  auto sc_issue = [&](int blk) {
#pragma unroll
    for (int i = 0; i < 8; ++i)   // one scale per row: always element 0
      sraw[i] = ((const unsigned short*)sc_src)[min(blk * 8 + i, sc_cols - 1)];
  };
  auto sc_store = [&](int blk) {
    if (sc_thread) {
#pragma unroll
      for (int i = 0; i < 8; ++i) ((unsigned short*)sc)[((blk & 1) * 8 + i) * SCROWS + tid] = sraw[i];
    }
  };
  // fold the int32 sums of sub-group gi of stage kt into the fp32 result:
  // out += float(sum) * (a * b), the accumulator holds 256 * sum and the weight scale the exact 2^-8
  auto fold_group = [&](int kt, int gi) {
    if constexpr (GROUPED) {
      const __half* s = sc + (((kt / SPB) & 1) * 8 + ((kt * GPS + gi) & 7)) * SCROWS;
      // the exact factor 2^-8 that undoes the x16 of both operands rides on the activation scale
      // (token-scale variant: on the final multiply), so the weight scales are used as loaded
      float sa[TM];
#pragma unroll
      for (int i = 0; i < TM; ++i) sa[i] = token_scale ? 1.f : __half2float(s[wm + i * 32 + frag_row]) * 0.00390625f;
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          const h4 t = *(const h4*)(s + BM + wn + j * 32 + 8 * q + 4 * frag_chunk);
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            if constexpr (token_scale) {              // one scale per token, applied after the loop
#pragma unroll
              for (int i = 0; i < TM; ++i)
                out[i][j][4 * q + e] = __builtin_fmaf((float)acc[i][j][4 * q + e], (float)t[e], out[i][j][4 * q + e]);
            } else {
              const float sb = (float)t[e];
#pragma unroll
              for (int i = 0; i < TM; ++i)
                out[i][j][4 * q + e] = __builtin_fmaf((float)acc[i][j][4 * q + e], sa[i] * sb, out[i][j][4 * q + e]);
            }
          }
        }
    }
  };

  // One-scale-per-row epilogue: the tile's scales are fetched now and parked in LDS behind the
  // ring, so that the epilogue does not start with a round trip to memory.
  __half* const lds_sa = (__half*)(lds + KS * STAGES * STAGE);   // [BM] then [BN]
  __half scale_reg[(BM + BN + QT * KS - 1) / (QT * KS)];
  if constexpr (EPI == kRowScale) {
#pragma unroll
    for (int i = 0; i < (BM + BN + QT * KS - 1) / (QT * KS); ++i) {
      const int e = tid + i * QT * KS;
      const bool second = SWIGLU && e - BM >= BNC;
      const int m = m0 + e, n = n0 + e - BM - (second ? BNC : 0);
      scale_reg[i] = e < BM ? (m < p.M ? p.As[m] : __float2half(1.f))
                            : (e < BM + BN && n < wN ? (second ? p.Bs2 : wBs)[n] : __float2half(1.f));
    }
  }
  if constexpr (GROUPED) sc_issue(0);
#pragma unroll
  for (int s = 0; s < STAGES - 1; ++s) issue_stage(s, s);
  wait_vmcnt<(STAGES - 2) * NI>();                    // stage 0 has landed (this wave's part)
  if constexpr (GROUPED) sc_store(0);
  if constexpr (EPI == kRowScale) {
#pragma unroll
    for (int i = 0; i < (BM + BN + QT * KS - 1) / (QT * KS); ++i) {
      const int e = tid + i * QT * KS;
      if (e < BM + BN) lds_sa[e] = scale_reg[i];
    }
  }
  __syncthreads();
#pragma unroll
  for (int f = 0; f < NF; ++f) pk[f] = *frag_ptr(0, f, off_k0);
#pragma unroll
  for (int f = 0; f < NF; ++f) {
    unpack8(pk[f], ulo[0][f], uhi[0][f]);
    pk[f] = *frag_ptr(0, f, off_k1);
  }

  int stage = 0;
  for (int kt = 0; kt < KTmax; ++kt) {
    const int nxt = stage + 1 == STAGES ? 0 : stage + 1;
    wait_vmcnt<(STAGES - 3) * NI>();                  // this wave's part of stage kt+1 has landed
    // ... everybody's has, and stage kt-1 is free: its last fragment reads were consumed an iteration ago;
    // the LDS reads still in flight here belong to stage kt, which nobody overwrites before the next barrier
    barrier_no_fence();
    if constexpr (GROUPED) {
      // the next block of eight group scales, requested at the end of the previous iteration
      if (kt % SPB == SPB - 1) sc_store(kt / SPB + 1);
    }
    {
      int fill = stage + STAGES - 1;
      if (fill >= STAGES) fill -= STAGES;
      issue_stage(fill, kt + STAGES - 1);
    }
    if constexpr (GROUPED) {
      // the request for the block of scales after that goes out right behind the stage's loads, one iteration before
      // its store: it has this whole iteration to arrive, and the full wait at the top of the next one covers it
      if ((kt + 1) % SPB == SPB - 1) sc_issue((kt + 1) / SPB + 1);
    }
    if constexpr (GROUPED && GROUP < 128) {
      const uint8_t* st = ring + stage * STAGE;
#pragma nounroll
      for (int gi = 0; gi < 128 / GROUP; ++gi) {
        v4i flo[NF], fhi[NF];
#pragma unroll
        for (int f = 0; f < NF; ++f) {
          const uint8_t* tile = st + (f < TM ? a_base + f * 2048 : b_base + (f - TM) * 2048) + frag_row * 64;
          if constexpr (GROUP == 64) {
            unpack8(*(const v4i*)(tile + (((2 * gi + frag_chunk) ^ sw) << 4)), flo[f], fhi[f]);
          } else {
            const v2i w = *(const v2i*)(tile + ((gi ^ sw) << 4) + 8 * frag_chunk);
            flo[f] = v4i{(w[0] << 4) & (int)0xF0F0F0F0, (w[1] << 4) & (int)0xF0F0F0F0, w[0] & (int)0xF0F0F0F0,
                         w[1] & (int)0xF0F0F0F0};
          }
        }
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j) {
            acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(flo[TM + j], flo[i], zero16, 0, 0, 0);
            if constexpr (GROUP == 64)
              acc[i][j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fhi[TM + j], fhi[i], acc[i][j], 0, 0, 0);
          }
        fold_group(kt, gi);
      }
    } else if (KS == 1 || kt < KT) {                  // (a quad with one stage fewer idles through the last iteration)
      // multiplies (kt, first half), prepares (kt, second half); then (kt, second half) and (kt+1, first half)
      half_step(std::integral_constant<bool, GROUPED>{}, 0, nxt, off_k0);
      half_step(std::false_type{}, 1, nxt, off_k1);
      if constexpr (GROUPED) fold_group(kt, 0);   // one stage is exactly one 128-wide group
    }
    stage = nxt;
  }
  wait_vmcnt<0>();                                    // drain the trailing reloads
  __syncthreads();                                    // every wave is done with the ring

  // ---- K split: add the quads' accumulators through LDS -------------------------------
  int rb = 0;                                         // first 32-row block of the wave tile this quad finishes
  if constexpr (KS > 1) {
    v4i* red = (v4i*)lds;
    const int t = tid % QT;
    if constexpr (ES == 2) {
      constexpr int UL = TE * TN * 4;                  // 16-byte units each quad receives per thread
      // quad 0 keeps row blocks [0, TE) and sends [TE, TM) into region 1; quad 1 the other way round
#pragma unroll
      for (int ii = 0; ii < TE; ++ii)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            v4i v;
#pragma unroll
            for (int e = 0; e < 4; ++e) v[e] = quad == 0 ? acc[TE + ii][j][4 * g + e] : acc[ii][j][4 * g + e];
            red[((1 - quad) * UL + (ii * TN + j) * 4 + g) * QT + t] = v;
          }
      __syncthreads();
#pragma unroll
      for (int ii = 0; ii < TE; ++ii)
#pragma unroll
        for (int j = 0; j < TN; ++j)
#pragma unroll
          for (int g = 0; g < 4; ++g) {
            const v4i v = red[(quad * UL + (ii * TN + j) * 4 + g) * QT + t];
#pragma unroll
            for (int e = 0; e < 4; ++e)
              acc[ii][j][4 * g + e] = (quad == 0 ? acc[ii][j][4 * g + e] : acc[TE + ii][j][4 * g + e]) + v[e];
          }
      rb = quad * TE;
    } else {
      constexpr int UL = TM * TN * 4;
      if (quad > 0) {
#pragma unroll
        for (int i = 0; i < TM; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j)
#pragma unroll
            for (int g = 0; g < 4; ++g)
              red[((quad - 1) * UL + (i * TN + j) * 4 + g) * QT + t] =
                  v4i{acc[i][j][4 * g], acc[i][j][4 * g + 1], acc[i][j][4 * g + 2], acc[i][j][4 * g + 3]};
      }
      __syncthreads();
      if (quad == 0) {
#pragma unroll
        for (int q = 0; q < KS - 1; ++q)
#pragma unroll
          for (int i = 0; i < TM; ++i)
#pragma unroll
            for (int j = 0; j < TN; ++j)
#pragma unroll
              for (int g = 0; g < 4; ++g) {
                const v4i v = red[(q * UL + (i * TN + j) * 4 + g) * QT + t];
#pragma unroll
                for (int e = 0; e < 4; ++e) acc[i][j][4 * g + e] += v[e];
              }
      }
    }
    __syncthreads();                                  // the staging tiles below reuse this memory
    if (quad >= ES) return;
  }

  // ---- epilogue: row blocks rb .. rb + TE - 1 of the wave tile, held in acc[0 .. TE) -----
  if constexpr (EPI == kInt32) {
#pragma unroll
    for (int i = 0; i < TE; ++i) {
      const int m = m0 + wm + (rb + i) * 32 + frag_row;
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const int n = n0 + wn + j * 32 + 8 * g + 4 * frag_chunk;
          int32_t* dst = (int32_t*)wD + (size_t)m * wN + n;
          if (m < p.M) {
            if (n + 4 <= wN && (wN & 3) == 0) {
              *(v4i*)dst = v4i{acc[i][j][4 * g] >> 8, acc[i][j][4 * g + 1] >> 8, acc[i][j][4 * g + 2] >> 8,
                               acc[i][j][4 * g + 3] >> 8};
            } else {
#pragma unroll
              for (int e = 0; e < 4; ++e)
                if (n + e < wN) dst[e] = acc[i][j][4 * g + e] >> 8;
            }
          }
        }
    }
  } else {
    // dequantise into this wave's private [WM][WN] fp16 tile in LDS ...
    uint8_t* ep = lds + (quad * WPQ + wave) * (TE * 32 * EPI_PITCH);
    float sa[TE];
    float sb[TN][4][4];
    if constexpr (GROUPED) {
      if constexpr (token_scale) {
#pragma unroll
        for (int i = 0; i < TE; ++i) {
          const int m = m0 + wm + (rb + i) * 32 + frag_row;
          sa[i] = (m < p.M ? __half2float(p.As[m]) : 1.f) * 0.00390625f;
        }
      }
    }
    if constexpr (EPI == kRowScale) {
#pragma unroll
      for (int i = 0; i < TE; ++i) sa[i] = __half2float(lds_sa[wm + (rb + i) * 32 + frag_row]);
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int g = 0; g < 4; ++g) {
          const h4 t = *(const h4*)(lds_sa + BM + wn + j * 32 + 8 * g + 4 * frag_chunk);
#pragma unroll
          for (int e = 0; e < 4; ++e) sb[j][g][e] = (float)t[e] * 0.00390625f;
        }
    }
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int nl = j * 32 + 8 * g + 4 * frag_chunk;   // column inside the wave tile
#pragma unroll
        for (int i = 0; i < TE; ++i) {
          h4 v;
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            float f;
            // acc holds 256 * sum (exactly representable in float32: the sum is below 2^24) and sb
            // carries the matching exact factor 2^-8, so this is float(sum) * (a * b) rounded once
            if constexpr (EPI == kRowScale) f = (float)acc[i][j][4 * g + e] * (sa[i] * sb[j][g][e]);
            else f = token_scale ? out[i][j][4 * g + e] * sa[i] : out[i][j][4 * g + e];
            v[e] = (_Float16)round_here(f);
          }
          *(h4*)(ep + (i * 32 + frag_row) * EPI_PITCH + nl * 2) = v;
        }
      }
    constexpr int CPR = WN / 8;                        // 16-byte chunks per row of the wave tile
    constexpr int RPI = 64 / CPR;                      // rows per store instruction
    const int crow = lane / CPR, cchunk = lane % CPR;
    const bool vec_ok = (wN & 7) == 0;
    if constexpr (SWIGLU) {
      // the gate tile (left wave column) and the up tile (right wave column) of this row band are both in LDS after
      // the barrier; each of the two waves combines half of the band's rows and stores 16-byte runs of the product
      __syncthreads();
      const int wcol = wave % WAVES_N;
      const uint8_t* gate_t = lds + (wave - wcol) * (TE * 32 * EPI_PITCH);
      const uint8_t* up_t = gate_t + TE * 32 * EPI_PITCH;
#pragma unroll
      for (int it = 0; it < TE * 32 / (2 * RPI); ++it) {
        const int row = wcol * (TE * 16) + it * RPI + crow;
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
    } else if constexpr (ROPE) {
      // the tile's 128 columns are one head: its first 64 channels sit in the left wave column's staging tile, the other
      // 64 in the right one's; each of the two waves finishes half of the band's rows, both halves of every row.
      // First every row's table entries and cache slot are requested (one memory latency for all of them, overlapping
      // the barrier), then the rows are rotated and stored.
      constexpr int NIT = TE * 32 / (2 * RPI);
      const int wcol = wave % WAVES_N;
      const int head = seg_tile;
      h8 c1[NIT], c2[NIT], s1[NIT], s2[NIT];
      long long slot[NIT];
      int bi[NIT];
      {
        const int m_first = m0 + wm + wcol * (TE * 16) + crow;
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
      const uint8_t* lo_t = lds + (wave - wcol) * (TE * 32 * EPI_PITCH);
      const uint8_t* hi_t = lo_t + TE * 32 * EPI_PITCH;
#pragma unroll
      for (int it = 0; it < NIT; ++it) {
        const int row = wcol * (TE * 16) + it * RPI + crow;
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
    } else {
    // ... and write it out as whole row segments (the tile is private to the wave: no barrier)
#pragma unroll
    for (int it = 0; it < TE * 32 / RPI; ++it) {
      const int row = it * RPI + crow;
      const int m = m0 + wm + rb * 32 + row, n = n0 + wn + cchunk * 8;
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
}

// output columns of a launch over all its weight matrices
int total_n(const GemmArgs& a) {
  int n = a.N;
  for (int s = 1; s < a.n_seg; ++s) n += a.seg_N[s];
  return n;
}

template <int BM, int BN, int WM, int WN, int STAGES, int EPI, int GROUP = 128, int KS = 1, bool SWIGLU = false,
          bool ROPE = false>
int launch(GemmArgs a, hipStream_t stream) {
  constexpr int BNC = SWIGLU ? BN / 2 : BN;           // output channels per tile
  a.tiles_m = (a.M + BM - 1) / BM;
  a.tiles_n = (a.N + BNC - 1) / BNC;
  for (int s = 1; s < a.n_seg; ++s) {                 // further weight matrices: their tiles follow
    a.seg_tile0[s] = a.tiles_n;
    a.tiles_n += (a.seg_N[s] + BN - 1) / BN;
  }
  a.group_m = a.tiles_m < 4 ? a.tiles_m : 4;
  // the ring(s), plus the tile's fp16 scales (one per row, or two blocks of eight groups per row)
  const size_t smem = (size_t)KS * STAGES * (BM + BN) * kStageBytes +
                      (EPI == kRowScale ? (BM + BN) * 2 : (EPI == kGroupScale || EPI == kTokenGroup) ? (BM + BN) * 32 : 0);
  auto kern = gemm_i4_kernel<BM, BN, WM, WN, STAGES, EPI, GROUP, KS, SWIGLU, ROPE>;
  static LdsGrant grant;                               // per instantiation
  if (int rc = reserve_lds((const void*)kern, smem, grant, "gemm")) return rc;
  hipLaunchKernelGGL(kern, dim3(a.tiles_m * a.tiles_n), dim3(64 * (BM / WM) * (BN / WN) * KS), smem, stream, a);
  return check_launch("gemm_i4");
}

// More 256 x 128 tiles than compute units: do 128 x 128 tiles spread evenly what the large ones spread unevenly?  The
// busiest of 256 compute units decides; it finishes a small tile in 0.575 of the time of a large one (measured).
bool prefers_small_tiles(long t256, long t128) { return 0.575 * (double)((t128 + 255) / 256) < (double)((t256 + 255) / 256); }

#ifndef FLH_GEMM_STAGES
#define FLH_GEMM_STAGES 3
#endif

// Tile and K-split choice for the one-scale-per-row and int32 epilogues: the largest tile that
// still gives every compute unit a workgroup (else the smallest), and for the smallest tile with
// at most two workgroups per compute unit, a K split that puts more waves on every SIMD.
// flh_gemm_set_tuning(tile, ks) overrides the choice process-wide (0 = automatic): the hook through which the
// tests reach every variant and a tuning run compares them.
template <int EPI>
int launch_by_shape(const GemmArgs& a, hipStream_t stream) {
  const int env_tile = g_tune_tile.load(std::memory_order_relaxed), env_ks = g_tune_ks.load(std::memory_order_relaxed);
  const int n_all = total_n(a);
  auto tiles = [&](int bm, int bn) { return (long)((a.M + bm - 1) / bm) * ((n_all + bn - 1) / bn); };
  const int kt = a.K >> 7;
  // measured on the Llama shapes at M = 128 ... 4096 (256 compute units): with more large tiles than compute units the
  // 256 x 128 tile wins (two workgroups share a compute unit) unless 128 x 128 tiles spread evenly what it spreads
  // unevenly (a compute unit finishes a small tile in 0.575 of the time of a large one); with at most one large tile per
  // compute unit a long K prefers the large tile split over two quads as soon as the 128 x 128 tiles would come two to a
  // compute unit, else the 128 x 128 tile (split over two quads when there is at most one per compute unit and K is
  // long); below 160 such tiles the 64 x 64 tile with its K splits
  const long t256 = tiles(256, 128), t128 = tiles(128, 128);
  int tile;
  if (t256 > 256) tile = prefers_small_tiles(t256, t128) ? 128 : 256;
  else if (t128 >= 256) tile = kt >= 64 && t128 > 256 ? 256 : 128;
  else tile = t128 >= 160 ? 128 : 64;
  if (env_tile == 256 || env_tile == 128 || env_tile == 64) tile = env_tile;
  const long n_tiles = tile == 256 ? t256 : tile == 128 ? t128 : tiles(64, 64);
  int ks = tile == 256 ? (n_tiles <= 256 ? 2 : 1)
                       : tile == 128 ? (n_tiles <= 256 && kt >= 64 ? 2 : 1) : n_tiles <= 256 ? 4 : n_tiles <= 512 ? 2 : 1;
  if (env_ks == 1 || env_ks == 2 || env_ks == 4) ks = env_ks;
  if (ks == 4 && tile != 64) ks = 2;
  while (ks > 1 && kt / ks < 2) ks >>= 1;
  if (tile == 256) {
    if (ks == 2) return launch<256, 128, 128, 64, FLH_GEMM_STAGES, EPI, 128, 2>(a, stream);
    // one workgroup per compute unit at most: the LDS a second one would have used buys a deeper ring
    // (measured: 7 % on K = 11008, neutral on K = 4096; with two resident workgroups it loses)
    if (n_tiles <= 256) return launch<256, 128, 128, 64, 4, EPI>(a, stream);
    return launch<256, 128, 128, 64, FLH_GEMM_STAGES, EPI>(a, stream);
  }
  if (tile == 128) {
    if (ks == 2) return launch<128, 128, 64, 64, 3, EPI, 128, 2>(a, stream);
    return launch<128, 128, 64, 64, 3, EPI>(a, stream);
  }
  if (ks == 4) return launch<64, 64, 32, 32, 3, EPI, 128, 4>(a, stream);
  if (ks == 2) return launch<64, 64, 32, 32, 3, EPI, 128, 2>(a, stream);
  return launch<64, 64, 32, 32, 3, EPI>(a, stream);
}

template <int EPI>
int launch_grouped(const GemmArgs& a, int group, bool small, hipStream_t stream) {
  if (small) {
    if (group == 64) return launch<64, 64, 32, 32, 3, EPI, 64>(a, stream);
    if (group == 32) return launch<64, 64, 32, 32, 3, EPI, 32>(a, stream);
    return launch<64, 64, 32, 32, 3, EPI>(a, stream);
  }
  if (group == 64) return launch<128, 128, 64, 64, 3, EPI, 64>(a, stream);
  if (group == 32) return launch<128, 128, 64, 64, 3, EPI, 32>(a, stream);
  return launch<128, 128, 64, 64, 3, EPI>(a, stream);
}

int gemm_dispatch(GemmArgs a, int epi, int group, hipStream_t stream) {
  if (a.M == 0 || a.N == 0) return FLH_OK;
  if (gemm_decode_supports(a, epi, group)) return gemm_decode_dispatch(a, epi, stream);
  switch (epi) {
    case kRowScale: return launch_by_shape<kRowScale>(a, stream);
    case kGroupScale: {
      // 128 x 128 tiles; a problem that would leave compute units without one takes 64 x 64 tiles
      const bool small = (long)((a.M + 127) / 128) * ((total_n(a) + 127) / 128) < 200;
      const bool token = a.a_cols == 1 && a.b_cols > 1;
      if (token) return launch_grouped<kTokenGroup>(a, group, small, stream);
      return launch_grouped<kGroupScale>(a, group, small, stream);
    }
    default: return launch_by_shape<kInt32>(a, stream);
  }
}

// SwiGLU launches: tile by the number of 128-column tiles of [gate | up] together; no K split (the epilogue pairs the
// two wave columns of a workgroup)
template <int EPI>
int launch_swiglu(const GemmArgs& a, int group, hipStream_t stream) {
  auto tiles = [&](int bm) { return (long)((a.M + bm - 1) / bm) * ((a.N + 63) / 64); };
  int tile = tiles(256) > 256 ? (prefers_small_tiles(tiles(256), tiles(128)) ? 128 : 256) : tiles(128) >= 160 ? 128 : 64;
  const int forced = g_tune_tile.load(std::memory_order_relaxed);
  if (forced == 256 || forced == 128 || forced == 64) tile = forced;
  if constexpr (EPI == kRowScale) {
    if (tile == 256) return launch<256, 128, 128, 64, FLH_GEMM_STAGES, EPI, 128, 1, true>(a, stream);
    if (tile == 128) return launch<128, 128, 64, 64, 3, EPI, 128, 1, true>(a, stream);
    return launch<64, 64, 32, 32, 3, EPI, 128, 1, true>(a, stream);
  } else {
    (void)group;                                       // groups of 128 only
    if (tile >= 128) return launch<128, 128, 64, 64, 3, EPI, 128, 1, true>(a, stream);
    return launch<64, 64, 32, 32, 3, EPI, 128, 1, true>(a, stream);
  }
}

// q / k / v launches with the rotary embedding and the cache write in the epilogue: 128-column tiles only
template <int EPI>
int launch_qkv_rope(const GemmArgs& a, hipStream_t stream) {
  const long tiles256 = (long)((a.M + 255) / 256) * (total_n(a) / 128), tiles128 = (long)((a.M + 127) / 128) * (total_n(a) / 128);
  int tile = tiles256 > 256 && !prefers_small_tiles(tiles256, tiles128) ? 256 : 128;
  const int forced = g_tune_tile.load(std::memory_order_relaxed);
  if (forced == 256 || forced == 128) tile = forced;
  if constexpr (EPI == kRowScale) {                    // (the group epilogues have one thread per scale row: 128 x 128 only)
    if (tile == 256) return launch<256, 128, 128, 64, FLH_GEMM_STAGES, EPI, 128, 1, false, true>(a, stream);
  }
  return launch<128, 128, 64, 64, 3, EPI, 128, 1, false, true>(a, stream);
}

int check_common(const void* A, const void* B, const void* D, size_t M, size_t N, size_t K) {
  if ((M && N) && (!A || !B || !D)) return fail(FLH_EINVAL, "gemm: null pointer");
  if (misaligned16(A, B, D)) return fail(FLH_EINVAL, "gemm: A, B and D must be 16-byte aligned");
  if (K == 0 || K % 128) return fail(FLH_EINVAL, "gemm: K (%zu) must be a positive multiple of 128", K);
  if (K > 131071 - 127) return fail(FLH_EINVAL, "gemm: K (%zu) too large for the int32 accumulator", K);
  if (M > (1u << 30) || N > (1u << 30)) return fail(FLH_EINVAL, "gemm: M/N too large");
  if (M * (K / 2) > 0xFFFFFFFFull || N * (K / 2) > 0xFFFFFFFFull)
    return fail(FLH_EINVAL, "gemm: packed operands above 4 GiB are not supported");
  return FLH_OK;
}

}  // namespace

}  // namespace flh

using namespace flh;


extern "C" int flh_gemm_set_tuning(int tile, int k_split) {
  if ((tile != 0 && tile != 64 && tile != 128 && tile != 256) || (k_split != 0 && k_split != 1 && k_split != 2 && k_split != 4))
    return fail(FLH_EINVAL, "gemm tuning: tile must be 0, 64, 128 or 256 and k_split 0, 1, 2 or 4");
  g_tune_tile.store(tile, std::memory_order_relaxed);
  g_tune_ks.store(k_split, std::memory_order_relaxed);
  return FLH_OK;
}

extern "C" int flh_gemm_i4_o16(const uint8_t* A, const uint8_t* B, const flh_half* a_scale, const flh_half* b_scale,
                               flh_half* D, size_t M, size_t N, size_t K, int a_cols, int b_cols, int group,
                               void* stream) {
  if (int e = check_common(A, B, D, M, N, K)) return e;
  if (M == 0 || N == 0) return FLH_OK;
  if (!a_scale || !b_scale) return fail(FLH_EINVAL, "gemm: null scale pointer");
  const bool grouped = a_cols != 1 || b_cols != 1;
  if (grouped) {
    if (group != 128 && group != 64 && group != 32)
      return fail(FLH_EINVAL, "gemm: group size %d not supported (32, 64 or 128)", group);
    const int ng = (int)(K / group);
    if ((a_cols != 1 && a_cols != ng) || (b_cols != 1 && b_cols != ng))
      return fail(FLH_EINVAL, "gemm: scale columns (%d, %d) must be 1 or K/group = %d", a_cols, b_cols, ng);
  }
  GemmArgs g{A, B, (const __half*)a_scale, (const __half*)b_scale, D, (int)M, (int)N, (int)K, a_cols, b_cols, 0, 0, 0};
  return gemm_dispatch(g, grouped ? kGroupScale : kRowScale, group, (hipStream_t)stream);
}

extern "C" int flh_gemm_i4_add_o16(const uint8_t* A, const uint8_t* B, const flh_half* a_scale, const flh_half* b_scale,
                                   const flh_half* residual, flh_half* D, size_t M, size_t N, size_t K, int a_cols,
                                   int b_cols, int group, void* stream) {
  if (int e = check_common(A, B, D, M, N, K)) return e;
  if (M == 0 || N == 0) return FLH_OK;
  if (!a_scale || !b_scale) return fail(FLH_EINVAL, "gemm: null scale pointer");
  if (!residual) return fail(FLH_EINVAL, "gemm (residual): null pointer");
  if (misaligned16(residual)) return fail(FLH_EINVAL, "gemm (residual): the residual must be 16-byte aligned");
  const bool grouped = a_cols != 1 || b_cols != 1;
  if (grouped) {
    if (group != 128 && group != 64 && group != 32)
      return fail(FLH_EINVAL, "gemm: group size %d not supported (32, 64 or 128)", group);
    const int ng = (int)(K / group);
    if ((a_cols != 1 && a_cols != ng) || (b_cols != 1 && b_cols != ng))
      return fail(FLH_EINVAL, "gemm: scale columns (%d, %d) must be 1 or K/group = %d", a_cols, b_cols, ng);
  }
  GemmArgs g{A, B, (const __half*)a_scale, (const __half*)b_scale, D, (int)M, (int)N, (int)K, a_cols, b_cols, 0, 0, 0};
  g.R = (const __half*)residual;
  return gemm_dispatch(g, grouped ? kGroupScale : kRowScale, group, (hipStream_t)stream);
}

extern "C" int flh_gemm_i4_swiglu_o16(const uint8_t* A, const uint8_t* B_gate, const uint8_t* B_up, const flh_half* a_scale,
                                      const flh_half* gate_scale, const flh_half* up_scale, flh_half* D, size_t M, size_t N,
                                      size_t K, int a_cols, int b_cols, int group, void* stream) {
  if (int e = check_common(A, B_gate, D, M, N, K)) return e;
  if ((M && N) && !B_up) return fail(FLH_EINVAL, "gemm: null pointer");
  if (misaligned16(B_up)) return fail(FLH_EINVAL, "gemm: A, B and D must be 16-byte aligned");
  if (M == 0 || N == 0) return FLH_OK;
  if (!a_scale || !gate_scale || !up_scale) return fail(FLH_EINVAL, "gemm: null scale pointer");
  const bool grouped = a_cols != 1 || b_cols != 1;
  if (grouped) {
    if (group != 128) return fail(FLH_EINVAL, "gemm (SwiGLU): group-scaled operands need groups of 128, not %d", group);
    const int ng = (int)(K / 128);
    if ((a_cols != 1 && a_cols != ng) || (b_cols != 1 && b_cols != ng))
      return fail(FLH_EINVAL, "gemm: scale columns (%d, %d) must be 1 or K/group = %d", a_cols, b_cols, ng);
  }
  GemmArgs g{A, B_gate, (const __half*)a_scale, (const __half*)gate_scale, D, (int)M, (int)N, (int)K, a_cols, b_cols, 0, 0, 0};
  g.B2 = B_up;
  g.Bs2 = (const __half*)up_scale;
  if (!grouped) return launch_swiglu<kRowScale>(g, group, (hipStream_t)stream);
  if (a_cols == 1) return launch_swiglu<kTokenGroup>(g, group, (hipStream_t)stream);
  return launch_swiglu<kGroupScale>(g, group, (hipStream_t)stream);
}

extern "C" int flh_gemm_i4_qkv_rope_o16(const uint8_t* A, const flh_half* a_scale, const uint8_t* const* B,
                                        const flh_half* const* b_scale, const flh_half* cos, const flh_half* sin,
                                        const int64_t* positions, flh_half* q_out, flh_half* k_cache, flh_half* v_cache,
                                        uint32_t batch, uint32_t T, uint32_t Hq, uint32_t Hkv, uint32_t max_len, size_t K,
                                        int a_cols, int b_cols, int group, void* stream) {
  if (!B || !b_scale) return fail(FLH_EINVAL, "gemm (q/k/v + rotary): null array");
  if (Hq == 0 || Hkv == 0 || max_len == 0) return fail(FLH_EINVAL, "gemm (q/k/v + rotary): heads and cache length must be positive");
  const size_t M = (size_t)batch * T;
  const size_t N[3] = {(size_t)Hq * 128, (size_t)Hkv * 128, (size_t)Hkv * 128};
  flh_half* const D[3] = {q_out, k_cache, v_cache};
  for (int s = 0; s < 3; ++s) {
    if (int e = check_common(A, B[s], D[s], M, N[s], K)) return e;
    if (!b_scale[s]) return fail(FLH_EINVAL, "gemm: null scale pointer");
  }
  if (M == 0) return FLH_OK;
  if (!a_scale || !cos || !sin || !positions) return fail(FLH_EINVAL, "gemm (q/k/v + rotary): null pointer");
  if (misaligned16(cos, sin)) return fail(FLH_EINVAL, "gemm (q/k/v + rotary): cos and sin must be 16-byte aligned");
  if ((uint64_t)batch * Hkv * max_len > (1ull << 40) / 128) return fail(FLH_EINVAL, "gemm (q/k/v + rotary): cache too large");
  const bool grouped = a_cols != 1 || b_cols != 1;
  if (grouped) {
    if (group != 128) return fail(FLH_EINVAL, "gemm (q/k/v + rotary): group-scaled operands need groups of 128, not %d", group);
    const int ng = (int)(K / 128);
    if ((a_cols != 1 && a_cols != ng) || (b_cols != 1 && b_cols != ng))
      return fail(FLH_EINVAL, "gemm: scale columns (%d, %d) must be 1 or K/group = %d", a_cols, b_cols, ng);
  }
  GemmArgs g{A, B[0], (const __half*)a_scale, (const __half*)b_scale[0], q_out, (int)M, (int)N[0], (int)K, a_cols, b_cols, 0, 0, 0};
  g.n_seg = 3;
  for (int s = 1; s < 3; ++s) {
    g.seg_B[s] = B[s];
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
  if (!grouped) return launch_qkv_rope<kRowScale>(g, (hipStream_t)stream);
  if (a_cols == 1 && b_cols > 1) return launch_qkv_rope<kTokenGroup>(g, (hipStream_t)stream);
  return launch_qkv_rope<kGroupScale>(g, (hipStream_t)stream);
}

extern "C" int flh_gemm_i4_o16_multi(const uint8_t* A, const flh_half* a_scale, int count, const uint8_t* const* B,
                                     const flh_half* const* b_scale, flh_half* const* D, const size_t* N, size_t M,
                                     size_t K, int a_cols, int b_cols, int group, void* stream) {
  if (count < 1 || count > kMaxGemmSegments)
    return fail(FLH_EINVAL, "gemm (several weight matrices): count = %d, must be 1 .. %d", count, kMaxGemmSegments);
  if (!B || !b_scale || !D || !N) return fail(FLH_EINVAL, "gemm (several weight matrices): null array");
  if (count == 1) return flh_gemm_i4_o16(A, B[0], a_scale, b_scale[0], D[0], M, N[0], K, a_cols, b_cols, group, stream);
  size_t n_all = 0;
  for (int s = 0; s < count; ++s) {
    if (N[s] == 0) return fail(FLH_EINVAL, "gemm (several weight matrices): N[%d] = 0", s);
    if (int e = check_common(A, B[s], D[s], M, N[s], K)) return e;
    if (!b_scale[s]) return fail(FLH_EINVAL, "gemm: null scale pointer");
    n_all += N[s];
  }
  if (n_all > (1u << 30)) return fail(FLH_EINVAL, "gemm: M/N too large");
  if (M == 0) return FLH_OK;
  if (!a_scale) return fail(FLH_EINVAL, "gemm: null scale pointer");
  const bool grouped = a_cols != 1 || b_cols != 1;
  if (grouped) {
    if (group != 128 && group != 64 && group != 32)
      return fail(FLH_EINVAL, "gemm: group size %d not supported (32, 64 or 128)", group);
    const int ng = (int)(K / group);
    if ((a_cols != 1 && a_cols != ng) || (b_cols != 1 && b_cols != ng))
      return fail(FLH_EINVAL, "gemm: scale columns (%d, %d) must be 1 or K/group = %d", a_cols, b_cols, ng);
  }
  GemmArgs g{A, B[0], (const __half*)a_scale, (const __half*)b_scale[0], D[0], (int)M, (int)N[0], (int)K, a_cols, b_cols, 0, 0, 0};
  g.n_seg = count;
  for (int s = 1; s < count; ++s) {
    g.seg_B[s] = B[s];
    g.seg_Bs[s] = (const __half*)b_scale[s];
    g.seg_D[s] = D[s];
    g.seg_N[s] = (int)N[s];
  }
  return gemm_dispatch(g, grouped ? kGroupScale : kRowScale, group, (hipStream_t)stream);
}

extern "C" int flh_gemm_i4_i32(const uint8_t* A, const uint8_t* B, int32_t* C, size_t M, size_t N, size_t K,
                               void* stream) {
  if (int e = check_common(A, B, C, M, N, K)) return e;
  GemmArgs g{A, B, nullptr, nullptr, C, (int)M, (int)N, (int)K, 1, 1, 0, 0, 0};
  return gemm_dispatch(g, kInt32, 0, (hipStream_t)stream);
}
