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
  static_assert(!GROUPED || SCROWS <= T, "one thread per scale row");

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
  auto issue_stage = [&](int stage, int kt) __attribute__((always_inline)) {
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
  // (the second half of the middle chunk gets an offset of its own that the compiler cannot see through: adjacent
  // 8-byte reads would be merged into one 16-byte read again and taken apart with copy instructions)
  int c1b = c1 + 8;
  asm("" : "+v"(c1b));
  const int a_base = (wm + frag_row) * kBlockBytes, b_base = (BM + wn + frag_row) * kBlockBytes;

  constexpr int NF = TM + TN;                          // fragments per stage (A first, then B)
  // The 48 bytes a lane reads of a row are the operands of two MFMAs, 24 bytes (six registers) each.  They are read as
  // 16 + 8 and 8 + 16 bytes, so that every piece lands in the registers of the operand it belongs to and no copy
  // instruction is needed to assemble an operand (a 16-byte read of the middle chunk would straddle the two).
  v4i fa[2][NF], fd[2][NF];                            // [parity][fragment]: bytes 0-15 and 32-47 of the lane's 48
  v2i fb[2][NF], fc[2][NF];                            // ... bytes 16-23 and 24-31
  // All fragments of a stage are read one stage ahead of the MFMAs that use them.
  // byte offset of fragment f's row inside a stage: every fragment gets an offset register of its own that the compiler
  // cannot see through, or it would merge
  // the 8-byte reads of two fragments (3072 bytes apart) into one instruction with four result registers and take
  // them apart again with copy instructions.
  int frag_off[NF];
#pragma unroll
  for (int f = 0; f < NF; ++f) {
    frag_off[f] = f < TM ? a_base + f * 32 * kBlockBytes : b_base + (f - TM) * 32 * kBlockBytes;
    if (f != 0 && f != TM) asm("" : "+v"(frag_off[f]));
  }
  auto read_frag = [&](auto par_tag, auto f_tag, int stage) __attribute__((always_inline)) {
    constexpr int par = decltype(par_tag)::value, f = decltype(f_tag)::value;
    const uint8_t* row = lds + stage * STAGE + frag_off[f];
    fa[par][f] = *(const v4i*)(row + c0);
    fb[par][f] = *(const v2i*)(row + c1);
    fc[par][f] = *(const v2i*)(row + c1b);
    fd[par][f] = *(const v4i*)(row + c2);
  };
  auto read_stage = [&](auto par_tag, int stage) __attribute__((always_inline)) {
    static_for<NF>([&](auto f_tag) { read_frag(par_tag, f_tag, stage); });
  };
  auto operand = [&](int par, int f, int m) {
    const v4i a = fa[par][f], d = fd[par][f];
    const v2i b = fb[par][f], c = fc[par][f];
    return m == 0 ? v8i{a[0], a[1], a[2], a[3], b[0], b[1], 0, 0} : v8i{c[0], c[1], d[0], d[1], d[2], d[3], 0, 0};
  };
  auto mfma_stage = [&](int par) __attribute__((always_inline)) {
#pragma unroll
    for (int m = 0; m < 2; ++m)
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(operand(par, TM + j, m), operand(par, i, m),
                                                                     acc[i][j], kBf6, kBf6, 0, 0, 0, 0);
  };

  // ---- group scales travel through LDS, eight groups (= eight K steps) at a time.  Thread t owns row t of the tile's
  // BM activation rows and BN weight rows (with one scale per token: of the BN weight rows only).  In the first step of
  // a block of eight it requests the row's eight scales of the NEXT block -- one 16-byte load where rows of scales are
  // dword-aligned runs of at least eight, else eight clamped 2-byte loads -- and in the block's second step, behind
  // that step's full wait and barrier, it stores them transposed into scl[block & 1][group - first][row], where a step
  // reads a lane's channel scale as one 2-byte piece and four tokens' scales as one 8-byte run.  (One 2-byte request
  // per row and group costs as many cache-line requests as the operands themselves.)  The two steps with this extra
  // work are code of their own; the other steps of a block stay free of branches, which the interleaving of matrix
  // and vector work below depends on.
  constexpr int SCR = token_scale ? BN : SCROWS;       // rows of scales kept
  constexpr int SCR0 = token_scale ? BM : 0;           // first tile row that has any
  __half* const scl = (__half*)(lds + STAGES * STAGE); // [2][8][SCR]
  const int sc_row = min(tid, SCROWS - 1);             // (threads past the last row repeat it)
  const bool sc_active = tid < SCROWS && tid >= SCR0;
  const int sc_cols = sc_row < BM ? p.a_cols : p.b_cols;
  const int sc_brow = sc_row - BM;                     // weight row of the tile this thread fetches scales for
  const bool sc_second = SWIGLU && sc_brow >= BNC;
  const unsigned short* const sc_src =
      (const unsigned short*)(sc_row < BM ? p.As + (size_t)min(m0 + sc_row, p.M - 1) * p.a_cols
                                          : (sc_second ? p.Bs2 : wBs) +
                                                (size_t)min(n0 + (sc_second ? sc_brow - BNC : sc_brow), wN - 1) * p.b_cols);
  // 16-byte requests need dword-aligned rows of at least eight scales; decided per launch and operand, so that every
  // thread of the workgroup derives the same first group of a block
  const int ng = p.K / 128;
  auto runs_ok = [&](const void* base, int cols) { return cols >= 8 && !(cols & 1) && !((uintptr_t)base & 3); };
  const bool fast_a = token_scale || runs_ok(p.As, p.a_cols);
  const bool fast_b = runs_ok(wBs, p.b_cols) && (!SWIGLU || runs_ok(p.Bs2, p.b_cols));
  auto first_of = [&](int blk, bool fast) { return fast ? min(8 * blk, ng - 8) : 8 * blk; };   // first group of a block
  v4i sraw = {0, 0, 0, 0};                             // eight scales, two per register
  auto sc_issue = [&](int blk) __attribute__((always_inline)) {
    if (sc_active) {
      const bool fast = sc_row < BM ? fast_a : fast_b;
      const int g0 = first_of(blk, fast);
      if (fast) {
        __builtin_memcpy(&sraw, __builtin_assume_aligned(sc_src + g0, 4), 16);
      } else {
#pragma unroll
        for (int i = 0; i < 4; ++i)
          sraw[i] = (int)((unsigned)sc_src[min(g0 + 2 * i, sc_cols - 1)] | (unsigned)sc_src[min(g0 + 2 * i + 1, sc_cols - 1)] << 16);
      }
    }
  };
  auto sc_store = [&](int blk) __attribute__((always_inline)) {
    if (sc_active) {
      unsigned short* dst = (unsigned short*)scl + (blk & 1) * 8 * SCR + (sc_row - SCR0);
#pragma unroll
      for (int i = 0; i < 8; ++i) dst[i * SCR] = (unsigned short)((unsigned)sraw[i >> 1] >> (16 * (i & 1)));
    }
  };
  // One group (= one stage): each 32 x 32 tile's two MFMAs start from zero, and the exact sums are folded into the
  // float32 result -- out = fma(sum, a_g * b_g, out) (token scale: fma(sum, b_g, out)) in ascending g, which is the
  // int8 kernel's arithmetic without its int -> float conversion.  The fold of a tile is sixteen vector instructions
  // that must not wait for the tile's own MFMAs, so the tiles form a software pipeline that runs across the stages:
  // step s issues the two MFMAs of tile s and, between and after them, folds tile s - 1 (whose sums are complete by
  // then); the last tile of a stage is folded during the first step of the next stage, with the scales of its own
  // stage kept in registers.  Every accumulator still sees its groups in ascending order.
  //
  // Operand roles.  With one scale per row (and for int32 output) the weights are the MFMA's first operand: an output
  // lane then holds one token (lane % 32) and four consecutive channels per register quad, which packs into 8-byte
  // writes of the staging tile.  With group scales the activations are the first operand instead: a lane holds one
  // CHANNEL (lane % 32) and, in register 4 q + e, the token 8 q + 4 (lane / 32) + e of the 32 x 32 tile -- the weight
  // scale of a group is then one register per lane and column block, and a tile's fold is sixteen plain float32
  // multiply-adds on it (the mixed-precision multiply-add that would take a half-precision scale straight from a
  // register issues at half that rate).
  v16f pend;                                           // sums of the tile whose fold is outstanding: a stage's last
  float pend_sb = 0.f;                                 // ... the weight scale of the lane's channel in that tile
  h4 pend_sa[4];                                       // ... and the activation scales of its sixteen tokens (group scales)
#pragma unroll
  for (int r = 0; r < 16; ++r) pend[r] = 0.f;
#pragma unroll
  for (int q = 0; q < 4; ++q) pend_sa[q] = h4{(_Float16)0.f, (_Float16)0.f, (_Float16)0.f, (_Float16)0.f};
  auto fold = [&](int i, int j, const v16f& t, float sb, const h4* sa4) __attribute__((always_inline)) {
#pragma unroll
    for (int q = 0; q < 4; ++q)
#pragma unroll
      for (int e = 0; e < 4; ++e)
        acc[i][j][4 * q + e] = __builtin_fmaf(t[4 * q + e], token_scale ? sb : (float)sa4[q][e] * sb, acc[i][j][4 * q + e]);
  };
  constexpr int FOLD_V = token_scale ? 16 : 32;        // vector instructions of one tile's fold
  // tile n of a stage: row blocks in order, column blocks back and forth; tile 0 is (0, 0)
  constexpr int LAST = TM * TN - 1;
  constexpr int LAST_I = LAST / TN, LAST_J = (LAST / TN) & 1 ? TN - 1 - LAST % TN : LAST % TN;
  auto mfma_fold = [&](auto par_tag, int kt, int stage, int nxt) __attribute__((always_inline)) {
    constexpr int par = decltype(par_tag)::value;
    // this step's group inside its block of eight (the last block of a row of scales may start early, see first_of)
    const int blk = kt >> 3;
    const __half* sgb = scl + ((blk & 1) * 8 + kt - first_of(blk, fast_b)) * SCR - SCR0;
    const __half* sga = scl + ((blk & 1) * 8 + kt - first_of(blk, fast_a)) * SCR - SCR0;
    const v16f zero = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    // this group's scales, then -- spread over the step -- the next stage's fragments
    float sb[TN];
    h4 sa[TM][4];
#pragma unroll
    for (int j = 0; j < TN; ++j)   // (kept as a float32 register: folded into the multiply-adds it would make them half rate)
      sb[j] = round_here(__half2float(sgb[BM + wn + j * 32 + frag_row]));
    if constexpr (!token_scale) {
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int q = 0; q < 4; ++q) sa[i][q] = *(const h4*)(sga + wm + i * 32 + 8 * q + 4 * frag_chunk);
    }
    read_stage(std::integral_constant<int, par ^ 1>{}, nxt);
    static_for<TM * TN>([&](auto n_tag) {
      constexpr int n = decltype(n_tag)::value;
      constexpr int i = n / TN, j = i & 1 ? TN - 1 - n % TN : n % TN;
      v16f cur = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(operand(par, i, 0), operand(par, TM + j, 0), zero, kBf6, kBf6,
                                                                 0, 0, 0, 0);
      cur = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(operand(par, i, 1), operand(par, TM + j, 1), cur, kBf6, kBf6, 0, 0,
                                                            0, 0);
      if constexpr (n == 0) {
        fold(LAST_I, LAST_J, pend, pend_sb, pend_sa);
      } else {
        constexpr int ip = (n - 1) / TN, jp = ip & 1 ? TN - 1 - (n - 1) % TN : (n - 1) % TN;
        fold(ip, jp, pend, sb[jp], sa[ip]);
      }
      pend = cur;
    });
    pend_sb = sb[LAST_J];
    if constexpr (!token_scale) {
#pragma unroll
      for (int q = 0; q < 4; ++q) pend_sa[q] = sa[LAST_I][q];
    }
    // issue order per tile: MFMA, half of the previous tile's fold, MFMA, the other half, with the LDS reads of the next
    // stage's fragments (four per fragment) spread evenly between them
    constexpr int NT = TM * TN, RD = 4 * NF, ADDR = 3;
    static_for<NT>([&](auto n_tag) {
      constexpr int n = decltype(n_tag)::value;
      // (ADDR more per slot: the address arithmetic of the fragment reads, which would otherwise pile up behind the
      // last MFMA)
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, FOLD_V / 2 + ADDR, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, RD * (2 * n + 1) / (2 * NT) - RD * (2 * n) / (2 * NT), 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x002, FOLD_V - FOLD_V / 2 + ADDR, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, RD * (2 * n + 2) / (2 * NT) - RD * (2 * n + 1) / (2 * NT), 0);
    });
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
  // one scale per token, applied after the groups: the tile's BM of them are parked in LDS behind the group scales now,
  // so that the epilogue does not start with a round trip to memory per row
  __half* const tok_sa = scl + 2 * 8 * SCR;            // [BM]
  if constexpr (token_scale) {
    if (tid < BM) tok_sa[tid] = p.As[min(m0 + tid, p.M - 1)];
  }
  if constexpr (GROUPED) sc_issue(0);
  // REFILL_OWN (three-stage rings): a stage's fragments are read into registers one step before they are multiplied, so
  // its slot is free a step before the classic ring order would refill it.  The whole ring is requested up front and a
  // step refills the slot of the stage it multiplies: every stage then has two steps to arrive instead of one, at the
  // same LDS footprint -- what weights that come from HBM rather than from the last-level cache need.
#ifndef FLH_F6_REFILL_OWN
#define FLH_F6_REFILL_OWN 1
#endif
  constexpr bool REFILL_OWN = FLH_F6_REFILL_OWN && STAGES == 3;
  constexpr int AHEAD = REFILL_OWN ? STAGES : STAGES - 1;   // stages in flight or waiting beyond the one being multiplied
#pragma unroll
  for (int s = 0; s < AHEAD; ++s) issue_stage(s, s);
  if constexpr (GROUPED) sc_store(0);                   // (the compiler waits for its own loads here)
  wait_stages(std::integral_constant<int, AHEAD - 1>{});   // stage 0 has landed (this wave's part)
  if constexpr (EPI == kRowScale) {
#pragma unroll
    for (int i = 0; i < (BM + BN + T - 1) / T; ++i) {
      const int e = tid + i * T;
      if (e < BM + BN) lds_sa[e] = scale_reg[i];
    }
  }
  __syncthreads();
  read_stage(std::integral_constant<int, 0>{}, 0);

  // one K step; `par` (a compile-time constant) says which half of the fragment registers feeds the MFMAs, `stage`
  // which ring slot holds the step's operands, `hook` whether the step also requests (1) or stores (2) the next block
  // of group scales
  auto k_step = [&](auto par_tag, auto hook_tag, const int stage, int kt) __attribute__((always_inline)) {
    constexpr int par = decltype(par_tag)::value, hook = decltype(hook_tag)::value;
    const int nxt = stage + 1 == STAGES ? 0 : stage + 1, fill = stage == 0 ? STAGES - 1 : stage - 1;
    wait_stages(std::integral_constant<int, AHEAD - 2>{});   // this wave's part of stage kt+1 has landed
    // ... everybody's has, and stage kt-1 is free: its fragment reads were consumed an iteration ago; the LDS
    // reads still in flight here belong to stage kt, which nobody overwrites before the next barrier -- unless this
    // step refills that very slot: then every wave lets its reads of stage kt finish before it signals
    if constexpr (REFILL_OWN) wait_lgkmcnt0();
    barrier_no_fence();
    // the next block's scales, requested in the previous step (everything outstanding has been waited for); the
    // buffer they go to was last read in the previous block, which every wave has left by now
    if constexpr (hook == 2) sc_store((kt >> 3) + 1);
    issue_stage(REFILL_OWN ? stage : fill, kt + AHEAD);
    if constexpr (hook == 1) sc_issue((kt >> 3) + 1);   // ordinary loads; the full wait at the top of the next step covers them
    if constexpr (GROUPED) {
      mfma_fold(par_tag, kt, stage, nxt);
    } else {
      // fragment reads run one stage ahead of the MFMAs that use them
      read_stage(std::integral_constant<int, par ^ 1>{}, nxt);
      mfma_stage(par);
    }
    __builtin_amdgcn_sched_barrier(0);
  };
  constexpr std::integral_constant<int, 0> c0_{};
  constexpr std::integral_constant<int, 1> c1_{};
  constexpr std::integral_constant<int, 2> c2_{};
  int kt = 0;
  if constexpr (GROUPED) {
    // blocks of eight steps: the first requests the next block's scales, the second stores them, the others come in
    // pairs (the fragment parity repeats); the ring slot is a run-time value (with more steps in one block of code the
    // compiler neither keeps the interleaving nor does without register copies)
    static_assert(STAGES == 3, "the scale requests rely on the full wait at the top of every step");
    int stage = 0;
    auto next = [&]() { stage = stage + 1 == STAGES ? 0 : stage + 1; };
    while (kt < KT) {
      const int n = min(8, KT - kt);
      k_step(c0_, c1_, stage, kt), next();
      if (n > 1) k_step(c1_, c2_, stage, kt + 1), next();
      int u = 2;
      for (; u + 2 <= n; u += 2) {
        k_step(c0_, c0_, stage, kt + u), next();
        k_step(c1_, c0_, stage, kt + u + 1), next();
      }
      if (u < n) k_step(c0_, c0_, stage, kt + u), next();
      kt += n;
    }
  } else {
    // as many steps per iteration as it takes for parity and ring slot to repeat: both are compile-time constants then,
    // every LDS address of a step is a per-lane register that never changes plus an immediate offset, and the loop has no
    // vector instruction besides the MFMAs
    constexpr int UNROLL = STAGES % 2 ? 2 * STAGES : STAGES;
    for (; kt + UNROLL <= KT; kt += UNROLL)
      static_for<UNROLL>([&](auto u) { k_step(std::integral_constant<int, decltype(u)::value % 2>{}, c0_, decltype(u)::value % STAGES, kt + decltype(u)::value); });
    static_for<UNROLL - 1>([&](auto u) {               // the remaining steps
      if (kt + decltype(u)::value < KT)
        k_step(std::integral_constant<int, decltype(u)::value % 2>{}, c0_, decltype(u)::value % STAGES, kt + decltype(u)::value);
    });
  }
  if constexpr (GROUPED) fold(LAST_I, LAST_J, pend, pend_sb, pend_sa);   // the last stage's last tile
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
    if constexpr (GROUPED) {
      // a lane holds one channel and sixteen tokens per 32 x 32 tile (see "operand roles" above)
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          h4 sa4 = {(_Float16)1.f, (_Float16)1.f, (_Float16)1.f, (_Float16)1.f};
          if constexpr (token_scale) sa4 = *(const h4*)(tok_sa + wm + i * 32 + 8 * q + 4 * frag_chunk);
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            const int ml = i * 32 + 8 * q + 4 * frag_chunk + e;   // row inside the wave tile
#pragma unroll
            for (int j = 0; j < TN; ++j) {
              const float f = token_scale ? acc[i][j][4 * q + e] * (float)sa4[e] : acc[i][j][4 * q + e];
              *(_Float16*)(ep + ml * EPI_PITCH + (j * 32 + frag_row) * 2) = (_Float16)round_here(f);
            }
          }
        }
    } else {
    float sa[TM];
#pragma unroll
    for (int i = 0; i < TM; ++i) sa[i] = __half2float(lds_sa[wm + i * 32 + frag_row]);
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int g = 0; g < 4; ++g) {
        const int nl = j * 32 + 8 * g + 4 * frag_chunk;   // column inside the wave tile
        const h4 t = *(const h4*)(lds_sa + BM + wn + nl);
#pragma unroll
        for (int i = 0; i < TM; ++i) {
          h4 v;
#pragma unroll
          for (int e = 0; e < 4; ++e)   // row scales: float(sum) * (a * b), the scale product is exact, the result rounded once
            v[e] = (_Float16)round_here(acc[i][j][4 * g + e] * (sa[i] * (float)t[e]));
          *(h4*)(ep + (i * 32 + frag_row) * EPI_PITCH + nl * 2) = v;
        }
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
                      (EPI == kRowScale ? (BM + BN) * 2 : EPI == kGroupScale ? (BM + BN) * 32 : EPI == kTokenGroup ? BN * 32 + BM * 2 : 0);
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
  // (the eight-wave tile of launch_f6_by_shape only when forced: with one workgroup per compute unit nothing overlaps
  // this epilogue's exchange and stores -- 155.5 against 150.0 us on weights from HBM, 152 against 133 us on cached ones)
  if constexpr (EPI == kRowScale)
    if (forced == 256) tile = 256;
  if (forced == 128 || forced == 64) tile = forced;
  if constexpr (EPI == kRowScale)
    if (tile == 256) return launch_f6<256, 128, 64, 64, 4, EPI, true>(a, stream);
  if (tile == 128) return launch_f6<128, 128, 64, 64, 3, EPI, true>(a, stream);
  return launch_f6<64, 64, 32, 32, 3, EPI, true>(a, stream);
}

// flh_gemm_set_tuning overrides the tile choice (256 / 128 / 64; the hook through which the tests cover every variant)
template <int EPI>
int launch_f6_by_shape(const GemmArgs& a, hipStream_t stream) {
  const int env_tile = g_tune_tile.load(std::memory_order_relaxed);
  const int n_all = total_n_f6(a);
  auto tiles = [&](int bm, int bn) { return (long)((a.M + bm - 1) / bm) * ((n_all + bn - 1) / bn); };
  // Measured at M = 2048 / 4096 on the Llama shapes.  With the same weights launched back to back (they then sit in the
  // last-level cache) two 128 x 128 workgroups per compute unit beat one 256 x 128 workgroup of eight waves by 2-6 %;
  // with weights that come from HBM -- every launch of a model, whose layers' weights do not fit that cache -- the
  // eight-wave tile with its four-stage ring is 12-16 % faster at every shape (gate + up 148 against 170 us, q + k + v
  // 79 against 90, down 61 against 72, o 27.5 against 31.5): it requests three quarters of the operand bytes per unit
  // of matrix work and a step further ahead.  It is taken as soon as there is one such tile per compute unit.
  int tile = tiles(256, 128) >= 256 ? 256 : tiles(128, 128) >= 256 ? 128 : 64;
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
  if (rows_only) {
    const int forced = g_tune_tile.load(std::memory_order_relaxed);
    const long tiles256 = (long)((g.M + 255) / 256) * ((total_n_f6(g) + 127) / 128);
    if (forced == 256 || (forced == 0 && tiles256 >= 256))
      return launch_f6<256, 128, 64, 64, 4, kRowScale, false, true>(g, (hipStream_t)stream);
    return launch_f6<128, 128, 64, 64, 3, kRowScale, false, true>(g, (hipStream_t)stream);
  }
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
