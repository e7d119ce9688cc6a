// Shared declarations of the int4 GEMM translation units.
#pragma once
#include <atomic>

#include "common.h"

namespace flh {

// kTokenGroup: group-scaled weights with one activation scale per token, applied after the groups
enum Epilogue { kRowScale = 0, kGroupScale = 1, kInt32 = 2, kTokenGroup = 3 };

constexpr int kMaxGemmSegments = 4;

// tile / K-split override of the shape heuristics (0 = automatic), set by flh_gemm_set_tuning
extern std::atomic<int> g_tune_tile, g_tune_ks;

struct GemmArgs {
  const uint8_t* A;     // [M, K/2] packed activations
  const uint8_t* B;     // [N, K/2] packed weights
  const __half* As;     // [M, a_cols]
  const __half* Bs;     // [N, b_cols]
  void* D;              // [M, N] fp16 (int32 for kInt32)
  int M, N, K;          // K in codes
  int a_cols, b_cols;   // scale columns (1 or K/group)
  int tiles_m, tiles_n, group_m;
  // Further weight matrices that share A (q / k / v, gate / up): segment s > 0 starts at output-column tile
  // seg_tile0[s] of the launch and has its own B, scales, output and N; segment 0 is B / Bs / D / N above.
  int n_seg;            // 0 or 1: a single weight matrix
  int seg_tile0[kMaxGemmSegments];
  int seg_N[kMaxGemmSegments];
  const uint8_t* seg_B[kMaxGemmSegments];
  const __half* seg_Bs[kMaxGemmSegments];
  void* seg_D[kMaxGemmSegments];
  // SwiGLU launches (gate = B / Bs, up = B2 / Bs2, N = channels of each, D [M, N] = fp16(fp16(silu(gate)) * up))
  const uint8_t* B2;
  const __half* Bs2;
  // q / k / v launches with the rotary embedding and the cache write in the epilogue (three segments q, k, v of heads of
  // 128 channels; row m = b * rope_T + t): q -> D [M, N] rotated; k -> seg_D[1] = key cache [B, rope_hkv, rope_max_len,
  // 128] at slot rope_pos[t], rotated; v -> seg_D[2] = value cache, as it is.  cos / sin [rope_T, 128].
  const __half* rope_cos;
  const __half* rope_sin;
  const long long* rope_pos;
  int rope_T, rope_max_len, rope_hkv;
  // residual (single weight matrix, fp16 output): D = fp16(R + fp16(the launch's result)), R [M, N]; may be D itself
  const __half* R;
};

// Small-M (decode) kernels: weight-streaming, split over K inside a workgroup.
constexpr int kDecodeMaxM = 64;
bool gemm_decode_supports(const GemmArgs& a, int epi, int group);
int gemm_decode_dispatch(const GemmArgs& a, int epi, hipStream_t stream);

}  // namespace flh
