// Causal attention of a block of new tokens over a key / value cache (prefill), fp16 with float32 softmax and
// accumulation, heads of 128 channels, grouped queries: what the reference's attention module hands to flash-attn
// after the rotary embedding and the cache update (flh/quantized_model/modeling_llama.py:426-460).  Inputs in the
// layouts the q / k / v GEMM of this library writes: queries token-major [B, T, Hq, 128], keys / values in cache slots
// [B, Hkv, max_len, 128]; query t of the block sees the slots 0 .. past + t.  Output token-major [B, T, Hq * 128], the
// layout the quantiser of o_proj reads.
//
// One workgroup = 4 waves = 128 consecutive queries of one head, 32 per wave; keys in blocks of 64, K and V tiles
// double-buffered in LDS by direct-to-LDS loads (row-major, 16-byte chunks XOR-swizzled by the row; the V tile has a
// swizzle of its own for the transpose loads).  Both products run
// on v_mfma_f32_32x32x16_f16 in transposed form, so that a lane owns one query throughout:
//
//   S^T[key, query] = sum_d K[key, d] Q[query, d]         A = K tile rows from LDS, B = the wave's queries (registers)
//   O^T[d, query]  += sum_key V[key, d] P[query, key]     A = V^T fragments, B = P^T as it sits in the S^T accumulators
//
// The S^T accumulator of lane (query n, half h) holds keys 8 g + 4 h + e (g, e in 0..3) of a 32-key tile, which as B
// operand of the second product means contraction slot 8 h + 4 g' + e <-> key 16 s + 8 g' + 4 h + e for step s; the V^T
// fragment is read to match with the LDS transpose load of this part (ds_read_b64_tr_b16: within 16 lanes, lane i
// receives element i % 4 of the 8-byte rows addressed by lanes i / 4 + 4 j, j = 0..3), i.e. four consecutive keys for
// the lane's channel straight from the row-major tile.  Online softmax in base 2 per lane; only the running maximum is
// exchanged between the two lanes of a query per key block.
#include <atomic>

#include "lane_ops.h"

namespace flh {

namespace {

constexpr int kHeadDim = 128;
constexpr int kQueriesPerBlock = 128;                  // 32 per wave
constexpr int kKeysPerStep = 64;
constexpr int kTileBytes = kKeysPerStep * kHeadDim * 2;   // one K or V tile in LDS (16 KiB)
constexpr int kOutPitch = kHeadDim * 2 + 16;           // bytes per query row of the output staging tile

typedef short s4 __attribute__((ext_vector_type(4)));
typedef short s8 __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) s4 lds_s4;

// byte offset inside a tile of the 16-byte chunk `c` (8 channels) of key row `r`
__device__ __forceinline__ int chunk_at(int r, int c) { return r * (kHeadDim * 2) + ((c ^ (r & 15)) << 4); }
// the same for a V tile, whose swizzle serves the transpose loads: one of them reads 64 bytes (four chunks) of each of
// four consecutive rows, which must fall into four different quarters of the 256-byte bank line
__device__ __forceinline__ int v_swizzle(int r) { return (r & 3) << 2; }
__device__ __forceinline__ int v_chunk_at(int r, int c) { return r * (kHeadDim * 2) + ((c ^ v_swizzle(r)) << 4); }

__global__ __launch_bounds__(256, 2) void prefill_attention_kernel(const __half* __restrict__ q,
                                                                   const __half* __restrict__ k_cache,
                                                                   const __half* __restrict__ v_cache,
                                                                   __half* __restrict__ out, int T, int Hq, int Hkv,
                                                                   int past, int max_len, float scale_log2) {
  extern __shared__ __align__(1024) uint8_t lds[];     // K[2], V[2] tiles; the output staging tile afterwards
  const int tid = threadIdx.x, lane = tid & 63, n = lane & 31, h = lane >> 5;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // workgroup -> (sequence, head, query block): every die takes a contiguous range of (sequence, head) pairs, so the
  // keys / values of a head (of a group of heads that share them) are fetched into one L2 only; within a head the long
  // blocks (late queries) come first
  const int n_blocks = (T + kQueriesPerBlock - 1) / kQueriesPerBlock;
  const unsigned L = xcd_contiguous(blockIdx.x, gridDim.x);
  const int head = (int)((L / n_blocks) % Hq), b = (int)(L / ((unsigned)n_blocks * Hq));
  // a die's 32 compute units take its workgroups in order, two each: every other row of 32 workgroups walks its heads'
  // blocks in the opposite direction, so that a compute unit's two residents are a long and a short block
  // (heads of 32 blocks or more fill whole rows: they keep the long blocks first)
  const bool ascending = n_blocks < 32 && (((L / n_blocks) / (32 / n_blocks)) & 1);
  const int qb = ascending ? (int)(L % n_blocks) : n_blocks - 1 - (int)(L % n_blocks);
  const int hkv = head / (Hq / Hkv);
  const int q_first = qb * kQueriesPerBlock + wave * 32;
  const int my_q = min(q_first + n, T - 1);            // rows past the end repeat the last query; never stored

  // this lane's query as B operand: channels 16 s + 8 h .. + 7
  h8 qf[8];
  {
    const __half* qrow = q + ((size_t)((size_t)b * T + my_q) * Hq + head) * kHeadDim;
#pragma unroll
    for (int s = 0; s < 8; ++s) qf[s] = *(const h8*)(qrow + 16 * s + 8 * h);
  }

  const int total_keys = past + T;
  const int block_keys = min(past + (qb + 1) * kQueriesPerBlock, total_keys);   // slots any query of the block sees
  const int n_steps = (block_keys + kKeysPerStep - 1) / kKeysPerStep;
  const __half* kbase = k_cache + ((size_t)b * Hkv + hkv) * (size_t)max_len * kHeadDim;
  const __half* vbase = v_cache + ((size_t)b * Hkv + hkv) * (size_t)max_len * kHeadDim;
  const unsigned lds0 = (unsigned)(size_t)lds;

  // one load instruction moves four key rows (1 KiB); a wave issues four for K and four for V per step.  A full step
  // takes its rows from a wave-uniform base (the step's first key) plus per-lane byte offsets that never change; the
  // last step of a sequence may run past the end and clamps its rows.
  unsigned k_off[4], v_off[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int r = (wave * 4 + i) * 4 + (lane >> 4);
    k_off[i] = (unsigned)(r * kHeadDim + ((lane & 15) ^ (r & 15)) * 8) * 2;
    v_off[i] = (unsigned)(r * kHeadDim + ((lane & 15) ^ v_swizzle(r)) * 8) * 2;
  }
  auto issue = [&](int step, int buf) {
    const int first = step * kKeysPerStep;
    if (first + kKeysPerStep <= total_keys) {
      const __half* kb = kbase + (size_t)first * kHeadDim;
      const __half* vb = vbase + (size_t)first * kHeadDim;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        load_to_lds16(kb, k_off[i], lds0 + buf * kTileBytes + (wave * 4 + i) * 1024);
        load_to_lds16(vb, v_off[i], lds0 + (2 + buf) * kTileBytes + (wave * 4 + i) * 1024);
      }
    } else {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const int inst = wave * 4 + i;                 // 0 .. 15
        const int r = inst * 4 + (lane >> 4);
        const size_t row = (size_t)min(first + r, total_keys - 1) * kHeadDim;
        load_to_lds16(kbase + row + ((lane & 15) ^ (r & 15)) * 8, lds0 + buf * kTileBytes + inst * 1024);
        load_to_lds16(vbase + row + ((lane & 15) ^ v_swizzle(r)) * 8, lds0 + (2 + buf) * kTileBytes + inst * 1024);
      }
    }
  };

  v16f o[4];                                           // O^T: [channel tile], lane = query, register r = channel 8 (r/4) + 4 h + r % 4
#pragma unroll
  for (int dt = 0; dt < 4; ++dt)
#pragma unroll
    for (int r = 0; r < 16; ++r) o[dt][r] = 0.f;
  float m_run = -INFINITY, l_run = 0.f;                // running maximum (scaled, base 2) and this lane's share of the sum
  const int q_limit = past + my_q;                     // last visible slot of this lane's query

  // per-lane offsets of the V^T transpose loads: lane i of a group of 16 addresses the 8-byte piece (i % 4) of the
  // 32-byte run of channels the group's sixteen lanes will own, in key row i / 4 of the four keys of one load
  const int grp = lane >> 4, gi = lane & 15;
  const int tr_key = gi >> 2;                          // + key0 of the load
  const int tr_half = (gi & 1) << 3;                   // byte inside the 16-byte chunk
  const int tr_chunk0 = ((grp & 1) << 1) + ((gi & 3) >> 1);   // + 4 dt: chunk of 8 channels inside the row
  // the lane's part of a transpose-load address for channel tile dt (the key rows of a load add a constant to it)
  int tr_off[4];
#pragma unroll
  for (int dt = 0; dt < 4; ++dt) tr_off[dt] = v_chunk_at(4 * (grp >> 1) + tr_key, 4 * dt + tr_chunk0) + tr_half;

  issue(0, 0);
  for (int step = 0; step < n_steps; ++step) {
    const int buf = step & 1;
    wait_vmcnt<0>();
    __syncthreads();                                   // tile `step` is complete; everybody is done with the other buffer
    if (step + 1 < n_steps) issue(step + 1, buf ^ 1);
    const uint8_t* kt_lds = lds + buf * kTileBytes;
    const uint8_t* vt_lds = lds + (2 + buf) * kTileBytes;

    // keys a wave's queries cannot see cost it nothing: a 32-key tile past the wave's last query is skipped
    // (the wave still takes part in the loads and barriers of the step)
    const int wave_limit = past + min(q_first + 31, T - 1);
    const int live_tiles = __builtin_amdgcn_readfirstlane(
        step * kKeysPerStep > wave_limit ? 0 : (step * kKeysPerStep + 32 > wave_limit ? 1 : 2));
    if (live_tiles == 0) continue;

    // ---- S^T = K Q^T for two tiles of 32 keys: all fragments are requested first, then the two accumulator chains
    // alternate (a tile the wave cannot see is computed and masked like any other: straight-line code schedules better)
    h8 kf[2][8];
#pragma unroll
    for (int s = 0; s < 8; ++s)
#pragma unroll
      for (int kt = 0; kt < 2; ++kt) kf[kt][s] = *(const h8*)(kt_lds + chunk_at(kt * 32 + n, 2 * s + h));
    __builtin_amdgcn_sched_barrier(0);                 // (keeps the compiler from sinking the reads to their uses)
    v16f st[2];
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int r = 0; r < 16; ++r) st[kt][r] = 0.f;
#pragma unroll
    for (int s = 0; s < 8; ++s)
#pragma unroll
      for (int kt = 0; kt < 2; ++kt) st[kt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(kf[kt][s], qf[s], st[kt], 0, 0, 0);
    // ---- causal mask, online softmax in base 2 on scale_log2 * s (register r of tile kt: key = 64 step + 32 kt +
    // 8 (r/4) + 4 h + r % 4)
    const int key0 = step * kKeysPerStep + 4 * h;
    const bool diagonal = __builtin_amdgcn_readfirstlane(step * kKeysPerStep + kKeysPerStep - 1 > past + q_first);
    float mx = -INFINITY;
    if (diagonal) {                                    // (a branch of its own: most steps carry no mask arithmetic at all;
      asm volatile("" ::: "memory");                   //  the empty statement keeps the compiler from predicating it)
#pragma unroll
      for (int kt = 0; kt < 2; ++kt)
#pragma unroll
        for (int r = 0; r < 16; ++r)
          if (key0 + 32 * kt + 8 * (r >> 2) + (r & 3) > q_limit) st[kt][r] = -INFINITY;
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int r = 0; r < 16; ++r) mx = fmaxf(mx, st[kt][r]);
    mx = fmaxf(mx, lane_xor_f<32>(mx)) * scale_log2;   // (the scale is positive: the maximum commutes with it)
    const float m_new = fmaxf(m_run, mx);              // finite from the first step on: slot 0 is visible to every query
    float sum = 0.f;
    h8 pb[2][2];                                       // P^T as B operand: [tile][step of 16 slots]
#pragma unroll
    for (int kt = 0; kt < 2; ++kt)
#pragma unroll
      for (int ks = 0; ks < 2; ++ks)
#pragma unroll
        for (int i = 0; i < 8; ++i) {
          const float p = __builtin_amdgcn_exp2f(__builtin_fmaf(st[kt][8 * ks + i], scale_log2, -m_new));
          sum += p;
          pb[kt][ks][i] = (_Float16)p;
        }
    // rescale what has been accumulated -- unless no lane's maximum moved (the common case after the first steps)
    if (__builtin_amdgcn_ballot_w64(m_new != m_run) != 0) {
      const float alpha = __builtin_amdgcn_exp2f(m_run - m_new);
      l_run *= alpha;
#pragma unroll
      for (int dt = 0; dt < 4; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) o[dt][r] *= alpha;
      m_run = m_new;
    }
    l_run += sum;
    // ---- O^T += V^T P^T
#pragma unroll
    for (int kt = 0; kt < 2; ++kt) {
      if (kt >= live_tiles) break;
#pragma unroll
      for (int ks = 0; ks < 2; ++ks) {
        // this half-wave's slots 8 h .. 8 h + 7 are keys 32 kt + 16 ks + 4 h + {0..3} and + 8 + {0..3}
        // (rows 32 kt + 16 ks and + 8 on: multiples of four, which the V swizzle does not see)
#pragma unroll
        for (int dt = 0; dt < 4; ++dt) {
          const uint8_t* at = vt_lds + tr_off[dt] + (32 * kt + 16 * ks) * (kHeadDim * 2);
          const s4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4*)at);
          const s4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_s4*)(at + 8 * (kHeadDim * 2)));
          const h8 a = __builtin_bit_cast(h8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
          o[dt] = __builtin_amdgcn_mfma_f32_32x32x16_f16(a, pb[kt][ks], o[dt], 0, 0, 0);
        }
      }
    }
  }

  // ---- normalise, transpose through LDS, store whole rows
  const float l_all = l_run + lane_xor_f<32>(l_run);
  const float inv = 1.0f / l_all;
  __syncthreads();                                     // every wave is done with the tiles
  uint8_t* stage = lds + wave * (32 * kOutPitch);
#pragma unroll
  for (int dt = 0; dt < 4; ++dt)
#pragma unroll
    for (int g = 0; g < 4; ++g) {
      h4 v;
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = (_Float16)(o[dt][4 * g + e] * inv);
      *(h4*)(stage + n * kOutPitch + (32 * dt + 8 * g + 4 * h) * 2) = v;
    }
  // (the staging tile is private to the wave: a wave-level wait is enough)
  __builtin_amdgcn_s_waitcnt(0xc07f);                  // lgkmcnt(0)
  __builtin_amdgcn_wave_barrier();
#pragma unroll
  for (int it = 0; it < 8; ++it) {
    const int row = it * 4 + (lane >> 4), c = lane & 15;
    const int tq = q_first + row;
    const v4i v = *(const v4i*)(stage + row * kOutPitch + c * 16);
    if (tq < T) *(v4i*)(out + ((size_t)((size_t)b * T + tq) * Hq + head) * kHeadDim + c * 8) = v;
  }
}

}  // namespace

}  // namespace flh

using namespace flh;

extern "C" int flh_prefill_attention_f16(const flh_half* q, const flh_half* k_cache, const flh_half* v_cache, flh_half* out,
                                         uint32_t B, uint32_t T, uint32_t Hq, uint32_t Hkv, uint32_t head_dim, uint32_t past,
                                         uint32_t max_len, float scale, void* stream) {
  if (!q || !k_cache || !v_cache || !out) return fail(FLH_EINVAL, "prefill_attention: null pointer");
  if (misaligned16(q, k_cache, v_cache, out)) return fail(FLH_EINVAL, "prefill_attention: tensors must be 16-byte aligned");
  if (head_dim != kHeadDim) return fail(FLH_EINVAL, "prefill_attention: head_dim (%u) must be 128", head_dim);
  if (Hq == 0 || Hkv == 0 || Hq % Hkv) return fail(FLH_EINVAL, "prefill_attention: %u query heads do not divide into %u key / value heads", Hq, Hkv);
  if ((uint64_t)past + T > max_len) return fail(FLH_EINVAL, "prefill_attention: past (%u) + T (%u) exceeds the cache length %u", past, T, max_len);
  if (B == 0 || T == 0) return FLH_OK;
  if ((uint64_t)B * Hq * ((T + kQueriesPerBlock - 1) / kQueriesPerBlock) > 0x7FFFFFFFull || (uint64_t)B * T * Hq * kHeadDim > (1ull << 40) || (uint64_t)B * Hkv * max_len * kHeadDim > (1ull << 40) ||
      (uint64_t)past + T > (1u << 30))
    return fail(FLH_EINVAL, "prefill_attention: problem too large");
  if (!(scale > 0.f)) return fail(FLH_EINVAL, "prefill_attention: the scale must be positive");
  const size_t smem = 4 * (size_t)kTileBytes;          // 64 KiB: two workgroups per compute unit
  static_assert(4 * 32 * kOutPitch <= 4 * kTileBytes, "the output staging tiles reuse the K / V buffers");
  static LdsGrant grant;
  if (int rc = reserve_lds((const void*)prefill_attention_kernel, smem, grant, "prefill_attention")) return rc;
  const unsigned blocks = (T + kQueriesPerBlock - 1) / kQueriesPerBlock;
  hipLaunchKernelGGL(prefill_attention_kernel, dim3(blocks * Hq * B), dim3(256), smem, (hipStream_t)stream, (const __half*)q,
                     (const __half*)k_cache, (const __half*)v_cache, (__half*)out, (int)T, (int)Hq, (int)Hkv, (int)past,
                     (int)max_len, scale * 1.4426950408889634f);
  return check_launch("prefill_attention");
}
