// Rotary position embedding of the query / key projections and the write of the new keys / values into a
// preallocated cache, in one launch: what a decode step otherwise spends a dozen elementwise launches on between the
// q / k / v GEMM and attention (transformers' apply_rotary_pos_emb and cache update as the reference calls them,
// flh/quantized_model/modeling_llama.py:403-424).  fp16 arithmetic with the roundings of the tensor expression
// x * cos + rotate_half(x) * sin evaluated op by op: fp16(fp16(x cos) + fp16(rot(x) sin)).
#include "common.h"

namespace flh {
namespace {

// One lane: the 8 consecutive channels at chunk c of one head vector of `d` channels AND their rotation partners d/2
// channels away (chunk c + d/16).  A lane reads both pieces before it writes either and no other lane touches them, so
// rotating the queries in place is safe for every head width (a lane per piece would have to rely on its partner's
// loads preceding its own store, which holds only while both sit in one wave).
// Item order: all query heads of a token, then its key heads, then its value heads.
__global__ __launch_bounds__(256) void rope_kv_cache_kernel(__half* __restrict__ q, const __half* __restrict__ k,
                                                            const __half* __restrict__ v, const __half* __restrict__ cos,
                                                            const __half* __restrict__ sin,
                                                            const long long* __restrict__ positions,
                                                            __half* __restrict__ k_cache, __half* __restrict__ v_cache,
                                                            uint32_t B, uint32_t T, uint32_t Hq, uint32_t Hkv, uint32_t d,
                                                            uint32_t max_len) {
  const uint32_t lph = d / 16;                         // lanes per head vector
  const uint32_t heads = Hq + 2 * Hkv;
  const uint32_t gl = blockIdx.x * 256u + threadIdx.x;
  const uint32_t item = gl / lph, chunk = gl % lph;
  if (item >= B * T * heads) return;
  const uint32_t token = item / heads, hh = item % heads;   // token = b * T + t
  const uint32_t b = token / T, t = token % T;
  const uint32_t lo = chunk * 8, hi = lo + d / 2;       // first channel of the lane's two pieces
  const long long pos = positions[t];
  const bool in_range = pos >= 0 && pos < (long long)max_len;
  if (hh >= Hq + Hkv) {                                // value head: copy into the cache slot
    const uint32_t hv = hh - Hq - Hkv;
    const __half* src = v + ((size_t)token * Hkv + hv) * d;
    const h8 v1 = *(const h8*)(src + lo), v2 = *(const h8*)(src + hi);
    if (in_range) {
      __half* dst = v_cache + (((size_t)b * Hkv + hv) * max_len + (size_t)pos) * d;
      *(h8*)(dst + lo) = v1;
      *(h8*)(dst + hi) = v2;
    }
    return;
  }
  const bool is_q = hh < Hq;
  const __half* src = is_q ? q + ((size_t)token * Hq + hh) * d : k + ((size_t)token * Hkv + (hh - Hq)) * d;
  const h8 x1 = *(const h8*)(src + lo), x2 = *(const h8*)(src + hi);
  const h8 c1 = *(const h8*)(cos + (size_t)t * d + lo), c2 = *(const h8*)(cos + (size_t)t * d + hi);
  const h8 s1 = *(const h8*)(sin + (size_t)t * d + lo), s2 = *(const h8*)(sin + (size_t)t * d + hi);
  h8 y1, y2;                                           // rotate_half: (x1, x2) -> (-x2, x1)
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    const _Float16 a1 = (_Float16)round_here((float)x1[e] * (float)c1[e]);
    const _Float16 r1 = (_Float16)round_here(-1.f * (float)x2[e] * (float)s1[e]);
    y1[e] = (_Float16)round_here((float)a1 + (float)r1);
    const _Float16 a2 = (_Float16)round_here((float)x2[e] * (float)c2[e]);
    const _Float16 r2 = (_Float16)round_here(1.f * (float)x1[e] * (float)s2[e]);
    y2[e] = (_Float16)round_here((float)a2 + (float)r2);
  }
  __half* dst = nullptr;
  if (is_q) dst = q + ((size_t)token * Hq + hh) * d;
  else if (in_range) dst = k_cache + (((size_t)b * Hkv + (hh - Hq)) * max_len + (size_t)pos) * d;
  if (dst) {
    *(h8*)(dst + lo) = y1;
    *(h8*)(dst + hi) = y2;
  }
}

}  // namespace
}  // namespace flh

using namespace flh;

extern "C" int flh_rope_kv_cache_f16(flh_half* q, const flh_half* k, const flh_half* v, const flh_half* cos,
                                     const flh_half* sin, const int64_t* positions, flh_half* k_cache, flh_half* v_cache,
                                     uint32_t B, uint32_t T, uint32_t Hq, uint32_t Hkv, uint32_t head_dim, uint32_t max_len,
                                     void* stream) {
  if (!q || !k || !v || !cos || !sin || !positions || !k_cache || !v_cache) return fail(FLH_EINVAL, "rope_kv_cache: null pointer");
  if (misaligned16(q, k, v, cos, sin, k_cache, v_cache)) return fail(FLH_EINVAL, "rope_kv_cache: tensors must be 16-byte aligned");
  if (head_dim == 0 || head_dim % 16 || head_dim > 512) return fail(FLH_EINVAL, "rope_kv_cache: head_dim (%u) must be a multiple of 16, at most 512", head_dim);
  if (Hq == 0 || Hkv == 0 || max_len == 0) return fail(FLH_EINVAL, "rope_kv_cache: heads and cache length must be positive");
  const uint64_t lanes = (uint64_t)B * T * (Hq + 2 * Hkv) * (head_dim / 16);
  if (lanes == 0) return FLH_OK;
  if (lanes > 0xFFFFFF00ull) return fail(FLH_EINVAL, "rope_kv_cache: too many elements for one launch");
  hipLaunchKernelGGL(rope_kv_cache_kernel, dim3((unsigned)((lanes + 255) / 256)), dim3(256), 0, (hipStream_t)stream,
                     (__half*)q, (const __half*)k, (const __half*)v, (const __half*)cos, (const __half*)sin,
                     (const long long*)positions, (__half*)k_cache, (__half*)v_cache, B, T, Hq, Hkv, head_dim, max_len);
  return check_launch("rope_kv_cache");
}
