// Attention of ONE new token per sequence over a preallocated fp16 key / value cache (the decode step), with grouped
// queries: out[b, h] = softmax(q[b, h] . K[b, h / rep]^T * scale) V[b, h / rep] over the first kv_len cache slots.
//
// Stands where the reference calls the flash-attn package (flh/quantized_model/modeling_llama.py:449-460,
// _flash_attention_forward on the cached keys / values); the stock fused attention kernels are built for long query
// blocks and take ~80 us for this shape, the same arithmetic as separate tensor operations ~30 us in five launches.
// Here the cached positions are split into chunks, one workgroup per (sequence, key / value head, chunk): scores and
// probabilities in float32, a partial (maximum, sum, weighted values) per chunk goes to a scratch buffer, and a second
// small kernel combines the chunks' partials -- two launches, every key and value read once, all query heads of a
// key / value head served by the same read.
#include <atomic>

#include "lane_ops.h"

namespace flh {
namespace {

constexpr int kAttnThreads = 256;

// partial of one (sequence, kv head, chunk): REP heads x (D weighted values, maximum, sum) as float
template <int D>
constexpr int partial_floats(int rep) { return rep * (D + 2); }

// One value of the rotary embedding with the roundings of the tensor expression x * cos + rotate_half(x) * sin evaluated
// op by op in fp16 (the same as the stand-alone kernel, rope_cache.hip): `first_half` says whether x sits in the first
// half of the head vector (its partner xp then enters negated).
__device__ __forceinline__ _Float16 rope_value(_Float16 x, _Float16 xp, _Float16 c, _Float16 s, bool first_half) {
  const _Float16 a = (_Float16)round_here((float)x * (float)c);
  const _Float16 r = (_Float16)round_here((first_half ? -1.f : 1.f) * (float)xp * (float)s);
  return (_Float16)round_here((float)a + (float)r);
}

// ROPE: the step's new token comes in un-rotated -- q, and k_new / v_new [B, Hkv, D] -- together with the cos / sin row of
// its position and the cache slot `positions[0]` it takes (the same for every sequence).  The queries are rotated while
// they are loaded; the workgroup whose chunk holds the slot rotates the new key, uses it and the new value in place of
// what the cache holds there, and writes both into the cache.  One launch less in front of attention, and the same
// bytes in the cache as the stand-alone rotary / cache kernel writes -- also for a slot in kv_len .. max_len - 1, which
// attention does not read: the first workgroup of every (sequence, key / value head) writes it there, as the
// stand-alone kernel would.
template <int D, int REP, int CHUNK, bool ROPE>
__global__ __launch_bounds__(kAttnThreads) void decode_attention_partial_kernel(
    const __half* __restrict__ q, __half* k_cache, __half* v_cache, float* __restrict__ partials, uint32_t Hkv,
    uint32_t kv_len, uint32_t max_len, uint32_t splits, float scale, const __half* __restrict__ k_new,
    const __half* __restrict__ v_new, const __half* __restrict__ cos, const __half* __restrict__ sin,
    const long long* __restrict__ positions) {
  static_assert(D == 128 || D == 64, "head dimension");
  static_assert(CHUNK == 64, "one key per lane in the softmax step");
  static_assert(REP <= 16, "the heads of a key / value head are the columns of one matrix tile");
  constexpr int KS = D / 32;                           // matrix steps over the channels
  constexpr int RPW = CHUNK / (kAttnThreads / 64);     // keys / value rows per wave: 16
  __shared__ __align__(16) _Float16 qs[REP * D];       // the query heads
  __shared__ float sc[REP][CHUNK];                     // scores, then probabilities
  __shared__ float red[kAttnThreads / 64][REP * D];    // the waves' weighted values
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t split = blockIdx.x % splits, bh = blockIdx.x / splits;   // bh = b * Hkv + kvh
  const uint32_t t0 = split * CHUNK;
  uint32_t slot = 0xFFFFFFFFu;                         // cache slot of the new token (ROPE), if it is inside kv_len
  if constexpr (ROPE) {
    const long long pos = positions[0];
    if (pos >= 0 && pos < (long long)kv_len) slot = (uint32_t)pos;
    if (pos >= (long long)kv_len && pos < (long long)max_len && split == 0 && wave == 0) {
      // a slot attention does not read: written, not used
      const _Float16 *kn = (const _Float16*)k_new + (size_t)bh * D, *vn = (const _Float16*)v_new + (size_t)bh * D;
      const _Float16 *cf = (const _Float16*)cos, *sf = (const _Float16*)sin;
      _Float16* kd = (_Float16*)k_cache + ((size_t)bh * max_len + (size_t)pos) * D;
      _Float16* vd = (_Float16*)v_cache + ((size_t)bh * max_len + (size_t)pos) * D;
      for (int c = lane; c < D; c += 64) {
        kd[c] = rope_value(kn[c], kn[c ^ (D / 2)], cf[c], sf[c], c < D / 2);
        vd[c] = vn[c];
      }
    }
  }
  const _Float16* qf = (const _Float16*)q + (size_t)bh * REP * D;   // q [B, Hq, D]: the REP heads of this kv head are adjacent
  for (int i = tid; i < REP * D; i += kAttnThreads) {
    if constexpr (ROPE) {
      const _Float16 *cf = (const _Float16*)cos, *sf = (const _Float16*)sin;
      const int d = i % D;
      qs[i] = rope_value(qf[i], qf[i ^ (D / 2)], cf[d], sf[d], d < D / 2);
    } else {
      qs[i] = qf[i];
    }
  }

  // Scores on the matrix cores: wave w owns the keys 16 w .. 16 w + 15 as the rows of a 16 x 16 tile whose columns are
  // the query heads; a lane holds eight consecutive channels (block `kb` of the step's 32) of key row `krow`.
  const int krow = lane & 15, kb = lane >> 4;
  const uint32_t t = t0 + wave * RPW + krow;
  const bool live = t < kv_len;
  h8 ka[KS];
  if (ROPE && t == slot) {                             // the new key: rotate it, keep it, and store it in its slot
    const __half* src = k_new + (size_t)bh * D;
    __half* dst = k_cache + ((size_t)bh * max_len + t) * D;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      const int c0 = ks * 32 + kb * 8, p0 = c0 ^ (D / 2);
      const h8 x = *(const h8*)(src + c0), xp = *(const h8*)(src + p0);
      const h8 cc = *(const h8*)(cos + c0), ss = *(const h8*)(sin + c0);
      h8 y;
#pragma unroll
      for (int e = 0; e < 8; ++e) y[e] = rope_value(x[e], xp[e], cc[e], ss[e], c0 < D / 2);
      ka[ks] = y;
      *(h8*)(dst + c0) = y;
    }
  } else {
    const __half* kr = k_cache + ((size_t)bh * max_len + (live ? t : 0)) * D + kb * 8;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) ka[ks] = *(const h8*)(kr + ks * 32);
  }
  // Values: wave w takes rows 16 w .. 16 w + 15 of the chunk, a lane one channel pair (one channel for D = 64) of
  // each; requested now, the loads travel while the scores and the softmax pieces are computed.  Rows past the live
  // range read the last live row again (any valid address) and are zeroed: their probability is zero, but 0 x NaN is not.
  const uint32_t n_live = kv_len > t0 ? min((uint32_t)CHUNK, kv_len - t0) : 0u;
  __half* vbase = v_cache + ((size_t)bh * max_len + t0) * D;
  float vv0[RPW], vv1[D == 128 ? RPW : 1];
#pragma unroll
  for (int i = 0; i < RPW; ++i) {
    const uint32_t row = wave * RPW + i;               // wave-uniform
    const bool fresh = ROPE && t0 + row == slot;
    const bool have = row < n_live;
    const __half* src = fresh ? v_new + (size_t)bh * D : vbase + (size_t)(have ? row : (n_live ? n_live - 1 : 0)) * D;
    if constexpr (D == 128) {
      h2 v = *(const h2*)(src + 2 * lane);
      if (fresh) *(h2*)(vbase + (size_t)row * D + 2 * lane) = v;
      vv0[i] = have ? (float)v[0] : 0.f;
      vv1[i] = have ? (float)v[1] : 0.f;
    } else {
      const __half v = src[lane];
      if (fresh) vbase[(size_t)row * D + lane] = v;
      vv0[i] = have ? __half2float(v) : 0.f;
    }
  }
  __syncthreads();                                     // the queries are in LDS
  {
    v4f acc = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      h8 qb = {0, 0, 0, 0, 0, 0, 0, 0};
      if (krow < REP) qb = *(const h8*)(qs + krow * D + ks * 32 + kb * 8);   // column `krow` of the tile: head krow
      acc = __builtin_amdgcn_mfma_f32_16x16x32_f16(ka[ks], qb, acc, 0, 0, 0);
    }
    // acc[i]: key 16 w + 4 kb + i, head krow
    if (krow < REP) {
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        const uint32_t key = wave * RPW + 4 * kb + i;
        sc[krow][key] = t0 + key < kv_len ? acc[i] * scale : -INFINITY;
      }
    }
  }
  __syncthreads();

  // softmax pieces of this chunk, head h by wave h (REP > 4: two heads per wave)
  float* out = partials + (size_t)blockIdx.x * partial_floats<D>(REP);
  for (int h = wave; h < REP; h += kAttnThreads / 64) {
    const float s = sc[h][lane];
    const float m = wave_max(s);
    const float p = m == -INFINITY ? 0.f : __expf(s - m);      // a chunk wholly past kv_len: nothing
    const float l = wave_sum(p);
    sc[h][lane] = p;
    if (lane == 0) {
      out[h * (D + 2) + D] = m;
      out[h * (D + 2) + D + 1] = l;
    }
  }
  __syncthreads();
  // weighted values: every wave its own rows for all heads, then the four waves' sums in a fixed order
#pragma unroll
  for (int h = 0; h < REP; ++h) {
    float a0 = 0.f, a1 = 0.f;
#pragma unroll
    for (int i = 0; i < RPW; ++i) {                    // probabilities past kv_len are zero, their values were not loaded
      const float p = sc[h][wave * RPW + i];
      a0 = __builtin_fmaf(p, vv0[i], a0);
      if constexpr (D == 128) a1 = __builtin_fmaf(p, vv1[i], a1);
    }
    if constexpr (D == 128) *(v2f*)(&red[wave][h * D + 2 * lane]) = v2f{a0, a1};
    else red[wave][h * D + lane] = a0;
  }
  __syncthreads();
  for (int i = tid; i < REP * D; i += kAttnThreads)
    out[(i / D) * (D + 2) + i % D] = (red[0][i] + red[1][i]) + (red[2][i] + red[3][i]);
}

// one workgroup of four waves per (sequence, query head): the chunks' partials -> fp16 output.  Every wave reads all
// maxima and sums (lane s: chunk s, 64 chunks per pass; two wave reductions) and accumulates the weighted values of
// every fourth chunk with the chunk's weight read from its lane; the four waves' sums meet in LDS.
template <int D>
__global__ __launch_bounds__(256) void decode_attention_combine_kernel(const float* __restrict__ partials,
                                                                       __half* __restrict__ out, uint32_t rep,
                                                                       uint32_t splits) {
  __shared__ float acc[4][2][64];
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const uint32_t bhq = blockIdx.x;                     // b * Hq + hq
  const uint32_t bh = bhq / rep, h = bhq % rep;
  const float* base = partials + (size_t)bh * splits * (rep * (D + 2)) + h * (D + 2);
  const size_t stride = (size_t)rep * (D + 2);
  float m = -INFINITY;
  for (uint32_t s0 = 0; s0 < splits; s0 += 64)
    if (s0 + lane < splits) m = __builtin_fmaxf(m, base[(s0 + lane) * stride + D]);
  m = wave_max(m);
  float l = 0.f, a0 = 0.f, a1 = 0.f;
  for (uint32_t s0 = 0; s0 < splits; s0 += 64) {
    float w = 0.f;
    if (s0 + lane < splits) {
      const float ms = base[(s0 + lane) * stride + D];
      w = ms == -INFINITY ? 0.f : __expf(ms - m);
      l = __builtin_fmaf(w, base[(s0 + lane) * stride + D + 1], l);
    }
    const uint32_t n = min(64u, splits - s0);
#pragma unroll 4
    for (uint32_t i = wave; i < n; i += 4) {
      const float wi = __int_as_float(__builtin_amdgcn_readlane(__float_as_int(w), (int)i));
      if constexpr (D == 128) {
        const v2f v = *(const v2f*)(base + (s0 + i) * stride + 2 * lane);
        a0 = __builtin_fmaf(wi, v[0], a0);
        a1 = __builtin_fmaf(wi, v[1], a1);
      } else {
        a0 = __builtin_fmaf(wi, base[(s0 + i) * stride + lane], a0);
      }
    }
  }
  l = wave_sum(l);
  acc[wave][0][lane] = a0;
  acc[wave][1][lane] = a1;
  __syncthreads();
  if (wave != 0) return;
  a0 = (acc[0][0][lane] + acc[1][0][lane]) + (acc[2][0][lane] + acc[3][0][lane]);
  a1 = (acc[0][1][lane] + acc[1][1][lane]) + (acc[2][1][lane] + acc[3][1][lane]);
  const float inv = l > 0.f ? 1.0f / l : 0.f;
  if constexpr (D == 128) {
    const h2 r = {(_Float16)(a0 * inv), (_Float16)(a1 * inv)};
    *(h2*)(out + (size_t)bhq * D + 2 * lane) = r;
  } else {
    out[(size_t)bhq * D + lane] = __float2half(a0 * inv);
  }
}

constexpr int kChunk = 64;

// the new token's inputs of the variant with the rotary embedding and the cache write inside (all null without it)
struct NewToken {
  const __half *k, *v, *cos, *sin;
  const long long* positions;
};

template <int D, int REP>
int launch_attention(const __half* q, __half* k, __half* v, __half* out, float* partials, uint32_t B, uint32_t Hkv,
                     uint32_t kv_len, uint32_t max_len, float scale, const NewToken& nt, hipStream_t stream) {
  const uint32_t splits = (kv_len + kChunk - 1) / kChunk;
  const dim3 grid(B * Hkv * splits), block(kAttnThreads);
  if (nt.k)
    hipLaunchKernelGGL((decode_attention_partial_kernel<D, REP, kChunk, true>), grid, block, 0, stream, q, k, v, partials,
                       Hkv, kv_len, max_len, splits, scale, nt.k, nt.v, nt.cos, nt.sin, nt.positions);
  else
    hipLaunchKernelGGL((decode_attention_partial_kernel<D, REP, kChunk, false>), grid, block, 0, stream, q, k, v, partials,
                       Hkv, kv_len, max_len, splits, scale, nt.k, nt.v, nt.cos, nt.sin, nt.positions);
  if (int rc = check_launch("decode_attention (partials)")) return rc;
  hipLaunchKernelGGL((decode_attention_combine_kernel<D>), dim3(B * Hkv * REP), dim3(256), 0, stream, partials, out,
                     (uint32_t)REP, splits);
  return check_launch("decode_attention (combine)");
}

}  // namespace
}  // namespace flh

using namespace flh;

extern "C" size_t flh_decode_attention_workspace_bytes(uint32_t B, uint32_t Hq, uint32_t head_dim, uint32_t kv_len) {
  const size_t splits = ((size_t)kv_len + kChunk - 1) / kChunk;
  return (size_t)B * Hq * splits * (head_dim + 2) * sizeof(float);
}

namespace {
int decode_attention_checked(const flh_half* q, flh_half* k_cache, flh_half* v_cache, flh_half* out, uint32_t B, uint32_t Hq,
                             uint32_t Hkv, uint32_t head_dim, uint32_t kv_len, uint32_t max_len, float scale,
                             void* workspace, size_t workspace_bytes, const NewToken& nt, void* stream) {
  if (!q || !k_cache || !v_cache || !out) return fail(FLH_EINVAL, "decode_attention: null pointer");
  if (misaligned16(q, k_cache, v_cache, out)) return fail(FLH_EINVAL, "decode_attention: tensors must be 16-byte aligned");
  if (head_dim != 128 && head_dim != 64) return fail(FLH_EINVAL, "decode_attention: head_dim (%u) must be 64 or 128", head_dim);
  if (Hkv == 0 || Hq % Hkv) return fail(FLH_EINVAL, "decode_attention: %u query heads do not divide over %u key / value heads", Hq, Hkv);
  const uint32_t rep = Hq / Hkv;
  if (rep != 1 && rep != 2 && rep != 4 && rep != 8)
    return fail(FLH_EINVAL, "decode_attention: %u query heads per key / value head (1, 2, 4 or 8 supported)", rep);
  if (kv_len == 0 || kv_len > max_len) return fail(FLH_EINVAL, "decode_attention: kv_len (%u) must be in 1 .. max_len (%u)", kv_len, max_len);
  if (B == 0) return FLH_OK;
  const size_t need = flh_decode_attention_workspace_bytes(B, Hq, head_dim, kv_len);
  if (!workspace || ((uintptr_t)workspace & 15)) return fail(FLH_EINVAL, "decode_attention: a 16-byte aligned workspace is required");
  if (workspace_bytes < need)
    return fail(FLH_EINVAL, "decode_attention: the workspace has %zu bytes, this call needs %zu", workspace_bytes, need);
  if ((uint64_t)B * Hkv * ((kv_len + kChunk - 1) / kChunk) > 0x7FFFFFFFull) return fail(FLH_EINVAL, "decode_attention: too many chunks");
  const __half* qh = (const __half*)q;
  __half *kh = (__half*)k_cache, *vh = (__half*)v_cache, *oh = (__half*)out;
  float* ws = (float*)workspace;
  hipStream_t st = (hipStream_t)stream;
#define FLH_ATTN(D, R) return launch_attention<D, R>(qh, kh, vh, oh, ws, B, Hkv, kv_len, max_len, scale, nt, st)
  if (head_dim == 128) {
    switch (rep) {
      case 1: FLH_ATTN(128, 1);
      case 2: FLH_ATTN(128, 2);
      case 4: FLH_ATTN(128, 4);
      default: FLH_ATTN(128, 8);
    }
  }
  switch (rep) {
    case 1: FLH_ATTN(64, 1);
    case 2: FLH_ATTN(64, 2);
    case 4: FLH_ATTN(64, 4);
    default: FLH_ATTN(64, 8);
  }
#undef FLH_ATTN
}
}  // namespace

extern "C" int flh_decode_attention_f16(const flh_half* q, const flh_half* k_cache, const flh_half* v_cache, flh_half* out,
                                        uint32_t B, uint32_t Hq, uint32_t Hkv, uint32_t head_dim, uint32_t kv_len,
                                        uint32_t max_len, float scale, void* workspace, size_t workspace_bytes,
                                        void* stream) {
  // (without a new token the kernel only reads the caches)
  return decode_attention_checked(q, (flh_half*)k_cache, (flh_half*)v_cache, out, B, Hq, Hkv, head_dim, kv_len, max_len, scale,
                                  workspace, workspace_bytes, NewToken{nullptr, nullptr, nullptr, nullptr, nullptr}, stream);
}

extern "C" int flh_decode_attention_rope_f16(const flh_half* q, const flh_half* k_new, const flh_half* v_new,
                                             const flh_half* cos, const flh_half* sin, const int64_t* positions,
                                             flh_half* k_cache, flh_half* v_cache, flh_half* out, uint32_t B, uint32_t Hq,
                                             uint32_t Hkv, uint32_t head_dim, uint32_t kv_len, uint32_t max_len, float scale,
                                             void* workspace, size_t workspace_bytes, void* stream) {
  if (!k_new || !v_new || !cos || !sin || !positions) return fail(FLH_EINVAL, "decode_attention (rotary): null pointer");
  if (misaligned16(k_new, v_new, cos, sin)) return fail(FLH_EINVAL, "decode_attention (rotary): tensors must be 16-byte aligned");
  return decode_attention_checked(q, k_cache, v_cache, out, B, Hq, Hkv, head_dim, kv_len, max_len, scale, workspace,
                                  workspace_bytes,
                                  NewToken{(const __half*)k_new, (const __half*)v_new, (const __half*)cos, (const __half*)sin,
                                           (const long long*)positions}, stream);
}

// ---- the same for callers that cannot allocate ---------------------------------------------------------------------
// The partials live in a static device array of a fixed size instead of a caller's workspace.  Every device the library
// runs on holds its own copy of the array until the process ends; the address of the current device's copy is looked
// up once per device.  Calls on one device share that array: calls that overlap in time (different streams) race.
constexpr size_t kScratchBytes = 16u << 20;            // 16 MiB: e.g. 31 sequences x 32 query heads x 2048 positions, d = 128
static __device__ __align__(256) unsigned char scratch[kScratchBytes];

namespace {
std::atomic<void*> g_scratch_ptr[kMaxDevices];         // per device: where that device's copy of `scratch` lives

int scratch_of_current_device(void** out) {
  int dev = 0;
  if (int rc = current_device(&dev, "decode_attention")) return rc;
  void* ptr = g_scratch_ptr[dev].load(std::memory_order_acquire);
  if (!ptr) {
    const hipError_t e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));   // of the current device
    if (e != hipSuccess || !ptr)
      return fail(FLH_ELAUNCH, "decode_attention: cannot locate the static scratch array: %s", hipGetErrorString(e));
    g_scratch_ptr[dev].store(ptr, std::memory_order_release);
  }
  *out = ptr;
  return FLH_OK;
}
}  // namespace

extern "C" size_t flh_decode_attention_static_scratch_bytes(void) { return kScratchBytes; }

extern "C" int flh_decode_attention_f16_static(const flh_half* q, const flh_half* k_cache, const flh_half* v_cache,
                                               flh_half* out, uint32_t B, uint32_t Hq, uint32_t Hkv, uint32_t head_dim,
                                               uint32_t kv_len, uint32_t max_len, float scale, void* stream) {
  const size_t need = flh_decode_attention_workspace_bytes(B, Hq, head_dim, kv_len);
  if (need > kScratchBytes)
    return fail(FLH_EINVAL, "decode_attention (static scratch): this call needs %zu bytes of scratch, the static array has "
                "%zu; use flh_decode_attention_f16 with a workspace", need, kScratchBytes);
  void* ptr = nullptr;
  if (int e = scratch_of_current_device(&ptr)) return e;
  // every chunk's partial is written before the combine kernel reads it: nothing has to start at zero
  return flh_decode_attention_f16(q, k_cache, v_cache, out, B, Hq, Hkv, head_dim, kv_len, max_len, scale, ptr,
                                  kScratchBytes, stream);
}
