// The PyTorch-ROCm extension in front of libflh_hip's C ABI: tensor checks, torch's current HIP stream, output
// allocation -- nothing else.  It takes the place of the reference's flh/cuda/flh_cuda_bindings.cpp (:75-313): the nine op
// names registered there (:301-313) with the same argument order, checks (TORCH_CHECK -> RuntimeError) and return
// values, plus the ops this library adds (whole-row rotate + quantise, launches over several weight matrices, the
// decode GEMM with its quantiser inside, the fused RMSNorm / SwiGLU producers).  Unlike the reference's bindings every
// launch goes to torch's current stream of the tensor's device.  Host-only C++: all device code lives behind
// include/flh_hip.h in libflh_hip.so.
//
// Exposed twice: as a pybind11 module (what flh_amd._CUDA resolves to; the cheapest call path from Python) and as
// dispatcher ops torch.ops.flh_hip.* (TORCH_LIBRARY) for callers that want schema'd operators.
#include <torch/extension.h>
#include <torch/library.h>

#include <ATen/hip/impl/HIPGuardImplMasqueradingAsCUDA.h>
#include <ATen/hip/impl/HIPStreamMasqueradingAsCUDA.h>

#include <cmath>
#include <mutex>
#include <vector>

#include "../../include/flh_hip.h"

namespace {

using torch::Tensor;

// torch's ROCm build presents its HIP devices and streams under the "cuda" device type
void* stream_of(const Tensor& t) {
  return (void*)c10::hip::getCurrentHIPStreamMasqueradingAsCUDA(t.device().index()).stream();
}

// flh_init once per device (device check + the constant tables of the matrix-core rotation)
void ensure_init(int device) {
  static std::mutex mu;
  static std::vector<bool> done;
  std::lock_guard<std::mutex> lock(mu);
  if ((int)done.size() <= device) done.resize(device + 1, false);
  if (!done[device]) {
    TORCH_CHECK(flh_init() == FLH_OK, "libflh_hip: ", flh_last_error());
    done[device] = true;
  }
}

struct Launch {   // device guard + set-up for one call
  c10::hip::OptionalHIPGuardMasqueradingAsCUDA guard;
  explicit Launch(const Tensor& t) {
    guard.set_device(t.device());
    ensure_init(t.device().index());
  }
};

void ok(int rc) { TORCH_CHECK(rc == FLH_OK, "libflh_hip: ", flh_last_error(), " (code ", rc, ")"); }

const flh_half* h(const Tensor& t) { return (const flh_half*)t.data_ptr(); }
flh_half* hm(Tensor& t) { return (flh_half*)t.data_ptr(); }
const uint8_t* u8(const Tensor& t) { return (const uint8_t*)t.data_ptr(); }

void check_gemm_inputs(const Tensor& A, const Tensor& B, const Tensor& A_scale, const Tensor& B_scale) {
  TORCH_CHECK(A.is_cuda() && B.is_cuda() && A_scale.is_cuda() && B_scale.is_cuda(), "tensors must be CUDA");
  TORCH_CHECK(A.scalar_type() == torch::kUInt8, "A must be uint8 packed int4");
  TORCH_CHECK(B.scalar_type() == torch::kUInt8, "B must be uint8 packed int4");
  TORCH_CHECK(A_scale.scalar_type() == torch::kFloat16, "A_scale must be float16");
  TORCH_CHECK(B_scale.scalar_type() == torch::kFloat16, "B_scale must be float16");
  TORCH_CHECK(A.is_contiguous() && B.is_contiguous() && A_scale.is_contiguous() && B_scale.is_contiguous(),
              "tensors must be contiguous");
  TORCH_CHECK(A.dim() == 2 && B.dim() == 2, "A/B must be 2D");
  TORCH_CHECK(B.size(1) == A.size(1), "B.shape[1] must equal A.shape[1]");
  TORCH_CHECK(B.device() == A.device() && A_scale.device() == A.device() && B_scale.device() == A.device(),
              "tensors must be on one device");
  TORCH_CHECK(A_scale.dim() == 2 && B_scale.dim() == 2, "scale must be 2D");
  TORCH_CHECK(A_scale.size(0) == A.size(0), "A_scale.shape[0] must equal M");
  TORCH_CHECK(B_scale.size(0) == B.size(0), "B_scale.shape[0] must equal N");
  TORCH_CHECK((A.size(1) * 2) % 128 == 0, "K must be a multiple of 128");
}

// ---- GEMM -------------------------------------------------------------------------------------------------------
Tensor gemm_checked(const Tensor& A, const Tensor& B, const Tensor& A_scale, const Tensor& B_scale, int64_t group) {
  const int64_t M = A.size(0), N = B.size(0), K = A.size(1) * 2;
  Tensor D = torch::empty({M, N}, A_scale.options());
  if (M == 0 || N == 0) return D;
  Launch l(A);
  ok(flh_gemm_i4_o16(u8(A), u8(B), h(A_scale), h(B_scale), hm(D), M, N, K, (int)A_scale.size(1), (int)B_scale.size(1),
                     (int)group, stream_of(A)));
  return D;
}

// generalised: scales [M, 1 | K/g], [N, 1 | K/g]
Tensor gemm_i4_dequant(const Tensor& A, const Tensor& B, const Tensor& A_scale, const Tensor& B_scale, int64_t group_size) {
  check_gemm_inputs(A, B, A_scale, B_scale);
  return gemm_checked(A, B, A_scale, B_scale, group_size);
}

// flh_cuda_bindings.cpp:75-113 (a scale width of 1 is accepted as an extension: one scale per row)
Tensor gemm_i4_dequant_o16(const Tensor& A, const Tensor& B, const Tensor& A_scale, const Tensor& B_scale) {
  check_gemm_inputs(A, B, A_scale, B_scale);
  const int64_t ng = A.size(1) * 2 / 128;
  TORCH_CHECK((A_scale.size(1) == 1 || A_scale.size(1) == ng) && (B_scale.size(1) == 1 || B_scale.size(1) == ng),
              "scale.shape[1] must be K/128 (or 1)");
  return gemm_checked(A, B, A_scale, B_scale, 128);
}

// flh_cuda_bindings.cpp:254-299
Tensor gemm_i4_dequant_o16_gs(const Tensor& A, const Tensor& B, const Tensor& A_scale, const Tensor& B_scale,
                              int64_t group_size) {
  check_gemm_inputs(A, B, A_scale, B_scale);
  TORCH_CHECK(group_size == 32 || group_size == 64 || group_size == 128, "group_size must be 32, 64, or 128");
  const int64_t K = A.size(1) * 2;
  TORCH_CHECK(K % group_size == 0, "K must be divisible by group_size");
  TORCH_CHECK(A_scale.size(1) == K / group_size, "A_scale.shape[1] must equal K/group_size");
  TORCH_CHECK(B_scale.size(1) == K / group_size, "B_scale.shape[1] must equal K/group_size");
  return gemm_checked(A, B, A_scale, B_scale, group_size);
}

// fp16(residual + gemm): a decoder layer's residual addition in the GEMM's epilogue; `out` may be the residual itself
Tensor gemm_i4_dequant_add(const Tensor& A, const Tensor& B, const Tensor& A_scale, const Tensor& B_scale,
                           const Tensor& residual, int64_t group_size, const c10::optional<Tensor>& out) {
  check_gemm_inputs(A, B, A_scale, B_scale);
  const int64_t M = A.size(0), N = B.size(0), K = A.size(1) * 2;
  auto shaped = [&](const Tensor& t, const char* what) {
    TORCH_CHECK(t.is_cuda() && t.scalar_type() == torch::kFloat16 && t.is_contiguous() && t.device() == A.device(), what,
                " must be a contiguous float16 CUDA tensor on the operands' device");
    TORCH_CHECK(t.numel() == M * N && t.dim() >= 1 && t.size(-1) == N, what, " must have the shape of the output");
  };
  shaped(residual, "the residual");
  if (out.has_value()) shaped(*out, "out");
  Tensor D = out.has_value() ? *out : torch::empty({M, N}, A_scale.options());
  if (M == 0 || N == 0) return D;
  Launch l(A);
  ok(flh_gemm_i4_add_o16(u8(A), u8(B), h(A_scale), h(B_scale), h(residual), hm(D), M, N, K, (int)A_scale.size(1),
                         (int)B_scale.size(1), (int)group_size, stream_of(A)));
  return D;
}

// causal attention of a block of new tokens over a cache (heads of 128 channels, grouped queries)
Tensor prefill_attention(const Tensor& q, const Tensor& k_cache, const Tensor& v_cache, int64_t past,
                         const c10::optional<double>& scale) {
  for (const Tensor* t : {&q, &k_cache, &v_cache})
    TORCH_CHECK(t->is_cuda() && t->scalar_type() == torch::kFloat16 && t->is_contiguous() && t->device() == q.device(),
                "tensors must be contiguous float16 CUDA tensors on one device");
  TORCH_CHECK(q.dim() == 4 && k_cache.dim() == 4 && k_cache.sizes() == v_cache.sizes() && k_cache.size(0) == q.size(0) &&
                  k_cache.size(3) == q.size(3),
              "q [B, T, Hq, d] and caches [B, Hkv, max_len, d] expected");
  const int64_t B = q.size(0), T = q.size(1), Hq = q.size(2), d = q.size(3), Hkv = k_cache.size(1), max_len = k_cache.size(2);
  TORCH_CHECK(d == 128, "head_dim must be 128");
  TORCH_CHECK(Hkv > 0 && Hq % Hkv == 0, "Hq must be a multiple of Hkv");
  TORCH_CHECK(past >= 0 && past + T <= max_len, "past + T must fit the cache");
  Tensor out = torch::empty({B, T, Hq * d}, q.options());
  if (B == 0 || T == 0) return out;
  Launch l(q);
  ok(flh_prefill_attention_f16(h(q), h(k_cache), h(v_cache), hm(out), (uint32_t)B, (uint32_t)T, (uint32_t)Hq, (uint32_t)Hkv,
                               (uint32_t)d, (uint32_t)past, (uint32_t)max_len,
                               (float)(scale.has_value() ? *scale : 1.0 / std::sqrt((double)d)), stream_of(q)));
  return out;
}

// gate and up projection of a SwiGLU MLP in one launch: fp16(fp16(silu(gate)) * up)
Tensor gemm_i4_swiglu(const Tensor& A, const Tensor& B_gate, const Tensor& B_up, const Tensor& A_scale,
                      const Tensor& gate_scale, const Tensor& up_scale, int64_t group_size) {
  check_gemm_inputs(A, B_gate, A_scale, gate_scale);
  check_gemm_inputs(A, B_up, A_scale, up_scale);
  TORCH_CHECK(B_up.sizes() == B_gate.sizes() && up_scale.sizes() == gate_scale.sizes(),
              "gate and up must have the same shapes");
  const int64_t M = A.size(0), N = B_gate.size(0), K = A.size(1) * 2;
  Tensor D = torch::empty({M, N}, A_scale.options());
  if (M == 0 || N == 0) return D;
  Launch l(A);
  ok(flh_gemm_i4_swiglu_o16(u8(A), u8(B_gate), u8(B_up), h(A_scale), h(gate_scale), h(up_scale), hm(D), M, N, K,
                            (int)A_scale.size(1), (int)gate_scale.size(1), (int)group_size, stream_of(A)));
  return D;
}

std::vector<Tensor> gemm_i4_dequant_multi(const Tensor& A, const std::vector<Tensor>& Bs, const Tensor& A_scale,
                                          const std::vector<Tensor>& B_scales, int64_t group_size) {
  TORCH_CHECK(Bs.size() == B_scales.size() && !Bs.empty() && Bs.size() <= 4,
              "one to four weight matrices, one scale tensor each");
  bool empty = A.size(0) == 0;
  for (size_t s = 0; s < Bs.size(); ++s) {
    check_gemm_inputs(A, Bs[s], A_scale, B_scales[s]);
    TORCH_CHECK(B_scales[s].size(1) == B_scales[0].size(1), "B_scale shapes");
    empty = empty || Bs[s].size(0) == 0;
  }
  std::vector<Tensor> Ds;
  if (empty) {
    for (size_t s = 0; s < Bs.size(); ++s) Ds.push_back(gemm_checked(A, Bs[s], A_scale, B_scales[s], group_size));
    return Ds;
  }
  const int64_t M = A.size(0), K = A.size(1) * 2;
  const uint8_t* b[4];
  const flh_half* bs[4];
  flh_half* d[4];
  size_t n[4];
  for (size_t s = 0; s < Bs.size(); ++s) {
    Ds.push_back(torch::empty({M, Bs[s].size(0)}, A_scale.options()));
    b[s] = u8(Bs[s]);
    bs[s] = h(B_scales[s]);
    d[s] = hm(Ds[s]);
    n[s] = (size_t)Bs[s].size(0);
  }
  Launch l(A);
  ok(flh_gemm_i4_o16_multi(u8(A), h(A_scale), (int)Bs.size(), b, bs, d, n, M, K, (int)A_scale.size(1),
                           (int)B_scales[0].size(1), (int)group_size, stream_of(A)));
  return Ds;
}

// ---- decode GEMM with the quantiser inside -----------------------------------------------------------------------
void check_rotate_gemm(const Tensor& x, const Tensor& B, const Tensor& S) {
  TORCH_CHECK(x.is_cuda() && B.is_cuda() && S.is_cuda() && B.device() == x.device() && S.device() == x.device(),
              "tensors must be CUDA and on one device");
  TORCH_CHECK(x.scalar_type() == torch::kFloat16 && x.dim() == 2 && x.is_contiguous(),
              "x must be a contiguous 2D float16 tensor");
  TORCH_CHECK(B.scalar_type() == torch::kUInt8 && B.dim() == 2 && B.is_contiguous() && B.size(1) * 2 == x.size(1),
              "B must be a contiguous uint8 [N, K/2] tensor");
  TORCH_CHECK(x.size(0) <= 4, "at most 4 tokens");
  TORCH_CHECK(x.size(1) == 4096, "K must be 4096");
  TORCH_CHECK(S.scalar_type() == torch::kFloat16 && S.is_contiguous() && S.dim() == 2 && S.size(0) == B.size(0) &&
                  (S.size(1) == 1 || S.size(1) == x.size(1) / 128),
              "B_scale must be a contiguous float16 [N, 1] or [N, K/128] tensor");
}

Tensor rotate_quantize_gemm_i4(const Tensor& x, const Tensor& B, const Tensor& B_scale) {
  check_rotate_gemm(x, B, B_scale);
  const int64_t M = x.size(0), N = B.size(0), K = x.size(1);
  Tensor D = torch::empty({M, N}, x.options());
  if (M == 0 || N == 0) return D;
  Launch l(x);
  ok(flh_rotate_quant_gemm_i4_o16(h(x), u8(B), h(B_scale), hm(D), M, N, K, (int)B_scale.size(1), stream_of(x)));
  return D;
}

std::vector<Tensor> rotate_quantize_gemm_i4_multi(const Tensor& x, const std::vector<Tensor>& Bs,
                                                  const std::vector<Tensor>& B_scales) {
  TORCH_CHECK(Bs.size() == B_scales.size() && !Bs.empty() && Bs.size() <= 4,
              "one to four weight matrices, one scale tensor each");
  const int64_t M = x.dim() == 2 ? x.size(0) : 0;
  std::vector<Tensor> Ds;
  const uint8_t* b[4];
  const flh_half* bs[4];
  flh_half* d[4];
  size_t n[4];
  int live = 0;
  for (size_t s = 0; s < Bs.size(); ++s) {
    check_rotate_gemm(x, Bs[s], B_scales[s]);
    TORCH_CHECK(B_scales[s].size(1) == B_scales[0].size(1), "the same scale width for every matrix");
    Ds.push_back(torch::empty({M, Bs[s].size(0)}, x.options()));
    if (Bs[s].size(0) == 0) continue;
    b[live] = u8(Bs[s]);
    bs[live] = h(B_scales[s]);
    d[live] = hm(Ds[s]);
    n[live] = (size_t)Bs[s].size(0);
    ++live;
  }
  if (M == 0 || live == 0) return Ds;
  Launch l(x);
  ok(flh_rotate_quant_gemm_i4_o16_multi(h(x), live, b, bs, d, n, M, x.size(1), (int)B_scales[0].size(1), stream_of(x)));
  return Ds;
}

// ---- group kernels ------------------------------------------------------------------------------------------------
void check_rows(const Tensor& x, int64_t width) {
  TORCH_CHECK(x.is_cuda(), "Input tensor must be on CUDA");
  TORCH_CHECK(x.scalar_type() == torch::kFloat16, "Input tensor must be float16 (half)");
  TORCH_CHECK(x.dim() == 2, "Input tensor must be 2D");
  TORCH_CHECK(x.size(1) == width, "Last dimension must be ", width);
  TORCH_CHECK(x.is_contiguous(), "Input tensor must be contiguous");
}

Tensor fwht_inplace(Tensor x, int64_t width) {   // flh_cuda_bindings.cpp:115-152: in place, returns the same tensor
  check_rows(x, width);
  if (x.size(0) == 0) return x;
  Launch l(x);
  ok(flh_fwht_f16_inplace(hm(x), (uint32_t)x.size(0), (int)width, stream_of(x)));
  return x;
}
Tensor hadamard_transform_half(Tensor x) { return fwht_inplace(x, 128); }
Tensor hadamard_transform_64_half(Tensor x) { return fwht_inplace(x, 64); }
Tensor hadamard_transform_32_half(Tensor x) { return fwht_inplace(x, 32); }

std::vector<Tensor> group_quant(const Tensor& x, int64_t group, bool hadamard, double scale_mul) {
  check_rows(x, group);
  const int64_t R = x.size(0);
  Tensor q = torch::empty({R, group / 2}, x.options().dtype(torch::kUInt8));
  Tensor s = torch::empty({R}, x.options());
  if (R) {
    Launch l(x);
    ok(flh_group_quant_i4(h(x), (uint8_t*)q.data_ptr(), hm(s), (uint32_t)R, (int)group, hadamard ? 1 : 0,
                          (float)scale_mul, stream_of(x)));
  }
  return {q, s};
}
void check_group(int64_t g) { TORCH_CHECK(g == 32 || g == 64 || g == 128, "group_size must be 32, 64, or 128"); }

// flh_cuda_bindings.cpp:154-252; scale_mul (extension): constant factor on the stored scales
std::vector<Tensor> hadamard_and_quantize_i4(const Tensor& x, double scale_mul) { return group_quant(x, 128, true, scale_mul); }
std::vector<Tensor> quant_and_pack_i4(const Tensor& x) { return group_quant(x, 128, false, 1.0); }
std::vector<Tensor> hadamard_and_quantize_i4_gs(const Tensor& x, int64_t group_size, double scale_mul) {
  check_group(group_size);
  TORCH_CHECK(x.dim() == 2 && x.size(1) == group_size, "Last dimension must equal group_size");
  return group_quant(x, group_size, true, scale_mul);
}
std::vector<Tensor> quant_and_pack_i4_gs(const Tensor& x, int64_t group_size, double scale_mul) {
  check_group(group_size);
  TORCH_CHECK(x.dim() == 2 && x.size(1) == group_size, "Last dimension must equal group_size");
  return group_quant(x, group_size, false, scale_mul);
}

// ---- whole-row rotate + quantise ------------------------------------------------------------------------------------
// mode: 0 none, 1 float32 butterflies (bit-exact for power-of-two K), 2 matrix cores
std::vector<Tensor> rotate_and_quantize_i4_mode(const Tensor& x, int64_t mode, int64_t had_group, int64_t scale_group,
                                                double clip_ratio, bool return_rotated) {
  TORCH_CHECK(x.is_cuda(), "Input tensor must be on CUDA");
  TORCH_CHECK(x.scalar_type() == torch::kFloat16, "Input tensor must be float16 (half)");
  TORCH_CHECK(x.dim() == 2 && x.is_contiguous(), "Input tensor must be 2D and contiguous");
  const int64_t M = x.size(0), K = x.size(1);
  const int64_t ns = scale_group > 0 ? K / scale_group : 1;
  Tensor q = torch::empty({M, K / 2}, x.options().dtype(torch::kUInt8));
  Tensor s = torch::empty({M, ns}, x.options());
  Tensor y;
  if (return_rotated) y = torch::empty_like(x);
  if (M) {
    Launch l(x);
    ok(flh_rotate_quant_i4(h(x), (uint8_t*)q.data_ptr(), hm(s), return_rotated ? hm(y) : nullptr, (uint32_t)M,
                           (uint32_t)K, (int)mode, (int)had_group, (int)scale_group, (float)clip_ratio, stream_of(x)));
  }
  if (return_rotated) return {q, s, y};
  return {q, s};
}

std::vector<Tensor> rmsnorm_rotate_and_quantize_i4_mode(const Tensor& x, const c10::optional<Tensor>& weight, double eps,
                                                        int64_t mode, double clip_ratio, bool return_rotated) {
  TORCH_CHECK(x.is_cuda(), "Input tensor must be on CUDA");
  TORCH_CHECK(x.scalar_type() == torch::kFloat16, "Input tensor must be float16 (half)");
  TORCH_CHECK(x.dim() == 2 && x.is_contiguous(), "Input tensor must be 2D and contiguous");
  const int64_t M = x.size(0), K = x.size(1);
  TORCH_CHECK(K == 512 || K == 1024 || K == 2048 || K == 4096 || K == 8192,
              "Last dimension must be 512, 1024, 2048, 4096 or 8192");
  if (weight.has_value())
    TORCH_CHECK(weight->is_cuda() && weight->scalar_type() == torch::kFloat16 && weight->is_contiguous() &&
                    weight->numel() == K && weight->device() == x.device(),
                "weight must be a contiguous float16 CUDA tensor of K values");
  Tensor q = torch::empty({M, K / 2}, x.options().dtype(torch::kUInt8));
  Tensor s = torch::empty({M, 1}, x.options());
  Tensor y;
  if (return_rotated) y = torch::empty_like(x);
  if (M) {
    Launch l(x);
    ok(flh_rmsnorm_rotate_quant_i4(h(x), weight.has_value() ? h(*weight) : nullptr, (float)eps, (uint8_t*)q.data_ptr(),
                                   hm(s), return_rotated ? hm(y) : nullptr, (uint32_t)M, (uint32_t)K, (int)mode,
                                   (float)clip_ratio, stream_of(x)));
  }
  if (return_rotated) return {q, s, y};
  return {q, s};
}

// ---- fused producers -------------------------------------------------------------------------------------------------
std::vector<Tensor> silu_mul_and_quantize_i4_gs(const Tensor& gate, const Tensor& up, int64_t group_size, bool hadamard,
                                                double scale_mul) {
  check_group(group_size);
  TORCH_CHECK(gate.is_cuda() && up.is_cuda() && gate.device() == up.device(), "Input tensors must be on CUDA");
  TORCH_CHECK(gate.scalar_type() == torch::kFloat16 && up.scalar_type() == torch::kFloat16,
              "Input tensors must be float16 (half)");
  TORCH_CHECK(gate.sizes() == up.sizes(), "gate and up must have the same shape");
  TORCH_CHECK(gate.is_contiguous() && up.is_contiguous(), "Input tensors must be contiguous");
  TORCH_CHECK(gate.dim() >= 1 && gate.size(-1) % group_size == 0, "Last dimension must be divisible by group_size");
  auto qs = gate.sizes().vec(), ss = gate.sizes().vec();
  qs.back() = gate.size(-1) / 2;
  ss.back() = gate.size(-1) / group_size;
  Tensor q = torch::empty(qs, gate.options().dtype(torch::kUInt8));
  Tensor s = torch::empty(ss, gate.options());
  if (s.numel()) {
    Launch l(gate);
    ok(flh_silu_mul_group_quant_i4(h(gate), h(up), (uint8_t*)q.data_ptr(), hm(s), (uint32_t)s.numel(), (int)group_size,
                                   hadamard ? 1 : 0, (float)scale_mul, stream_of(gate)));
  }
  return {q, s};
}

std::vector<Tensor> rmsnorm_and_quantize_i4_gs(const Tensor& x, const c10::optional<Tensor>& weight, double eps,
                                               int64_t group_size, bool hadamard, double scale_mul) {
  check_group(group_size);
  TORCH_CHECK(x.is_cuda(), "Input tensor must be on CUDA");
  TORCH_CHECK(x.scalar_type() == torch::kFloat16, "Input tensor must be float16 (half)");
  TORCH_CHECK(x.is_contiguous() && x.dim() >= 1, "Input tensor must be contiguous");
  const int64_t K = x.size(-1);
  TORCH_CHECK(K % group_size == 0 && K > 0 && K <= 16384,
              "Last dimension must be divisible by group_size and at most 16384");
  if (weight.has_value())
    TORCH_CHECK(weight->is_cuda() && weight->scalar_type() == torch::kFloat16 && weight->is_contiguous() &&
                    weight->numel() == K && weight->device() == x.device(),
                "weight must be a contiguous float16 CUDA tensor of K values");
  auto qs = x.sizes().vec(), ss = x.sizes().vec();
  qs.back() = K / 2;
  ss.back() = K / group_size;
  Tensor q = torch::empty(qs, x.options().dtype(torch::kUInt8));
  Tensor s = torch::empty(ss, x.options());
  const int64_t M = x.numel() / K;
  if (M) {
    Launch l(x);
    ok(flh_rmsnorm_group_quant_i4(h(x), weight.has_value() ? h(*weight) : nullptr, (uint8_t*)q.data_ptr(), hm(s),
                                  (uint32_t)M, (uint32_t)K, (float)eps, (int)group_size, hadamard ? 1 : 0,
                                  (float)scale_mul, stream_of(x)));
  }
  return {q, s};
}

// ---- rotary embedding + cache write -----------------------------------------------------------------------------------
Tensor rope_kv_cache_(Tensor q, const Tensor& k, const Tensor& v, const Tensor& cos, const Tensor& sin,
                      const Tensor& positions, Tensor k_cache, Tensor v_cache) {
  for (const Tensor* t : std::initializer_list<const Tensor*>{&q, &k, &v, &cos, &sin, &k_cache, &v_cache})
    TORCH_CHECK(t->is_cuda() && t->scalar_type() == torch::kFloat16 && t->is_contiguous() && t->device() == q.device(),
                "tensors must be contiguous float16 CUDA tensors on one device");
  TORCH_CHECK(q.dim() == 4 && k.dim() == 4 && v.sizes() == k.sizes() && k.size(0) == q.size(0) && k.size(1) == q.size(1) &&
                  k.size(3) == q.size(3), "q [B, T, Hq, d] and k, v [B, T, Hkv, d] expected");
  const int64_t B = q.size(0), T = q.size(1), Hq = q.size(2), d = q.size(3), Hkv = k.size(2);
  TORCH_CHECK(cos.dim() == 2 && cos.size(0) == T && cos.size(1) == d && sin.sizes() == cos.sizes(), "cos / sin must be [T, d]");
  TORCH_CHECK(positions.is_cuda() && positions.scalar_type() == torch::kInt64 && positions.is_contiguous() &&
                  positions.numel() == T && positions.device() == q.device(),
              "positions must be a contiguous int64 CUDA tensor of T entries");
  TORCH_CHECK(k_cache.dim() == 4 && k_cache.sizes() == v_cache.sizes() && k_cache.size(0) == B && k_cache.size(1) == Hkv &&
                  k_cache.size(3) == d, "caches must be [B, Hkv, max_len, d]");
  TORCH_CHECK(d % 16 == 0, "head_dim must be a multiple of 16");
  if (q.numel() == 0) return q;
  Launch l(q);
  ok(flh_rope_kv_cache_f16(hm(q), h(k), h(v), h(cos), h(sin), (const int64_t*)positions.data_ptr(), hm(k_cache), hm(v_cache),
                           (uint32_t)B, (uint32_t)T, (uint32_t)Hq, (uint32_t)Hkv, (uint32_t)d, (uint32_t)k_cache.size(2),
                           stream_of(q)));
  return q;
}

}  // namespace

// dispatcher ops (torch.ops.flh_hip.*): the reference's nine names and the general forms
TORCH_LIBRARY(flh_hip, m) {
  m.def("gemm_i4_dequant_o16(Tensor A, Tensor B, Tensor A_scale, Tensor B_scale) -> Tensor", &gemm_i4_dequant_o16);
  m.def("gemm_i4_dequant_o16_gs(Tensor A, Tensor B, Tensor A_scale, Tensor B_scale, int group_size) -> Tensor",
        &gemm_i4_dequant_o16_gs);
  m.def("gemm_i4_dequant(Tensor A, Tensor B, Tensor A_scale, Tensor B_scale, int group_size) -> Tensor", &gemm_i4_dequant);
  m.def("gemm_i4_dequant_multi(Tensor A, Tensor[] Bs, Tensor A_scale, Tensor[] B_scales, int group_size) -> Tensor[]",
        &gemm_i4_dequant_multi);
  m.def("hadamard_transform_half(Tensor(a!) x) -> Tensor(a!)", &hadamard_transform_half);
  m.def("hadamard_transform_64_half(Tensor(a!) x) -> Tensor(a!)", &hadamard_transform_64_half);
  m.def("hadamard_transform_32_half(Tensor(a!) x) -> Tensor(a!)", &hadamard_transform_32_half);
  m.def("hadamard_and_quantize_i4(Tensor x, float scale_mul=1.0) -> Tensor[]", &hadamard_and_quantize_i4);
  m.def("quant_and_pack_i4(Tensor x) -> Tensor[]", &quant_and_pack_i4);
  m.def("hadamard_and_quantize_i4_gs(Tensor x, int group_size, float scale_mul=1.0) -> Tensor[]",
        &hadamard_and_quantize_i4_gs);
  m.def("quant_and_pack_i4_gs(Tensor x, int group_size, float scale_mul=1.0) -> Tensor[]", &quant_and_pack_i4_gs);
  m.def("rotate_and_quantize_i4(Tensor x, int mode, int had_group=0, int scale_group=0, float clip_ratio=1.0, "
        "bool return_rotated=False) -> Tensor[]", &rotate_and_quantize_i4_mode);
  m.def("rotate_quantize_gemm_i4(Tensor x, Tensor B, Tensor B_scale) -> Tensor", &rotate_quantize_gemm_i4);
}

PYBIND11_MODULE(TORCH_EXTENSION_NAME, m) {
  namespace py = pybind11;
  m.doc() = "tensor-level front of libflh_hip (see include/flh_hip.h)";
  m.def("gemm_i4_dequant_o16", &gemm_i4_dequant_o16, py::arg("A"), py::arg("B"), py::arg("A_scale"), py::arg("B_scale"));
  m.def("gemm_i4_dequant_o16_gs", &gemm_i4_dequant_o16_gs, py::arg("A"), py::arg("B"), py::arg("A_scale"),
        py::arg("B_scale"), py::arg("group_size"));
  m.def("gemm_i4_dequant", &gemm_i4_dequant, py::arg("A"), py::arg("B"), py::arg("A_scale"), py::arg("B_scale"),
        py::arg("group_size") = 128);
  m.def("gemm_i4_dequant_multi", &gemm_i4_dequant_multi, py::arg("A"), py::arg("Bs"), py::arg("A_scale"),
        py::arg("B_scales"), py::arg("group_size") = 128);
  m.def("gemm_i4_swiglu", &gemm_i4_swiglu, py::arg("A"), py::arg("B_gate"), py::arg("B_up"), py::arg("A_scale"),
        py::arg("gate_scale"), py::arg("up_scale"), py::arg("group_size") = 128);
  m.def("gemm_i4_dequant_add", &gemm_i4_dequant_add, py::arg("A"), py::arg("B"), py::arg("A_scale"), py::arg("B_scale"),
        py::arg("residual"), py::arg("group_size") = 128, py::arg("out") = py::none());
  m.def("prefill_attention", &prefill_attention, py::arg("q"), py::arg("k_cache"), py::arg("v_cache"), py::arg("past"),
        py::arg("scale") = py::none());
  m.def("rotate_quantize_gemm_i4", &rotate_quantize_gemm_i4, py::arg("x"), py::arg("B"), py::arg("B_scale"));
  m.def("rotate_quantize_gemm_i4_multi", &rotate_quantize_gemm_i4_multi, py::arg("x"), py::arg("Bs"), py::arg("B_scales"));
  m.def("rope_kv_cache_", &rope_kv_cache_, py::arg("q"), py::arg("k"), py::arg("v"), py::arg("cos"), py::arg("sin"),
        py::arg("positions"), py::arg("k_cache"), py::arg("v_cache"));
  m.def("hadamard_transform_half", &hadamard_transform_half, py::arg("x"));
  m.def("hadamard_transform_128_half", &hadamard_transform_half, py::arg("x"));   // the name flh/cuda/hadamard.py:35 calls
  m.def("hadamard_transform_64_half", &hadamard_transform_64_half, py::arg("x"));
  m.def("hadamard_transform_32_half", &hadamard_transform_32_half, py::arg("x"));
  m.def("hadamard_and_quantize_i4", &hadamard_and_quantize_i4, py::arg("x"), py::kw_only(), py::arg("scale_mul") = 1.0);
  m.def("quant_and_pack_i4", &quant_and_pack_i4, py::arg("x"));
  m.def("hadamard_and_quantize_i4_gs", &hadamard_and_quantize_i4_gs, py::arg("x"), py::arg("group_size"), py::kw_only(),
        py::arg("scale_mul") = 1.0);
  m.def("quant_and_pack_i4_gs", &quant_and_pack_i4_gs, py::arg("x"), py::arg("group_size"), py::kw_only(),
        py::arg("scale_mul") = 1.0);
  m.def("rotate_and_quantize_i4_mode", &rotate_and_quantize_i4_mode, py::arg("x"), py::arg("mode"),
        py::arg("had_group") = 0, py::arg("scale_group") = 0, py::arg("clip_ratio") = 1.0,
        py::arg("return_rotated") = false);
  m.def("rmsnorm_rotate_and_quantize_i4_mode", &rmsnorm_rotate_and_quantize_i4_mode, py::arg("x"), py::arg("weight"),
        py::arg("eps"), py::arg("mode") = 1, py::arg("clip_ratio") = 1.0, py::arg("return_rotated") = false);
  m.def("silu_mul_and_quantize_i4_gs", &silu_mul_and_quantize_i4_gs, py::arg("gate"), py::arg("up"),
        py::arg("group_size"), py::arg("hadamard") = false, py::kw_only(), py::arg("scale_mul") = 1.0);
  m.def("rmsnorm_and_quantize_i4_gs", &rmsnorm_and_quantize_i4_gs, py::arg("x"), py::arg("weight"), py::arg("eps"),
        py::arg("group_size"), py::arg("hadamard") = false, py::kw_only(), py::arg("scale_mul") = 1.0);
}
