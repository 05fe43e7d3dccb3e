// Shared helpers of the ragged serving kernels (gfx950 only).
//
// Every kernel here is templated on the activation type: bf16 (stored as
// unsigned short) when a model is served in bfloat16, float when it is served
// in true 32-bit. Statistics, scores, gates, decays and recurrent state are
// float in both; only loads and stores differ.
#pragma once

#include <torch/extension.h>
#include <ATen/hip/HIPContext.h>

#include "../common.h"

namespace cai {
namespace serving {

using bf16s = unsigned short;

DEV_INLINE float ldf(const float* p) { return *p; }
DEV_INLINE float ldf(const bf16s* p) { return bf2f(*p); }
DEV_INLINE void stf(float* p, float v) { *p = v; }
DEV_INLINE void stf(bf16s* p, float v) { *p = f2bf(v); }

DEV_INLINE float sigmoidf_(float x) { return 1.0f / (1.0f + expf(-x)); }
DEV_INLINE float softplusf_(float x) { return fmaxf(x, 0.0f) + log1pf(expf(-fabsf(x))); }

// 8 consecutive elements of a row as floats (16-byte aligned for bf16, 32-byte for float)
DEV_INLINE void load8(const float* p, float* o) {
  const float4v a = *reinterpret_cast<const float4v*>(p), b = *reinterpret_cast<const float4v*>(p + 4);
  o[0] = a[0]; o[1] = a[1]; o[2] = a[2]; o[3] = a[3]; o[4] = b[0]; o[5] = b[1]; o[6] = b[2]; o[7] = b[3];
}
DEV_INLINE void load8(const bf16s* p, float* o) {
  const short8 a = *reinterpret_cast<const short8*>(p);
#pragma unroll
  for (int e = 0; e < 8; ++e) o[e] = bf2f((bf16s)a[e]);
}
DEV_INLINE void store8(float* p, const float* v) {
  *reinterpret_cast<float4v*>(p) = float4v{v[0], v[1], v[2], v[3]};
  *reinterpret_cast<float4v*>(p + 4) = float4v{v[4], v[5], v[6], v[7]};
}
DEV_INLINE void store8(bf16s* p, const float* v) {
  short8 a;
#pragma unroll
  for (int e = 0; e < 8; ++e) a[e] = (short)f2bf(v[e]);
  *reinterpret_cast<short8*>(p) = a;
}
// two consecutive elements
DEV_INLINE void load2(const float* p, float& a, float& b) {
  const float2v t = *reinterpret_cast<const float2v*>(p);
  a = t[0]; b = t[1];
}
DEV_INLINE void load2(const bf16s* p, float& a, float& b) {
  const unsigned int t = *reinterpret_cast<const unsigned int*>(p);
  a = bf2f((bf16s)(t & 0xffffu)); b = bf2f((bf16s)(t >> 16));
}

inline hipStream_t stream() { return at::hip::getCurrentHIPStream().stream(); }

inline bool is_bf16(const at::Tensor& t) { return t.scalar_type() == at::kBFloat16; }
inline bool is_f32(const at::Tensor& t) { return t.scalar_type() == at::kFloat; }

inline void check_act(const at::Tensor& t, const char* name) {
  TORCH_CHECK(t.is_cuda(), name, " must be a GPU tensor");
  TORCH_CHECK(is_bf16(t) || is_f32(t), name, " must be bfloat16 or float32");
}

// Small per-channel vectors (norm weights, biases, taps, decays) are float32.
inline at::Tensor f32c(const at::Tensor& t) { return t.to(at::kFloat).contiguous(); }

inline void check_i32(const at::Tensor& t, const char* name) {
  TORCH_CHECK(t.is_cuda() && t.scalar_type() == at::kInt && t.is_contiguous(), name,
              " must be a contiguous int32 GPU tensor");
}

template <typename T> inline T* ptr(const at::Tensor& t);
template <> inline float* ptr<float>(const at::Tensor& t) { return t.data_ptr<float>(); }
template <> inline bf16s* ptr<bf16s>(const at::Tensor& t) {
  return reinterpret_cast<bf16s*>(t.data_ptr<at::BFloat16>());
}

// Run `body` with `T` bound to the storage type of `t`.
#define SERVING_DISPATCH_ACT(t, T, ...)                \
  do {                                                 \
    if (::cai::serving::is_bf16(t)) {                  \
      using T = ::cai::serving::bf16s;                 \
      __VA_ARGS__                                      \
    } else {                                           \
      using T = float;                                 \
      __VA_ARGS__                                      \
    }                                                  \
  } while (0)

}  // namespace serving
}  // namespace cai
