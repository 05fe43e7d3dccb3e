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
