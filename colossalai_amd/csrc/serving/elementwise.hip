// Element-wise serving kernels: token shift with carried previous row,
// squared ReLU, gated SiLU of a packed tensor, logit soft-cap, ragged scatter
// of keys/values into pages.
#include "serving_common.h"

namespace cai {
namespace serving {

// One block per token. prev_row = previous token of the same sequence: the
// row above inside a portion, the slot's saved row at a portion's start, zeros
// at position 0. The block of a portion's FIRST token also saves the portion's
// LAST row into the slot, each thread after its own read of the same element,
// so one launch both consumes and refreshes the slot.
template <typename TO>
__global__ __launch_bounds__(256) void token_shift_kernel(
    TO* __restrict__ out, const float* __restrict__ x, const float* __restrict__ mu, float* __restrict__ prev,
    long prev_stride, const int* __restrict__ cu, const int* __restrict__ start, const int* __restrict__ slots,
    const int* __restrict__ tok_seq, int W) {
  const int n = blockIdx.x;
  const int b = tok_seq[n];
  const int first = cu[b], last = cu[b + 1] - 1;
  const float* xr = x + (long)n * W;
  if (n == first) {
    float* pv = prev + (long)slots[b] * prev_stride;
    const bool fresh = start[b] == 0;
    const float* xl = x + (long)last * W;
    for (int w = threadIdx.x; w < W; w += blockDim.x) {
      const float p = fresh ? 0.0f : pv[w];
      const float xv = xr[w];
      const float keep = xl[w];
      stf(out + (long)n * W + w, xv + (p - xv) * mu[w]);
      pv[w] = keep;
    }
  } else {
    const float* xp = xr - W;
    for (int w = threadIdx.x; w < W; w += blockDim.x) {
      const float xv = xr[w];
      stf(out + (long)n * W + w, xv + (xp[w] - xv) * mu[w]);
    }
  }
}

at::Tensor token_shift(at::Tensor x, at::Tensor mu, at::Tensor prev, at::Tensor cu, at::Tensor start,
                       at::Tensor slots, at::Tensor tok_seq, at::ScalarType out_dtype) {
  TORCH_CHECK(x.is_cuda() && is_f32(x) && x.dim() == 2 && x.is_contiguous(), "x must be contiguous float32 [N, W]");
  TORCH_CHECK(is_f32(prev) && prev.dim() == 2 && prev.size(1) == x.size(1) && prev.stride(1) == 1,
              "prev must be float32 [slots, W] with unit inner stride");
  check_i32(cu, "cu"); check_i32(start, "start"); check_i32(slots, "slots"); check_i32(tok_seq, "tok_seq");
  const long N = x.size(0);
  const int W = (int)x.size(1);
  TORCH_CHECK(tok_seq.numel() == N && cu.numel() == start.numel() + 1 && slots.numel() == start.numel());
  at::Tensor muf = f32c(mu);
  TORCH_CHECK(muf.numel() == W);
  at::Tensor out = at::empty({N, W}, x.options().dtype(out_dtype));
  if (N == 0) return out;
  SERVING_DISPATCH_ACT(out, T, {
    hipLaunchKernelGGL(token_shift_kernel<T>, dim3((unsigned)N), dim3(256), 0, stream(), ptr<T>(out),
                       x.data_ptr<float>(), muf.data_ptr<float>(), prev.data_ptr<float>(), (long)prev.stride(0),
                       cu.data_ptr<int>(), start.data_ptr<int>(), slots.data_ptr<int>(), tok_seq.data_ptr<int>(), W);
  });
  HIP_CHECK_LAST();
  return out;
}

template <typename T>
__global__ __launch_bounds__(256) void relu_squared_kernel(T* __restrict__ out, const T* __restrict__ in, long n) {
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x) {
    // the square is taken of the value as the activation type holds it
    const float v = fmaxf(ldf(in + i), 0.0f);
    stf(out + i, v * v);
  }
}

at::Tensor relu_squared(at::Tensor x) {
  check_act(x, "x");
  TORCH_CHECK(x.is_contiguous());
  at::Tensor out = at::empty_like(x);
  const long n = x.numel();
  if (n == 0) return out;
  SERVING_DISPATCH_ACT(x, T, {
    hipLaunchKernelGGL(relu_squared_kernel<T>, dim3(capped_grid((n + 255) / 256, 4096)), dim3(256), 0, stream(),
                       ptr<T>(out), ptr<T>(x), n);
  });
  HIP_CHECK_LAST();
  return out;
}

__global__ __launch_bounds__(256) void softcap_kernel(float* __restrict__ out, const float* __restrict__ in, float cap,
                                                      long n) {
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (long)gridDim.x * blockDim.x)
    out[i] = cap * tanhf(in[i] / cap);
}

at::Tensor softcap(at::Tensor x, double cap) {
  TORCH_CHECK(x.is_cuda() && is_f32(x) && x.is_contiguous(), "x must be contiguous float32");
  at::Tensor out = at::empty_like(x);
  const long n = x.numel();
  if (n == 0) return out;
  hipLaunchKernelGGL(softcap_kernel, dim3(capped_grid((n + 255) / 256, 4096)), dim3(256), 0, stream(),
                     out.data_ptr<float>(), x.data_ptr<float>(), (float)cap, n);
  HIP_CHECK_LAST();
  return out;
}

// k [N, G*D] / v [N, G*Dv] rows (row-strided) -> pool rows rows[n].
template <typename TI, typename TP>
__global__ __launch_bounds__(256) void paged_kv_write_kernel(
    TP* __restrict__ kpool, TP* __restrict__ vpool, const TI* __restrict__ k, const TI* __restrict__ v, long k_stride,
    long v_stride, const int* __restrict__ rows, int KW, int VW) {
  const int n = blockIdx.x;
  const long r = rows[n];
  for (int i = threadIdx.x; i < KW; i += blockDim.x) stf(kpool + r * KW + i, ldf(k + (long)n * k_stride + i));
  for (int i = threadIdx.x; i < VW; i += blockDim.x) stf(vpool + r * VW + i, ldf(v + (long)n * v_stride + i));
}

void paged_kv_write(at::Tensor k, at::Tensor v, at::Tensor kpool, at::Tensor vpool, at::Tensor rows) {
  check_act(k, "k"); check_act(v, "v");
  TORCH_CHECK(k.dim() == 3 && v.dim() == 3 && kpool.dim() == 4 && vpool.dim() == 4);
  TORCH_CHECK(kpool.is_contiguous() && vpool.is_contiguous() && kpool.scalar_type() == vpool.scalar_type());
  TORCH_CHECK(k.scalar_type() == v.scalar_type() && k.scalar_type() == kpool.scalar_type(),
              "keys, values and pools share one dtype");
  check_i32(rows, "rows");
  const long N = k.size(0);
  const int KW = (int)(k.size(1) * k.size(2)), VW = (int)(v.size(1) * v.size(2));
  TORCH_CHECK(v.size(0) == N && rows.numel() == N);
  TORCH_CHECK(kpool.size(2) * kpool.size(3) == KW && vpool.size(2) * vpool.size(3) == VW, "pool row width mismatch");
  TORCH_CHECK(k.stride(2) == 1 && k.stride(1) == k.size(2) && v.stride(2) == 1 && v.stride(1) == v.size(2),
              "k/v rows must be dense (row stride free)");
  if (N == 0) return;
  SERVING_DISPATCH_ACT(k, T, {
    hipLaunchKernelGGL((paged_kv_write_kernel<T, T>), dim3((unsigned)N), dim3(256), 0, stream(), ptr<T>(kpool),
                       ptr<T>(vpool), ptr<T>(k), ptr<T>(v), (long)k.stride(0), (long)v.stride(0),
                       rows.data_ptr<int>(), KW, VW);
  });
  HIP_CHECK_LAST();
}

// packed [N, 2F] = [gate | up], rows strided by ps -> out [N, F] = silu(gate) * up, formed in float32.
// VEC: eight elements per thread (F and the row stride are multiples of 8 and the base is aligned).
template <typename T, bool VEC>
__global__ __launch_bounds__(256) void silu_mul_kernel(T* __restrict__ out, const T* __restrict__ packed, long ps,
                                                       long N, int F) {
  constexpr int PER = VEC ? 8 : 1;
  const long total = N * F / PER;
  for (long i = (long)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (long)gridDim.x * blockDim.x) {
    const long n = i * PER / F;
    const int f = (int)(i * PER % F);
    if (VEC) {
      float g[8], u[8];
      load8(packed + n * ps + f, g);
      load8(packed + n * ps + F + f, u);
#pragma unroll
      for (int e = 0; e < 8; ++e) g[e] = g[e] * sigmoidf_(g[e]) * u[e];
      store8(out + n * F + f, g);
    } else {
      const float g = ldf(packed + n * ps + f), u = ldf(packed + n * ps + F + f);
      stf(out + i, g * sigmoidf_(g) * u);
    }
  }
}

at::Tensor silu_mul(at::Tensor packed) {
  check_act(packed, "packed");
  TORCH_CHECK(packed.dim() == 2 && packed.stride(1) == 1 && packed.size(1) % 2 == 0, "packed must be [N, 2F] with dense rows");
  const long N = packed.size(0);
  const int F = (int)(packed.size(1) / 2);
  at::Tensor out = at::empty({N, F}, packed.options());
  if (N * F == 0) return out;
  const bool vec = F % 8 == 0 && packed.stride(0) % 8 == 0 && reinterpret_cast<uintptr_t>(packed.data_ptr()) % 32 == 0;
  SERVING_DISPATCH_ACT(packed, T, {
    if (vec)
      hipLaunchKernelGGL((silu_mul_kernel<T, true>), dim3(capped_grid((N * F / 8 + 255) / 256, 8192)), dim3(256), 0, stream(),
                         ptr<T>(out), ptr<T>(packed), (long)packed.stride(0), N, F);
    else
      hipLaunchKernelGGL((silu_mul_kernel<T, false>), dim3(capped_grid((N * F + 255) / 256, 4096)), dim3(256), 0, stream(),
                         ptr<T>(out), ptr<T>(packed), (long)packed.stride(0), N, F);
  });
  HIP_CHECK_LAST();
  return out;
}

}  // namespace serving
}  // namespace cai
