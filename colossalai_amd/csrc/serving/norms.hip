// Normalisation kernels of the serving path (float32 statistics):
//   grouped_rms_norm   : per-group RMS scaling of a row, optional in-place add
//                        to the float32 residual stream;
//   head_rms_norm_gate : per-head RMS norm of [N, H, D] with a shared [D]
//                        weight and an optional sigmoid gate;
//   merge_rms_norm     : two branch rows, each full-width RMS-normed with its
//                        own weight, averaged, group-normed and added to the
//                        residual — one pass, the merged row staged in LDS;
//   add_rms_norm       : residual += a (+ b) in place and, when a weight is
//                        given, the RMS norm of the new residual row for the
//                        next pre-norm layer, in one launch.
#include "serving_common.h"

namespace cai {
namespace serving {

// One wave per (row, group).
template <typename TI, typename TO>
__global__ __launch_bounds__(256) void grouped_rms_norm_kernel(
    TO* __restrict__ out, float* __restrict__ residual, const TI* __restrict__ x, const float* __restrict__ w,
    long units, int groups, int gs, float eps) {
  const int lane = threadIdx.x & 63;
  const long unit = (long)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (unit >= units) return;
  const long row = unit / groups;
  const int g = (int)(unit % groups);
  const long base = (row * groups + g) * (long)gs;
  float ssq = 0.0f;
#pragma unroll 8
  for (int i = lane; i < gs; i += 64) {  // unrolled: the loads of a row are in flight together
    const float v = ldf(x + base + i);
    ssq += v * v;
  }
  ssq = wave_reduce_sum(ssq);
  const float inv = 1.0f / sqrtf(ssq / (float)gs + eps);
#pragma unroll 8
  for (int i = lane; i < gs; i += 64) {
    const float y = ldf(x + base + i) * inv * w[g * gs + i];
    if (residual != nullptr) residual[base + i] += y;
    else stf(out + base + i, y);
  }
}

at::Tensor grouped_rms_norm(at::Tensor x, at::Tensor weight, int64_t groups, double eps,
                            c10::optional<at::Tensor> residual, at::ScalarType out_dtype) {
  check_act(x, "x");
  TORCH_CHECK(x.dim() == 2 && x.is_contiguous(), "x must be contiguous [N, W]");
  const long N = x.size(0);
  const int W = (int)x.size(1);
  TORCH_CHECK(groups > 0 && W % groups == 0);
  at::Tensor w = f32c(weight);
  TORCH_CHECK(w.numel() == W);
  float* res = nullptr;
  at::Tensor out;
  if (residual.has_value()) {
    TORCH_CHECK(is_f32(*residual) && residual->is_contiguous() && residual->sizes() == x.sizes(),
                "residual must be contiguous float32 of x's shape");
    res = residual->data_ptr<float>();
    out = *residual;
  } else {
    out = at::empty({N, W}, x.options().dtype(out_dtype));
  }
  if (N == 0) return out;
  const long units = N * groups;
  const unsigned grid = (unsigned)((units + 3) / 4);
  SERVING_DISPATCH_ACT(x, TI, {
    if (res != nullptr) {
      hipLaunchKernelGGL((grouped_rms_norm_kernel<TI, float>), dim3(grid), dim3(256), 0, stream(), (float*)nullptr, res,
                         ptr<TI>(x), w.data_ptr<float>(), units, (int)groups, W / (int)groups, (float)eps);
    } else {
      SERVING_DISPATCH_ACT(out, TO, {
        hipLaunchKernelGGL((grouped_rms_norm_kernel<TI, TO>), dim3(grid), dim3(256), 0, stream(), ptr<TO>(out),
                           (float*)nullptr, ptr<TI>(x), w.data_ptr<float>(), units, (int)groups, W / (int)groups,
                           (float)eps);
      });
    }
  });
  HIP_CHECK_LAST();
  return out;
}

// One wave per (n, h). x row-strided: element (n, h, d) at n*xs + h*D + d.
template <typename TI, typename TG, typename TO>
__global__ __launch_bounds__(256) void head_rms_norm_gate_kernel(
    TO* __restrict__ out, const TI* __restrict__ x, long xs, const float* __restrict__ w, const TG* __restrict__ gate,
    long gs, long units, int H, int D, float eps) {
  const int lane = threadIdx.x & 63;
  const long unit = (long)blockIdx.x * (blockDim.x >> 6) + (threadIdx.x >> 6);
  if (unit >= units) return;
  const long n = unit / H;
  const int h = (int)(unit % H);
  const TI* xr = x + n * xs + (long)h * D;
  float ssq = 0.0f;
  for (int i = lane; i < D; i += 64) {
    const float v = ldf(xr + i);
    ssq += v * v;
  }
  ssq = wave_reduce_sum(ssq);
  const float inv = 1.0f / sqrtf(ssq / (float)D + eps);
  for (int i = lane; i < D; i += 64) {
    float y = ldf(xr + i) * inv * w[i];
    if (gate != nullptr) y *= sigmoidf_(ldf(gate + n * gs + (long)h * D + i));
    stf(out + (n * H + h) * (long)D + i, y);
  }
}

at::Tensor head_rms_norm_gate(at::Tensor x, at::Tensor weight, double eps, c10::optional<at::Tensor> gate,
                              at::ScalarType out_dtype) {
  check_act(x, "x");
  TORCH_CHECK(x.dim() == 3 && x.stride(2) == 1 && x.stride(1) == x.size(2), "x must be [N, H, D] with dense rows");
  const long N = x.size(0);
  const int H = (int)x.size(1), D = (int)x.size(2);
  at::Tensor w = f32c(weight);
  TORCH_CHECK(w.numel() == D);
  at::Tensor out = at::empty({N, H, D}, x.options().dtype(out_dtype));
  if (N == 0) return out;
  long gs = 0;
  if (gate.has_value()) {
    check_act(*gate, "gate");
    TORCH_CHECK(gate->dim() == 2 && gate->size(0) == N && gate->size(1) == (long)H * D && gate->stride(1) == 1);
    gs = gate->stride(0);
  }
  const long units = N * H;
  const unsigned grid = (unsigned)((units + 3) / 4);
  SERVING_DISPATCH_ACT(x, TI, {
    SERVING_DISPATCH_ACT(out, TO, {
      if (gate.has_value()) {
        SERVING_DISPATCH_ACT(*gate, TG, {
          hipLaunchKernelGGL((head_rms_norm_gate_kernel<TI, TG, TO>), dim3(grid), dim3(256), 0, stream(), ptr<TO>(out),
                             ptr<TI>(x), (long)x.stride(0), w.data_ptr<float>(), ptr<TG>(*gate), gs, units, H, D,
                             (float)eps);
        });
      } else {
        hipLaunchKernelGGL((head_rms_norm_gate_kernel<TI, float, TO>), dim3(grid), dim3(256), 0, stream(),
                           ptr<TO>(out), ptr<TI>(x), (long)x.stride(0), w.data_ptr<float>(), (const float*)nullptr,
                           0L, units, H, D, (float)eps);
      }
    });
  });
  HIP_CHECK_LAST();
  return out;
}

// One block per row; the merged row lives in LDS (W floats).
template <typename T>
__global__ __launch_bounds__(256) void merge_rms_norm_kernel(
    float* __restrict__ residual, const T* __restrict__ a, const float* __restrict__ wa, const T* __restrict__ b,
    const float* __restrict__ wb, const float* __restrict__ wo, int W, int groups, float eps) {
  extern __shared__ float merged[];
  __shared__ float red[8];
  const long row = blockIdx.x;
  const T* ar = a + row * W;
  const T* br = b + row * W;
  float sa = 0.0f, sb = 0.0f;
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    const float va = ldf(ar + i), vb = ldf(br + i);
    sa += va * va;
    sb += vb * vb;
  }
  sa = block_reduce_sum(sa, red);
  sb = block_reduce_sum(sb, red);
  const float ia = 1.0f / sqrtf(sa / (float)W + eps), ib = 1.0f / sqrtf(sb / (float)W + eps);
  for (int i = threadIdx.x; i < W; i += blockDim.x)
    merged[i] = 0.5f * (ldf(ar + i) * ia * wa[i] + ldf(br + i) * ib * wb[i]);
  __syncthreads();
  const int gs = W / groups, lane = threadIdx.x & 63, nw = blockDim.x >> 6;
  for (int g = threadIdx.x >> 6; g < groups; g += nw) {
    float s = 0.0f;
    for (int i = lane; i < gs; i += 64) {
      const float v = merged[g * gs + i];
      s += v * v;
    }
    s = wave_reduce_sum(s);
    const float inv = 1.0f / sqrtf(s / (float)gs + eps);
    for (int i = lane; i < gs; i += 64) residual[row * W + g * gs + i] += merged[g * gs + i] * inv * wo[g * gs + i];
  }
}

at::Tensor merge_rms_norm(at::Tensor a, at::Tensor wa, at::Tensor b, at::Tensor wb, double eps, at::Tensor out_w,
                          int64_t groups, at::Tensor residual) {
  check_act(a, "a");
  TORCH_CHECK(a.dim() == 2 && a.is_contiguous() && b.is_contiguous() && a.sizes() == b.sizes() &&
              a.scalar_type() == b.scalar_type());
  TORCH_CHECK(is_f32(residual) && residual.is_contiguous() && residual.sizes() == a.sizes());
  const long N = a.size(0);
  const int W = (int)a.size(1);
  TORCH_CHECK(groups > 0 && W % groups == 0 && W * 4 <= 64 * 1024, "row too wide for the LDS-staged merge");
  at::Tensor fa = f32c(wa), fb = f32c(wb), fo = f32c(out_w);
  TORCH_CHECK(fa.numel() == W && fb.numel() == W && fo.numel() == W);
  if (N == 0) return residual;
  SERVING_DISPATCH_ACT(a, T, {
    hipLaunchKernelGGL(merge_rms_norm_kernel<T>, dim3((unsigned)N), dim3(256), (size_t)W * 4, stream(),
                       residual.data_ptr<float>(), ptr<T>(a), fa.data_ptr<float>(), ptr<T>(b), fb.data_ptr<float>(),
                       fo.data_ptr<float>(), W, (int)groups, (float)eps);
  });
  HIP_CHECK_LAST();
  return residual;
}

// One block per row. Pass 1 forms r = residual + (a + b) in float32, stores it and sums r^2; pass 2
// (only with a weight) re-reads the elements this same thread stored and writes the normed row.
template <typename TA, typename TB, typename TO>
__global__ __launch_bounds__(256) void add_rms_norm_kernel(
    TO* __restrict__ out, float* __restrict__ residual, const TA* __restrict__ a, const TB* __restrict__ b,
    const float* __restrict__ w, int W, float eps) {
  __shared__ float red[8];
  const long row = blockIdx.x;
  float* rr = residual + row * W;
  float ssq = 0.0f;
#pragma unroll 4
  for (int i = threadIdx.x; i < W; i += blockDim.x) {
    float add = ldf(a + row * W + i);
    if (b != nullptr) add += ldf(b + row * W + i);
    const float r = rr[i] + add;
    rr[i] = r;
    ssq += r * r;
  }
  if (w == nullptr) return;
  ssq = block_reduce_sum(ssq, red);
  const float inv = 1.0f / sqrtf(ssq / (float)W + eps);
  for (int i = threadIdx.x; i < W; i += blockDim.x) stf(out + row * W + i, rr[i] * inv * w[i]);
}

// Row-in-registers form for rows of up to 2048 * CH elements (W a multiple of 8, 32-byte aligned
// operands): each thread owns CH chunks of 8 consecutive elements, reads every operand once with
// 16/32-byte loads, keeps the summed row in registers across the reduction and writes residual and
// normed row once.
template <typename TA, typename TB, typename TO, int CH>
__global__ __launch_bounds__(256) void add_rms_norm_rows_kernel(
    TO* __restrict__ out, float* __restrict__ residual, const TA* __restrict__ a, const TB* __restrict__ b,
    const float* __restrict__ w, int W, float eps) {
  __shared__ float red[8];
  const long row = blockIdx.x;
  float r[CH][8];
  float ssq = 0.0f;
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const int i = (threadIdx.x + 256 * c) * 8;
    if (i < W) {
      float av[8], bv[8];
      load8(residual + row * W + i, r[c]);
      load8(a + row * W + i, av);
      if (b != nullptr) load8(b + row * W + i, bv);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        r[c][e] += b != nullptr ? av[e] + bv[e] : av[e];
        ssq += r[c][e] * r[c][e];
      }
      store8(residual + row * W + i, r[c]);
    }
  }
  if (w == nullptr) return;
  ssq = block_reduce_sum(ssq, red);
  const float inv = 1.0f / sqrtf(ssq / (float)W + eps);
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const int i = (threadIdx.x + 256 * c) * 8;
    if (i < W) {
      float wv[8];
      load8(w + i, wv);
#pragma unroll
      for (int e = 0; e < 8; ++e) wv[e] *= r[c][e] * inv;
      store8(out + row * W + i, wv);
    }
  }
}

c10::optional<at::Tensor> add_rms_norm(at::Tensor residual, at::Tensor a, c10::optional<at::Tensor> b,
                                       c10::optional<at::Tensor> weight, double eps, at::ScalarType out_dtype) {
  check_act(a, "a");
  TORCH_CHECK(residual.is_cuda() && is_f32(residual) && residual.dim() == 2 && residual.is_contiguous(),
              "residual must be contiguous float32 [N, W]");
  TORCH_CHECK(a.is_contiguous() && a.sizes() == residual.sizes(), "a must be contiguous and of the residual's shape");
  if (b.has_value()) {
    check_act(*b, "b");
    TORCH_CHECK(b->is_contiguous() && b->sizes() == residual.sizes(), "b must be contiguous and of the residual's shape");
  }
  const long N = residual.size(0);
  const int W = (int)residual.size(1);
  at::Tensor w, out;
  const float* wp = nullptr;
  if (weight.has_value()) {
    w = f32c(*weight);
    TORCH_CHECK(w.numel() == W);
    wp = w.data_ptr<float>();
    out = at::empty({N, W}, residual.options().dtype(out_dtype));
    check_act(out, "out");
  }
  if (N > 0) {
    // without a weight nothing is written through `out`: any instantiation of TO will do
    const at::Tensor& like = weight.has_value() ? out : residual;
    auto al32 = [](const at::Tensor& t) { return reinterpret_cast<uintptr_t>(t.data_ptr()) % 32 == 0; };
    const bool rows = W % 8 == 0 && W <= 2048 * 4 && al32(residual) && al32(a) && (!b.has_value() || al32(*b)) &&
                      (!weight.has_value() || (al32(out) && al32(w)));
    const float* nob = nullptr;
#define ADD_NORM_LAUNCH(TB_, bp)                                                                                        \
  do {                                                                                                                  \
    if (rows && W <= 2048)                                                                                              \
      hipLaunchKernelGGL((add_rms_norm_rows_kernel<TA, TB_, TO, 1>), dim3((unsigned)N), dim3(256), 0, stream(), op,    \
                         residual.data_ptr<float>(), ptr<TA>(a), bp, wp, W, (float)eps);                                \
    else if (rows && W <= 4096)                                                                                         \
      hipLaunchKernelGGL((add_rms_norm_rows_kernel<TA, TB_, TO, 2>), dim3((unsigned)N), dim3(256), 0, stream(), op,    \
                         residual.data_ptr<float>(), ptr<TA>(a), bp, wp, W, (float)eps);                                \
    else if (rows)                                                                                                      \
      hipLaunchKernelGGL((add_rms_norm_rows_kernel<TA, TB_, TO, 4>), dim3((unsigned)N), dim3(256), 0, stream(), op,    \
                         residual.data_ptr<float>(), ptr<TA>(a), bp, wp, W, (float)eps);                                \
    else                                                                                                                \
      hipLaunchKernelGGL((add_rms_norm_kernel<TA, TB_, TO>), dim3((unsigned)N), dim3(256), 0, stream(), op,            \
                         residual.data_ptr<float>(), ptr<TA>(a), bp, wp, W, (float)eps);                                \
  } while (0)
    SERVING_DISPATCH_ACT(a, TA, {
      SERVING_DISPATCH_ACT(like, TO, {
        TO* op = weight.has_value() ? ptr<TO>(out) : (TO*)nullptr;
        if (b.has_value()) {
          SERVING_DISPATCH_ACT(*b, TB, { ADD_NORM_LAUNCH(TB, ptr<TB>(*b)); });
        } else {
          ADD_NORM_LAUNCH(float, nob);
        }
      });
    });
#undef ADD_NORM_LAUNCH
    HIP_CHECK_LAST();
  }
  if (!weight.has_value()) return c10::nullopt;
  return out;
}

}  // namespace serving
}  // namespace cai
