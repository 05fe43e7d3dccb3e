// Grouped matrix product of routed experts on the matrix cores (bfloat16):
//   out[r, :] = act(a[src(r), :] . w[e(r)]^T)   for rows r sorted by expert,
// with the experts' row ranges given by a device-side offsets vector, so that a
// step of any size runs all its experts in ONE launch and nothing goes to the
// host. `src` optionally gathers the rows of `a` (the up product reads the
// tokens' rows in place, no gathered copy is made); act is the identity or
// relu(.)^2 on the float32 accumulator.
//
// Block = 128 rows of one expert x 128 output columns, four waves in a 2 x 2
// arrangement of 64 x 64 (four 32x32x16 MFMA accumulators each). Both operands
// are K-contiguous, which is what the MFMA fragments want: a tile of 128 x 32
// is fetched with 16-byte loads into registers while the previous one is
// multiplied, then stored to LDS rows of 40 elements (16 rows of 16-byte reads
// then cover all 64 banks). A block finds its (expert, row tile) by walking the
// offsets; the grid is sized for the worst case sum_e ceil(rows_e / 128) <=
// ceil(P / 128) + E and surplus blocks leave at once.
#include "serving_common.h"

namespace cai {
namespace serving {

constexpr int GG_TM = 128, GG_TN = 128, GG_TK = 32, GG_PITCH = GG_TK + 8;
constexpr int GG_MAX_EXPERTS = 1024;

template <bool RELU_SQ>
__global__ __launch_bounds__(256) void expert_grouped_gemm_kernel(
    bf16s* __restrict__ out, const bf16s* __restrict__ a, const int* __restrict__ a_rows, const bf16s* __restrict__ w,
    const int* __restrict__ offsets, int E, int M, int K) {
  __shared__ __align__(16) bf16s As[2][GG_TM * GG_PITCH];
  __shared__ __align__(16) bf16s Bs[2][GG_TN * GG_PITCH];
  const int tid = threadIdx.x, wid = tid >> 6, lane = tid & 63;
  // which expert and which of its row tiles: the offsets come into LDS with one load per thread, every thread then
  // walks them there
  __shared__ int offs[GG_MAX_EXPERTS + 1];
  for (int i = tid; i <= E; i += 256) offs[i] = offsets[i];
  __syncthreads();
  int t = blockIdx.x, e = 0, row0 = 0, row_end = 0;
  bool found = false;
  for (; e < E; ++e) {
    const int lo = offs[e], hi = offs[e + 1];
    const int nt = (hi - lo + GG_TM - 1) / GG_TM;
    if (t < nt) {
      row0 = lo + t * GG_TM;
      row_end = hi;
      found = true;
      break;
    }
    t -= nt;
  }
  if (!found) return;  // the whole block: blockIdx.x is past the last tile
  const int col0 = blockIdx.y * GG_TN;

  // staging: chunk c = tid + 256 r of a 128 x 32 tile is row c / 4, elements 8 (c % 4) .. + 8
  const bf16s* ap[2];
  const bf16s* bp[2];
  int lds_off[2];
#pragma unroll
  for (int r = 0; r < 2; ++r) {
    const int c = tid + 256 * r, row = c >> 2, kc = (c & 3) * 8;
    const int grow = min(row0 + row, row_end - 1);  // rows past the expert's end repeat its last row and are not stored
    const long src = a_rows != nullptr ? a_rows[grow] : grow;
    ap[r] = a + src * K + kc;
    const int gcol = min(col0 + row, M - 1);
    bp[r] = w + ((long)e * M + gcol) * K + kc;
    lds_off[r] = row * GG_PITCH + kc;
  }
  bf16x8_v ra[2], rb[2];
  auto fetch = [&](int k0) {
#pragma unroll
    for (int r = 0; r < 2; ++r) {
      ra[r] = ld_g16b(ap[r] + k0);
      rb[r] = ld_g16b(bp[r] + k0);
    }
  };
  auto stash = [&](int buf) {
#pragma unroll
    for (int r = 0; r < 2; ++r) {
      *reinterpret_cast<bf16x8_v*>(&As[buf][lds_off[r]]) = ra[r];
      *reinterpret_cast<bf16x8_v*>(&Bs[buf][lds_off[r]]) = rb[r];
    }
  };

  const int wr = wid >> 1, wc = wid & 1, col = lane & 31, hf = lane >> 5;
  f32x16 acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int x = 0; x < 16; ++x) acc[i][j][x] = 0.0f;

  const int steps = K / GG_TK;
  fetch(0);
  stash(0);
  __syncthreads();
  for (int s = 0; s < steps; ++s) {
    const int buf = s & 1;
    const bool more = s + 1 < steps;
    if (more) fetch((s + 1) * GG_TK);
#pragma unroll
    for (int ks = 0; ks < GG_TK / 16; ++ks) {
      bf16x8_v af[2], bfr[2];
#pragma unroll
      for (int i = 0; i < 2; ++i)
        af[i] = *reinterpret_cast<const bf16x8_v*>(&As[buf][(wr * 64 + i * 32 + col) * GG_PITCH + ks * 16 + hf * 8]);
#pragma unroll
      for (int j = 0; j < 2; ++j)
        bfr[j] = *reinterpret_cast<const bf16x8_v*>(&Bs[buf][(wc * 64 + j * 32 + col) * GG_PITCH + ks * 16 + hf * 8]);
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bfr[j], acc[i][j], 0, 0, 0);
    }
    if (more) stash(buf ^ 1);
    __syncthreads();
  }
  // C layout of a 32 x 32 accumulator: element x of a lane is row (x & 3) + 8 (x >> 2) + 4 hf, column lane & 31
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j) {
      const int feat = col0 + wc * 64 + j * 32 + col;
#pragma unroll
      for (int x = 0; x < 16; ++x) {
        const int r = row0 + wr * 64 + i * 32 + (x & 3) + 8 * (x >> 2) + 4 * hf;
        if (r < row_end && feat < M) {
          float v = acc[i][j][x];
          if (RELU_SQ) {
            v = fmaxf(v, 0.0f);
            v *= v;
          }
          out[(long)r * M + feat] = f2bf(v);
        }
      }
    }
}

at::Tensor expert_grouped_gemm(at::Tensor a, c10::optional<at::Tensor> a_rows, at::Tensor w, at::Tensor offsets,
                               int64_t rows, bool relu_squared) {
  TORCH_CHECK(a.is_cuda() && is_bf16(a) && a.dim() == 2 && a.is_contiguous(), "a must be contiguous bfloat16 [rows, K]");
  TORCH_CHECK(w.is_cuda() && is_bf16(w) && w.dim() == 3 && w.is_contiguous(), "w must be contiguous bfloat16 [E, M, K]");
  check_i32(offsets, "offsets");
  const int E = (int)w.size(0), M = (int)w.size(1), K = (int)w.size(2);
  TORCH_CHECK(a.size(1) == K && offsets.numel() == E + 1, "shapes of a / w / offsets do not fit");
  TORCH_CHECK(K % GG_TK == 0, "the contraction size must be a multiple of 32");
  TORCH_CHECK(E <= GG_MAX_EXPERTS, "more experts than the grouped product's offsets buffer holds");
  TORCH_CHECK(reinterpret_cast<uintptr_t>(a.data_ptr()) % 16 == 0 && reinterpret_cast<uintptr_t>(w.data_ptr()) % 16 == 0);
  const int* rows_ptr = nullptr;
  if (a_rows.has_value()) {
    check_i32(*a_rows, "a_rows");
    TORCH_CHECK(a_rows->numel() == rows, "one source row per output row");
    rows_ptr = a_rows->data_ptr<int>();
  } else {
    TORCH_CHECK(a.size(0) == rows, "without a gather the rows of a are the output rows");
  }
  at::Tensor out = at::empty({rows, M}, a.options());
  if (rows == 0) return out;
  // worst case of sum_e ceil(rows_e / 128) when the rows are spread over the experts
  const dim3 grid((unsigned)((rows + GG_TM - 1) / GG_TM + E), (unsigned)((M + GG_TN - 1) / GG_TN));
  if (relu_squared)
    hipLaunchKernelGGL(expert_grouped_gemm_kernel<true>, grid, dim3(256), 0, stream(), ptr<bf16s>(out), ptr<bf16s>(a),
                       rows_ptr, ptr<bf16s>(w), offsets.data_ptr<int>(), E, M, K);
  else
    hipLaunchKernelGGL(expert_grouped_gemm_kernel<false>, grid, dim3(256), 0, stream(), ptr<bf16s>(out), ptr<bf16s>(a),
                       rows_ptr, ptr<bf16s>(w), offsets.data_ptr<int>(), E, M, K);
  HIP_CHECK_LAST();
  return out;
}

}  // namespace serving
}  // namespace cai
