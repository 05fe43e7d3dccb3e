// Attention of a ragged batch over paged keys/values with a sliding window,
// kept first tokens, a linear distance penalty and a per-head output gate.
//
// One wave per (token, query head). The visible keys of a token are two
// position ranges: the kept prefix [0, min(keep_first, lo)) and the window
// [lo, pos] with lo = max(0, pos - window + 1) (lo = 0 without a window); the
// wave walks their concatenation 64 keys at a time. Phase 1: lane = key, each
// lane takes the full dot product of its key with the query (query in LDS,
// key row read with its own page lookup). Online softmax in float32 across
// the 64-key blocks. Phase 2: lane = value channel, the block's weights and
// pool rows are broadcast from LDS. A prompt portion and a decode token run
// the same code, so a position's result depends on nothing but the pages.
#include "serving_common.h"

namespace cai {
namespace serving {

constexpr int MAX_VD_PER_LANE = 4;  // value size up to 256
constexpr int ATT_WAVES = 4;        // (token, head) units per block

template <typename T>
__global__ __launch_bounds__(64 * ATT_WAVES) void paged_attention_kernel(
    T* __restrict__ out, const T* __restrict__ q, long q_stride, const T* __restrict__ kpool,
    const T* __restrict__ vpool, const int* __restrict__ block_tables, int bt_stride, const int* __restrict__ tok_seq,
    const int* __restrict__ positions, const float* __restrict__ slopes, const T* __restrict__ gate, long gate_stride,
    long units, int H, int G, int D, int Dv, int page_shift, float scale, int window, int keep_first) {
  extern __shared__ float lds[];
  const int wid = threadIdx.x >> 6, lane = threadIdx.x & 63;
  float* qs = lds + wid * (D + 128);   // [D] query
  float* pw = qs + D;                  // [64] weights of the block
  int* prow = reinterpret_cast<int*>(pw + 64);  // [64] pool rows of the block
  const long unit = (long)blockIdx.x * ATT_WAVES + wid;
  if (unit >= units) return;  // whole wave leaves; nothing below synchronises across waves
  const long n = unit / H;
  const int h = (int)(unit % H);
  const int g = h / (H / G);
  const int b = tok_seq[n];
  const int pos = positions[n];
  const int* bt = block_tables + (long)b * bt_stride;
  const int page_mask = (1 << page_shift) - 1;

  for (int i = lane; i < D; i += 64) qs[i] = ldf(q + n * q_stride + (long)h * D + i);
  const float slope = slopes != nullptr ? slopes[h] : 0.0f;

  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  const int n_keep = window > 0 ? min(keep_first, lo) : 0;
  const int total = n_keep + (pos - lo + 1);

  float m = -INFINITY, l = 0.0f;
  float acc[MAX_VD_PER_LANE];
#pragma unroll
  for (int i = 0; i < MAX_VD_PER_LANE; ++i) acc[i] = 0.0f;

  for (int base = 0; base < total; base += 64) {
    const int idx = base + lane;
    const bool valid = idx < total;
    float s = -INFINITY;
    int row = 0;
    if (valid) {
      const int j = idx < n_keep ? idx : lo + (idx - n_keep);
      row = (bt[j >> page_shift] << page_shift) + (j & page_mask);
      const T* kr = kpool + ((long)row * G + g) * D;
      float dot = 0.0f;
      for (int d = 0; d < D; ++d) dot += qs[d] * ldf(kr + d);
      s = dot * scale - slope * (float)(pos - j);
    }
    const float bm = wave_reduce_max(s);
    const float m_new = fmaxf(m, bm);
    const float w = valid ? expf(s - m_new) : 0.0f;
    const float corr = expf(m - m_new);  // m = -inf on the first block: exp(-inf) = 0
    l = l * corr + wave_reduce_sum(w);
    m = m_new;
    pw[lane] = w;
    prow[lane] = row;
    // the wave is its own producer and consumer of pw/prow: LDS ops of one wave complete in order
    __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0)
    const int cnt = min(64, total - base);
#pragma unroll
    for (int i = 0; i < MAX_VD_PER_LANE; ++i) {
      const int dv = lane + 64 * i;
      if (dv < Dv) {
        float a = acc[i] * corr;
        for (int jj = 0; jj < cnt; ++jj) a += pw[jj] * ldf(vpool + ((long)prow[jj] * G + g) * Dv + dv);
        acc[i] = a;
      }
    }
    __builtin_amdgcn_s_waitcnt(0xc07f);
  }
  float scale_out = 1.0f / l;
  if (gate != nullptr) scale_out *= sigmoidf_(ldf(gate + n * gate_stride + h));
#pragma unroll
  for (int i = 0; i < MAX_VD_PER_LANE; ++i) {
    const int dv = lane + 64 * i;
    if (dv < Dv) stf(out + (n * H + h) * (long)Dv + dv, acc[i] * scale_out);
  }
}

at::Tensor paged_attention(at::Tensor q, at::Tensor kpool, at::Tensor vpool, at::Tensor block_tables, at::Tensor cu,
                           at::Tensor start, at::Tensor tok_seq, at::Tensor positions, double scale, int64_t window,
                           int64_t keep_first, c10::optional<at::Tensor> slopes, c10::optional<at::Tensor> gate) {
  check_act(q, "q");
  TORCH_CHECK(q.dim() == 3 && q.stride(2) == 1 && q.stride(1) == q.size(2), "q must be [N, H, D] with dense rows");
  TORCH_CHECK(kpool.dim() == 4 && vpool.dim() == 4 && kpool.is_contiguous() && vpool.is_contiguous());
  TORCH_CHECK(kpool.scalar_type() == q.scalar_type() && vpool.scalar_type() == q.scalar_type(),
              "query and pools share one dtype");
  const long N = q.size(0);
  const int H = (int)q.size(1), D = (int)q.size(2);
  const int page = (int)kpool.size(1), G = (int)kpool.size(2), Dv = (int)vpool.size(3);
  TORCH_CHECK(kpool.size(3) == D && vpool.size(2) == G && vpool.size(1) == page && vpool.size(0) == kpool.size(0));
  TORCH_CHECK(H % G == 0 && Dv <= 64 * MAX_VD_PER_LANE && page > 0 && (page & (page - 1)) == 0);
  check_i32(block_tables, "block_tables"); check_i32(tok_seq, "tok_seq"); check_i32(positions, "positions");
  TORCH_CHECK(block_tables.dim() == 2 && tok_seq.numel() == N && positions.numel() == N);
  TORCH_CHECK(window >= 0 && keep_first >= 0);
  int page_shift = 0;
  while ((1 << page_shift) < page) ++page_shift;
  at::Tensor sl;
  const float* slp = nullptr;
  if (slopes.has_value()) {
    sl = f32c(*slopes);
    TORCH_CHECK(sl.numel() == H);
    slp = sl.data_ptr<float>();
  }
  long gstride = 0;
  if (gate.has_value()) {
    TORCH_CHECK(gate->scalar_type() == q.scalar_type() && gate->dim() == 2 && gate->size(0) == N &&
                gate->size(1) == H && gate->stride(1) == 1, "gate must be [N, H] of q's dtype");
    gstride = gate->stride(0);
  }
  at::Tensor out = at::empty({N, H, Dv}, q.options());
  if (N == 0) return out;
  const long units = N * H;
  const unsigned grid = (unsigned)((units + ATT_WAVES - 1) / ATT_WAVES);
  const size_t smem = (size_t)ATT_WAVES * (D + 128) * sizeof(float);
  SERVING_DISPATCH_ACT(q, T, {
    hipLaunchKernelGGL(paged_attention_kernel<T>, dim3(grid), dim3(64 * ATT_WAVES), smem, stream(), ptr<T>(out),
                       ptr<T>(q), (long)q.stride(0), ptr<T>(kpool), ptr<T>(vpool), block_tables.data_ptr<int>(),
                       (int)block_tables.stride(0), tok_seq.data_ptr<int>(), positions.data_ptr<int>(), slp,
                       gate.has_value() ? ptr<T>(*gate) : (const T*)nullptr, gstride, units, H, G, D, Dv, page_shift,
                       (float)scale, (int)window, (int)keep_first);
  });
  HIP_CHECK_LAST();
  return out;
}

}  // namespace serving
}  // namespace cai
