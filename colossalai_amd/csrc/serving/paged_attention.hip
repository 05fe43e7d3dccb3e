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
constexpr int ATT_WAVES = 4;        // waves of a block: they split the keys of one (token, head)

DEV_INLINE float dot_row(const float* kr, const float* qs, int D, bool vec) {
  float dot = 0.0f;
  if (vec) {
    for (int d = 0; d < D; d += 4) {
      const float4v kv = *reinterpret_cast<const float4v*>(kr + d);
      const float4v qv = *reinterpret_cast<const float4v*>(qs + d);
      dot += kv[0] * qv[0] + kv[1] * qv[1] + kv[2] * qv[2] + kv[3] * qv[3];
    }
  } else {
    for (int d = 0; d < D; ++d) dot += qs[d] * kr[d];
  }
  return dot;
}

DEV_INLINE float dot_row(const bf16s* kr, const float* qs, int D, bool vec) {
  float dot = 0.0f;
  if (vec) {
    for (int d = 0; d < D; d += 8) {
      const short8 kv = *reinterpret_cast<const short8*>(kr + d);
      const float4v qa = *reinterpret_cast<const float4v*>(qs + d);
      const float4v qb = *reinterpret_cast<const float4v*>(qs + d + 4);
      dot += bf2f((bf16s)kv[0]) * qa[0] + bf2f((bf16s)kv[1]) * qa[1] + bf2f((bf16s)kv[2]) * qa[2] +
             bf2f((bf16s)kv[3]) * qa[3] + bf2f((bf16s)kv[4]) * qb[0] + bf2f((bf16s)kv[5]) * qb[1] +
             bf2f((bf16s)kv[6]) * qb[2] + bf2f((bf16s)kv[7]) * qb[3];
    }
  } else {
    for (int d = 0; d < D; ++d) dot += qs[d] * bf2f(kr[d]);
  }
  return dot;
}

// Scalar kernel (decode tokens, float32 serving, shapes the MFMA kernel does not take).
// One block per (token, head); its four waves take every fourth 64-key block and merge
// their partial softmax states through LDS.
template <typename T>
__global__ __launch_bounds__(64 * ATT_WAVES) void paged_attention_kernel(
    T* __restrict__ out, const T* __restrict__ q, long q_stride, const T* __restrict__ kpool,
    const T* __restrict__ vpool, const int* __restrict__ block_tables, int bt_stride, const int* __restrict__ tok_seq,
    const int* __restrict__ positions, const float* __restrict__ slopes, const T* __restrict__ gate, long gate_stride,
    int H, int G, int D, int Dv, int page_shift, float scale, int window, int keep_first, int kvec) {
  extern __shared__ __align__(16) float lds[];
  const int wid = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int Dp = (D + 3) & ~3;
  float* qs = lds;                                   // [Dp] query
  float* pw = lds + Dp + wid * 128;                  // [64] weights of this wave's key block
  int* prow = reinterpret_cast<int*>(pw + 64);       // [64] pool rows of the block
  float* part = lds + Dp + ATT_WAVES * 128;          // [waves][2 + Dv] partial states
  const long n = blockIdx.x / H;
  const int h = (int)(blockIdx.x % H);
  const int g = h / (H / G);
  const int b = tok_seq[n];
  const int pos = positions[n];
  const int* bt = block_tables + (long)b * bt_stride;
  const int page_mask = (1 << page_shift) - 1;

  for (int i = threadIdx.x; i < D; i += blockDim.x) qs[i] = ldf(q + n * q_stride + (long)h * D + i);
  __syncthreads();
  const float slope = slopes != nullptr ? slopes[h] : 0.0f;

  const int lo = window > 0 ? max(0, pos - window + 1) : 0;
  const int n_keep = window > 0 ? min(keep_first, lo) : 0;
  const int total = n_keep + (pos - lo + 1);

  float m = -INFINITY, l = 0.0f;
  float acc[MAX_VD_PER_LANE];
#pragma unroll
  for (int i = 0; i < MAX_VD_PER_LANE; ++i) acc[i] = 0.0f;

  for (int base = wid * 64; base < total; base += 64 * ATT_WAVES) {
    const int idx = base + lane;
    const bool valid = idx < total;
    float s = -INFINITY;
    int row = 0;
    if (valid) {
      const int j = idx < n_keep ? idx : lo + (idx - n_keep);
      row = (bt[j >> page_shift] << page_shift) + (j & page_mask);
      s = dot_row(kpool + ((long)row * G + g) * D, qs, D, kvec != 0) * scale - slope * (float)(pos - j);
    }
    const float m_new = fmaxf(m, wave_reduce_max(s));  // a block holds at least one valid key
    const float w = valid ? expf(s - m_new) : 0.0f;
    const float corr = expf(m - m_new);  // m = -inf on the first block: exp(-inf) = 0
    l = l * corr + wave_reduce_sum(w);
    m = m_new;
    pw[lane] = w;
    prow[lane] = row;
    // the wave is its own producer and consumer of pw/prow: wait for its LDS writes
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
  float* mine = part + wid * (2 + Dv);
  if (lane == 0) { mine[0] = m; mine[1] = l; }
#pragma unroll
  for (int i = 0; i < MAX_VD_PER_LANE; ++i) {
    const int dv = lane + 64 * i;
    if (dv < Dv) mine[2 + dv] = acc[i];
  }
  __syncthreads();
  float mm = -INFINITY;
  for (int w = 0; w < ATT_WAVES; ++w) mm = fmaxf(mm, part[w * (2 + Dv)]);
  float ll = 0.0f;
  for (int w = 0; w < ATT_WAVES; ++w) {
    const float mw = part[w * (2 + Dv)];
    if (mw != -INFINITY) ll += part[w * (2 + Dv) + 1] * expf(mw - mm);
  }
  float scale_out = 1.0f / ll;
  if (gate != nullptr) scale_out *= sigmoidf_(ldf(gate + n * gate_stride + h));
  for (int dv = threadIdx.x; dv < Dv; dv += blockDim.x) {
    float o = 0.0f;
    for (int w = 0; w < ATT_WAVES; ++w) {
      const float mw = part[w * (2 + Dv)];
      if (mw != -INFINITY) o += part[w * (2 + Dv) + 2 + dv] * expf(mw - mm);
    }
    stf(out + (n * H + h) * (long)Dv + dv, o * scale_out);
  }
}

// MFMA kernel (bfloat16 prompt portions). One wave per (32-token tile of one sequence, head);
// the four waves of a block take four neighbouring heads of the same tile. All per-token
// quantities are lane-local because the products are formed transposed:
//   S^T = K Q^T   (A = key rows, B = query rows: both read along the head size, 16 B a lane)
//   O^T = V^T P^T (B = the float32 weights in the C layout they were born in, split into a
//                  high and a low bfloat16 half so that no weight loses its float32 mantissa
//                  to the matrix unit; A = values gathered with the same key order)
// so column = token = lane & 31 everywhere: running max, running sum, rescaling and the gate
// never cross lanes except for one exchange between the two half-waves.
template <int DS, int VT>
__global__ __launch_bounds__(256) void paged_attention_mfma_kernel(
    bf16s* __restrict__ out, const bf16s* __restrict__ q, long q_stride, const bf16s* __restrict__ kpool,
    const bf16s* __restrict__ vpool, const int* __restrict__ block_tables, int bt_stride, const int* __restrict__ cu,
    const int* __restrict__ start, const float* __restrict__ slopes, const bf16s* __restrict__ gate, long gate_stride,
    int H, int G, int page_shift, float scale, int window, int keep_first) {
  constexpr int D = DS * 16, Dv = VT * 32;
  const int wid = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int h = blockIdx.y * 4 + wid;
  if (h >= H) return;  // waves never synchronise with each other
  int tile = blockIdx.x, b = 0;
  for (;; ++b) {  // the grid holds exactly sum_b ceil(count_b / 32) tiles
    const int nt = (cu[b + 1] - cu[b] + 31) >> 5;
    if (tile < nt) break;
    tile -= nt;
  }
  const int cnt = cu[b + 1] - cu[b];
  const int col = lane & 31, hf = lane >> 5;
  const int t_off = tile * 32;
  const bool tok_ok = t_off + col < cnt;
  const int my_i = tok_ok ? t_off + col : cnt - 1;
  const long n = cu[b] + my_i;
  const int s0 = start[b];
  const int pos = s0 + my_i;
  const int p0 = s0 + t_off, p1 = s0 + min(t_off + 31, cnt - 1);
  const int g = h / (H / G);
  const int* bt = block_tables + (long)b * bt_stride;
  const int page_mask = (1 << page_shift) - 1;
  const float slope = slopes != nullptr ? slopes[h] : 0.0f;

  bf16x8_v qf[DS];
#pragma unroll
  for (int s = 0; s < DS; ++s) qf[s] = ld_g16b(q + n * q_stride + (long)h * D + 16 * s + hf * 8);

  const int lo_min = window > 0 ? max(0, p0 - window + 1) : 0;
  const int wstart = lo_min & ~31;
  const int n_sink = window > 0 ? min(keep_first, wstart) : 0;  // kept keys below the window's first tile
  const int sink_tiles = (n_sink + 31) >> 5;
  const int tiles = sink_tiles + ((p1 - wstart) >> 5) + 1;

  float m = -INFINITY, l = 0.0f;
  f32x16 oacc[VT];
#pragma unroll
  for (int t = 0; t < VT; ++t)
#pragma unroll
    for (int i = 0; i < 16; ++i) oacc[t][i] = 0.0f;

  for (int it = 0; it < tiles; ++it) {
    const bool sink = it < sink_tiles;
    const int kbase = sink ? it * 32 : wstart + (it - sink_tiles) * 32;
    const int klimit = sink ? n_sink : p1 + 1;  // keys of this tile at or above it are not this tile's to count
    // S^T tile: rows = keys kbase..kbase+31, columns = the 32 tokens
    const int jk = min(kbase + col, p1);
    const long krow = ((long)bt[jk >> page_shift] << page_shift) + (jk & page_mask);
    const bf16s* kr = kpool + (krow * G + g) * D + hf * 8;
    f32x16 sacc;
#pragma unroll
    for (int i = 0; i < 16; ++i) sacc[i] = 0.0f;
#pragma unroll
    for (int s = 0; s < DS; ++s)
      sacc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(ld_g16b(kr + 16 * s), qf[s], sacc, 0, 0, 0);
    float sv[16];
    float tmax = -INFINITY;
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const int j = kbase + (i & 3) + 8 * (i >> 2) + 4 * hf;
      const bool seen = tok_ok && j < klimit && j <= pos && (window == 0 || pos - j < window || j < keep_first);
      sv[i] = seen ? sacc[i] * scale - slope * (float)(pos - j) : -INFINITY;
      tmax = fmaxf(tmax, sv[i]);
    }
    tmax = fmaxf(tmax, __shfl_xor(tmax, 32));
    const float m_new = fmaxf(m, tmax);
    const float corr = (m == -INFINITY) ? 1.0f : __expf(m - m_new);  // nothing accumulated yet: nothing to rescale
    float psum = 0.0f;
    bf16x8_v phi[2], plo[2];
#pragma unroll
    for (int i = 0; i < 16; ++i) {
      const float p = (sv[i] == -INFINITY) ? 0.0f : __expf(sv[i] - m_new);
      psum += p;
      const __bf16 hi = (__bf16)p;
      phi[i >> 3][i & 7] = hi;
      plo[i >> 3][i & 7] = (__bf16)(p - (float)hi);
    }
    l = l * corr + psum;
    m = m_new;
#pragma unroll
    for (int t = 0; t < VT; ++t)
#pragma unroll
      for (int i = 0; i < 16; ++i) oacc[t][i] *= corr;
    // O^T += V^T P^T: contraction slot (hf, e) of step s2 is key kbase + 16 s2 + 8 (e >> 2) + 4 hf + (e & 3)
#pragma unroll
    for (int s2 = 0; s2 < 2; ++s2) {
      long vrow[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const int j = min(kbase + 16 * s2 + 8 * (e >> 2) + 4 * hf + (e & 3), p1);
        vrow[e] = ((((long)bt[j >> page_shift] << page_shift) + (j & page_mask)) * G + g) * Dv + col;
      }
#pragma unroll
      for (int t = 0; t < VT; ++t) {
        bf16x8_v va;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const bf16s raw = vpool[vrow[e] + t * 32];
          va[e] = *reinterpret_cast<const __bf16*>(&raw);
        }
        oacc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va, phi[s2], oacc[t], 0, 0, 0);
        oacc[t] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(va, plo[s2], oacc[t], 0, 0, 0);
      }
    }
  }
  l += __shfl_xor(l, 32);
  if (!tok_ok) return;
  float scale_out = 1.0f / l;
  if (gate != nullptr) scale_out *= sigmoidf_(ldf(gate + n * gate_stride + h));
  bf16s* orow = out + (n * H + h) * (long)Dv;
#pragma unroll
  for (int t = 0; t < VT; ++t)
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      short4v pk;
#pragma unroll
      for (int c = 0; c < 4; ++c) pk[c] = (short)f2bf(oacc[t][4 * a + c] * scale_out);
      *reinterpret_cast<short4v*>(orow + t * 32 + 8 * a + 4 * hf) = pk;
    }
}

at::Tensor paged_attention(at::Tensor q, at::Tensor kpool, at::Tensor vpool, at::Tensor block_tables, at::Tensor cu,
                           at::Tensor start, at::Tensor tok_seq, at::Tensor positions, double scale, int64_t window,
                           int64_t keep_first, c10::optional<at::Tensor> slopes, c10::optional<at::Tensor> gate,
                           int64_t num_tiles) {
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
  check_i32(cu, "cu"); check_i32(start, "start");
  // prompt portions in bfloat16 go to the matrix cores when the head sizes fit a tiling;
  // num_tiles = sum over sequences of ceil(new tokens / 32), 0 asks for the scalar kernel
  const bool aligned = q.stride(0) % 8 == 0 && reinterpret_cast<uintptr_t>(q.data_ptr()) % 16 == 0;
  const bool mfma_shape = (D == 32 && Dv == 32) || ((D == 64 || D == 128) && (Dv == 64 || Dv == 128));
  if (num_tiles > 0 && is_bf16(q) && aligned && mfma_shape) {
    const dim3 grid((unsigned)num_tiles, (unsigned)((H + 3) / 4));
#define MFMA_CASE(DS_, VT_)                                                                                          \
  hipLaunchKernelGGL((paged_attention_mfma_kernel<DS_, VT_>), grid, dim3(256), 0, stream(), ptr<bf16s>(out),        \
                     ptr<bf16s>(q), (long)q.stride(0), ptr<bf16s>(kpool), ptr<bf16s>(vpool),                        \
                     block_tables.data_ptr<int>(), (int)block_tables.stride(0), cu.data_ptr<int>(),                 \
                     start.data_ptr<int>(), slp, gate.has_value() ? ptr<bf16s>(*gate) : (const bf16s*)nullptr,      \
                     gstride, H, G, page_shift, (float)scale, (int)window, (int)keep_first)
    if (D == 32) MFMA_CASE(2, 1);
    else if (D == 64 && Dv == 64) MFMA_CASE(4, 2);
    else if (D == 64 && Dv == 128) MFMA_CASE(4, 4);
    else if (D == 128 && Dv == 64) MFMA_CASE(8, 2);
    else MFMA_CASE(8, 4);
#undef MFMA_CASE
    HIP_CHECK_LAST();
    return out;
  }
  const int Dp = (D + 3) & ~3;
  const size_t smem = (size_t)(Dp + ATT_WAVES * 128 + ATT_WAVES * (2 + Dv)) * sizeof(float);
  const int kvec = (is_bf16(q) ? D % 8 == 0 : D % 4 == 0) ? 1 : 0;
  SERVING_DISPATCH_ACT(q, T, {
    hipLaunchKernelGGL(paged_attention_kernel<T>, dim3((unsigned)(N * H)), dim3(64 * ATT_WAVES), smem, stream(),
                       ptr<T>(out), ptr<T>(q), (long)q.stride(0), ptr<T>(kpool), ptr<T>(vpool),
                       block_tables.data_ptr<int>(), (int)block_tables.stride(0), tok_seq.data_ptr<int>(),
                       positions.data_ptr<int>(), slp, gate.has_value() ? ptr<T>(*gate) : (const T*)nullptr, gstride,
                       H, G, D, Dv, page_shift, (float)scale, (int)window, (int)keep_first, kvec);
  });
  HIP_CHECK_LAST();
  return out;
}

}  // namespace serving
}  // namespace cai
