// fp32 paged attention for models served in float32: every operand, score, weight and sum is a
// 32-bit float (no MFMA, no reduced-precision product), over the same paged cache layouts as the
// bf16 kernels (K [page, Hkv, P, D], V [page, Hkv, D, P]) with float elements.
//
// One 256-thread workgroup per (query row, query head).  A row knows its sequence (block-table
// row) and absolute position, so prompt chunks and decode rows are the same launch.  Visible keys:
// j <= pos and (j >= lo(pos, window) or j < keep) -- sliding window (window > 0), chunked
// attention (window < -1), kept first keys.  They are visited in chunks of CH keys: one thread per
// key forms q.k, the block reduces max and sum (online softmax across chunks), then one thread per
// output dim accumulates p.V.  Built for exactness at test sizes, not for speed.
// sinks (optional, fp32 [Hq]): a per-head logit that joins the softmax denominator once, unscaled,
// with no key and no value (exp(sink) is added to the sum of the weights).
#include "common.h"

namespace {

constexpr int CH = 1024;
constexpr int MAXD = 768;   // widest head (three output dims per thread)

__device__ __forceinline__ float block_max256(float v, float* red) {
  v = wave_max(v);
  const int w = threadIdx.x >> 6, l = threadIdx.x & 63;
  if (l == 0) red[w] = v;
  __syncthreads();
  const float t = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
  __syncthreads();
  return t;
}

__global__ __launch_bounds__(256) void paged_attention_f32_kernel(
    const float* __restrict__ q, int64_t q_stride, const float* __restrict__ k_cache,
    const float* __restrict__ v_cache, const int* __restrict__ block_tables, int bt_stride,
    const int* __restrict__ row_seq, const int* __restrict__ row_pos, float* __restrict__ out, int64_t out_stride,
    int Hq, int Hkv, int D, int P, float scale, int window, int keep, const float* __restrict__ sinks) {
  __shared__ float qs[MAXD];
  __shared__ float sc[CH];
  __shared__ float red[4];
  const int64_t t = blockIdx.x;
  const int h = blockIdx.y, tid = threadIdx.x;
  const int kvh = h / (Hq / Hkv);
  const int pos = row_pos[t];
  float* orow = out + t * out_stride + (int64_t)h * D;
  if (pos < 0) {   // padding row: no keys
    for (int d = tid; d < D; d += 256) orow[d] = 0.f;
    return;
  }
  const int* bt = block_tables + (int64_t)row_seq[t] * bt_stride;
  const int lo = window > 0 ? max(0, pos - window + 1) : (window < -1 ? pos - pos % (-window) : 0);
  const int kept = keep > 0 ? min(keep, lo) : 0;     // kept keys that lie before the window
  const int n_vis = kept + (pos - lo + 1);
  for (int d = tid; d < D; d += 256) qs[d] = q[t * q_stride + (int64_t)h * D + d];
  __syncthreads();
  float m = -__builtin_inff(), l = 0.f, acc[3] = {0.f, 0.f, 0.f};   // output dims tid, tid + 256, tid + 512
  for (int c0 = 0; c0 < n_vis; c0 += CH) {
    const int n = min(CH, n_vis - c0);
    float cm = -__builtin_inff();
    for (int i = tid; i < n; i += 256) {
      const int key = c0 + i < kept ? c0 + i : lo + (c0 + i - kept);
      const float* kp = k_cache + (((int64_t)bt[key / P] * Hkv + kvh) * P + key % P) * D;
      float s = 0.f;
      for (int d = 0; d < D; ++d) s += qs[d] * kp[d];
      s *= scale;
      sc[i] = s;
      cm = fmaxf(cm, s);
    }
    cm = block_max256(cm, red);           // (also orders the sc[] writes before the reads below)
    const float m_new = fmaxf(m, cm);
    float ps = 0.f;
    for (int i = tid; i < n; i += 256) {
      const float p = expf(sc[i] - m_new);
      sc[i] = p;
      ps += p;
    }
    ps = block_sum<256>(ps, red);
    const float alpha = expf(m - m_new);  // first chunk: exp(-inf) = 0
    l = l * alpha + ps;
    m = m_new;
#pragma unroll
    for (int j = 0; j < 3; ++j) {
      const int d = tid + 256 * j;
      if (d < D) {
        acc[j] *= alpha;
        for (int i = 0; i < n; ++i) {
          const int key = c0 + i < kept ? c0 + i : lo + (c0 + i - kept);
          acc[j] += sc[i] * v_cache[(((int64_t)bt[key / P] * Hkv + kvh) * D + d) * P + key % P];
        }
      }
    }
    __syncthreads();
  }
  if (sinks != nullptr) {
    const float sk = sinks[h], m_new = fmaxf(m, sk), alpha = expf(m - m_new);
    l = l * alpha + expf(sk - m_new);
#pragma unroll
    for (int j = 0; j < 3; ++j) acc[j] *= alpha;
  }
#pragma unroll
  for (int j = 0; j < 3; ++j)
    if (tid + 256 * j < D) orow[tid + 256 * j] = acc[j] / l;
}

}  // namespace

OME_API int ome_paged_attention_f32(const float* q, int64_t q_stride, const float* k_cache, const float* v_cache,
                                    const int* block_tables, int bt_stride, const int* row_seq, const int* row_pos,
                                    float* out, int64_t out_stride, int T, int Hq, int Hkv, int D, int P, float scale,
                                    int window, int keep_first, const float* sinks, hipStream_t stream) {
  if (T <= 0) return 0;
  if (D <= 0 || D > MAXD || P <= 0 || Hkv <= 0 || Hq % Hkv != 0) return -2;
  paged_attention_f32_kernel<<<dim3(T, Hq), 256, 0, stream>>>(q, q_stride, k_cache, v_cache, block_tables, bt_stride,
                                                              row_seq, row_pos, out, out_stride, Hq, Hkv, D, P, scale,
                                                              window, window > 0 && keep_first > 0 ? keep_first : 0,
                                                              sinks);
  OME_CHECK_LAUNCH();
  return 0;
}
