// HGRN2 mixer core: gated linear recurrence whose forget gate also sets what is written, fused with
// the activations before it and the per-head RMS norm after it.
//
//   q_t = silu(q_raw),  f_t = l + (1 - l) * sigmoid(f_raw + f_bias)          (per head and channel d)
//   S_t = diag(f_t) S_{t-1} + (1 - f_t) v_t^T        S [dim, vdim] per head, fp32, per request slot
//   o_t = S_t^T q_t,   out_t = o_t / sqrt(mean_v(o_t^2) + eps) * w           (w [vdim], shared by heads)
//
// q_raw / f_raw / v are row-strided views of one fused projection (bf16, or float for fp32 models);
// gates, state, the dot products and the norm are fp32, `out` is rounded once.
//
// One 256-thread workgroup per (head, sequence) walks the sequence's rows.  Thread (g, v) keeps
// rows d = g, g + G, ... of column v of the state in registers (G = 256 / vdim thread groups), so
// the recurrence itself needs no LDS traffic for S.  Rows are taken TB at a time: (A) all threads
// turn the block's raw gates / queries into fp32 (f, q) pairs in LDS, (B) each thread runs its
// state slice over the TB rows and leaves a partial o per row, (C) the partials of the G groups
// are summed, (D) one wave per row reduces the mean square and writes the normed output.  Three
// barriers per TB rows.  Decode rows are sequences of length one (state in, state out).
#include "common.h"

namespace {

constexpr int TB = 8;

template <typename T, int MAXR>
__global__ __launch_bounds__(256) void hgrn2_scan_kernel(
    const T* __restrict__ q, const T* __restrict__ f, const T* __restrict__ v, int64_t in_stride,
    const T* __restrict__ f_bias, const T* __restrict__ lower, const T* __restrict__ w, float* __restrict__ state,
    T* __restrict__ out, int64_t out_stride, const int* __restrict__ cu, const int* __restrict__ slot,
    const int* __restrict__ reset, int H, int dim, int vdim, int G, float eps) {
  extern __shared__ float sm[];
  float2* fq = (float2*)sm;                      // [TB][dim]
  float* vv = sm + 2 * TB * dim;                 // [TB][vdim]
  float* part = vv + TB * vdim;                  // [TB][G][vdim]
  const int h = blockIdx.x, s = blockIdx.y, tid = threadIdx.x;
  const int r0 = cu[s], r1 = cu[s + 1];
  if (r1 <= r0) return;
  const int g = tid / vdim, vc = tid - g * vdim;
  const bool active = g < G;
  float* gst = state + ((int64_t)slot[s] * H + h) * dim * vdim;
  float S[MAXR];
  const bool fresh = reset[s] != 0;
#pragma unroll
  for (int i = 0; i < MAXR; ++i) {
    const int d = g + i * G;
    S[i] = (active && d < dim && !fresh) ? gst[(int64_t)d * vdim + vc] : 0.f;
  }
  for (int rb = r0; rb < r1; rb += TB) {
    const int nb = min(TB, r1 - rb);
    for (int idx = tid; idx < nb * dim; idx += 256) {
      const int tb = idx / dim, d = idx - tb * dim;
      const int64_t o = (int64_t)(rb + tb) * in_stride + h * dim + d;
      const float lo = (float)lower[h * dim + d];
      const float fr = (float)f[o] + (float)f_bias[h * dim + d];
      const float qr = (float)q[o];
      fq[idx] = make_float2(lo + (1.f - lo) / (1.f + expf(-fr)), qr / (1.f + expf(-qr)));
    }
    for (int idx = tid; idx < nb * vdim; idx += 256) {
      const int tb = idx / vdim, c = idx - tb * vdim;
      vv[idx] = (float)v[(int64_t)(rb + tb) * in_stride + h * vdim + c];
    }
    __syncthreads();
    if (active) {
      for (int tb = 0; tb < nb; ++tb) {
        const float vt = vv[tb * vdim + vc];
        const float2* fr = fq + tb * dim + g;
        float acc = 0.f;
#pragma unroll
        for (int i = 0; i < MAXR; ++i) {
          if (g + i * G < dim) {
            const float2 p = fr[i * G];
            S[i] = p.x * (S[i] - vt) + vt;
            acc += S[i] * p.y;
          }
        }
        part[(tb * G + g) * vdim + vc] = acc;
      }
    }
    __syncthreads();
    for (int idx = tid; idx < nb * vdim; idx += 256) {
      const int tb = idx / vdim, c = idx - tb * vdim;
      float o = 0.f;
      for (int k = 0; k < G; ++k) o += part[(tb * G + k) * vdim + c];
      part[tb * G * vdim + c] = o;
    }
    __syncthreads();
    for (int tb = tid >> 6; tb < nb; tb += 4) {
      const float* o = part + tb * G * vdim;
      float ss = 0.f;
      for (int c = tid & 63; c < vdim; c += 64) ss += o[c] * o[c];
      ss = wave_sum(ss);
      const float rs = 1.f / sqrtf(ss / (float)vdim + eps);
      T* orow = out + (int64_t)(rb + tb) * out_stride + h * vdim;
      for (int c = tid & 63; c < vdim; c += 64) orow[c] = (T)(o[c] * rs * (float)w[c]);
    }
    // (the next block's first barrier orders these reads of `part` before its phase B writes)
  }
  if (active) {
#pragma unroll
    for (int i = 0; i < MAXR; ++i) {
      const int d = g + i * G;
      if (d < dim) gst[(int64_t)d * vdim + vc] = S[i];
    }
  }
}

}  // namespace

OME_API int ome_hgrn2_scan(const void* q, const void* f, const void* v, int64_t in_stride, const void* f_bias,
                           const void* lower, const void* w, float* state, void* out, int64_t out_stride,
                           const int* cu, const int* slot, const int* reset, int S, int H, int dim, int vdim, float eps,
                           int f32, hipStream_t stream) {
  if (S <= 0 || H <= 0) return 0;
  if (dim <= 0 || vdim <= 0 || vdim > 256) return -2;
  int G = 256 / vdim;
  if (G > dim) G = dim;
  const int nr = (dim + G - 1) / G;
  if (nr > 128) return -3;
  const size_t lds = sizeof(float) * (size_t)TB * (2 * dim + vdim + G * vdim);
  if (lds > 64 * 1024) return -4;
  dim3 grid(H, S);
#define HGRN2_LAUNCH(TT, R)                                                                                          \
  hgrn2_scan_kernel<TT, R><<<grid, 256, lds, stream>>>((const TT*)q, (const TT*)f, (const TT*)v, in_stride,          \
                                                       (const TT*)f_bias, (const TT*)lower, (const TT*)w, state,     \
                                                       (TT*)out, out_stride, cu, slot, reset, H, dim, vdim, G, eps)
#define HGRN2_ROWS(TT)                \
  if (nr <= 4) HGRN2_LAUNCH(TT, 4);   \
  else if (nr <= 16) HGRN2_LAUNCH(TT, 16); \
  else if (nr <= 64) HGRN2_LAUNCH(TT, 64); \
  else HGRN2_LAUNCH(TT, 128)
  if (f32) {
    HGRN2_ROWS(float);
  } else {
    HGRN2_ROWS(bf16);
  }
#undef HGRN2_ROWS
#undef HGRN2_LAUNCH
  OME_CHECK_LAUNCH();
  return 0;
}
