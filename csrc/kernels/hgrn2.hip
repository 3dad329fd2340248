// HGRN2 mixer core: gated linear recurrence whose forget gate also sets what is written, fused with
// the activations before it; the per-head RMS norm after it is a second, row-parallel kernel.
//
//   q_t = silu(q_raw),  f_t = l + (1 - l) * sigmoid(f_raw + f_bias)          (per head and channel d)
//   S_t = diag(f_t) S_{t-1} + (1 - f_t) v_t^T        S [dim, vdim] per head, fp32, per request slot
//   o_t = S_t^T q_t,   out_t = o_t / sqrt(mean_v(o_t^2) + eps) * w           (w [vdim], shared by heads)
//
// q_raw / f_raw / v are row-strided views of one fused projection (bf16, or float for fp32 models);
// gates, state, the dot products and the norm are fp32, `out` is rounded once.
//
// Scan: one 256-thread workgroup per (head, slice of VC value columns, sequence) walks the
// sequence's rows -- columns of S evolve independently, so slicing vdim multiplies the workgroups
// (heads x sequences alone would leave most of the chip idle) and shortens each thread's share.
// Thread (g, c) keeps rows d = g, g + G, ... of column c in registers (G = 256 / VC groups), so the
// recurrence needs no LDS traffic for S.  Rows are taken TB at a time: (A) all threads turn the
// block's raw gates / queries into fp32 (f, q) pairs in LDS, (B) each thread runs its state slice
// over the TB rows and leaves a partial o per row, (C) the G partials are summed into the fp32
// scratch `o`.  Two barriers per TB rows.  Decode rows are sequences of length one.
#include "common.h"

namespace {

constexpr int TB_MAX = 16;   // rows per pair of barriers (fewer when a wide head's gates would not fit in LDS)

template <typename T, int MAXR>
__global__ __launch_bounds__(256) void hgrn2_scan_kernel(
    const T* __restrict__ q, const T* __restrict__ f, const T* __restrict__ v, int64_t in_stride,
    const T* __restrict__ f_bias, const T* __restrict__ lower, float* __restrict__ state, float* __restrict__ o,
    const int* __restrict__ cu, const int* __restrict__ slot, const int* __restrict__ reset, int H, int dim,
    int vdim, int VC, int VS, int G, int TB) {
  extern __shared__ float sm[];
  float2* fq = (float2*)sm;                      // [TB][dim]
  float* vv = sm + 2 * TB * dim;                 // [TB][VC]
  float* part = vv + TB * VC;                    // [TB][G][VC]
  const int h = blockIdx.x / VS, c0 = (blockIdx.x % VS) * VC, s = blockIdx.y, tid = threadIdx.x;
  const int nc = min(VC, vdim - c0);
  const int r0 = cu[s], r1 = cu[s + 1];
  if (r1 <= r0) return;
  const int g = tid / VC, vc = tid - g * VC;
  const bool active = g < G && vc < nc;
  float* gst = state + ((int64_t)slot[s] * H + h) * dim * vdim + c0;
  float S[MAXR];
  const bool fresh = reset[s] != 0;
#pragma unroll
  for (int i = 0; i < MAXR; ++i) {
    const int d = g + i * G;
    S[i] = (active && d < dim && !fresh) ? gst[(int64_t)d * vdim + vc] : 0.f;
  }
  const int HV = H * vdim;
  for (int rb = r0; rb < r1; rb += TB) {
    const int nb = min(TB, r1 - rb);
    for (int idx = tid; idx < nb * dim; idx += 256) {
      const int tb = idx / dim, d = idx - tb * dim;
      const int64_t off = (int64_t)(rb + tb) * in_stride + h * dim + d;
      const float lo = (float)lower[h * dim + d];
      const float fr = (float)f[off] + (float)f_bias[h * dim + d];
      const float qr = (float)q[off];
      fq[idx] = make_float2(lo + (1.f - lo) / (1.f + expf(-fr)), qr / (1.f + expf(-qr)));
    }
    for (int idx = tid; idx < nb * nc; idx += 256) {
      const int tb = idx / nc, c = idx - tb * nc;
      vv[tb * VC + c] = (float)v[(int64_t)(rb + tb) * in_stride + h * vdim + c0 + c];
    }
    __syncthreads();
    if (active) {
      for (int tb = 0; tb < nb; ++tb) {
        const float vt = vv[tb * VC + vc];
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
        part[(tb * G + g) * VC + vc] = acc;
      }
    }
    __syncthreads();
    for (int idx = tid; idx < nb * nc; idx += 256) {
      const int tb = idx / nc, c = idx - tb * nc;
      float a = 0.f;
      for (int k = 0; k < G; ++k) a += part[(tb * G + k) * VC + c];
      o[(int64_t)(rb + tb) * HV + h * vdim + c0 + c] = a;
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

// out[r, :] = o[r, :] / sqrt(mean(o[r, :]^2) + eps) * w over rows of n fp32 values (one row = one
// head of one token); one wave per row.
template <typename T>
__global__ __launch_bounds__(256) void head_rms_norm_kernel(const float* __restrict__ o, const T* __restrict__ w,
                                                            T* __restrict__ out, int64_t rows, int n, float eps) {
  const int64_t r = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
  if (r >= rows) return;
  const int lane = threadIdx.x & 63;
  const float* x = o + r * n;
  float ss = 0.f;
  for (int c = lane; c < n; c += 64) ss += x[c] * x[c];
  ss = wave_sum(ss);
  const float rs = 1.f / sqrtf(ss / (float)n + eps);
  for (int c = lane; c < n; c += 64) out[r * n + c] = (T)(x[c] * rs * (float)w[c]);
}

}  // namespace

// o: fp32 scratch [rows, H * vdim] (rows = cu[S]); out: [rows, H * vdim] contiguous.
OME_API int ome_hgrn2_scan(const void* q, const void* f, const void* v, int64_t in_stride, const void* f_bias,
                           const void* lower, const void* w, float* state, float* o, void* out, int rows,
                           const int* cu, const int* slot, const int* reset, int S, int H, int dim, int vdim, float eps,
                           int f32, hipStream_t stream) {
  if (S <= 0 || H <= 0 || rows <= 0) return 0;
  if (dim <= 0 || vdim <= 0) return -2;
  int VC = vdim >= 64 ? 32 : vdim;
  // few long sequences: narrower slices, so that at least ~2 workgroups per CU walk them
  while (VC > 8 && VC % 2 == 0 && (int64_t)H * ((vdim + VC - 1) / VC) * S < 512) VC /= 2;
  const int VS = (vdim + VC - 1) / VC;
  int G = 256 / VC;
  if (G > dim) G = dim;
  const int nr = (dim + G - 1) / G;
  if (nr > 128) return -3;
  int TB = rows <= S ? 1 : TB_MAX;   // (decode: every sequence is one row)
  while (TB > 1 && sizeof(float) * (size_t)TB * (2 * dim + VC + G * VC) > 48 * 1024) TB /= 2;
  const size_t lds = sizeof(float) * (size_t)TB * (2 * dim + VC + G * VC);
  if (lds > 64 * 1024 || S > 65535) return -4;
  dim3 grid(H * VS, S);
#define HGRN2_LAUNCH(TT, R)                                                                                       \
  hgrn2_scan_kernel<TT, R><<<grid, 256, lds, stream>>>((const TT*)q, (const TT*)f, (const TT*)v, in_stride,       \
                                                       (const TT*)f_bias, (const TT*)lower, state, o, cu, slot,  \
                                                       reset, H, dim, vdim, VC, VS, G, TB)
#define HGRN2_ROWS(TT)                     \
  if (nr <= 4) HGRN2_LAUNCH(TT, 4);        \
  else if (nr <= 8) HGRN2_LAUNCH(TT, 8);   \
  else if (nr <= 16) HGRN2_LAUNCH(TT, 16); \
  else if (nr <= 32) HGRN2_LAUNCH(TT, 32); \
  else if (nr <= 64) HGRN2_LAUNCH(TT, 64); \
  else HGRN2_LAUNCH(TT, 128)
  const int64_t nrows = (int64_t)rows * H;
  const int nblk = (int)((nrows + 3) / 4);
  if (f32) {
    HGRN2_ROWS(float);
    head_rms_norm_kernel<float><<<nblk, 256, 0, stream>>>(o, (const float*)w, (float*)out, nrows, vdim, eps);
  } else {
    HGRN2_ROWS(bf16);
    head_rms_norm_kernel<bf16><<<nblk, 256, 0, stream>>>(o, (const bf16*)w, (bf16*)out, nrows, vdim, eps);
  }
#undef HGRN2_ROWS
#undef HGRN2_LAUNCH
  OME_CHECK_LAUNCH();
  return 0;
}
