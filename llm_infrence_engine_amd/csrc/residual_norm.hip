// Kernels of layers that normalise a sublayer's output before it joins the residual stream:
//   x <- x + w_post * y / sqrt(mean(y^2) + eps)        (y: the sublayer's output, x: the float residual stream)
// fused, when asked, with the norm that the next sublayer reads:  h = w_next * x / sqrt(mean(x^2) + eps_next);
// and the small sum that opens a pass over a looped stretch of layers: x <- x (+ kept) (+ vec).
// Everything is float; activations are rounded once on store.
#include "common.h"
#include "api.h"

namespace {

// One block per row.  The row of y (then of x) is kept in LDS when it fits (`staged`), else read again.
template <typename TY, typename TO>
__global__ void __launch_bounds__(256)
rms_norm_add_kernel(const TY* __restrict__ y, size_t y_stride, const float* __restrict__ w_post, float eps_post,
                    float* __restrict__ x, const float* __restrict__ w_next, float eps_next, TO* __restrict__ out,
                    int H, int staged) {
  __shared__ float red[16];
  extern __shared__ float buf[];
  const int r = blockIdx.x;
  const TY* yr = y + (size_t)r * y_stride;
  float* xr = x + (size_t)r * H;
  float ss = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    const float v = to_float(yr[i]);
    if (staged) buf[i] = v;
    ss = fmaf(v, v, ss);
  }
  ss = block_sum(ss, red);
  const float inv = 1.0f / sqrtf(ss / (float)H + eps_post);
  float s2 = 0.f;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    const float v = staged ? buf[i] : to_float(yr[i]);
    const float nx = xr[i] + w_post[i] * (v * inv);
    xr[i] = nx;
    if (staged) buf[i] = nx;
    s2 = fmaf(nx, nx, s2);
  }
  if (out == nullptr) return;
  s2 = block_sum(s2, red);
  const float inv2 = 1.0f / sqrtf(s2 / (float)H + eps_next);
  TO* o = out + (size_t)r * H;
  for (int i = threadIdx.x; i < H; i += blockDim.x) {
    const float v = staged ? buf[i] : xr[i];
    o[i] = from_float<TO>(w_next[i] * (v * inv2));
  }
}

__global__ void add_rows_kernel(float* __restrict__ x, const float* __restrict__ kept, const float* __restrict__ vec,
                                size_t total, int H) {
  const size_t stride = (size_t)gridDim.x * blockDim.x;
  for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += stride) {
    float v = x[i];
    if (kept) v += kept[i];
    if (vec) v += vec[i % H];
    x[i] = v;
  }
}

}  // namespace

extern "C" int ms_rms_norm_add(const void* y, long long y_stride, int y_dtype, const float* w_post, float eps_post, float* x,
                               const float* w_next, float eps_next, void* out, int out_dtype, int n_rows, int hidden,
                               hipStream_t stream) {
  if (n_rows <= 0) return MS_OK;
  if (hidden <= 0 || (out != nullptr && w_next == nullptr)) return MS_BAD_ARG;
  const int staged = hidden <= 12288;
  const size_t lds = staged ? (size_t)hidden * sizeof(float) : 0;
  dim3 grid(n_rows), block(256);
#define LAUNCH(TY, TO)                                                                                             \
  rms_norm_add_kernel<TY, TO><<<grid, block, lds, stream>>>((const TY*)y, (size_t)y_stride, w_post, eps_post, x,  \
                                                            w_next, eps_next, (TO*)out, hidden, staged)
  if (y_dtype == MS_F32 && out_dtype == MS_F32) LAUNCH(float, float);
  else if (y_dtype == MS_F32 && out_dtype == MS_BF16) LAUNCH(float, bf16);
  else if (y_dtype == MS_BF16 && out_dtype == MS_F32) LAUNCH(bf16, float);
  else if (y_dtype == MS_BF16 && out_dtype == MS_BF16) LAUNCH(bf16, bf16);
  else return MS_BAD_ARG;
#undef LAUNCH
  return ms_launch_status();
}

extern "C" int ms_add_rows(float* x, const float* kept, const float* vec, int n_rows, int hidden, hipStream_t stream) {
  if (n_rows <= 0) return MS_OK;
  if (hidden <= 0) return MS_BAD_ARG;
  const size_t total = (size_t)n_rows * hidden;
  int blocks = (int)((total + 1023) / 1024);
  if (blocks > 4096) blocks = 4096;
  add_rows_kernel<<<blocks, 256, 0, stream>>>(x, kept, vec, total, hidden);
  return ms_launch_status();
}
