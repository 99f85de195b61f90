// Softmax forward / backward and the fused softmax-cross-entropy backward over
// an [outer, dim, inner] view.  Two layouts:
//   inner == 1 : rows of `dim` contiguous elements, one workgroup per row;
//   inner  > 1 : (softmax over the channel axis of NCHW) one thread per
//                (outer, inner) position, striding over `dim`; consecutive
//                threads touch consecutive addresses.
#include "common.h"

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / MN_WAVE;

__device__ __forceinline__ float block_max(float v, float* lds) {
  v = wave_max(v);
  __syncthreads();
  if (threadIdx.x % MN_WAVE == 0) lds[threadIdx.x / MN_WAVE] = v;
  __syncthreads();
  float r = lds[0];
#pragma unroll
  for (int w = 1; w < kWaves; ++w) r = fmaxf(r, lds[w]);
  return r;
}
__device__ __forceinline__ float block_sum(float v, float* lds) {
  v = wave_sum(v);
  __syncthreads();
  if (threadIdx.x % MN_WAVE == 0) lds[threadIdx.x / MN_WAVE] = v;
  __syncthreads();
  float r = 0.f;
#pragma unroll
  for (int w = 0; w < kWaves; ++w) r += lds[w];
  return r;
}

// fmaxf ignores NaN, but exp(NaN - max) is NaN, so a NaN anywhere in a row
// still turns the whole row into NaN through the sum.
enum Mode { FWD = 0, XENT = 1 };

template <int MODE>
__global__ __launch_bounds__(kThreads) void softmax_row_kernel(const float* x, float* y,
                                                               const int64_t* labels, int64_t dim,
                                                               float scale) {
  __shared__ float lds[kWaves];
  const size_t row = blockIdx.x;
  const float* xr = x + row * dim;
  float* yr = y + row * dim;
  float m = -INFINITY;
  for (int64_t i = threadIdx.x; i < dim; i += kThreads) m = fmaxf(m, xr[i]);
  m = block_max(m, lds);
  if (m == -INFINITY) m = 0.f;  // row of -inf: exp(-inf - 0) = 0, sum 0 -> NaN like exp(-inf+inf)
  float s = 0.f;
  for (int64_t i = threadIdx.x; i < dim; i += kThreads) s += expf(xr[i] - m);
  s = block_sum(s, lds);
  const float inv = 1.f / s;
  const int64_t lab = MODE == XENT ? labels[row] : -1;
  for (int64_t i = threadIdx.x; i < dim; i += kThreads) {
    float p = expf(xr[i] - m) * inv;
    if (MODE == XENT) p = (p - (i == lab ? 1.f : 0.f)) * scale;
    yr[i] = p;
  }
}

__global__ __launch_bounds__(kThreads) void softmax_bwd_row_kernel(const float* dy, const float* y,
                                                                   float* dx, int64_t dim) {
  __shared__ float lds[kWaves];
  const size_t row = blockIdx.x;
  const float* gr = dy + row * dim;
  const float* yr = y + row * dim;
  float* dr = dx + row * dim;
  float s = 0.f;
  for (int64_t i = threadIdx.x; i < dim; i += kThreads) s += gr[i] * yr[i];
  s = block_sum(s, lds);
  for (int64_t i = threadIdx.x; i < dim; i += kThreads) {
    const float p = yr[i];
    dr[i] = gr[i] * p - p * s;
  }
}

template <int MODE>
__global__ __launch_bounds__(kThreads) void softmax_spatial_kernel(const float* x, float* y,
                                                                   const int64_t* labels,
                                                                   int64_t dim, int64_t inner,
                                                                   size_t positions, float scale) {
  const size_t t = (size_t)blockIdx.x * kThreads + threadIdx.x;
  if (t >= positions) return;
  const size_t o = t / inner;
  const size_t i = t - o * inner;
  const float* xp = x + o * dim * inner + i;
  float* yp = y + o * dim * inner + i;
  float m = -INFINITY;
  for (int64_t d = 0; d < dim; ++d) m = fmaxf(m, xp[d * inner]);
  if (m == -INFINITY) m = 0.f;
  float s = 0.f;
  for (int64_t d = 0; d < dim; ++d) s += expf(xp[d * inner] - m);
  const float inv = 1.f / s;
  const int64_t lab = MODE == XENT ? labels[t] : -1;
  for (int64_t d = 0; d < dim; ++d) {
    float p = expf(xp[d * inner] - m) * inv;
    if (MODE == XENT) p = (p - (d == lab ? 1.f : 0.f)) * scale;
    yp[d * inner] = p;
  }
}

__global__ __launch_bounds__(kThreads) void softmax_bwd_spatial_kernel(const float* dy,
                                                                       const float* y, float* dx,
                                                                       int64_t dim, int64_t inner,
                                                                       size_t positions) {
  const size_t t = (size_t)blockIdx.x * kThreads + threadIdx.x;
  if (t >= positions) return;
  const size_t o = t / inner;
  const size_t base = o * dim * inner + (t - o * inner);
  float s = 0.f;
  for (int64_t d = 0; d < dim; ++d) s += dy[base + d * inner] * y[base + d * inner];
  for (int64_t d = 0; d < dim; ++d) {
    const float p = y[base + d * inner];
    dx[base + d * inner] = dy[base + d * inner] * p - p * s;
  }
}

int check(int64_t outer, int64_t dim, int64_t inner) {
  if (outer < 0 || dim < 0 || inner < 0) return MN_EINVAL;
  if (outer >= (1ll << 31) || (inner > 1 && outer * inner >= (1ll << 39))) return MN_EUNSUPPORTED;
  return MN_OK;
}

}  // namespace

extern "C" {

int mn_softmax_fwd_f32(const float* x, float* y, int64_t outer, int64_t dim, int64_t inner,
                       mn_stream_t stream) {
  const int st = check(outer, dim, inner);
  if (st != MN_OK) return st;
  if (outer == 0 || dim == 0 || inner == 0) return MN_OK;
  if (!x || !y) return MN_EINVAL;
  hipStream_t s = mn_stream(stream);
  if (inner == 1) {
    softmax_row_kernel<FWD><<<(unsigned)outer, kThreads, 0, s>>>(x, y, nullptr, dim, 1.f);
  } else {
    const size_t pos = (size_t)outer * inner;
    softmax_spatial_kernel<FWD><<<(unsigned)((pos + kThreads - 1) / kThreads), kThreads, 0, s>>>(
        x, y, nullptr, dim, inner, pos, 1.f);
  }
  return mn_launch_status();
}

int mn_softmax_bwd_f32(const float* dy, const float* y, float* dx, int64_t outer, int64_t dim,
                       int64_t inner, mn_stream_t stream) {
  const int st = check(outer, dim, inner);
  if (st != MN_OK) return st;
  if (outer == 0 || dim == 0 || inner == 0) return MN_OK;
  if (!dy || !y || !dx) return MN_EINVAL;
  hipStream_t s = mn_stream(stream);
  if (inner == 1) {
    softmax_bwd_row_kernel<<<(unsigned)outer, kThreads, 0, s>>>(dy, y, dx, dim);
  } else {
    const size_t pos = (size_t)outer * inner;
    softmax_bwd_spatial_kernel<<<(unsigned)((pos + kThreads - 1) / kThreads), kThreads, 0, s>>>(
        dy, y, dx, dim, inner, pos);
  }
  return mn_launch_status();
}

int mn_xent_bwd_f32(const float* logits, const int64_t* labels, float* dlogits, int64_t outer,
                    int64_t dim, int64_t inner, float scale, mn_stream_t stream) {
  const int st = check(outer, dim, inner);
  if (st != MN_OK) return st;
  if (outer == 0 || dim == 0 || inner == 0) return MN_OK;
  if (!logits || !labels || !dlogits) return MN_EINVAL;
  hipStream_t s = mn_stream(stream);
  if (inner == 1) {
    softmax_row_kernel<XENT><<<(unsigned)outer, kThreads, 0, s>>>(logits, dlogits, labels, dim,
                                                                  scale);
  } else {
    const size_t pos = (size_t)outer * inner;
    softmax_spatial_kernel<XENT><<<(unsigned)((pos + kThreads - 1) / kThreads), kThreads, 0, s>>>(
        logits, dlogits, labels, dim, inner, pos, scale);
  }
  return mn_launch_status();
}

}  // extern "C"
