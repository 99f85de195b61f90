// BatchNorm kernels over an [N, C, HW] view (NCHW): training forward, forward
// from saved statistics, backward from the input and backward from the output.
//
// Work decomposition (all kernels): channel c owns N*HW elements, visited as
// the flat sequence j = n*HWV + i (HWV = HW / VEC vectors per image slab).
// That sequence is cut into S equal pieces, one workgroup each, so the grid is
// C*S workgroups whatever the shape; workgroup b handles channel b / S, piece
// b % S.  Reductions are two-level and atomic-free: every workgroup writes one
// partial pair to the workspace, and the consumer kernel re-adds the S partials
// of its channel in a fixed order, so results are reproducible.
#include "common.h"

namespace mn_bn {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / MN_WAVE;
constexpr int kMaxSplit = 64;
constexpr int kU = 4;  // vectors in flight per thread per tensor

template <int VEC>
struct Vec;
template <>
struct Vec<4> {
  typedef float4_t type;
};
template <>
struct Vec<1> {
  typedef float type;
};

struct Shape {
  int C;
  int S;         // pieces per channel
  uint32_t HWV;  // vectors per (n, c) slab
  uint32_t HW;   // elements per slab
  uint64_t L;    // vectors per piece
  uint64_t tot;  // vectors per channel = N * HWV
};

// Walks the vectors of one piece with a stride of kThreads, keeping (n, i)
// without a division per step.
struct Cursor {
  uint64_t j, jend;
  uint32_t n, i, qstep, rstep, HWV;
  __device__ __forceinline__ Cursor(const Shape& sh, int piece) {
    HWV = sh.HWV;
    const uint64_t j0 = (uint64_t)piece * sh.L;
    jend = min(j0 + sh.L, sh.tot);
    j = j0 + threadIdx.x;
    n = (uint32_t)(j / HWV);
    i = (uint32_t)(j - (uint64_t)n * HWV);
    qstep = kThreads / HWV;
    rstep = kThreads - qstep * HWV;
  }
  __device__ __forceinline__ bool valid() const { return j < jend; }
  __device__ __forceinline__ void next() {
    j += kThreads;
    n += qstep;
    i += rstep;
    if (i >= HWV) {
      i -= HWV;
      ++n;
    }
  }
  // element offset of the current vector for channel c
  template <int VEC>
  __device__ __forceinline__ size_t off(int C, int c, uint32_t HW) const {
    return ((size_t)n * C + c) * HW + (size_t)i * VEC;
  }
};

template <int VEC>
__device__ __forceinline__ typename Vec<VEC>::type ldv(const float* p) {
  return ld_stream(reinterpret_cast<const typename Vec<VEC>::type*>(p));
}
template <int VEC>
__device__ __forceinline__ void stv(float* p, typename Vec<VEC>::type v) {
  st_stream(reinterpret_cast<typename Vec<VEC>::type*>(p), v);
}
__device__ __forceinline__ float comp(const float4_t& v, int k) { return v[k]; }
__device__ __forceinline__ float comp(const float& v, int) { return v; }
__device__ __forceinline__ void setc(float4_t& v, int k, float a) { v[k] = a; }
__device__ __forceinline__ void setc(float& v, int, float a) { v = a; }

// ---------------------------------------------------------------- reduce --
// partial[c][piece] = ( sum a , sum a*(b - shift[c]) )       (backward)
//                  or ( sum (b - K) , sum (b - K)^2 )         (STATS: forward)
// with K = first element of the channel (also stored in pivot[c]).
template <int VEC, bool STATS>
__global__ __launch_bounds__(kThreads) void bn_reduce_kernel(const Shape sh, const float* a,
                                                             const float* b, const float* shift,
                                                             float* partial, float* pivot) {
  __shared__ float lds[2 * kWaves];
  typedef typename Vec<VEC>::type V;
  const int c = blockIdx.x / sh.S;
  const int piece = blockIdx.x - c * sh.S;
  float sft;
  if (STATS) {
    sft = b[(size_t)c * sh.HW];
    if (piece == 0 && threadIdx.x == 0) pivot[c] = sft;
  } else {
    sft = shift ? shift[c] : 0.f;
  }
  float s0 = 0.f, s1 = 0.f;
  Cursor cur(sh, piece);
  while (cur.valid()) {
    V va[kU], vb[kU];
    bool ok[kU];
#pragma unroll
    for (int u = 0; u < kU; ++u) {
      ok[u] = cur.valid();
      if (ok[u]) {
        const size_t o = cur.off<VEC>(sh.C, c, sh.HW);
        vb[u] = ldv<VEC>(b + o);
        if (!STATS) va[u] = ldv<VEC>(a + o);
      }
      cur.next();
    }
#pragma unroll
    for (int u = 0; u < kU; ++u) {
      if (ok[u]) {
#pragma unroll
        for (int k = 0; k < VEC; ++k) {
          const float d = comp(vb[u], k) - sft;
          if (STATS) {
            s0 += d;
            s1 += d * d;
          } else {
            const float g = comp(va[u], k);
            s0 += g;
            s1 += g * d;
          }
        }
      }
    }
  }
  block_sum2<kWaves>(s0, s1, lds);
  if (threadIdx.x == 0) {
    partial[2 * (size_t)blockIdx.x] = s0;
    partial[2 * (size_t)blockIdx.x + 1] = s1;
  }
}

// Re-add the S partial pairs of channel c; every thread gets the totals.
__device__ __forceinline__ void channel_totals(const float* partial, int c, int S, float& t0,
                                               float& t1) {
  // S <= 64: lane l of each wave fetches partial l, then a fixed-order lane tree
  const int lane = threadIdx.x % MN_WAVE;
  float p0 = 0.f, p1 = 0.f;
  if (lane < S) {
    p0 = partial[2 * ((size_t)c * S + lane)];
    p1 = partial[2 * ((size_t)c * S + lane) + 1];
  }
  t0 = wave_sum(p0);
  t1 = wave_sum(p1);
}

// ------------------------------------------------------------ bwd: apply --
// dx = (dy - (t - shift)*proj - gmean) * gscale, coefficients per channel.
// FROM_Y: t = y, shift = beta, proj = dot/(M*gamma^2); dgamma = dot/gamma
// else  : t = x, shift = mean, proj = dot*invstd^2/M;  dgamma = dot*invstd
template <int VEC, bool FROM_Y>
__global__ __launch_bounds__(kThreads) void bn_bwd_apply_kernel(
    const Shape sh, const float* dy, const float* t, const float* gamma, const float* shift,
    const float* invstd, const float* partial, float* dx, float* dgamma, float* dbeta,
    float inv_m) {
  typedef typename Vec<VEC>::type V;
  const int c = blockIdx.x / sh.S;
  const int piece = blockIdx.x - c * sh.S;
  float gsum, dot;
  channel_totals(partial, c, sh.S, gsum, dot);
  const float w = gamma ? gamma[c] : 1.f;
  const float sft = shift ? shift[c] : 0.f;
  const float istd = invstd[c];
  float proj, dg;
  if (FROM_Y) {
    const float inv_w = 1.f / w;
    proj = dot * inv_m * inv_w * inv_w;
    dg = dot * inv_w;
  } else {
    proj = dot * inv_m * istd * istd;
    dg = dot * istd;
  }
  const float gmean = gsum * inv_m;
  const float gscale = istd * w;
  if (piece == 0 && threadIdx.x == 0) {
    if (dgamma) dgamma[c] = dg;
    if (dbeta) dbeta[c] = gsum;
  }
  if (!dx) return;
  Cursor cur(sh, piece);
  while (cur.valid()) {
    V vg[kU], vt[kU];
    size_t o[kU];
    bool ok[kU];
#pragma unroll
    for (int u = 0; u < kU; ++u) {
      ok[u] = cur.valid();
      if (ok[u]) {
        o[u] = cur.off<VEC>(sh.C, c, sh.HW);
        vg[u] = ldv<VEC>(dy + o[u]);
        vt[u] = ldv<VEC>(t + o[u]);
      }
      cur.next();
    }
#pragma unroll
    for (int u = 0; u < kU; ++u) {
      if (ok[u]) {
        V r;
#pragma unroll
        for (int k = 0; k < VEC; ++k)
          setc(r, k, (comp(vg[u], k) - (comp(vt[u], k) - sft) * proj - gmean) * gscale);
        stv<VEC>(dx + o[u], r);
      }
    }
  }
}

// ------------------------------------------------------------ fwd: apply --
// y = (x - mean) * (invstd*gamma) + beta.  FINALIZE: mean / invstd come from
// the partial sums of bn_reduce_kernel<STATS> and piece 0 also writes
// save_mean, save_invstd and the running statistics.
template <int VEC, bool FINALIZE>
__global__ __launch_bounds__(kThreads) void bn_fwd_apply_kernel(
    const Shape sh, const float* x, const float* mean_in, const float* invstd_in,
    const float* gamma, const float* beta, const float* partial, const float* pivot, float* y,
    float* save_mean, float* save_invstd, float* running_mean, float* running_var, float inv_m,
    float unbias, float momentum, float eps) {
  typedef typename Vec<VEC>::type V;
  const int c = blockIdx.x / sh.S;
  const int piece = blockIdx.x - c * sh.S;
  float mean, istd;
  if (FINALIZE) {
    float s1, s2;
    channel_totals(partial, c, sh.S, s1, s2);
    const float dm = s1 * inv_m;
    mean = pivot[c] + dm;
    const float var = fmaxf(s2 * inv_m - dm * dm, 0.f);
    istd = 1.f / sqrtf(var + eps);
    if (piece == 0 && threadIdx.x == 0) {
      save_mean[c] = mean;
      save_invstd[c] = istd;
      if (running_mean) running_mean[c] = (1.f - momentum) * running_mean[c] + momentum * mean;
      if (running_var)
        running_var[c] = (1.f - momentum) * running_var[c] + momentum * (var * unbias);
    }
  } else {
    mean = mean_in[c];
    istd = invstd_in[c];
  }
  const float scale = istd * (gamma ? gamma[c] : 1.f);
  const float bias = beta ? beta[c] : 0.f;
  Cursor cur(sh, piece);
  while (cur.valid()) {
    V vx[kU];
    size_t o[kU];
    bool ok[kU];
#pragma unroll
    for (int u = 0; u < kU; ++u) {
      ok[u] = cur.valid();
      if (ok[u]) {
        o[u] = cur.off<VEC>(sh.C, c, sh.HW);
        vx[u] = ldv<VEC>(x + o[u]);
      }
      cur.next();
    }
#pragma unroll
    for (int u = 0; u < kU; ++u) {
      if (ok[u]) {
        V r;
#pragma unroll
        for (int k = 0; k < VEC; ++k) setc(r, k, (comp(vx[u], k) - mean) * scale + bias);
        stv<VEC>(y + o[u], r);
      }
    }
  }
}

// ------------------------------------------------------------------ host --
struct Plan {
  Shape sh;
  int vec;
  unsigned blocks;
};

// `target_blocks`: aim of the split, ~16 workgroups per CU on 256 CUs.
static bool make_plan(int64_t N, int64_t C, int64_t HW, bool aligned16, int target_blocks,
                      Plan& p) {
  if (N <= 0 || C <= 0 || HW <= 0) return false;
  if (C > (1 << 24) || HW >= (1ll << 31) || N >= (1ll << 31)) return false;
  p.vec = (HW % 4 == 0 && aligned16) ? 4 : 1;
  const uint64_t hwv = (uint64_t)HW / p.vec;
  const uint64_t tot = (uint64_t)N * hwv;
  int64_t S = (target_blocks + C - 1) / C;
  const int64_t cap = (int64_t)((tot + kThreads * kU - 1) / (kThreads * kU));  // >= 1 batch each
  if (S > cap) S = cap;
  if (S > kMaxSplit) S = kMaxSplit;
  if (S < 1) S = 1;
  p.sh.C = (int)C;
  p.sh.S = (int)S;
  p.sh.HWV = (uint32_t)hwv;
  p.sh.HW = (uint32_t)HW;
  p.sh.tot = tot;
  p.sh.L = (tot + S - 1) / S;
  p.blocks = (unsigned)(C * S);
  return true;
}

constexpr int kTargetBlocks = 4096;

static size_t ws_bytes_for(int64_t C) { return (size_t)C * (2 * kMaxSplit + 1) * sizeof(float); }

int bwd_launch(bool from_y, const float* dy, const float* t, const float* gamma, const float* shift,
               const float* invstd, float* dx, float* dgamma, float* dbeta, int64_t N, int64_t C,
               int64_t HW, void* ws, size_t ws_bytes, hipStream_t s, int target_blocks) {
  if (N == 0 || C == 0 || HW == 0) return MN_OK;
  if (!dy || !t || !invstd || !ws) return MN_EINVAL;
  if (ws_bytes < ws_bytes_for(C) || !mn_aligned(ws, 4)) return MN_EINVAL;
  Plan p;
  const bool al = mn_aligned(dy, 16) && mn_aligned(t, 16) && (!dx || mn_aligned(dx, 16));
  if (!make_plan(N, C, HW, al, target_blocks, p)) return MN_EUNSUPPORTED;
  float* partial = static_cast<float*>(ws);
  const float inv_m = 1.f / (float)((double)N * (double)HW);
  if (p.vec == 4)
    bn_reduce_kernel<4, false><<<p.blocks, kThreads, 0, s>>>(p.sh, dy, t, shift, partial, nullptr);
  else
    bn_reduce_kernel<1, false><<<p.blocks, kThreads, 0, s>>>(p.sh, dy, t, shift, partial, nullptr);
#define MN_BN_APPLY(V, FY)                                                                      \
  bn_bwd_apply_kernel<V, FY><<<p.blocks, kThreads, 0, s>>>(p.sh, dy, t, gamma, shift, invstd,   \
                                                           partial, dx, dgamma, dbeta, inv_m)
  if (p.vec == 4) {
    if (from_y) MN_BN_APPLY(4, true); else MN_BN_APPLY(4, false);
  } else {
    if (from_y) MN_BN_APPLY(1, true); else MN_BN_APPLY(1, false);
  }
#undef MN_BN_APPLY
  return mn_launch_status();
}

}  // namespace mn_bn

extern "C" {

size_t mn_bn_ws_bytes(int64_t N, int64_t C, int64_t HW) {
  (void)N;
  (void)HW;
  return C > 0 ? mn_bn::ws_bytes_for(C) : 0;
}

int mn_bn_fwd_train_f32(const float* x, const float* gamma, const float* beta, float* running_mean,
                        float* running_var, float* y, float* save_mean, float* save_invstd,
                        int64_t N, int64_t C, int64_t HW, double momentum, double eps, void* ws,
                        size_t ws_bytes, mn_stream_t stream) {
  using namespace mn_bn;
  if (N < 0 || C < 0 || HW < 0) return MN_EINVAL;
  if (N == 0 || C == 0 || HW == 0) return MN_OK;
  if (!x || !y || !save_mean || !save_invstd || !ws) return MN_EINVAL;
  if (ws_bytes < ws_bytes_for(C) || !mn_aligned(ws, 4)) return MN_EINVAL;
  Plan p;
  if (!make_plan(N, C, HW, mn_aligned(x, 16) && mn_aligned(y, 16), kTargetBlocks, p))
    return MN_EUNSUPPORTED;
  hipStream_t s = mn_stream(stream);
  float* partial = static_cast<float*>(ws);
  float* pivot = partial + 2 * (size_t)C * kMaxSplit;
  const double M = (double)N * (double)HW;
  const float inv_m = (float)(1.0 / M);
  const float unbias = M > 1.0 ? (float)(M / (M - 1.0)) : 1.f;
  if (p.vec == 4) {
    bn_reduce_kernel<4, true><<<p.blocks, kThreads, 0, s>>>(p.sh, nullptr, x, nullptr, partial,
                                                            pivot);
    bn_fwd_apply_kernel<4, true><<<p.blocks, kThreads, 0, s>>>(
        p.sh, x, nullptr, nullptr, gamma, beta, partial, pivot, y, save_mean, save_invstd,
        running_mean, running_var, inv_m, unbias, (float)momentum, (float)eps);
  } else {
    bn_reduce_kernel<1, true><<<p.blocks, kThreads, 0, s>>>(p.sh, nullptr, x, nullptr, partial,
                                                            pivot);
    bn_fwd_apply_kernel<1, true><<<p.blocks, kThreads, 0, s>>>(
        p.sh, x, nullptr, nullptr, gamma, beta, partial, pivot, y, save_mean, save_invstd,
        running_mean, running_var, inv_m, unbias, (float)momentum, (float)eps);
  }
  return mn_launch_status();
}

int mn_bn_fwd_apply_f32(const float* x, const float* mean, const float* invstd, const float* gamma,
                        const float* beta, float* y, int64_t N, int64_t C, int64_t HW,
                        mn_stream_t stream) {
  using namespace mn_bn;
  if (N < 0 || C < 0 || HW < 0) return MN_EINVAL;
  if (N == 0 || C == 0 || HW == 0) return MN_OK;
  if (!x || !y || !mean || !invstd) return MN_EINVAL;
  Plan p;
  if (!make_plan(N, C, HW, mn_aligned(x, 16) && mn_aligned(y, 16), kTargetBlocks, p))
    return MN_EUNSUPPORTED;
  hipStream_t s = mn_stream(stream);
  if (p.vec == 4)
    bn_fwd_apply_kernel<4, false><<<p.blocks, kThreads, 0, s>>>(
        p.sh, x, mean, invstd, gamma, beta, nullptr, nullptr, y, nullptr, nullptr, nullptr, nullptr,
        0.f, 0.f, 0.f, 0.f);
  else
    bn_fwd_apply_kernel<1, false><<<p.blocks, kThreads, 0, s>>>(
        p.sh, x, mean, invstd, gamma, beta, nullptr, nullptr, y, nullptr, nullptr, nullptr, nullptr,
        0.f, 0.f, 0.f, 0.f);
  return mn_launch_status();
}

int mn_bn_bwd_from_x_f32(const float* dy, const float* x, const float* gamma, const float* mean,
                         const float* invstd, float* dx, float* dgamma, float* dbeta, int64_t N,
                         int64_t C, int64_t HW, void* ws, size_t ws_bytes, mn_stream_t stream) {
  if (N < 0 || C < 0 || HW < 0 || !mean) return MN_EINVAL;
  return mn_bn::bwd_launch(false, dy, x, gamma, mean, invstd, dx, dgamma, dbeta, N, C, HW, ws,
                           ws_bytes, mn_stream(stream), mn_bn::kTargetBlocks);
}

int mn_bn_bwd_from_y_f32(const float* dy, const float* y, const float* gamma, const float* beta,
                         const float* invstd, float* dx, float* dgamma, float* dbeta, int64_t N,
                         int64_t C, int64_t HW, void* ws, size_t ws_bytes, mn_stream_t stream) {
  if (N < 0 || C < 0 || HW < 0) return MN_EINVAL;
  return mn_bn::bwd_launch(true, dy, y, gamma, beta, invstd, dx, dgamma, dbeta, N, C, HW, ws,
                           ws_bytes, mn_stream(stream), mn_bn::kTargetBlocks);
}

}  // extern "C"
