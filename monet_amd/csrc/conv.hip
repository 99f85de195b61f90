// 2-D convolution as implicit GEMM on the fp32 matrix cores
// (v_mfma_f32_32x32x2_f32), NCHW tensors, no layout change in HBM.
//
// Forward and backward-data are the same "gather GEMM":
//     D[m][col] = sum over (ch, tap)  A(m, ch, tap) * src[n, ch, oh*ish + dh[tap], ow*isw + dw[tap]]
// with col = (n, oh, ow).  Forward: A = weights, src = x, taps = the R*S window.
// Backward-data: A = weights read through strides (or a transposed copy in the
// workspace), src = dy; for stride > 1 the input positions are split by parity
// class so that every class is a dense stride-1 gather over the taps that can
// reach it (no multiplies by structural zeros).
//
// Backward-weight is a GEMM whose reduction runs over (n, p, q); the reduction
// is split across workgroups (split-K) and combined either with atomics into a
// cleared dw (no workspace) or through per-split partials in the workspace
// followed by a fixed-order reduction (deterministic).
//
// Tiling: a workgroup of 4 wavefronts computes a BM x BN = 128 x 128 tile of D;
// each wavefront owns 64 x 64 as 2 x 2 MFMA tiles (64 accumulator VGPRs).
// Operand tiles (BK = 16 deep) are staged through LDS k-major, double buffered:
// the global loads of tile t+1 are in flight while tile t is multiplied.
#include "common.h"

namespace mn_conv {

typedef float float16_t __attribute__((ext_vector_type(16)));

constexpr int kThreads = 256;
constexpr int BM = 128, BN = 128, BK = 16;
constexpr int kPad = 1;  // LDS row padding (floats)
constexpr int kMaxTaps = 49;

// n / d for n < 2^20, d < 4096 (mul = floor(2^32 / d) + 1).
struct FastDiv {
  uint32_t mul, d;
  __device__ __forceinline__ uint32_t div(uint32_t n) const {
    return d == 1 ? n : __umulhi(n, mul);
  }
};
static FastDiv make_fastdiv(uint32_t d) {
  FastDiv f;
  f.d = d ? d : 1;
  f.mul = (uint32_t)((1ull << 32) / f.d + 1);
  return f;
}

// One launch of the gather GEMM (forward, or one parity class of backward-data).
struct Gather {
  int M, Kd, T;
  FastDiv divT;
  int N, OH, OW;        // column space; ncols = N*OH*OW
  uint32_t ncols;
  int Cs, Hs, Ws;       // source tensor [N, Cs, Hs, Ws]
  int ish, isw;         // source coordinate = oh*ish + dh[tap]
  int DH, DW;           // destination tensor [N, M, DH, DW]
  int osh, osw, oh0, ow0;  // destination coordinate = oh*osh + oh0
  long long lda;        // A(m, ch, tap) = a[m*lda + ch*cha + aoff[tap]]
  long long cha;
  int16_t dh[kMaxTaps], dw[kMaxTaps];
  int32_t aoff[kMaxTaps];
};

struct Lds {
  float a[2][BK][BM + kPad];
  float b[2][BK][BN + kPad];
  int tdh[kMaxTaps], tdw[kMaxTaps], taoff[kMaxTaps];
};

// Wavefront-level multiply of one staged k-tile: wave (wm, wn) owns rows
// wm*64.. and columns wn*64.. of the workgroup tile.
__device__ __forceinline__ void mma_tile(const float (*As)[BM + kPad], const float (*Bs)[BN + kPad],
                                         int wm, int wn, int lane, float16_t (&acc)[2][2]) {
  const int r = lane & 31, half = lane >> 5;
#pragma unroll
  for (int ks = 0; ks < BK; ks += 2) {
    const int k = ks + half;
    const float a0 = As[k][wm * 64 + r];
    const float a1 = As[k][wm * 64 + 32 + r];
    const float b0 = Bs[k][wn * 64 + r];
    const float b1 = Bs[k][wn * 64 + 32 + r];
    acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b0, acc[0][0], 0, 0, 0);
    acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b1, acc[0][1], 0, 0, 0);
    acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b0, acc[1][0], 0, 0, 0);
    acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b1, acc[1][1], 0, 0, 0);
  }
}

// Row of accumulator register v within a 32x32 MFMA tile, for this lane.
__device__ __forceinline__ int acc_row(int v, int lane) {
  return 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
}

// FAST: the source has a multiple of BK channels and every tensor is < 4 GB.
// Then the reduction index runs tap-major (kk = tap*Cs + ch): a k-tile lies
// inside one tap, so the window test and the spatial offset are computed once
// per tile and thread, every address is a 32-bit byte offset = per-thread
// constant + per-tile scalar, and almost no vector ALU work competes with the
// matrix cores.  Otherwise (e.g. 3 input channels) kk = ch*T + tap and every
// element is decomposed on its own.
template <bool FAST>
__global__ __launch_bounds__(kThreads) void gather_gemm_kernel(const Gather g,
                                                               const float* __restrict__ a,
                                                               const float* __restrict__ src,
                                                               const float* __restrict__ bias,
                                                               float* __restrict__ dst) {
  __shared__ Lds lds;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int m0 = blockIdx.y * BM;
  const uint32_t n0 = blockIdx.x * BN;
  if (tid < g.T) {
    lds.tdh[tid] = g.dh[tid];
    lds.tdw[tid] = g.dw[tid];
    lds.taoff[tid] = g.aoff[tid];
  }
  __syncthreads();

  // B loader: this thread always fetches column bcol, rows brow0 + 2*i
  constexpr int kBRows = BN * BK / kThreads, kARows = BM * BK / kThreads;
  const int bcol = tid & (BN - 1), brow0 = tid / BN;
  const uint32_t col = n0 + bcol;
  const bool col_ok = col < g.ncols;
  int ohs = 0, ows = 0;
  uint32_t img = 0;
  {
    const uint32_t c = col_ok ? col : 0;
    img = c / ((uint32_t)g.OH * g.OW);
    const uint32_t rem = c - img * (uint32_t)g.OH * g.OW;
    const uint32_t oh = rem / g.OW, ow = rem - oh * g.OW;
    ohs = oh * g.ish;
    ows = ow * g.isw;
  }
  const size_t srcbase = (size_t)img * g.Cs * g.Hs * g.Ws;
  // A loader: this thread always fetches k-column ak, rows arow0 + 16*i
  const int ak = tid & (BK - 1), arow0 = tid / BK;

  // FAST: per-thread constant byte offsets
  const uint32_t plane_b = (uint32_t)g.Hs * g.Ws * 4u;
  const uint32_t pix_b = ((img * (uint32_t)g.Cs * g.Hs + ohs) * (uint32_t)g.Ws + ows) * 4u +
                         brow0 * plane_b;
  uint32_t am_b[kARows];
  uint32_t am_ok = 0;
  if (FAST) {
#pragma unroll
    for (int i = 0; i < kARows; ++i) {
      const int m = m0 + arow0 + (kThreads / BK) * i;
      const bool ok = m < g.M;
      am_b[i] = ok ? (uint32_t)(((long long)m * g.lda + (long long)ak * g.cha) * 4) : 0u;
      am_ok |= (ok ? 1u : 0u) << i;
    }
  }

  float ra[kARows], rb[kBRows];
  bool b_ok = true;  // FAST: whether rb holds window elements or must be staged as zeros
  // FAST fetch of the k-tile at (tap t, first channel c0); t and c0 are uniform.
  // Only issues the loads: masking happens in stage(), after the multiply of the
  // current tile, so the loads stay in flight behind the matrix instructions.
  auto fetch_fast = [&](int t, int c0) {
    const int dh = lds.tdh[t], dw = lds.tdw[t];
    const int hh = ohs + dh, ww = ows + dw;
    b_ok = col_ok && (unsigned)hh < (unsigned)g.Hs && (unsigned)ww < (unsigned)g.Ws;
    const uint32_t sb = (uint32_t)((((long long)c0 * g.Hs + dh) * g.Ws + dw) * 4);
    const uint32_t base = b_ok ? pix_b + sb : brow0 * plane_b;
    const char* sp = reinterpret_cast<const char*>(src);
#pragma unroll
    for (int i = 0; i < kBRows; ++i)
      rb[i] = *reinterpret_cast<const float*>(sp + (base + (kThreads / BN) * i * plane_b));
    const uint32_t sa = (uint32_t)(((long long)c0 * g.cha + lds.taoff[t]) * 4);
    const char* ap = reinterpret_cast<const char*>(a);
#pragma unroll
    for (int i = 0; i < kARows; ++i) {
      const bool mok = (am_ok >> i) & 1u;
      ra[i] = *reinterpret_cast<const float*>(ap + (am_b[i] + (mok ? sa : 0u)));
    }
  };
  auto fetch = [&](int k0) {
#pragma unroll
    for (int i = 0; i < kBRows; ++i) {
      const uint32_t kk = k0 + brow0 + (kThreads / BN) * i;
      float v = 0.f;
      if (col_ok && kk < (uint32_t)g.Kd) {
        const uint32_t ch = g.divT.div(kk);
        const uint32_t t = kk - ch * g.T;
        const int hh = ohs + lds.tdh[t], ww = ows + lds.tdw[t];
        if ((unsigned)hh < (unsigned)g.Hs && (unsigned)ww < (unsigned)g.Ws)
          v = src[srcbase + ((size_t)ch * g.Hs + hh) * g.Ws + ww];
      }
      rb[i] = v;
    }
    const uint32_t kk = k0 + ak;
    uint32_t ch = 0, t = 0;
    const bool k_ok = kk < (uint32_t)g.Kd;
    if (k_ok) {
      ch = g.divT.div(kk);
      t = kk - ch * g.T;
    }
    const long long koff = k_ok ? (long long)ch * g.cha + lds.taoff[t] : 0;
#pragma unroll
    for (int i = 0; i < kARows; ++i) {
      const int m = m0 + arow0 + (kThreads / BK) * i;
      ra[i] = (k_ok && m < g.M) ? a[(long long)m * g.lda + koff] : 0.f;
    }
  };
  auto stage = [&](int buf) {
#pragma unroll
    for (int i = 0; i < kBRows; ++i)
      lds.b[buf][brow0 + (kThreads / BN) * i][bcol] = (!FAST || b_ok) ? rb[i] : 0.f;
#pragma unroll
    for (int i = 0; i < kARows; ++i)
      lds.a[buf][ak][arow0 + (kThreads / BK) * i] =
          (!FAST || ((am_ok >> i) & 1u)) ? ra[i] : 0.f;
  };

  float16_t acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  const int ktiles = (g.Kd + BK - 1) / BK;
  if (ktiles > 0) {
    int t = 0, c0 = 0;  // FAST: position of the tile being fetched
    auto fetch_next = [&](int kt) {
      if (FAST) {
        fetch_fast(t, c0);
        c0 += BK;
        if (c0 == g.Cs) {
          c0 = 0;
          ++t;
        }
      } else {
        fetch(kt * BK);
      }
    };
    fetch_next(0);
    stage(0);
    __syncthreads();
    for (int kt = 0; kt < ktiles; ++kt) {
      const int buf = kt & 1;
      if (kt + 1 < ktiles) fetch_next(kt + 1);
      mma_tile(lds.a[buf], lds.b[buf], wm, wn, lane, acc);
      if (kt + 1 < ktiles) stage(buf ^ 1);
      __syncthreads();
    }
  }

  // epilogue: lane owns columns (ni*32 + lane%32) and 16 rows per MFMA tile
#pragma unroll
  for (int ni = 0; ni < 2; ++ni) {
    const uint32_t c = n0 + wn * 64 + ni * 32 + (lane & 31);
    if (c >= g.ncols) continue;
    const uint32_t n = c / ((uint32_t)g.OH * g.OW);
    const uint32_t rem = c - n * (uint32_t)g.OH * g.OW;
    const uint32_t oh = rem / g.OW, ow = rem - oh * g.OW;
    const size_t plane = (size_t)g.DH * g.DW;
    float* out = dst + (size_t)n * g.M * plane + (size_t)(oh * g.osh + g.oh0) * g.DW +
                 (ow * g.osw + g.ow0);
#pragma unroll
    for (int mi = 0; mi < 2; ++mi) {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int m = m0 + wm * 64 + mi * 32 + acc_row(v, lane);
        if (m < g.M) {
          float r = acc[mi][ni][v];
          if (bias) r += bias[m];
          out[(size_t)m * plane] = r;
        }
      }
    }
  }
}

// ------------------------------------------------------- backward weight --
// dw[k][c][r][s] = sum over (n, p, q) dy[n,k,p,q] * x[n,c,p*sH + r*dH - pH, q*sW + s*dW - pW]
// GEMM: rows = k (M = K), columns = (c, r, s) (Ncol = C*R*S), depth = (n, p, q).
struct WGrad {
  int K, C, R, S, H, W, P, Q, N;
  int sH, sW, pH, pW, dH, dW;
  uint32_t depth;       // N*P*Q
  uint32_t ncols;       // C*R*S
  FastDiv divRS, divS;
  uint32_t tiles_per_split;  // k-tiles handled by one blockIdx.z
  int mode;             // 0: store, 1: atomicAdd into dw, 2: store partial [z][K][ncols]
};

constexpr int WBK = 32;  // depth of a staged tile for backward-weight

struct WLds {
  float a[2][WBK][BM + kPad];
  float b[2][WBK][BN + kPad];
};

__device__ __forceinline__ void mma_tile_w(const float (*As)[BM + kPad],
                                           const float (*Bs)[BN + kPad], int wm, int wn, int lane,
                                           float16_t (&acc)[2][2]) {
  const int r = lane & 31, half = lane >> 5;
#pragma unroll
  for (int ks = 0; ks < WBK; ks += 2) {
    const int k = ks + half;
    const float a0 = As[k][wm * 64 + r];
    const float a1 = As[k][wm * 64 + 32 + r];
    const float b0 = Bs[k][wn * 64 + r];
    const float b1 = Bs[k][wn * 64 + 32 + r];
    acc[0][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b0, acc[0][0], 0, 0, 0);
    acc[0][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b1, acc[0][1], 0, 0, 0);
    acc[1][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b0, acc[1][0], 0, 0, 0);
    acc[1][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b1, acc[1][1], 0, 0, 0);
  }
}

__global__ __launch_bounds__(kThreads) void wgrad_kernel(const WGrad g,
                                                         const float* __restrict__ dy,
                                                         const float* __restrict__ x,
                                                         float* __restrict__ out) {
  __shared__ WLds lds;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  const int m0 = blockIdx.y * BM;
  const uint32_t n0 = blockIdx.x * BN;
  const uint32_t PQ = (uint32_t)g.P * g.Q;

  // this thread always fetches depth lane kd = tid % 32 and rows row0 + 8*i of both tiles
  const int kdl = tid & (WBK - 1), row0 = tid / WBK;
  constexpr int kRows = BM * WBK / kThreads;  // 16

  // the (c, r, s) of this thread's 16 B rows never change: keep offset and window shift
  int bo_h[kRows], bo_w[kRows];
  uint32_t bo_c[kRows];
#pragma unroll
  for (int i = 0; i < kRows; ++i) {
    const uint32_t cc = n0 + row0 + (kThreads / WBK) * i;
    if (cc < g.ncols) {
      const uint32_t c = g.divRS.div(cc);
      const uint32_t rs = cc - c * (uint32_t)(g.R * g.S);
      const uint32_t r = g.divS.div(rs), s = rs - r * g.S;
      bo_c[i] = c;
      bo_h[i] = (int)r * g.dH - g.pH;
      bo_w[i] = (int)s * g.dW - g.pW;
    } else {
      bo_c[i] = 0xFFFFFFFFu;
      bo_h[i] = 0;
      bo_w[i] = 0;
    }
  }

  float ra[kRows], rb[kRows];
  auto fetch = [&](uint32_t d0) {
    const uint32_t d = d0 + kdl;
    const bool d_ok = d < g.depth;
    uint32_t n = 0, p = 0, q = 0;
    if (d_ok) {
      n = d / PQ;
      const uint32_t pq = d - n * PQ;
      p = pq / g.Q;
      q = pq - p * g.Q;
    }
    const float* dyp = dy + (size_t)n * g.K * PQ + (size_t)p * g.Q + q;
    const float* xp = x + (size_t)n * g.C * g.H * g.W;
    const int h0 = (int)p * g.sH, w0 = (int)q * g.sW;
#pragma unroll
    for (int i = 0; i < kRows; ++i) {
      const int m = m0 + row0 + (kThreads / WBK) * i;
      ra[i] = (d_ok && m < g.K) ? dyp[(size_t)m * PQ] : 0.f;
      float v = 0.f;
      if (d_ok && bo_c[i] != 0xFFFFFFFFu) {
        const int hh = h0 + bo_h[i], ww = w0 + bo_w[i];
        if ((unsigned)hh < (unsigned)g.H && (unsigned)ww < (unsigned)g.W)
          v = xp[((size_t)bo_c[i] * g.H + hh) * g.W + ww];
      }
      rb[i] = v;
    }
  };
  auto stage = [&](int buf) {
#pragma unroll
    for (int i = 0; i < kRows; ++i) {
      lds.a[buf][kdl][row0 + (kThreads / WBK) * i] = ra[i];
      lds.b[buf][kdl][row0 + (kThreads / WBK) * i] = rb[i];
    }
  };

  float16_t acc[2][2];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  const uint32_t total_tiles = (g.depth + WBK - 1) / WBK;
  const uint32_t t_begin = blockIdx.z * g.tiles_per_split;
  const uint32_t t_end = min(t_begin + g.tiles_per_split, total_tiles);
  if (t_begin < t_end) {
    fetch(t_begin * WBK);
    stage(0);
    __syncthreads();
    for (uint32_t kt = t_begin; kt < t_end; ++kt) {
      const int buf = (kt - t_begin) & 1;
      if (kt + 1 < t_end) fetch((kt + 1) * WBK);
      mma_tile_w(lds.a[buf], lds.b[buf], wm, wn, lane, acc);
      if (kt + 1 < t_end) stage(buf ^ 1);
      __syncthreads();
    }
  }

  float* base = out;
  if (g.mode == 2) base += (size_t)blockIdx.z * g.K * g.ncols;
#pragma unroll
  for (int ni = 0; ni < 2; ++ni) {
    const uint32_t c = n0 + wn * 64 + ni * 32 + (lane & 31);
    if (c >= g.ncols) continue;
#pragma unroll
    for (int mi = 0; mi < 2; ++mi) {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int m = m0 + wm * 64 + mi * 32 + acc_row(v, lane);
        if (m < g.K) {
          float* o = base + (size_t)m * g.ncols + c;
          if (g.mode == 1)
            atomicAdd(o, acc[mi][ni][v]);
          else
            *o = acc[mi][ni][v];
        }
      }
    }
  }
}

// dw[i] = sum over splits of partial[z][i], fixed order.
__global__ __launch_bounds__(kThreads) void wgrad_reduce_kernel(const float* __restrict__ partial,
                                                                float* __restrict__ dw, size_t n,
                                                                int splits) {
  const size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x;
  if (i >= n) return;
  float s = 0.f;
  for (int z = 0; z < splits; ++z) s += partial[(size_t)z * n + i];
  dw[i] = s;
}

__global__ __launch_bounds__(kThreads) void fill_zero_kernel(float* p, size_t n) {
  const size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x;
  if (i < n) p[i] = 0.f;
}

// wt[c][k][r][s] = w[k][c][r][s]
__global__ __launch_bounds__(kThreads) void transpose_weights_kernel(const float* __restrict__ w,
                                                                     float* __restrict__ wt, int K,
                                                                     int C, int RS) {
  const size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x;
  const size_t n = (size_t)K * C * RS;
  if (i >= n) return;
  const int rs = i % RS;
  const size_t kc = i / RS;
  const int k = kc % K;
  const int c = kc / K;
  wt[i] = w[((size_t)k * C + c) * RS + rs];
}

// ------------------------------------------------------------------ host --
static int check(const mn_conv2d* g) {
  if (!g) return MN_EINVAL;
  if (g->N < 0 || g->C <= 0 || g->K <= 0 || g->H <= 0 || g->W <= 0 || g->R <= 0 || g->S <= 0)
    return MN_EINVAL;
  if (g->sH <= 0 || g->sW <= 0 || g->dH <= 0 || g->dW <= 0 || g->pH < 0 || g->pW < 0)
    return MN_EINVAL;
  if (g->groups != 1) return MN_EUNSUPPORTED;
  if (g->R * g->S > kMaxTaps) return MN_EUNSUPPORTED;
  const long long P = ((long long)g->H + 2 * g->pH - (long long)g->dH * (g->R - 1) - 1) / g->sH + 1;
  const long long Q = ((long long)g->W + 2 * g->pW - (long long)g->dW * (g->S - 1) - 1) / g->sW + 1;
  if (P != g->P || Q != g->Q || P <= 0 || Q <= 0) return MN_EINVAL;
  // index ranges the kernels rely on
  if ((long long)g->C * g->R * g->S >= (1 << 20) || (long long)g->K * g->R * g->S >= (1 << 20))
    return MN_EUNSUPPORTED;
  if ((long long)g->N * g->H * g->W >= (1ll << 31) || (long long)g->N * g->P * g->Q >= (1ll << 31))
    return MN_EUNSUPPORTED;
  return MN_OK;
}

static void launch_gather(const Gather& g, const float* a, const float* src, const float* bias,
                          float* dst, unsigned long long src_bytes, unsigned long long a_bytes,
                          hipStream_t s) {
  if (g.ncols == 0 || g.M == 0) return;
  dim3 grid((g.ncols + BN - 1) / BN, (g.M + BM - 1) / BM);
  const unsigned long long limit = 1ull << 32;
  const bool fast = g.T > 0 && g.Cs % BK == 0 && src_bytes < limit && a_bytes < limit;
  if (fast)
    gather_gemm_kernel<true><<<grid, kThreads, 0, s>>>(g, a, src, bias, dst);
  else
    gather_gemm_kernel<false><<<grid, kThreads, 0, s>>>(g, a, src, bias, dst);
}

// Split of the (n, p, q) reduction: enough workgroups for ~2 per CU.
static void wgrad_split(const mn_conv2d* g, int* splits, int* tiles_per_split) {
  const long long depth = (long long)g->N * g->P * g->Q;
  const long long total_tiles = (depth + WBK - 1) / WBK;
  const long long out_tiles =
      (((long long)g->C * g->R * g->S + BN - 1) / BN) * (((long long)g->K + BM - 1) / BM);
  long long want = (512 + out_tiles - 1) / out_tiles;
  if (want > total_tiles) want = total_tiles;
  if (want > 256) want = 256;
  if (want < 1) want = 1;
  const long long tps = (total_tiles + want - 1) / want;
  *tiles_per_split = (int)(tps < 1 ? 1 : tps);
  *splits = (int)((total_tiles + *tiles_per_split - 1) / (*tiles_per_split));
  if (*splits < 1) *splits = 1;
}


}  // namespace mn_conv

extern "C" {

int mn_conv_n_variants(int direction) {
  switch (direction) {
    case MN_CONV_FWD:
      return 1;
    case MN_CONV_BWD_DATA:
      return 2;
    case MN_CONV_BWD_WEIGHT:
      return 2;
    default:
      return 0;
  }
}

int mn_conv_ws_bytes(const mn_conv2d* g, int direction, int variant, int dtype, size_t* bytes) {
  using namespace mn_conv;
  if (!bytes) return MN_EINVAL;
  *bytes = 0;
  const int st = check(g);
  if (st != MN_OK) return st;
  if (dtype != MN_F32) return MN_EUNSUPPORTED;
  if (variant < 0 || variant >= mn_conv_n_variants(direction)) return MN_EUNSUPPORTED;
  const size_t wsize = (size_t)g->K * g->C * g->R * g->S * sizeof(float);
  if (direction == MN_CONV_BWD_DATA && variant == 1) *bytes = wsize;
  if (direction == MN_CONV_BWD_WEIGHT && variant == 1) {
    int splits, tiles;
    wgrad_split(g, &splits, &tiles);
    *bytes = splits > 1 ? wsize * splits : 0;
  }
  return MN_OK;
}

int mn_conv_fwd(const mn_conv2d* g, const void* x, const void* w, const void* bias, void* y,
                void* ws, size_t ws_bytes, int variant, int dtype, mn_stream_t stream) {
  using namespace mn_conv;
  (void)ws;
  (void)ws_bytes;
  const int st = check(g);
  if (st != MN_OK) return st;
  if (dtype != MN_F32) return MN_EUNSUPPORTED;
  if (variant != 0) return MN_EUNSUPPORTED;
  if (g->N == 0) return MN_OK;
  if (!x || !w || !y) return MN_EINVAL;
  Gather q = {};
  q.M = g->K;
  q.T = g->R * g->S;
  q.Kd = g->C * q.T;
  q.divT = make_fastdiv(q.T);
  q.N = g->N;
  q.OH = g->P;
  q.OW = g->Q;
  q.ncols = (uint32_t)((long long)g->N * g->P * g->Q);
  q.Cs = g->C;
  q.Hs = g->H;
  q.Ws = g->W;
  q.ish = g->sH;
  q.isw = g->sW;
  q.DH = g->P;
  q.DW = g->Q;
  q.osh = q.osw = 1;
  q.lda = (long long)g->C * q.T;
  q.cha = q.T;
  for (int r = 0; r < g->R; ++r)
    for (int s = 0; s < g->S; ++s) {
      const int t = r * g->S + s;
      q.dh[t] = (int16_t)(r * g->dH - g->pH);
      q.dw[t] = (int16_t)(s * g->dW - g->pW);
      q.aoff[t] = t;
    }
  launch_gather(q, (const float*)w, (const float*)x, (const float*)bias, (float*)y,
                4ull * g->N * g->C * g->H * g->W, 4ull * g->K * g->C * g->R * g->S,
                mn_stream(stream));
  return mn_launch_status();
}

int mn_conv_bwd_data(const mn_conv2d* g, const void* dy, const void* w, void* dx, void* ws,
                     size_t ws_bytes, int variant, int dtype, mn_stream_t stream) {
  using namespace mn_conv;
  const int st = check(g);
  if (st != MN_OK) return st;
  if (dtype != MN_F32) return MN_EUNSUPPORTED;
  if (variant < 0 || variant > 1) return MN_EUNSUPPORTED;
  if (g->N == 0) return MN_OK;
  if (!dy || !w || !dx) return MN_EINVAL;
  hipStream_t s = mn_stream(stream);
  const int RS = g->R * g->S;
  const float* a = (const float*)w;
  long long lda = RS, cha = (long long)g->C * RS;  // read w[k][c][r][s] as A(c, k, rs)
  if (variant == 1) {
    const size_t n = (size_t)g->K * g->C * RS;
    if (!ws || ws_bytes < n * sizeof(float) || !mn_aligned(ws, 4)) return MN_EINVAL;
    transpose_weights_kernel<<<(unsigned)((n + kThreads - 1) / kThreads), kThreads, 0, s>>>(
        (const float*)w, (float*)ws, g->K, g->C, RS);
    a = (const float*)ws;
    lda = (long long)g->K * RS;
    cha = RS;
  }
  // one dense gather per parity class (a, b) of (h + pH, w + pW) modulo the stride
  for (int ca = 0; ca < g->sH; ++ca) {
    for (int cb = 0; cb < g->sW; ++cb) {
      Gather q = {};
      q.M = g->C;
      q.oh0 = ((ca - g->pH) % g->sH + g->sH) % g->sH;
      q.ow0 = ((cb - g->pW) % g->sW + g->sW) % g->sW;
      q.OH = q.oh0 < g->H ? (g->H - q.oh0 + g->sH - 1) / g->sH : 0;
      q.OW = q.ow0 < g->W ? (g->W - q.ow0 + g->sW - 1) / g->sW : 0;
      int T = 0;
      for (int r = 0; r < g->R; ++r) {
        if ((r * g->dH) % g->sH != ca) continue;
        for (int sx = 0; sx < g->S; ++sx) {
          if ((sx * g->dW) % g->sW != cb) continue;
          q.dh[T] = (int16_t)((q.oh0 + g->pH - r * g->dH) / g->sH);
          q.dw[T] = (int16_t)((q.ow0 + g->pW - sx * g->dW) / g->sW);
          q.aoff[T] = r * g->S + sx;
          ++T;
        }
      }
      q.T = T;
      q.Kd = g->K * T;
      q.divT = make_fastdiv(T);
      q.N = g->N;
      q.ncols = (uint32_t)((long long)g->N * q.OH * q.OW);
      q.Cs = g->K;
      q.Hs = g->P;
      q.Ws = g->Q;
      q.ish = q.isw = 1;
      q.DH = g->H;
      q.DW = g->W;
      q.osh = g->sH;
      q.osw = g->sW;
      q.lda = lda;
      q.cha = cha;
      launch_gather(q, a, (const float*)dy, nullptr, (float*)dx, 4ull * g->N * g->K * g->P * g->Q,
                    4ull * g->K * g->C * g->R * g->S, s);
    }
  }
  return mn_launch_status();
}

int mn_conv_bwd_weight(const mn_conv2d* g, const void* dy, const void* x, void* dw, void* ws,
                       size_t ws_bytes, int variant, int dtype, mn_stream_t stream) {
  using namespace mn_conv;
  const int st = check(g);
  if (st != MN_OK) return st;
  if (dtype != MN_F32) return MN_EUNSUPPORTED;
  if (variant < 0 || variant > 1) return MN_EUNSUPPORTED;
  if (!dw) return MN_EINVAL;
  hipStream_t s = mn_stream(stream);
  const size_t nw = (size_t)g->K * g->C * g->R * g->S;
  if (g->N == 0) {
    fill_zero_kernel<<<(unsigned)((nw + kThreads - 1) / kThreads), kThreads, 0, s>>>((float*)dw, nw);
    return mn_launch_status();
  }
  if (!dy || !x) return MN_EINVAL;
  WGrad q = {};
  q.K = g->K;
  q.C = g->C;
  q.R = g->R;
  q.S = g->S;
  q.H = g->H;
  q.W = g->W;
  q.P = g->P;
  q.Q = g->Q;
  q.N = g->N;
  q.sH = g->sH;
  q.sW = g->sW;
  q.pH = g->pH;
  q.pW = g->pW;
  q.dH = g->dH;
  q.dW = g->dW;
  q.depth = (uint32_t)((long long)g->N * g->P * g->Q);
  q.ncols = (uint32_t)(g->C * g->R * g->S);
  q.divRS = make_fastdiv(g->R * g->S);
  q.divS = make_fastdiv(g->S);
  int splits, tps;
  wgrad_split(g, &splits, &tps);
  q.tiles_per_split = tps;
  float* out = (float*)dw;
  if (splits == 1) {
    q.mode = 0;
  } else if (variant == 0) {
    q.mode = 1;
    fill_zero_kernel<<<(unsigned)((nw + kThreads - 1) / kThreads), kThreads, 0, s>>>((float*)dw, nw);
  } else {
    q.mode = 2;
    if (!ws || ws_bytes < nw * sizeof(float) * splits || !mn_aligned(ws, 4)) return MN_EINVAL;
    out = (float*)ws;
  }
  dim3 grid((q.ncols + BN - 1) / BN, (g->K + BM - 1) / BM, splits);
  wgrad_kernel<<<grid, kThreads, 0, s>>>(q, (const float*)dy, (const float*)x, out);
  if (q.mode == 2)
    wgrad_reduce_kernel<<<(unsigned)((nw + kThreads - 1) / kThreads), kThreads, 0, s>>>(
        (const float*)ws, (float*)dw, nw, splits);
  return mn_launch_status();
}

}  // extern "C"
