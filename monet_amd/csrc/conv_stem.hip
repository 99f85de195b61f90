// The first convolution of an ImageNet network (3 -> 64 channels, 7x7, stride 2, padding 3) as
// kernels of its own.  Reference slot: the same cudnnConvolution* calls as every other
// convolution (monet/lm_ops/conv.cpp:21-46); the general gather GEMM runs this shape at 0.45 of
// the fp32 matrix rate because the reduction (3 x 49 = 147) is no multiple of its 16-deep tiles
// and every element needs its own window test and address.
//
// Here the whole reduction is ONE tile.  Forward: a workgroup owns 64 output channels x 4 output
// rows x 128 columns (one image); the 13 input rows of each channel that those outputs read lie
// in LDS with their left and right padding written out as zeros (no window test in the loop),
// the weights lie beside them as [reduction][channel].  A wavefront takes 32 columns of all four
// rows and both halves of the channels: per 2-deep step of v_mfma_f32_32x32x2_f32 two weight
// reads and four pixel reads from LDS feed eight matrix instructions, with addresses that are
// compile-time constants of the unrolled loop.  74 KB of LDS: two workgroups fit a CU, so one
// stages while the other multiplies.  Backward-weight (variant 1 as well): further down.
#include "common.h"

namespace mn_stem {

constexpr int kThreads = 256;
constexpr int C = 3, R = 7, S = 7, K = 64;         // the only shape these kernels take
constexpr int kDepth = C * R * S;                  // 147
constexpr int kSteps = (kDepth + 1) / 2;           // 74 matrix steps of depth 2 (the last half empty)
constexpr int kRowsOut = 4;                        // output rows per workgroup
constexpr int kRowsIn = 2 * kRowsOut + R - 2;      // 13 input rows per channel
constexpr int kMaxW = 224;                         // widest input row
constexpr int kPadLeft = 4;                        // zeros in front of a row (3 needed; 4 keeps 16-byte alignment)
constexpr int kRowLen = 232;                       // floats per LDS row: the zeros, the row, zeros
constexpr int kColsOut = 128;                      // columns a workgroup covers (4 wavefronts x 32)
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef float float4_t __attribute__((ext_vector_type(4)));

// wt[k][m] = w[m][k] for k < 147, zero for k = 147
__global__ __launch_bounds__(kThreads) void transpose_weights_kernel(const float* __restrict__ w,
                                                                     float* __restrict__ wt) {
  const int i = blockIdx.x * kThreads + threadIdx.x;
  if (i >= 2 * kSteps * K) return;
  const int k = i / K, m = i - k * K;
  wt[i] = k < kDepth ? w[m * kDepth + k] : 0.f;
}

struct Geo {
  int N, H, W, P, Q;
  int row_blocks;   // workgroups per image
};

// LDS offset (floats) of reduction element k for output column 0 of output row 0:
// k = (c * 7 + r) * 7 + s  ->  row (c, r), column s - 3 + kPadLeft  (input column 2 ow + s - 3)
__device__ __forceinline__ constexpr int tap_offset(int k) {
  return k < kDepth ? ((k / (R * S)) * kRowsIn + (k / S) % R) * kRowLen + k % S + kPadLeft - 3 : 0;
}

// One 16-byte piece of the staged input rows (piece i of [C * kRowsIn][kRowLen / 4]): the value to
// write to LDS.  Branch-free when the rows allow 16-byte loads: the load is always issued (from
// the start of the tensor when the piece lies outside the image) and the result replaced by zeros,
// so that all pieces of a thread are in flight together; a branch around each load made the
// compiler wait for one load before it issued the next.
template <bool VEC>
__device__ __forceinline__ float4_t staged_piece(const float* __restrict__ x, int n, int H, int W,
                                                 int h_first, int i) {
  const int row = i / (kRowLen / 4), q = i - row * (kRowLen / 4);
  const int c = row / kRowsIn, h = h_first + row - c * kRowsIn;
  const int wcol = 4 * q - kPadLeft;
  const bool row_ok = row < C * kRowsIn && (unsigned)h < (unsigned)H;
  const size_t off = (((size_t)n * C + c) * H + h) * W + wcol;
  float4_t v = {0.f, 0.f, 0.f, 0.f};
  if (VEC) {
    const bool ok = row_ok && (unsigned)wcol < (unsigned)W;
    const float4_t got = *reinterpret_cast<const float4_t*>(x + (ok ? off : 0));
    v = ok ? got : v;
  } else if (row_ok) {
#pragma unroll
    for (int e = 0; e < 4; ++e)
      if ((unsigned)(wcol + e) < (unsigned)W) v[e] = x[off + e];
  }
  return v;
}

template <bool VEC>  // rows that allow 16-byte loads (W % 4 == 0, x 16-byte aligned)
__global__ __launch_bounds__(kThreads, 2) void forward_kernel(const Geo g, const float* __restrict__ x,
                                                              const float* __restrict__ wt,
                                                              const float* __restrict__ bias,
                                                              float* __restrict__ y) {
  __shared__ __attribute__((aligned(16))) float lds_w[2 * kSteps][K];
  __shared__ __attribute__((aligned(16))) float lds_x[C * kRowsIn][kRowLen];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const uint32_t blk = blockIdx.x;
  const int n = blk / g.row_blocks, oh0 = (blk - n * g.row_blocks) * kRowsOut;

  // Staging: every load of the workgroup is issued before the first LDS write (a loop of load,
  // wait, store pays the memory latency once per trip: the workgroup then waited as long as it
  // multiplied).  Weights: a straight copy of 148 x 64 floats.  Input rows 2 oh0 - 3 .. + 12 of
  // the three channels, each as kPadLeft zeros, W floats, zeros; 16-byte pieces when the rows
  // allow it.
  constexpr int kWItems = (2 * kSteps * K / 4 + kThreads - 1) / kThreads;
  constexpr int kXItems = (C * kRowsIn * (kRowLen / 4) + kThreads - 1) / kThreads;
  {
    float4_t wv[kWItems], xv[kXItems];
#pragma unroll
    for (int u = 0; u < kWItems; ++u) {
      const int i = tid + u * kThreads;
      wv[u] = reinterpret_cast<const float4_t*>(wt)[i < 2 * kSteps * K / 4 ? i : 0];  // (not written when beyond)
    }
    const int h_first = 2 * oh0 - 3;
#pragma unroll
    for (int u = 0; u < kXItems; ++u) xv[u] = staged_piece<VEC>(x, n, g.H, g.W, h_first, tid + u * kThreads);
#pragma unroll
    for (int u = 0; u < kWItems; ++u) {
      const int i = tid + u * kThreads;
      if (i < 2 * kSteps * K / 4) reinterpret_cast<float4_t*>(&lds_w[0][0])[i] = wv[u];
    }
#pragma unroll
    for (int u = 0; u < kXItems; ++u) {
      const int i = tid + u * kThreads;
      if (i < C * kRowsIn * (kRowLen / 4)) reinterpret_cast<float4_t*>(&lds_x[0][0])[i] = xv[u];
    }
  }
  __syncthreads();

  float16_t acc[kRowsOut][2];
#pragma unroll
  for (int j = 0; j < kRowsOut; ++j)
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[j][i][v] = 0.f;
  const int half = lane >> 5, col = wave * 32 + (lane & 31);
  // lanes 32-63 hold the odd reduction element of a step
  const float* const pw = &lds_w[half][lane & 31];
  // (columns past the row compute with the last real column's pixels and are not stored)
  const float* const px = &lds_x[0][0] + 2 * min(col, g.Q - 1);
#pragma unroll
  for (int s = 0; s < kSteps; ++s) {
    const int off = half ? tap_offset(2 * s + 1) : tap_offset(2 * s);
    const float a0 = pw[2 * s * K], a1 = pw[2 * s * K + 32];
    float b[kRowsOut];
#pragma unroll
    for (int j = 0; j < kRowsOut; ++j) b[j] = px[off + 2 * j * kRowLen];
#pragma unroll
    for (int j = 0; j < kRowsOut; ++j) {
      acc[j][0] = __builtin_amdgcn_mfma_f32_32x32x2f32(a0, b[j], acc[j][0], 0, 0, 0);
      acc[j][1] = __builtin_amdgcn_mfma_f32_32x32x2f32(a1, b[j], acc[j][1], 0, 0, 0);
    }
  }
  // a register holds one output channel for 32 consecutive columns: 128 contiguous bytes per
  // half-wavefront and store
  if (col >= g.Q) return;
#pragma unroll
  for (int j = 0; j < kRowsOut; ++j) {
    const int oh = oh0 + j;
    if (oh >= g.P) break;
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int m = 32 * i + 8 * (v >> 2) + 4 * half + (v & 3);
        const float bv = bias ? bias[m] : 0.f;
        __builtin_nontemporal_store(acc[j][i][v] + bv, &y[(((size_t)n * K + m) * g.P + oh) * g.Q + col]);
      }
  }
}

// ---------------------------------------------------------------- backward weight --
// dW[k][col] = sum over (n, oh, ow) of dy[n][k][oh][ow] * x[n][c][2 oh - 3 + r][2 ow - 3 + s],
// col = (c, r, s): a 64 x 147 result reduced over N * P * Q positions.  The general kernel builds
// the 147 columns with a window test and an address per element; here the input rows lie in LDS
// exactly as in the forward kernel (padding written out as zeros), a column is a per-lane LDS
// offset that never changes, and the output gradient comes straight from global memory: a lane
// holds output k (or 32 + k) and loads 4 consecutive positions as one 16-byte vector.
// The reduction index of a matrix step is free as long as both operands agree: within a group
// of 8 positions lanes 0-31 take positions 0..3 and lanes 32-63 positions 4..7, one per step.
// A workgroup walks (image, 4 output rows) items; a wavefront takes 32 of the outputs and two of
// the four rows, with its 32 x 160 result (147 columns padded to five 32-wide tiles) in 80
// accumulation registers per lane; at the end the two wavefronts of each half of the outputs are
// added in order through LDS and the workgroup writes one partial result, which
// wgrad_reduce_kernel adds in order (reproducible).
constexpr int kColTiles = 5;
constexpr int kColsPad = 32 * kColTiles;
constexpr int kAhead = 4;                          // groups of the output gradient in flight
constexpr int kMaxGroups = kColsOut / 8;           // groups of 8 positions in the widest row

struct WGeo {
  int N, H, W, P, Q;
  int row_blocks;
  uint32_t items;  // N * row_blocks
};

// EVEN8: Q % 8 == 0, W % 4 == 0, x and dy 16-byte aligned: vector loads, no position beyond a row.
// NG: groups per row when known at compile time (14 for the 224 x 224 image), else 0: with a trip
// count only known at run time the exits from the unrolled loop are block boundaries, at which
// the compiler waits for every load in flight.
template <bool EVEN8, int NG>
__global__ __launch_bounds__(kThreads, 2) void wgrad_kernel(const WGeo g, const float* __restrict__ x,
                                                            const float* __restrict__ dy,
                                                            float* __restrict__ partial,
                                                            float* __restrict__ dbp) {
  __shared__ __attribute__((aligned(16))) float lds_x[C * kRowsIn][kRowLen];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int half = lane >> 5, r = lane & 31;
  // a wavefront owns 32 outputs (kh) and two of the four output rows (rsel, rsel + 2): 80
  // accumulation registers, which leaves room for the staging loads to be in flight together
  // (with all 64 outputs of one row per wavefront, 160, the compiler issued them one by one)
  const int kh = wave & 1, rsel = wave >> 1;
  const float* const flat = &lds_x[0][0];
  // LDS offset of this lane's column in tile t for position 0 of its half of a group, row rsel
  int tap[kColTiles];
#pragma unroll
  for (int t = 0; t < kColTiles; ++t) {
    const int k = 32 * t + r;
    const int off = k < kDepth ? ((k / (R * S)) * kRowsIn + (k / S) % R) * kRowLen + k % S + kPadLeft - 3 : 0;
    tap[t] = off + 2 * rsel * kRowLen + 8 * half;
  }
  float16_t acc[kColTiles];
#pragma unroll
  for (int t = 0; t < kColTiles; ++t)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[t][v] = 0.f;
  float bsum = 0.f;  // bias gradient: the sum of this lane's share of dy (output 32 kh + r)

  constexpr int kXItems = (C * kRowsIn * (kRowLen / 4) + kThreads - 1) / kThreads;
  const int ngroups = NG ? NG : (g.Q + 7) >> 3;
  for (uint32_t item = blockIdx.x; item < g.items; item += gridDim.x) {
    const int n = item / g.row_blocks, oh0 = (item - n * g.row_blocks) * kRowsOut;
    // The output gradient comes straight from global memory, kAhead groups ahead of the matrix
    // instructions (a group of 20 MFMAs covers 0.5 us); the first groups of the first row are
    // requested before the input rows are staged.
    const float* const dyk = dy + ((size_t)n * K + 32 * kh + r) * g.P * g.Q + 4 * half;
    auto load = [&](const float* row, int gq, float4_t& a) {
      gq = gq < ngroups ? gq : ngroups - 1;  // past the end: the last group again, not used
      if (EVEN8) {
        a = *reinterpret_cast<const float4_t*>(row + 8 * gq);
      } else {
#pragma unroll
        for (int j = 0; j < 4; ++j) a[j] = 8 * gq + 4 * half + j < g.Q ? row[8 * gq + j] : 0.f;
      }
    };
    auto row_of = [&](int rr) {  // rows beyond the image: the last real row, not used
      const int oh = oh0 + rsel + 2 * rr;
      return dyk + (size_t)(oh < g.P ? oh : g.P - 1) * g.Q;
    };
    float4_t a[kAhead];
    {
      const float* const row = row_of(0);
#pragma unroll
      for (int d = 0; d < kAhead; ++d) load(row, d, a[d]);
    }
    {
      // input rows 2 oh0 - 3 .. + 12 of the three channels; all loads before the first LDS write
      float4_t xv[kXItems];
      const int h_first = 2 * oh0 - 3;
#pragma unroll
      for (int u = 0; u < kXItems; ++u) xv[u] = staged_piece<EVEN8>(x, n, g.H, g.W, h_first, tid + u * kThreads);
      __syncthreads();  // the rows of the previous item are no longer read
#pragma unroll
      for (int u = 0; u < kXItems; ++u) {
        const int i = tid + u * kThreads;
        if (i < C * kRowsIn * (kRowLen / 4)) reinterpret_cast<float4_t*>(&lds_x[0][0])[i] = xv[u];
      }
      __syncthreads();
    }
#pragma unroll
    for (int rr = 0; rr < 2; ++rr) {
      if (oh0 + rsel + 2 * rr >= g.P) break;  // uniform per wavefront
      const float* const row = row_of(rr);
      if (rr) {
#pragma unroll
        for (int d = 0; d < kAhead; ++d) load(row, d, a[d]);
        __builtin_amdgcn_sched_barrier(0);
      }
#pragma unroll
      for (int gq = 0; gq < (NG ? NG : kMaxGroups); ++gq) {
        if (!NG && gq >= ngroups) break;
        const float4_t c = a[gq % kAhead];
        bsum += (c[0] + c[1]) + (c[2] + c[3]);
        load(row, gq + kAhead, a[gq % kAhead]);
        // (the scheduler otherwise sinks the load to just before its use, kAhead groups later)
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          float b[kColTiles];
#pragma unroll
          for (int t = 0; t < kColTiles; ++t) {
            int px2 = 16 * gq + 2 * j + 4 * rr * kRowLen;  // twice the position (this lane's half is in tap[])
            if (!EVEN8) {
              // a position beyond the row multiplies a zero of dy: read the last real one instead
              const int px = 8 * gq + 4 * half + j;
              px2 -= 2 * (px > g.Q - 1 ? px - (g.Q - 1) : 0);
            }
            b[t] = flat[tap[t] + px2];
          }
#pragma unroll
          for (int t = 0; t < kColTiles; ++t)
            acc[t] = __builtin_amdgcn_mfma_f32_32x32x2f32(c[j], b[t], acc[t], 0, 0, 0);
        }
      }
    }
  }
  // outputs 0..31, then 32..63: the two wavefronts that hold them, in order, through the LDS the
  // rows occupied
  float* const red = &lds_x[0][0];
  {
    // bias gradient first: the two halves of a wavefront, then the two wavefronts of an output
    __syncthreads();
    const float both = bsum + __shfl_xor(bsum, 32);
    if (rsel == 1 && half == 0) red[32 * kh + r] = both;
    __syncthreads();
    if (rsel == 0 && half == 0) dbp[(size_t)blockIdx.x * K + 32 * kh + r] = both + red[32 * kh + r];
  }
  static_assert(32 * kColsPad <= C * kRowsIn * kRowLen, "reduction buffer");
#pragma unroll
  for (int h = 0; h < 2; ++h) {
#pragma unroll
    for (int w = 0; w < 2; ++w) {
      __syncthreads();
      if (kh == h && rsel == w) {
#pragma unroll
        for (int t = 0; t < kColTiles; ++t)
#pragma unroll
          for (int v = 0; v < 16; ++v) {
            const int idx = (8 * (v >> 2) + 4 * half + (v & 3)) * kColsPad + 32 * t + r;
            red[idx] = (w ? red[idx] : 0.f) + acc[t][v];
          }
      }
    }
    __syncthreads();
    for (int i = tid; i < 32 * kDepth; i += kThreads) {
      const int m = i / kDepth, col = i - m * kDepth;
      partial[((size_t)blockIdx.x * K + 32 * h + m) * kDepth + col] = red[m * kColsPad + col];
    }
  }
}

// dw = sum of the workgroups' partial results, in a fixed order: 16 outputs x 16 slices of the
// partials per workgroup (one thread per output walking all 512 partials is a chain of loads
// 37 KB apart: 0.25 ms), the slices then added in order through LDS.
__global__ __launch_bounds__(kThreads) void wgrad_reduce_kernel(const float* __restrict__ partial,
                                                                const float* __restrict__ dbp,
                                                                float* __restrict__ dw,
                                                                float* __restrict__ db, int parts) {
  static_assert(K * kDepth % 16 == 0 && K % 16 == 0 && kThreads == 256, "16 outputs x 16 slices per workgroup");
  __shared__ float red[16][17];
  const int o = threadIdx.x & 15, sl = threadIdx.x >> 4;
  // blocks past the weight gradient reduce the bias gradient the same way
  const int nwb = K * kDepth / 16;
  const bool bias = (int)blockIdx.x >= nwb;
  const float* const src = bias ? dbp : partial;
  const int stride = bias ? K : K * kDepth;
  const int i = (bias ? (int)blockIdx.x - nwb : (int)blockIdx.x) * 16 + o;
  const int per = (parts + 15) / 16;
  const int p0 = sl * per, p1 = min(parts, p0 + per);
  float s = 0.f;
#pragma unroll 8
  for (int p = p0; p < p1; ++p) s += src[(size_t)p * stride + i];
  red[sl][o] = s;
  __syncthreads();
  if (sl == 0) {
    float t = 0.f;
#pragma unroll
    for (int q = 0; q < 16; ++q) t += red[q][o];
    (bias ? db : dw)[i] = t;
  }
}

static uint32_t wgrad_workgroups(const mn_conv2d* g) {
  int dev = 0, cus = 256;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
    cus = 256;
  const long long items = (long long)g->N * ((g->P + kRowsOut - 1) / kRowsOut);
  return (uint32_t)(items < 2ll * cus ? items : 2ll * cus);  // two workgroups fit a CU
}

static bool stem_shape(const mn_conv2d* g) {
  return g->C == C && g->K == K && g->R == R && g->S == S && g->sH == 2 && g->sW == 2 && g->pH == 3 &&
         g->pW == 3 && g->dH == 1 && g->dW == 1 && g->groups == 1 && g->W <= kMaxW &&
         g->Q <= kColsOut && g->W + kPadLeft + 4 <= kRowLen;
}

}  // namespace mn_stem

// Entry points used by conv.hip (fp32).  MN_EUNSUPPORTED for every other shape.
int mn_stem_ws_bytes(const mn_conv2d* g, int direction, size_t* bytes) {
  using namespace mn_stem;
  *bytes = 0;
  if (!stem_shape(g)) return MN_EUNSUPPORTED;
  if (direction == MN_CONV_BWD_WEIGHT) {
    if ((long long)g->N * g->P >= (1ll << 30)) return MN_EUNSUPPORTED;
    *bytes = (size_t)wgrad_workgroups(g) * K * (kDepth + 1) * sizeof(float);  // + the bias gradient
    return MN_OK;
  }
  if (direction != MN_CONV_FWD) return MN_EUNSUPPORTED;
  *bytes = (size_t)2 * kSteps * K * sizeof(float);
  return MN_OK;
}

int mn_stem_bwd_weight(const mn_conv2d* g, const float* dy, const float* x, float* dw, float* db,
                       void* ws, size_t ws_bytes, hipStream_t s) {
  using namespace mn_stem;
  size_t need;
  const int st = mn_stem_ws_bytes(g, MN_CONV_BWD_WEIGHT, &need);
  if (st != MN_OK) return st;
  if (g->N == 0 || need == 0) return MN_EUNSUPPORTED;
  if (!ws || ws_bytes < need || !mn_aligned(ws, 16)) return MN_EINVAL;
  const uint32_t grid = wgrad_workgroups(g);
  WGeo q = {g->N, g->H, g->W, g->P, g->Q, (g->P + kRowsOut - 1) / kRowsOut, 0};
  q.items = (uint32_t)g->N * q.row_blocks;
  const bool even8 = (g->Q & 7) == 0 && (g->W & 3) == 0 && mn_aligned(dy, 16) && mn_aligned(x, 16);
  float* const partial = (float*)ws;
  float* const dbp = partial + (size_t)grid * K * kDepth;
  if (even8 && g->Q == 112)
    wgrad_kernel<true, 14><<<grid, kThreads, 0, s>>>(q, x, dy, partial, dbp);
  else if (even8)
    wgrad_kernel<true, 0><<<grid, kThreads, 0, s>>>(q, x, dy, partial, dbp);
  else
    wgrad_kernel<false, 0><<<grid, kThreads, 0, s>>>(q, x, dy, partial, dbp);
  wgrad_reduce_kernel<<<K * kDepth / 16 + (db ? K / 16 : 0), kThreads, 0, s>>>(partial, dbp, dw, db, (int)grid);
  return mn_launch_status();
}

int mn_stem_fwd(const mn_conv2d* g, const float* x, const float* w, const float* bias, float* y,
                void* ws, size_t ws_bytes, hipStream_t s) {
  using namespace mn_stem;
  size_t need;
  const int st = mn_stem_ws_bytes(g, MN_CONV_FWD, &need);
  if (st != MN_OK) return st;
  if (!ws || ws_bytes < need || !mn_aligned(ws, 16)) return MN_EINVAL;
  Geo q = {g->N, g->H, g->W, g->P, g->Q, (g->P + kRowsOut - 1) / kRowsOut};
  const long long blocks = (long long)g->N * q.row_blocks;
  if (blocks == 0) return MN_OK;
  if (blocks >= (1ll << 31)) return MN_EUNSUPPORTED;
  transpose_weights_kernel<<<(2 * kSteps * K + kThreads - 1) / kThreads, kThreads, 0, s>>>(w, (float*)ws);
  if ((g->W & 3) == 0 && mn_aligned(x, 16))
    forward_kernel<true><<<(unsigned)blocks, kThreads, 0, s>>>(q, x, (const float*)ws, bias, y);
  else
    forward_kernel<false><<<(unsigned)blocks, kThreads, 0, s>>>(q, x, (const float*)ws, bias, y);
  return mn_launch_status();
}
