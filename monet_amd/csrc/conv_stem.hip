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
// stages while the other multiplies.
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
      wv[u] = i < 2 * kSteps * K / 4 ? reinterpret_cast<const float4_t*>(wt)[i] : float4_t{0.f, 0.f, 0.f, 0.f};
    }
    const int h_first = 2 * oh0 - 3;
    const bool vec = (g.W & 3) == 0 && (reinterpret_cast<uintptr_t>(x) & 15) == 0;
#pragma unroll
    for (int u = 0; u < kXItems; ++u) {
      const int i = tid + u * kThreads;
      const int row = i / (kRowLen / 4), q = i - row * (kRowLen / 4);
      const int c = row / kRowsIn, h = h_first + row - c * kRowsIn;
      const int wcol = 4 * q - kPadLeft;
      const float* src = x + (((size_t)n * C + c) * g.H + h) * g.W + wcol;
      float4_t v = {0.f, 0.f, 0.f, 0.f};
      if (row < C * kRowsIn && (unsigned)h < (unsigned)g.H) {
        if (vec) {
          if ((unsigned)wcol < (unsigned)g.W) v = *reinterpret_cast<const float4_t*>(src);
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if ((unsigned)(wcol + e) < (unsigned)g.W) v[e] = src[e];
        }
      }
      xv[u] = v;
    }
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
  if (direction != MN_CONV_FWD) return MN_EUNSUPPORTED;
  *bytes = (size_t)2 * kSteps * K * sizeof(float);
  return MN_OK;
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
  forward_kernel<<<(unsigned)blocks, kThreads, 0, s>>>(q, x, (const float*)ws, bias, y);
  return mn_launch_status();
}
