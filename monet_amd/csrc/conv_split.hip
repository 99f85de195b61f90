// fp32 1x1 (pointwise, stride 1, no padding) convolution on the bf16 matrix cores with fp32
// accuracy: every fp32 operand is cut into three bf16 slices,
//     x = x0 + x1 + x2,  x0 = bf16(x), x1 = bf16(x - x0), x2 = bf16(x - x0 - x1)
// (the differences are exact in fp32, 3 x 8 significant bits cover the 24 of an fp32 value), and
// the six slice products of magnitude >= 2^-16 of the full product are accumulated in fp32 on
// v_mfma_f32_32x32x16_bf16:
//     x*w ~ x0 w0 + x0 w1 + x1 w0 + x0 w2 + x1 w1 + x2 w0     (dropped: 2^-24 of the product)
// Six bf16 matrix instructions (32 cycles each, 16 deep) do the work of eight fp32 ones
// (v_mfma_f32_32x32x2_f32: 64 cycles each, 2 deep) in 3/8 of the matrix time, and one set of
// operand fragments feeds six instructions instead of one, so LDS and global traffic per
// matrix cycle are low.  Non-finite inputs give NaN (inf - inf in the split).
//
// NCHW fp32 tensors as everywhere in the fp32 path.  The GEMM of one direction is
//     OUT[n][m][p] = sum_r Wm[m][r] * IN[n][r][p]
//   forward        m = k, r = c, Wm = w          backward-data  m = c, r = k, Wm = w^T
//   backward-weight dW[k][c] = sum_(n,p) dY[n][k][p] * X[n][c][p]  (reduction over pixels)
// The weight matrix is split once per call by a small kernel into the workspace; activations
// are split on their way into LDS: a thread loads four pixels (one float4) of four reduction rows,
// splits them in registers and stores, per pixel and slice, the four reduction elements as one
// 8-byte LDS write, which is the transposition the matrix instruction needs (a lane feeds it 8
// consecutive reduction elements of one pixel).
#include "common.h"

namespace mn_split {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef uint16_t bf16_t;
typedef uint32_t uint2_t __attribute__((ext_vector_type(2)));

constexpr int kThreads = 256;
constexpr int BK = 32;        // reduction depth of a staged tile
constexpr int LDK = BK + 8;   // LDS row length in elements (80 bytes: conflict-free 16-byte reads)
constexpr uint32_t kBeyond = 0x80000000u;  // byte offset past any buffer (tensors are < 2 GB)

// Three bf16 slices of two fp32 values, packed (low half = first value).  Truncating split:
// slice = upper 16 bits, remainder exact.
__device__ __forceinline__ void split2(float a, float b, uint32_t (&s)[3]) {
  uint32_t ua = __float_as_uint(a), ub = __float_as_uint(b);
#pragma unroll
  for (int i = 0; i < 3; ++i) {
    s[i] = __builtin_amdgcn_perm(ub, ua, 0x07060302u);  // (hi16(b) << 16) | hi16(a)
    if (i < 2) {
      ua = __float_as_uint(__uint_as_float(ua) - __uint_as_float(ua & 0xFFFF0000u));
      ub = __float_as_uint(__uint_as_float(ub) - __uint_as_float(ub & 0xFFFF0000u));
    }
  }
}

// Row of accumulator register v within a 32x32 MFMA tile (column = lane % 32).
__device__ __forceinline__ int acc_row(int v, int lane) {
  return 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
}

// Slices of Wm[m][r] (bf16), laid out by 16-deep stage of the reduction so that what a workgroup
// fetches per stage is contiguous (whole cache lines): ws[((r / 16) * 3 + s) * Mpad + m][r % 16];
// rows m >= M are zero.
// transposed == 0: Wm[m][r] = w[m * R + r]; transposed == 1: Wm[m][r] = w[r * M + m].
__global__ __launch_bounds__(kThreads) void split_weights_kernel(const float* __restrict__ w,
                                                                 bf16_t* __restrict__ ws, int M,
                                                                 int Mpad, int R, int transposed) {
  const size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x;  // pair of r
  const size_t pairs = (size_t)Mpad * R / 2;
  if (i >= pairs) return;
  const int m = (int)(i / (R / 2)), r = (int)(i % (R / 2)) * 2;
  float a = 0.f, b = 0.f;
  if (m < M) {
    a = transposed ? w[(size_t)r * M + m] : w[(size_t)m * R + r];
    b = transposed ? w[(size_t)(r + 1) * M + m] : w[(size_t)m * R + r + 1];
  }
  uint32_t s[3];
  split2(a, b, s);
#pragma unroll
  for (int k = 0; k < 3; ++k)
    reinterpret_cast<uint32_t*>(ws)[((((size_t)(r / 16) * 3 + k) * Mpad + m) * 16 + r % 16) / 2] = s[k];
}

struct PointH {
  uint32_t NP, HW;        // flat pixels N*HW, pixels per image
  int M, Mpad, R;         // output channels (padded to 256), reduction length
  uint32_t in_bytes, w_bytes;
  int accumulate;         // OUT += result
};

constexpr int kPointThreads = 512;
constexpr int BKP = 16;        // reduction depth of a staged tile (one matrix step)
constexpr int LDP = BKP + 8;   // LDS row: 48 bytes (3 x 16: 16 consecutive rows hit 16 different 16-byte slots)

// OUT[n][m][p] (+= or =) sum_r Wm[m][r] IN[n][r][p] (+ bias[m]).
// 8 wavefronts, WMB of them along the output channels (32 each) and 8 / WMB along the pixels
// (32 * TN each): tile = 32 WMB channels x 256 TN / WMB flat pixels, 16 deep per stage, LDS double
// buffered with one barrier per stage.  What bounds this kernel is the L2 -> CU traffic (about
// 10 TB/s over the whole device), so tiles are as large as LDS and registers allow: per stage a
// workgroup fetches 3 x 2 x BM x 16 bytes of weight slices and 4 x BP x 16 bytes of activations.
template <int WMB, int TN>
__global__ __launch_bounds__(kPointThreads) __attribute__((amdgpu_waves_per_eu(2, 2))) void pointwise_kernel(
    const PointH g, const float* __restrict__ in, const bf16_t* __restrict__ wsl,
    const float* __restrict__ bias, float* __restrict__ out) {
  constexpr int WPB = 8 / WMB;
  constexpr int BM = 32 * WMB, BP = 32 * TN * WPB;
  constexpr int kWTotal = 3 * BM * 2;                                  // 16-byte chunks of a weight stage
  constexpr int kWChunks = (kWTotal + kPointThreads - 1) / kPointThreads;
  __shared__ __attribute__((aligned(16))) bf16_t lds_w[2][3][BM][LDP];
  __shared__ __attribute__((aligned(16))) bf16_t lds_x[2][3][BP][LDP];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / WPB, wp = wave % WPB;
  // XCD-aware order: contiguous ranges of pixel tiles per XCD, the channel tiles of a pixel tile
  // one after the other (they read the same pixels)
  const uint32_t slot = xcd_slot();
  const uint32_t bx = slot / gridDim.y, by = slot - bx * gridDim.y;
  const uint32_t p0 = bx * BP;
  const int m0 = by * BM;

  const __amdgpu_buffer_rsrc_t in_buf =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(in), 0, g.in_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t w_buf =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(wsl), 0, g.w_bytes, 0x00020000);
  // activation loader: pixels 4q..4q+3 (one float4), reduction rows 4h..4h+3 of the stage
  // (four consecutive lanes take four consecutive pixel groups: 64 contiguous bytes per row and
  // load, which is what the address coalescer merges; one row per lane costs it a cycle per lane)
  const int h = (tid >> 2) & 3, q = (tid & 3) | ((tid >> 4) << 2);
  const bool loader = 4 * q < BP;
  const bool wave_loads = __builtin_amdgcn_readfirstlane(wave) * 64 < BP;   // uniform: any loader in this wavefront
  uint32_t x_off = kBeyond;   // byte offset of (row 4h of the first stage, pixel 4q); row stride HW*4
  if (loader) {
    const uint32_t f = p0 + 4 * q;
    const uint32_t n = f / g.HW, p = f - n * g.HW;
    if (f < g.NP) x_off = ((n * (uint32_t)g.R + 4 * h) * g.HW + p) * 4u;
  }
  const uint32_t row_bytes = g.HW * 4u;
  // weight loader: chunk e = tid + 512 i -> slice e / (2 BM), row (e / 2) % BM, 16-byte chunk e % 2
  uint32_t w_off[kWChunks];
#pragma unroll
  for (int i = 0; i < kWChunks; ++i) {
    const int e = tid + kPointThreads * i;
    const int sl = e / (2 * BM), row = (e >> 1) % BM, ch = e & 1;
    w_off[i] = e < kWTotal ? (((uint32_t)sl * g.Mpad + m0 + row) * 16u + ch * 8) * 2u : kBeyond;
  }
  // Loads complete in issue order and every stage issues the same loads, so two register sets
  // keep the loads of stage t+2 in flight while stage t is multiplied and stage t+1 is staged.
  float4_t rx0[4], rx1[4];
  uint4_t rw0[kWChunks], rw1[kWChunks];
  // (the scalar offsets are made uniform explicitly: a load whose scalar operand the compiler
  // holds in a vector register is wrapped in a loop over its distinct values, which also stops
  // the scheduler from moving anything across it; threads that load no pixels point beyond the
  // buffer instead of branching around the loads)
  auto fetch = [&](float4_t (&rx)[4], uint4_t (&rw)[kWChunks], int r0) {  // r0 uniform
    const int so_w = __builtin_amdgcn_readfirstlane((r0 / BKP) * 3 * g.Mpad * BKP * 2);
    const int so_x = __builtin_amdgcn_readfirstlane(r0 * (int)row_bytes);
#pragma unroll
    for (int i = 0; i < kWChunks; ++i)
      rw[i] = __builtin_amdgcn_raw_buffer_load_b128(w_buf, w_off[i], so_w, 0);
    if (wave_loads) {
#pragma unroll
      for (int j = 0; j < 4; ++j)
        rx[j] = __builtin_bit_cast(float4_t, __builtin_amdgcn_raw_buffer_load_b128(
                                                 in_buf, x_off + j * row_bytes, so_x, 0));
    }
  };
  auto stage = [&](int buf, const float4_t (&rx)[4], const uint4_t (&rw)[kWChunks]) {
#pragma unroll
    for (int i = 0; i < kWChunks; ++i) {
      const int e = tid + kPointThreads * i;
      const int sl = e / (2 * BM), row = (e >> 1) % BM, ch = e & 1;
      if (e < kWTotal) *reinterpret_cast<uint4_t*>(&lds_w[buf][sl][row][ch * 8]) = rw[i];
    }
    if (loader) {
      // pixel pp of this thread: reduction elements 4h..4h+3 as two packed pairs per slice
#pragma unroll
      for (int pp = 0; pp < 4; ++pp) {
        uint32_t lo[3], hi[3];
        split2(rx[0][pp], rx[1][pp], lo);
        split2(rx[2][pp], rx[3][pp], hi);
#pragma unroll
        for (int sl = 0; sl < 3; ++sl)
          *reinterpret_cast<uint2_t*>(&lds_x[buf][sl][4 * q + pp][4 * h]) = uint2_t{lo[sl], hi[sl]};
      }
    }
  };

  float16_t acc[TN];
#pragma unroll
  for (int j = 0; j < TN; ++j)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[j][v] = 0.f;

  const int r = lane & 31, kq = (lane >> 5) * 8;
  // column blocks in groups of at most three: their 9 pixel fragments are live together with the
  // 3 weight fragments (all 3 TN at once do not fit the register file at TN = 5, 6)
  auto multiply = [&](int buf) {
    bf16x8 af[3];
#pragma unroll
    for (int sl = 0; sl < 3; ++sl)
      af[sl] = *reinterpret_cast<const bf16x8*>(&lds_w[buf][sl][wm * 32 + r][kq]);
#pragma unroll
    for (int j0 = 0; j0 < TN; j0 += 3) {
      constexpr int JG = 3;
      bf16x8 bfr[3][JG];
#pragma unroll
      for (int sl = 0; sl < 3; ++sl)
#pragma unroll
        for (int j = 0; j < JG; ++j)
          if (j0 + j < TN)
            bfr[sl][j] = *reinterpret_cast<const bf16x8*>(&lds_x[buf][sl][(wp * TN + j0 + j) * 32 + r][kq]);
      // smallest products first
#pragma unroll
      for (int order = 2; order >= 0; --order)
#pragma unroll
        for (int sa = 0; sa <= order; ++sa)
#pragma unroll
          for (int j = 0; j < JG; ++j)
            if (j0 + j < TN)
              acc[j0 + j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[sa], bfr[order - sa][j], acc[j0 + j], 0, 0, 0);
    }
  };
  const int stages = g.R / BKP;
  fetch(rx0, rw0, 0);
  if (stages > 1) fetch(rx1, rw1, BKP);
  stage(0, rx0, rw0);
  __syncthreads();
  for (int t = 0; t < stages; t += 2) {
    // stage t is in LDS buffer 0, stage t+1 in flight in set 1
    if (t + 2 < stages) fetch(rx0, rw0, (t + 2) * BKP);
    multiply(0);
    if (t + 1 >= stages) break;
    stage(1, rx1, rw1);
    __syncthreads();
    // stage t+1 is in LDS buffer 1, stage t+2 in flight in set 0
    if (t + 3 < stages) fetch(rx1, rw1, (t + 3) * BKP);
    multiply(1);
    if (t + 2 < stages) stage(0, rx0, rw0);
    __syncthreads();
  }

  // epilogue: for a fixed register, lanes 0..31 hold 32 consecutive pixels of one output channel
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const uint32_t f = p0 + (wp * TN + j) * 32 + (lane & 31);
    if (f >= g.NP) continue;
    const uint32_t n = f / g.HW, p = f - n * g.HW;
    float* o = out + (size_t)n * g.M * g.HW + p;
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int m = m0 + wm * 32 + acc_row(v, lane);
      if (m >= g.M) continue;
      float val = acc[j][v];
      if (bias) val += bias[m];
      float* dst = o + (size_t)m * g.HW;
      if (g.accumulate)
        *dst += val;
      else
        st_stream(dst, val);
    }
  }
}

static bool pointwise_shape(const mn_conv2d* g) {
  return g->R == 1 && g->S == 1 && g->sH == 1 && g->sW == 1 && g->pH == 0 && g->pW == 0 &&
         g->groups == 1;
}

static int pad_rows(int m) { return (m + 255) / 256 * 256; }

// Tile choice: BM = 256 / 128 / 64 by the number of output channels; the pixel extent among
// the instantiated ones by the number of rounds the workgroups (one per CU at a time) make over
// the 256 CUs times the extent, weighted by what the extents measured per unit of work at the
// ResNet-50 batch-184 shapes (narrower tiles re-read the weight slices more often; the 160-pixel
// tile of the 256-channel kernel only pays where it saves a round).
struct PointTile { int wmb, tn, bm, bp; double weight; };
static PointTile pick_point_tile(int M, uint32_t NP) {
  static const PointTile wide[] = {{8, 4, 256, 128, 1.0}, {8, 5, 256, 160, 1.1}};
  static const PointTile mid[] = {{4, 4, 128, 256, 1.0}, {4, 3, 128, 192, 1.05}, {4, 2, 128, 128, 1.3}};
  static const PointTile narrow[] = {{2, 2, 64, 256, 1.0}, {2, 1, 64, 128, 1.3}};
  const PointTile* c = M > 128 ? wide : M > 64 ? mid : narrow;
  const int n = M > 128 ? 2 : M > 64 ? 3 : 2;
  PointTile best = c[0];
  double best_cost = 1e30;
  for (int i = 0; i < n; ++i) {
    const long long tiles = (long long)((NP + c[i].bp - 1) / c[i].bp) * ((M + c[i].bm - 1) / c[i].bm);
    const double cost = (double)((tiles + 255) / 256) * c[i].bp * c[i].weight;
    if (cost < best_cost) {
      best_cost = cost;
      best = c[i];
    }
  }
  return best;
}

}  // namespace mn_split

// Entry points used by the variant dispatch in conv.hip -----------------------------------

// Workspace: the three bf16 slices of the weight matrix, rows padded to the tile.
int mn_split_ws_bytes(const mn_conv2d* g, int direction, size_t* bytes) {
  using namespace mn_split;
  *bytes = 0;
  if (!pointwise_shape(g)) return MN_EUNSUPPORTED;
  const long long hw = (long long)g->H * g->W;
  if (hw % 4 != 0) return MN_EUNSUPPORTED;
  if (direction == MN_CONV_BWD_WEIGHT) return MN_EUNSUPPORTED;
  const int M = direction == MN_CONV_FWD ? g->K : g->C, R = direction == MN_CONV_FWD ? g->C : g->K;
  if (R % BKP != 0) return MN_EUNSUPPORTED;
  // 32-bit byte offsets through buffer descriptors
  if ((long long)g->N * g->C * hw * 4 >= (1ll << 31) || (long long)g->N * g->K * hw * 4 >= (1ll << 31))
    return MN_EUNSUPPORTED;
  *bytes = (size_t)3 * pad_rows(M) * R * sizeof(bf16_t);
  return MN_OK;
}

// direction: MN_CONV_FWD (in = x, out = y) or MN_CONV_BWD_DATA (in = dy, out = dx)
int mn_split_pointwise(const mn_conv2d* g, int direction, const float* in, const float* w,
                       const float* bias, float* out, bool accumulate, void* ws, size_t ws_bytes,
                       hipStream_t s) {
  using namespace mn_split;
  size_t need;
  const int st = mn_split_ws_bytes(g, direction, &need);
  if (st != MN_OK) return st;
  if (!ws || ws_bytes < need || !mn_aligned(ws, 16) || !mn_aligned(in, 16) || !mn_aligned(out, 4))
    return MN_EINVAL;
  PointH q = {};
  q.HW = (uint32_t)(g->H * g->W);
  q.NP = (uint32_t)((long long)g->N * q.HW);
  q.M = direction == MN_CONV_FWD ? g->K : g->C;
  q.R = direction == MN_CONV_FWD ? g->C : g->K;
  q.Mpad = pad_rows(q.M);
  q.in_bytes = (uint32_t)((unsigned long long)q.NP * q.R * 4ull);
  q.w_bytes = (uint32_t)need;
  q.accumulate = accumulate ? 1 : 0;
  if (q.NP == 0) return MN_OK;
  const size_t pairs = (size_t)q.Mpad * q.R / 2;
  split_weights_kernel<<<(unsigned)((pairs + kThreads - 1) / kThreads), kThreads, 0, s>>>(
      w, (bf16_t*)ws, q.M, q.Mpad, q.R, direction == MN_CONV_BWD_DATA ? 1 : 0);
  const PointTile t = pick_point_tile(q.M, q.NP);
  dim3 grid((q.NP + t.bp - 1) / t.bp, (q.M + t.bm - 1) / t.bm);
  const bf16_t* wsl = (const bf16_t*)ws;
#define MN_POINT(WMB, TN) \
  if (t.wmb == WMB && t.tn == TN) pointwise_kernel<WMB, TN><<<grid, kPointThreads, 0, s>>>(q, in, wsl, bias, out)
  MN_POINT(8, 5); MN_POINT(8, 4);
  MN_POINT(4, 4); MN_POINT(4, 3); MN_POINT(4, 2);
  MN_POINT(2, 2); MN_POINT(2, 1);
#undef MN_POINT
  return mn_launch_status();
}
