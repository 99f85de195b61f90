// fp32 1x1 (pointwise, stride 1, no padding) convolution on the bf16 matrix cores with fp32
// accuracy: every fp32 operand is cut into three bf16 slices,
//     x = x0 + x1 + x2,  x0 = upper 16 bits of x, x1 = upper 16 bits of (x - x0), x2 likewise
// (a bf16 value is the upper half of an fp32 one, the differences are exact in fp32, and 3 x 8
// significant bits cover the 24 of an fp32 value), and the six slice products of magnitude
// >= 2^-16 of the full product are accumulated in fp32 on v_mfma_f32_32x32x16_bf16:
//     x*w ~ x0 w0 + x0 w1 + x1 w0 + x0 w2 + x1 w1 + x2 w0     (dropped: 2^-24 of the product)
// Six bf16 matrix instructions (32 cycles each, 16 deep) do the work of eight fp32 ones
// (v_mfma_f32_32x32x2_f32: 64 cycles each, 2 deep) in 3/8 of the matrix time, and one set of
// operand fragments feeds six instructions instead of one, so LDS and global traffic per
// matrix cycle are low.  Measured error: 1e-7 .. 6e-7 of the output's largest magnitude (the
// fp32 matrix instruction: 3e-7 .. 5e-7).  Non-finite inputs give NaN (inf - inf in the split).
//
// NCHW fp32 tensors as everywhere in the fp32 path.  The GEMM of one direction is
//     OUT[n][m][p] = sum_r Wm[m][r] * IN[n][r][p]
//   forward        m = k, r = c, Wm = w          backward-data  m = c, r = k, Wm = w^T
// (backward-weight, a reduction over pixels with both operands to split, is not built).
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
// Eight wavefronts with two roles.  Wavefronts 0-3 (one per SIMD) only multiply: CMW of them
// along the output channels (64 each) and 4 / CMW along the pixels (32 TN each), so the tile is
// 64 CMW channels x 128 TN / CMW flat pixels; per 16-deep stage one of them reads 3 x (2 + TN)
// fragments from LDS and issues 12 TN matrix instructions, nothing else.  Wavefronts 4-7 (the
// second one of each SIMD) only feed: they fetch the next stages' weight slices and activations
// into registers (two stages ahead), split the activations and write LDS, double buffered with
// one barrier per stage.  With every wavefront doing both, as workgroups of such kernels usually
// do, the phases of a stage ran one after the other on all of them (a block of loads holds
// back the matrix instructions behind it until the memory path has taken it, about 16 cycles per
// load and CU; after the barrier everybody reads fragments; then everybody stages) and the matrix
// pipe was busy a third of the time.
template <int CMW, int TN>
__global__ __launch_bounds__(kPointThreads) __attribute__((amdgpu_waves_per_eu(2, 2))) void pointwise_kernel(
    const PointH g, const float* __restrict__ in, const bf16_t* __restrict__ wsl,
    const float* __restrict__ bias, float* __restrict__ out) {
  constexpr int CPW = 4 / CMW;                    // multiplying wavefronts along the pixels
  constexpr int BM = 64 * CMW, BP = 32 * TN * CPW;
  constexpr int kFeeders = 256;                   // threads of the feeding wavefronts
  constexpr int kWTotal = 3 * BM * 2;             // 16-byte chunks of a weight stage
  constexpr int kWChunks = (kWTotal + kFeeders - 1) / kFeeders;
  static_assert(BP <= kFeeders, "one activation item (4 rows x 4 pixels) per feeding thread");
  __shared__ __attribute__((aligned(16))) bf16_t lds_w[2][3][BM][LDP];
  __shared__ __attribute__((aligned(16))) bf16_t lds_x[2][3][BP][LDP];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // Persistent workgroups (at most one per CU) take tiles slot, slot + gridDim.x, ...: the
  // feeding wavefronts start on the next tile while the multiplying ones still store the last
  // one.  Tiles are numbered pixel tile by pixel tile, the channel tiles of a pixel tile one
  // after the other (they read the same pixels), and the slot order gives every XCD a contiguous
  // range of them at any time.
  const uint32_t slot = xcd_slot();
  const uint32_t mtiles = (uint32_t)(g.M + BM - 1) / BM;
  const uint32_t tiles = ((g.NP + BP - 1) / BP) * mtiles;
  const int stages = g.R / BKP;

  if (wave >= 4) {
    // ------------------------------------------------------------------ feeding wavefronts
    const int ft = tid - 256;
    const __amdgpu_buffer_rsrc_t in_buf =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(in), 0, g.in_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t w_buf =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(wsl), 0, g.w_bytes, 0x00020000);
    // activation item: pixels 4q..4q+3 (one float4), reduction rows 4h..4h+3 of the stage (four
    // consecutive lanes take four consecutive pixel groups: 64 contiguous bytes per row and load)
    const int h = (ft >> 2) & 3, q = (ft & 3) | ((ft >> 4) << 2);
    const bool loader = 4 * q < BP;
    const bool wave_loads = (wave - 4) * 64 < BP;   // uniform: any loader in this wavefront
    const uint32_t row_bytes = g.HW * 4u;
    uint32_t x_off;             // byte offset of (row 4h of the first stage, pixel 4q); row stride HW*4
    uint32_t w_off[kWChunks];   // weight chunk e = ft + 256 i -> slice e / (2 BM), row (e / 2) % BM, 16-byte chunk e % 2
    // kSets register sets: the loads of a stage are issued kSets stages before it is written to
    // LDS (four sets measured the same as two on every ResNet-50 shape: what bounds the feeding
    // wavefronts is the splitting and the LDS writes, about 1.5 us per 16 KB stage, not latency)
    constexpr int kSets = 2;
    float4_t rx[kSets][4];
    uint4_t rw[kSets][kWChunks];
    // (the scalar offsets are made uniform explicitly: a load whose scalar operand the compiler
    // holds in a vector register is wrapped in a loop over its distinct values)
    auto fetch = [&](float4_t (&rx)[4], uint4_t (&rw)[kWChunks], int t) {  // t uniform
      const int so_w = __builtin_amdgcn_readfirstlane(t * 3 * g.Mpad * BKP * 2);
      const int so_x = __builtin_amdgcn_readfirstlane(t * BKP * (int)row_bytes);
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
        const int e = ft + kFeeders * i;
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
    // The stages of all tiles of this workgroup form one stream: the loads run two stages ahead of
    // the LDS writes across tile boundaries, so a new tile starts without waiting for memory.
    uint32_t ftile = slot;   // tile and stage of the next fetch
    int fstage = 0;
    auto offsets = [&](uint32_t tile) {
      const uint32_t p0 = (tile / mtiles) * BP;
      const int m0 = (int)(tile % mtiles) * BM;
      x_off = kBeyond;
      if (loader) {
        const uint32_t f = p0 + 4 * q;
        const uint32_t n = f / g.HW, p = f - n * g.HW;
        if (f < g.NP) x_off = ((n * (uint32_t)g.R + 4 * h) * g.HW + p) * 4u;
      }
#pragma unroll
      for (int i = 0; i < kWChunks; ++i) {
        const int e = ft + kFeeders * i;
        const int sl = e / (2 * BM), row = (e >> 1) % BM, ch = e & 1;
        w_off[i] = e < kWTotal ? (((uint32_t)sl * g.Mpad + m0 + row) * 16u + ch * 8) * 2u : kBeyond;
      }
    };
    auto fetch_next = [&](float4_t (&rx)[4], uint4_t (&rw)[kWChunks]) {
      if (ftile >= tiles) return;
      fetch(rx, rw, fstage);
      if (++fstage == stages) {
        fstage = 0;
        ftile += gridDim.x;
        if (ftile < tiles) offsets(ftile);
      }
    };
    const uint32_t my_tiles = slot < tiles ? (tiles - slot + gridDim.x - 1) / gridDim.x : 0;
    const uint32_t total = my_tiles * (uint32_t)stages;
    if (total == 0) return;
    offsets(ftile);
    // stream stage s goes into LDS buffer s % 2 while stage s-1 is multiplied
#pragma unroll
    for (int k = 0; k < kSets; ++k) fetch_next(rx[k], rw[k]);
    stage(0, rx[0], rw[0]);
    fetch_next(rx[0], rw[0]);
    __syncthreads();
    for (uint32_t s = 0; s < total; s += kSets) {
#pragma unroll
      for (int u = 0; u < kSets; ++u) {
        if (s + u >= total) break;
        const int k = (u + 1) % kSets;   // register set of stream stage s + u + 1
        if (s + u + 1 < total) stage((u + 1) & 1, rx[k], rw[k]);
        fetch_next(rx[k], rw[k]);
        __syncthreads();
      }
    }
    return;
  }

  // -------------------------------------------------------------------- multiplying wavefronts
  const int wm = wave / CPW, wp = wave % CPW;
  float16_t acc[2][TN];
  auto clear = [&]() {
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
  };
  const int r = lane & 31, kq = (lane >> 5) * 8;
  // (one loop body for both LDS buffers, the buffer is an address offset: two copies of the body
  // with an exit between them made the compiler carry copies of the accumulators and spill)
  const bf16_t* aw = &lds_w[0][0][wm * 64 + r][kq];
  const bf16_t* ax = &lds_x[0][0][wp * TN * 32 + r][kq];
  // Column blocks go in groups of at most three, so that at most 3 x (2 + 3) fragments are live
  auto multiply = [&](int buf) {
    const bf16_t* bw = aw + buf * (3 * BM * LDP);
    const bf16_t* bx = ax + buf * (3 * BP * LDP);
    bf16x8 af[3][2];
#pragma unroll
    for (int sl = 0; sl < 3; ++sl)
#pragma unroll
      for (int i = 0; i < 2; ++i)
        af[sl][i] = *reinterpret_cast<const bf16x8*>(bw + (sl * BM + 32 * i) * LDP);
#pragma unroll
    for (int j0 = 0; j0 < TN; j0 += 3) {
      constexpr int JG = 3;
      bf16x8 bfr[3][JG];
#pragma unroll
      for (int sl = 0; sl < 3; ++sl)
#pragma unroll
        for (int j = 0; j < JG; ++j)
          if (j0 + j < TN)
            bfr[sl][j] = *reinterpret_cast<const bf16x8*>(bx + (sl * BP + 32 * (j0 + j)) * LDP);
      // smallest products first
#pragma unroll
      for (int order = 2; order >= 0; --order)
#pragma unroll
        for (int sa = 0; sa <= order; ++sa)
#pragma unroll
          for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < JG; ++j)
              if (j0 + j < TN)
                acc[i][j0 + j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(bfr[order - sa][j], af[sa][i], acc[i][j0 + j], 0, 0, 0);
    }
  };
  // The pixels are the rows of the matrix instruction and the channels its columns: a lane holds,
  // for ONE output channel, four consecutive pixels in four consecutive registers, i.e. one
  // 16-byte store (with the operands the other way round every register is a store of its own,
  // 16 TN x 2 per wavefront and tile, and the stores of a tile took as long as a third of its
  // matrix work at 256 reduction channels).
  auto store_tile = [&](uint32_t tile) {
    const uint32_t p0 = (tile / mtiles) * BP;
    const int m0 = (int)(tile % mtiles) * BM;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
      const int m = m0 + wm * 64 + 32 * i + (lane & 31);
      if (m >= g.M) continue;
      const float b = bias ? bias[m] : 0.f;
#pragma unroll
      for (int j = 0; j < TN; ++j) {
#pragma unroll
        for (int v4 = 0; v4 < 4; ++v4) {
          const uint32_t f = p0 + (wp * TN + j) * 32 + 8 * v4 + 4 * (lane >> 5);   // 4 pixels of one image
          if (f >= g.NP) continue;
          const uint32_t n = f / g.HW, p = f - n * g.HW;
          float4_t* dst = reinterpret_cast<float4_t*>(out + ((size_t)n * g.M + m) * g.HW + p);
          float4_t val = {acc[i][j][4 * v4] + b, acc[i][j][4 * v4 + 1] + b, acc[i][j][4 * v4 + 2] + b,
                          acc[i][j][4 * v4 + 3] + b};
          if (g.accumulate)
            *dst = *dst + val;
          else
            st_stream(dst, val);
        }
      }
    }
  };
  if (slot >= tiles) return;
  __syncthreads();   // stream stage 0 is in LDS
  int parity = 0;    // LDS buffer of the tile's first stage
  for (uint32_t tile = slot; tile < tiles; tile += gridDim.x) {
    clear();
    for (int t = 0; t < stages; ++t) {
      multiply((t + parity) & 1);
      __syncthreads();
    }
    parity = (parity + stages) & 1;
    store_tile(tile);
  }
}

static bool pointwise_shape(const mn_conv2d* g) {
  return g->R == 1 && g->S == 1 && g->sH == 1 && g->sW == 1 && g->pH == 0 && g->pW == 0 &&
         g->groups == 1;
}

static int pad_rows(int m) { return (m + 255) / 256 * 256; }

// Tile choice: BM = 256 / 128 / 64 by the number of output channels; the pixel extent among the
// instantiated ones by the number of rounds the workgroups (one per CU) make over the CUs times
// the extent, weighted by what the extents measured per unit of work at the ResNet-50 batch-184
// shapes (narrower tiles re-read the weight slices more often).
struct PointTile { int cmw, tn, bm, bp; double weight; };
static PointTile pick_point_tile(int M, uint32_t NP, int cus) {
  static const PointTile wide[] = {{4, 5, 256, 160, 1.0}, {4, 4, 256, 128, 1.05}};
  static const PointTile mid[] = {{2, 4, 128, 256, 1.0}, {2, 3, 128, 192, 1.03}, {2, 2, 128, 128, 1.3}};
  static const PointTile narrow[] = {{1, 2, 64, 256, 1.0}, {1, 1, 64, 128, 1.4}};
  const PointTile* c = M > 128 ? wide : M > 64 ? mid : narrow;
  const int n = M > 128 ? 2 : M > 64 ? 3 : 2;
  PointTile best = c[0];
  double best_cost = 1e30;
  for (int i = 0; i < n; ++i) {
    const long long tiles = (long long)((NP + c[i].bp - 1) / c[i].bp) * ((M + c[i].bm - 1) / c[i].bm);
    const double cost = (double)((tiles + cus - 1) / cus) * c[i].bp * c[i].weight;
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
  if (!ws || ws_bytes < need || !mn_aligned(ws, 16) || !mn_aligned(in, 16) || !mn_aligned(out, 16))
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
  int dev = 0, cus = 256;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
    cus = 256;
  const PointTile t = pick_point_tile(q.M, q.NP, cus);
  const long long ntiles = (long long)((q.NP + t.bp - 1) / t.bp) * ((q.M + t.bm - 1) / t.bm);
  const dim3 grid((unsigned)(ntiles < cus ? ntiles : cus));   // persistent workgroups, one per CU
  const bf16_t* wsl = (const bf16_t*)ws;
#define MN_POINT(CMW, TN) \
  if (t.cmw == CMW && t.tn == TN) pointwise_kernel<CMW, TN><<<grid, kPointThreads, 0, s>>>(q, in, wsl, bias, out)
  MN_POINT(4, 5); MN_POINT(4, 4);
  MN_POINT(2, 4); MN_POINT(2, 3); MN_POINT(2, 2);
  MN_POINT(1, 2); MN_POINT(1, 1);
#undef MN_POINT
  return mn_launch_status();
}
