// 2-D convolution on bf16 tensors with fp32 accumulation on the gfx950 matrix
// cores (v_mfma_f32_32x32x16_bf16).
//
// Layout: channels-last.  Activations [N, H, W, C], weights [K, R, S, C],
// outputs [N, P, Q, K] (what torch calls memory_format=channels_last for a
// logically NCHW tensor).  With the channel innermost, the reduction index of
// the implicit GEMM is contiguous in memory for BOTH operands of forward and
// backward-data, which is what the matrix instruction wants: every lane feeds
// it 8 consecutive reduction elements (16 bytes) per operand, so operand tiles
// go global -> LDS -> registers as 16-byte vectors with no transposition, and
// a window shift moves addresses by whole pixels (multiples of 2*C bytes), so
// taps never break the 16-byte alignment.
//
//   forward        D[pix][k] = sum_(tap, c) X[pix @ tap][c] * W[k][tap][c]
//   backward-data  D[pix][c] = sum_(tap, k) dY[pix @ tap][k] * W'[c][tap][k]
//                  (W' = weights transposed into the workspace; stride > 1 is
//                  split by parity class like the fp32 path)
//   backward-weight dW[k][tap][c] = sum_pix dY[pix][k] * X[pix @ tap][c]
//                  Here the reduction (pixels) is the STRIDED index, so the
//                  16-byte chunks (8 channels of one pixel) are transposed on
//                  their way into LDS (lane-pair exchange + dword stores) to
//                  put pixels innermost.  The
//                  reduction is split across workgroups; partial sums are fp32
//                  in the workspace and a second kernel adds them in a fixed
//                  order and rounds once to bf16.
//
// Workgroup = 4 wavefronts (2 x 2); tile 128 rows x BN columns x 32 deep,
// double buffered in LDS with rows padded to 80 bytes (conflict-free 16-byte
// reads).  Channel counts must be multiples of 32 (reduction side) or 64
// (backward-weight columns).
#include "common.h"

namespace mn_conv16 {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));
typedef uint16_t bf16_t;  // storage type

constexpr int kThreads = 256;
constexpr int BM = 128;     // rows of a workgroup tile (gather kernels)
constexpr int BK = 32;      // reduction depth of a staged tile
constexpr int LDK = BK + 8; // LDS row length in elements (80 bytes)
constexpr int kMaxTaps = 49;
constexpr uint32_t kNoRow = 0xFFFFFFFFu;

__device__ __forceinline__ bf16_t f2bf(float f) {
  uint32_t u = __float_as_uint(f);
  if ((u & 0x7FFFFFFFu) > 0x7F800000u) return (bf16_t)((u >> 16) | 0x40u);  // quiet NaN
  u += 0x7FFFu + ((u >> 16) & 1u);  // round to nearest even
  return (bf16_t)(u >> 16);
}
__device__ __forceinline__ float bf2f(bf16_t h) { return __uint_as_float((uint32_t)h << 16); }

// Row of accumulator register v within a 32x32 MFMA tile (column = lane % 32).
__device__ __forceinline__ int acc_row(int v, int lane) {
  return 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
}

// acc[i][j] += A rows (wm-th half) x B rows (wn-th half), both staged [row][k].
template <int TM, int TN, int ROWS_A, int ROWS_B, int DEPTH = BK>
__device__ __forceinline__ void mma_tile(const bf16_t (*As)[DEPTH + 8], const bf16_t (*Bs)[DEPTH + 8],
                                         int wm, int wn, int lane, float16_t (&acc)[TM][TN]) {
  const int r = lane & 31, kq = (lane >> 5) * 8;
#pragma unroll
  for (int ks = 0; ks < DEPTH; ks += 16) {
    bf16x8 af[TM], bfr[TN];
#pragma unroll
    for (int i = 0; i < TM; ++i)
      af[i] = *reinterpret_cast<const bf16x8*>(&As[wm * (ROWS_A / 2) + 32 * i + r][ks + kq]);
#pragma unroll
    for (int j = 0; j < TN; ++j)
      bfr[j] = *reinterpret_cast<const bf16x8*>(&Bs[wn * (ROWS_B / 2) + 32 * j + r][ks + kq]);
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bfr[j], acc[i][j], 0, 0, 0);
  }
}

// ---------------------------------------------------- forward / backward-data
struct GatherH {
  uint32_t npix;          // rows of this launch = N * OH * OW
  int OH, OW;
  int Nout;               // columns = channels of dst
  int Cs, Hs, Ws;         // source [N, Hs, Ws, Cs]
  int ish, isw;           // source position = oh*ish + dh[tap]
  int DH, DW, osh, osw, oh0, ow0;  // dst [N, DH, DW, Nout], position = oh*osh + oh0
  int T;                  // taps of this launch
  uint32_t wrow;          // elements between consecutive weight rows
  uint32_t wstep;         // bytes between consecutive 16-deep steps of the weight operand: 32 for
                          // rows in place, 1024 for the fragment-packed layout
  uint32_t src_bytes, w_bytes;  // sizes of the two operand tensors (set by the launcher)
  int16_t dh[kMaxTaps], dw[kMaxTaps];
  int32_t woff[kMaxTaps]; // element offset of tap t inside a weight row
};

// The channel operand (weights) never passes through LDS: every wavefront loads the fragments
// of its own 32-channel blocks straight from global memory into the registers the matrix
// instruction reads (a lane's fragment is 16 contiguous bytes of one weight row), one
// 64-deep tile ahead of their use.  Only the pixel operand (gathered rows, shared by the
// wavefronts of a workgroup row) is staged in LDS.  That halves the LDS traffic per matrix
// instruction, which is what bounded a kernel that staged both operands (a 128 x 128 x 32
// tile is 8 instructions = 256 cycles per wavefront, and read 32 KB + wrote 16 KB of LDS).
// The weights come in one of two layouts, told apart by `wstep`:
//  * in place ([rows][reduction], wstep = 32): a fragment load touches 32 rows, 32 bytes each;
//  * packed ([32-row block][16-deep step][lane], wstep = 1024): a fragment is 1 KB contiguous.
// Everything else a wavefront issues per tile is kept small:
//  * the pixel operand is fetched with raw buffer loads: the per-thread byte offset of a row is
//    fixed for a whole tap (a row outside the window or the tensor gets an offset beyond the
//    buffer and reads as zero: no masks when staging), the per-tile part (channel offset) is the
//    scalar offset of the instruction: no vector arithmetic per tile;
//  * two register sets: the loads of tile t+2 are issued before tile t is multiplied and
//    are staged during tile t+1.
template <int BN, int DEPTH>
__global__ __launch_bounds__(kThreads) void gather_bf16_kernel(const GatherH g,
                                                               const bf16_t* __restrict__ src,
                                                               const bf16_t* __restrict__ w,
                                                               const bf16_t* __restrict__ bias,
                                                               bf16_t* __restrict__ dst) {
  constexpr int TN = BN / 64;                 // MFMA tiles per wavefront along the columns
  constexpr int KS = DEPTH / 16;              // matrix steps per staged tile
  constexpr int kCPR = DEPTH / 8;             // 16-byte chunks per staged row
  constexpr int kRPP = kThreads / kCPR;       // rows covered by one pass of the workgroup
  constexpr int kARows = BM / kRPP;           // chunks per thread
  constexpr int LDR = DEPTH + 8;              // LDS row length (elements): 80 or 144 bytes
  constexpr uint32_t kBeyond = 0x80000000u;   // byte offset past any buffer (tensors are < 2 GB)
  __shared__ __attribute__((aligned(16))) bf16_t lds_a[2][BM][LDR];
  __shared__ int tdh[kMaxTaps], tdw[kMaxTaps], twoff[kMaxTaps];
  __shared__ uint32_t row_dst[BM];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  // XCD-aware order: contiguous ranges of position tiles per XCD, the channel tiles of a
  // position tile one after the other (they gather the same pixels)
  const uint32_t slot = xcd_slot();
  const uint32_t bx = slot / gridDim.y, by = slot - bx * gridDim.y;
  const uint32_t p0 = bx * BM;
  const int n0 = by * BN;
  const uint32_t plane = (uint32_t)g.OH * g.OW;
  if (tid < g.T) {
    tdh[tid] = g.dh[tid];
    tdw[tid] = g.dw[tid];
    twoff[tid] = g.woff[tid];
  }
  if (tid < BM) {
    const uint32_t pix = p0 + tid;
    uint32_t off = kNoRow;
    if (pix < g.npix) {
      const uint32_t n = pix / plane, rem = pix - n * plane;
      const uint32_t oh = rem / g.OW, ow = rem - oh * g.OW;
      off = ((n * g.DH + oh * g.osh + g.oh0) * (uint32_t)g.DW + ow * g.osw + g.ow0) * (uint32_t)g.Nout;
    }
    row_dst[tid] = off;
  }
  // A loader: 16-byte chunk `chunk` of rows arow + kRPP*i
  const int chunk = tid % kCPR, arow = tid / kCPR;
  int ohs[kARows], ows[kARows];
  uint32_t abase[kARows];
  bool aok[kARows];
#pragma unroll
  for (int i = 0; i < kARows; ++i) {
    const uint32_t pix = p0 + arow + kRPP * i;
    aok[i] = pix < g.npix;
    const uint32_t pp = aok[i] ? pix : 0u;
    const uint32_t n = pp / plane, rem = pp - n * plane;
    const uint32_t oh = rem / g.OW, ow = rem - oh * g.OW;
    ohs[i] = oh * g.ish;
    ows[i] = ow * g.isw;
    abase[i] = n * (uint32_t)g.Hs * g.Ws;
  }
  // weight fragments of this wavefront's column blocks: per-lane byte offset, fixed for the launch
  uint32_t b_off[TN];
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int blk = (n0 + wn * (BN / 2) + 32 * j) / 32;   // 32-row block of the weight operand
    const int col = blk * 32 + (lane & 31);
    if (g.wstep == 1024)
      b_off[j] = ((uint32_t)blk * (g.wrow / 16) * 64 + lane) * 16u;
    else
      b_off[j] = col < g.Nout ? ((uint32_t)col * g.wrow + (lane >> 5) * 8) * 2u : kBeyond;
  }
  __syncthreads();

  const __amdgpu_buffer_rsrc_t src_buf =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(src), 0, g.src_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t w_buf =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(w), 0, g.w_bytes, 0x00020000);
  // per-tap state: byte offsets of this thread's rows of the source (or kBeyond)
  uint32_t a_off[kARows];
  auto enter_tap = [&](int t) {  // t uniform
    const int dh = tdh[t], dw = tdw[t];
#pragma unroll
    for (int i = 0; i < kARows; ++i) {
      const int hh = ohs[i] + dh, ww = ows[i] + dw;
      const bool ok = aok[i] && (unsigned)hh < (unsigned)g.Hs && (unsigned)ww < (unsigned)g.Ws;
      a_off[i] = ok ? ((abase[i] + hh * g.Ws + ww) * (uint32_t)g.Cs + chunk * 8) * 2u : kBeyond;
    }
  };
  auto fetch = [&](uint4_t (&ra)[kARows], int c0) {  // c0 uniform
#pragma unroll
    for (int i = 0; i < kARows; ++i)
      ra[i] = __builtin_amdgcn_raw_buffer_load_b128(src_buf, a_off[i], c0 * 2, 0);
  };
  auto stage = [&](int buf, const uint4_t (&ra)[kARows]) {
#pragma unroll
    for (int i = 0; i < kARows; ++i)
      *reinterpret_cast<uint4_t*>(&lds_a[buf][arow + kRPP * i][chunk * 8]) = ra[i];
  };

  float16_t acc[2][TN];
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  const int per_tap = g.Cs / DEPTH;
  const int ktiles = g.T * per_tap;
  if (ktiles > 0) {
    uint4_t ra0[kARows], ra1[kARows];
    // weight fragments of the two tiles in flight: set b holds the tile that LDS buffer b holds;
    // a step's fragments are reloaded with those of the tile after next as soon as it is done.
    // Loads complete in issue order, so every operand is fetched the same distance (two tiles)
    // ahead: a deeper prefetch of one operand would only make the waits for the other longer
    uint4_t bq[2][KS][TN];
    int t = 0, c0 = 0;    // position of the next pixel tile to fetch
    int tb = 0, cb = 0;   // position of the next weight tile to fetch
    enter_tap(0);
    auto advance = [&]() {
      c0 += DEPTH;
      if (c0 == g.Cs) {
        c0 = 0;
        ++t;
        if (t < g.T) enter_tap(t);
      }
    };
    // uniform byte offset of weight tile (tb, cb), then move to the next tile (the last tile is
    // loaded again instead of branching around the loads)
    auto wtile = [&]() {
      const uint32_t k16 = (uint32_t)(__builtin_amdgcn_readfirstlane(twoff[tb]) + cb) / 16u;
      if (tb * per_tap * DEPTH + cb + DEPTH < ktiles * DEPTH) {
        cb += DEPTH;
        if (cb == g.Cs) {
          cb = 0;
          ++tb;
        }
      }
      return k16 * g.wstep;
    };
    auto wfetch = [&](uint4_t (&b)[KS][TN], uint32_t woff) {
#pragma unroll
      for (int s = 0; s < KS; ++s)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          b[s][j] = __builtin_amdgcn_raw_buffer_load_b128(w_buf, b_off[j], woff + s * g.wstep, 0);
    };
    auto mma_tile = [&](int buf, uint4_t (&b)[KS][TN], uint32_t wnext) {
      const int r = lane & 31, kq = (lane >> 5) * 8;
#pragma unroll
      for (int s = 0; s < KS; ++s) {
        bf16x8 af[2];
#pragma unroll
        for (int i = 0; i < 2; ++i)
          af[i] = *reinterpret_cast<const bf16x8*>(&lds_a[buf][wm * 64 + 32 * i + r][s * 16 + kq]);
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          const bf16x8 bfr = __builtin_bit_cast(bf16x8, b[s][j]);
#pragma unroll
          for (int i = 0; i < 2; ++i)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bfr, acc[i][j], 0, 0, 0);
          b[s][j] = __builtin_amdgcn_raw_buffer_load_b128(w_buf, b_off[j], wnext + s * g.wstep, 0);
        }
      }
    };
    wfetch(bq[0], wtile());   // tile 0
    fetch(ra0, c0);
    advance();
    wfetch(bq[1], wtile());   // tile 1 (tile 0 again if there is only one)
    if (ktiles > 1) {
      fetch(ra1, c0);
      advance();
    }
    stage(0, ra0);
    __syncthreads();
    for (int kt = 0; kt + 1 < ktiles; kt += 2) {
      // tile kt is in LDS buffer 0, tile kt+1 in flight in set 1
      if (kt + 2 < ktiles) {
        fetch(ra0, c0);
        advance();
      }
      mma_tile(0, bq[0], wtile());
      stage(1, ra1);
      __syncthreads();
      // tile kt+1 is in LDS buffer 1, tile kt+2 in flight in set 0
      if (kt + 3 < ktiles) {
        fetch(ra1, c0);
        advance();
      }
      mma_tile(1, bq[1], wtile());
      if (kt + 2 < ktiles) stage(0, ra0);
      __syncthreads();
    }
    // an odd number of tiles: the last one was staged into buffer 0
    if (ktiles & 1) mma_tile(0, bq[0], wtile());
  }

  // epilogue: for a fixed register, lanes 0..31 hold 32 consecutive channels of one position
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const int col = n0 + wn * (BN / 2) + 32 * j + (lane & 31);
    if (col >= g.Nout) continue;
    const float b = bias ? bf2f(bias[col]) : 0.f;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const uint32_t off = row_dst[wm * 64 + 32 * i + acc_row(v, lane)];
        if (off != kNoRow) dst[off + col] = f2bf(acc[i][j][v] + b);
      }
    }
  }
}

// The large-tile form of the same gather GEMM: 64 CMW output channels x 128 TN / CMW positions x 64
// deep per stage, eight wavefronts with two roles.  Wavefronts 0-3 (one per SIMD) only multiply:
// CMW of them along the channels (64 each), 4 / CMW along the positions (32 TN each, 2 x TN
// accumulator tiles); per stage one reads 4 x (2 + TN) fragments from LDS for 8 TN matrix
// instructions.  Wavefronts 4-7 (the second one of each
// SIMD) only feed: they fetch the next stages' weight rows and gathered pixel rows into
// registers two stages ahead and write them to LDS, double buffered, one barrier per stage.
// With every wavefront doing both (the 128 x 128 kernel above) the phases of a stage run one
// after the other on all of them, and what a CU pulls through its vector memory path per matrix
// instruction is twice as much: 0.54 PFLOP/s at the ResNet-50 layer3 shape against the
// 2.5 PFLOP/s peak.  Workgroups are persistent (at most one per CU) and walk the tile list.
// Needs Cs % 64 == 0 and Nout % 64 == 0.  PACKED = weights in fragment order (wstep == 1024): the
// multiplying wavefronts load their weight fragments straight into registers, so LDS only carries
// the pixel rows (a stage moves 52 KB in and 112 KB out of LDS otherwise, as many LDS cycles as
// the stage has matrix cycles).
constexpr int kRoleThreads = 512;
constexpr int kRoleDepth = 64;
constexpr int kRoleLd = kRoleDepth + 8;   // LDS row: 144 bytes (9 x 16: conflict-free 16-byte reads)

template <int CMW, int TN, bool PACKED>
__global__ __launch_bounds__(kRoleThreads) __attribute__((amdgpu_waves_per_eu(2, 2))) void gather_roles_kernel(
    const GatherH g, const bf16_t* __restrict__ src, const bf16_t* __restrict__ w,
    const bf16_t* __restrict__ bias, bf16_t* __restrict__ dst) {
  constexpr int CPW = 4 / CMW;
  constexpr int BMW = 64 * CMW, BP = 32 * TN * CPW;
  static_assert(BP <= 256, "one row of the position table per multiplying thread");
  constexpr int kFeeders = 256;
  constexpr int kWChunks = BMW * (kRoleDepth / 8) / kFeeders;
  constexpr int kXChunks = (BP * (kRoleDepth / 8) + kFeeders - 1) / kFeeders;
  constexpr uint32_t kBeyond = 0x80000000u;   // byte offset past any buffer (tensors are < 2 GB)
  __shared__ __attribute__((aligned(16))) bf16_t lds_w[PACKED ? 1 : 2][PACKED ? 1 : BMW][kRoleLd];
  __shared__ __attribute__((aligned(16))) bf16_t lds_x[2][BP][kRoleLd];
  __shared__ int tdh[kMaxTaps], tdw[kMaxTaps], twoff[kMaxTaps];
  __shared__ uint32_t row_dst[2][BP];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const uint32_t slot = xcd_slot();
  const uint32_t ntiles_n = ((uint32_t)g.Nout + BMW - 1) / BMW;
  const uint32_t tiles = ((g.npix + BP - 1) / BP) * ntiles_n;
  const uint32_t plane = (uint32_t)g.OH * g.OW;
  const int per_tap = g.Cs / kRoleDepth;
  const int stages = g.T * per_tap;
  if (tid < g.T) {
    tdh[tid] = g.dh[tid];
    tdw[tid] = g.dw[tid];
    twoff[tid] = g.woff[tid];
  }
  __syncthreads();

  if (wave >= 4) {
    // ------------------------------------------------------------------ feeding wavefronts
    const int ft = tid - 256;
    const __amdgpu_buffer_rsrc_t src_buf =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(src), 0, g.src_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t w_buf =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(w), 0, g.w_bytes, 0x00020000);
    // chunk e = ft + 256 i of an operand tile: row e / 8, 16-byte chunk e % 8 (a row's 128 bytes
    // are contiguous in memory and across 8 lanes)
    const int ch = ft & 7, row0 = ft >> 3;
    uint32_t w_off[kWChunks];
    int ohs[kXChunks], ows[kXChunks];
    uint32_t abase[kXChunks];
    bool aok[kXChunks];
    uint32_t a_off[kXChunks];
    constexpr int kSets = 4;   // register sets = stages the loads run ahead of the LDS writes
    uint4_t rw[kSets][kWChunks], rx[kSets][kXChunks];
    for (uint32_t tile = slot; tile < tiles; tile += gridDim.x) {
      const uint32_t p0 = (tile / ntiles_n) * BP;
      const int n0 = (int)(tile % ntiles_n) * BMW;
      if constexpr (!PACKED) {
#pragma unroll
        for (int i = 0; i < kWChunks; ++i) {
          const int col = n0 + row0 + 32 * i;
          w_off[i] = col < g.Nout ? ((uint32_t)col * g.wrow + ch * 8) * 2u : kBeyond;
        }
      }
#pragma unroll
      for (int i = 0; i < kXChunks; ++i) {
        const uint32_t r = row0 + 32 * i, pix = p0 + r;
        aok[i] = r < BP && pix < g.npix;
        const uint32_t pp = aok[i] ? pix : 0u;
        const uint32_t n = pp / plane, rem = pp - n * plane;
        const uint32_t oh = rem / g.OW, ow = rem - oh * g.OW;
        ohs[i] = oh * g.ish;
        ows[i] = ow * g.isw;
        abase[i] = n * (uint32_t)g.Hs * g.Ws;
      }
      int t = -1, c0 = g.Cs;   // position of the next stage to fetch
      uint32_t so_w = 0;
      auto fetch = [&](uint4_t (&qw)[kWChunks], uint4_t (&qx)[kXChunks]) {
        c0 += kRoleDepth;
        if (c0 >= g.Cs) {   // enter the next tap (uniform)
          c0 = 0;
          ++t;
          const int dh = tdh[t], dw = tdw[t];
#pragma unroll
          for (int i = 0; i < kXChunks; ++i) {
            const int hh = ohs[i] + dh, ww = ows[i] + dw;
            const bool ok = aok[i] && (unsigned)hh < (unsigned)g.Hs && (unsigned)ww < (unsigned)g.Ws;
            a_off[i] = ok ? ((abase[i] + hh * g.Ws + ww) * (uint32_t)g.Cs + ch * 8) * 2u : kBeyond;
          }
          so_w = (uint32_t)__builtin_amdgcn_readfirstlane(twoff[t]) * 2u;
        }
        const int so = __builtin_amdgcn_readfirstlane(c0 * 2);
        const int sw = __builtin_amdgcn_readfirstlane((int)so_w + c0 * 2);
        if constexpr (!PACKED) {
#pragma unroll
          for (int i = 0; i < kWChunks; ++i)
            qw[i] = __builtin_amdgcn_raw_buffer_load_b128(w_buf, w_off[i], sw, 0);
        }
#pragma unroll
        for (int i = 0; i < kXChunks; ++i)
          qx[i] = __builtin_amdgcn_raw_buffer_load_b128(src_buf, a_off[i], so, 0);
      };
      auto stage = [&](int buf, const uint4_t (&qw)[kWChunks], const uint4_t (&qx)[kXChunks]) {
        if constexpr (!PACKED) {
#pragma unroll
          for (int i = 0; i < kWChunks; ++i)
            *reinterpret_cast<uint4_t*>(&lds_w[buf][row0 + 32 * i][ch * 8]) = qw[i];
        }
#pragma unroll
        for (int i = 0; i < kXChunks; ++i)
          if (row0 + 32 * i < BP) *reinterpret_cast<uint4_t*>(&lds_x[buf][row0 + 32 * i][ch * 8]) = qx[i];
      };
#pragma unroll
      for (int k = 0; k < kSets; ++k)
        if (k < stages) fetch(rw[k], rx[k]);
      stage(0, rw[0], rx[0]);
      if (kSets < stages) fetch(rw[0], rx[0]);
      __syncthreads();
      for (int s2 = 0; s2 < stages; s2 += kSets) {
#pragma unroll
        for (int u = 0; u < kSets; ++u) {
          if (s2 + u >= stages) break;
          const int k = (u + 1) % kSets;   // register set of stage s2 + u + 1
          if (s2 + u + 1 < stages) stage((u + 1) & 1, rw[k], rx[k]);
          if (s2 + u + 1 + kSets < stages) fetch(rw[k], rx[k]);
          __syncthreads();
        }
      }
    }
    return;
  }

  // -------------------------------------------------------------------- multiplying wavefronts
  const int wm = wave / CPW, wp = wave % CPW;   // 64 channels x 32 TN positions each
  const int r = lane & 31, kq = (lane >> 5) * 8;
  const bf16_t* aw = PACKED ? nullptr : &lds_w[0][wm * 64 + r][kq];
  const __amdgpu_buffer_rsrc_t wq_buf =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(w), 0, g.w_bytes, 0x00020000);
  // PACKED: this wavefront's weight fragments come straight from memory, one 1 KB load per
  // fragment, fetched a whole stage ahead into the registers the previous stage has just used
  constexpr int kSteps = kRoleDepth / 16;
  uint4_t wreg[kSteps][2];
  uint32_t wq_off[2];
  const bf16_t* ax = &lds_x[0][wp * TN * 32 + r][kq];
  float16_t acc[2][TN];
  int parity = 0;
  for (uint32_t tile = slot; tile < tiles; tile += gridDim.x, parity ^= 1) {
    const uint32_t p0 = (tile / ntiles_n) * BP;
    const int n0 = (int)(tile % ntiles_n) * BMW;
    if (tid < BP) {
      const uint32_t pix = p0 + tid;
      uint32_t off = kNoRow;
      if (pix < g.npix) {
        const uint32_t n = pix / plane, rem = pix - n * plane;
        const uint32_t oh = rem / g.OW, ow = rem - oh * g.OW;
        off = ((n * g.DH + oh * g.osh + g.oh0) * (uint32_t)g.DW + ow * g.osw + g.ow0) * (uint32_t)g.Nout;
      }
      row_dst[parity][tid] = off;
    }
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
    // position in the reduction of the stage whose weights are fetched next (PACKED)
    int wt = -1, wc0 = g.Cs;
    uint32_t wtap = 0;
    auto next_weights = [&]() -> int {   // scalar byte offset of that stage's first fragment
      wc0 += kRoleDepth;
      if (wc0 >= g.Cs) {
        wc0 = 0;
        ++wt;
        wtap = (uint32_t)__builtin_amdgcn_readfirstlane(twoff[wt]);
      }
      return __builtin_amdgcn_readfirstlane((int)(((wtap + (uint32_t)wc0) >> 4) * 1024u));
    };
    if constexpr (PACKED) {
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const uint32_t blk = (uint32_t)(n0 + wm * 64 + 32 * i) / 32;
        wq_off[i] = (blk * (g.wrow / 16) * 64 + lane) * 16u;   // blocks past the rows: past the buffer
      }
      const int so = next_weights();
#pragma unroll
      for (int q = 0; q < kSteps; ++q)
#pragma unroll
        for (int i = 0; i < 2; ++i)
          wreg[q][i] = __builtin_amdgcn_raw_buffer_load_b128(wq_buf, wq_off[i], so + q * 1024, 0);
    }
    __syncthreads();   // stage 0 is in LDS
    int so_next = 0;
    for (int s2 = 0; s2 < stages; ++s2) {
      const bf16_t* bw = aw + (s2 & 1) * (BMW * kRoleLd);
      const bf16_t* bx = ax + (s2 & 1) * (BP * kRoleLd);
      if constexpr (PACKED) {
        // the last stage fetches its own weights once more instead of branching around the loads
        if (s2 + 1 < stages) so_next = next_weights();
        else so_next = __builtin_amdgcn_readfirstlane((int)(((wtap + (uint32_t)wc0) >> 4) * 1024u));
      }
#pragma unroll
      for (int ks = 0; ks < kRoleDepth; ks += 16) {
        bf16x8 af[2], bfr[TN];
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          if constexpr (PACKED) af[i] = __builtin_bit_cast(bf16x8, wreg[ks / 16][i]);
          else af[i] = *reinterpret_cast<const bf16x8*>(bw + 32 * i * kRoleLd + ks);
        }
#pragma unroll
        for (int j = 0; j < TN; ++j) bfr[j] = *reinterpret_cast<const bf16x8*>(bx + 32 * j * kRoleLd + ks);
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int j = 0; j < TN; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bfr[j], acc[i][j], 0, 0, 0);
        if constexpr (PACKED) {
#pragma unroll
          for (int i = 0; i < 2; ++i)
            wreg[ks / 16][i] = __builtin_amdgcn_raw_buffer_load_b128(wq_buf, wq_off[i], so_next + (ks / 16) * 1024, 0);
        }
      }
      __syncthreads();
    }
    // channels are the rows of the matrix instruction: a lane holds four consecutive channels of
    // one position in four consecutive registers = one 8-byte store; lanes l and l + 32 write
    // neighbouring 8 bytes
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
      for (int v4 = 0; v4 < 4; ++v4) {
        const int col = n0 + wm * 64 + 32 * i + 8 * v4 + 4 * (lane >> 5);
        if (col >= g.Nout) continue;
        float b4[4] = {0.f, 0.f, 0.f, 0.f};
        if (bias) {
#pragma unroll
          for (int e = 0; e < 4; ++e) b4[e] = bf2f(bias[col + e]);
        }
#pragma unroll
        for (int j = 0; j < TN; ++j) {
          const uint32_t off = row_dst[parity][(wp * TN + j) * 32 + (lane & 31)];
          if (off == kNoRow) continue;
          uint32_t lo = (uint32_t)f2bf(acc[i][j][4 * v4] + b4[0]) | ((uint32_t)f2bf(acc[i][j][4 * v4 + 1] + b4[1]) << 16);
          uint32_t hi = (uint32_t)f2bf(acc[i][j][4 * v4 + 2] + b4[2]) | ((uint32_t)f2bf(acc[i][j][4 * v4 + 3] + b4[3]) << 16);
          typedef uint32_t u2 __attribute__((ext_vector_type(2)));
          *reinterpret_cast<u2*>(dst + off + col) = u2{lo, hi};
        }
      }
    }
  }
}

// Weight operand in fragment order: wp[(blk * steps + s) * 64 + lane] (16-byte units) = the 8
// elements rows[blk * 32 + lane % 32][s * 16 + (lane / 32) * 8 ...] of a [rows][len] matrix
// (rows beyond the matrix are zero).  With transposed == 0 the matrix is the weight tensor
// itself (rows = K, len = T * C); with transposed == 1 it is wt[c][t * K + k] = w[k][t][c]
// (rows = C, len = T * K), the operand of backward-data.
__global__ __launch_bounds__(kThreads) void pack_weights_bf16_kernel(
    const bf16_t* __restrict__ w, bf16_t* __restrict__ wp, int K, int C, int T, int transposed) {
  const int rows = transposed ? C : K, len = T * (transposed ? K : C);
  const int steps = len / 16, blocks = (rows + 31) / 32;
  const size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x;   // 16-byte unit
  if (i >= (size_t)blocks * steps * 64) return;
  const int lane = (int)(i % 64);
  const size_t bs = i / 64;
  const int s = (int)(bs % steps), blk = (int)(bs / steps);
  const int row = blk * 32 + (lane & 31), k0 = s * 16 + (lane >> 5) * 8;
  bf16_t v[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    bf16_t x = 0;
    if (row < rows) {
      if (!transposed) {
        x = w[(size_t)row * len + k0 + e];
      } else {
        const int t = (k0 + e) / K, k = (k0 + e) - t * K;
        x = w[((size_t)k * T + t) * C + row];
      }
    }
    v[e] = x;
  }
  uint4_t o;
#pragma unroll
  for (int e = 0; e < 4; ++e) o[e] = (uint32_t)v[2 * e] | ((uint32_t)v[2 * e + 1] << 16);
  reinterpret_cast<uint4_t*>(wp)[i] = o;
}

// wt[(c*T + t)*K + k] = w[(k*T + t)*C + c]
__global__ __launch_bounds__(kThreads) void transpose_weights_bf16_kernel(
    const bf16_t* __restrict__ w, bf16_t* __restrict__ wt, int K, int C, int T) {
  const size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x;
  const size_t n = (size_t)K * C * T;
  if (i >= n) return;
  const int k = (int)(i % K);
  const size_t ct = i / K;
  const int t = (int)(ct % T), c = (int)(ct / T);
  wt[i] = w[((size_t)k * T + t) * C + c];
}

__global__ __launch_bounds__(kThreads) void fill_zero_bf16_kernel(bf16_t* p, size_t n) {
  for (size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x; i < n;
       i += (size_t)gridDim.x * kThreads)
    p[i] = 0;
}

// ------------------------------------------------------------ backward weight
struct WGradH {
  int K, C, T, S;            // T = R*S taps
  int H, W, P, Q;
  int sH, sW, pH, pW, dH, dW;
  uint32_t depth;            // N*P*Q
  uint32_t tiles_per_split;  // 32-position tiles per blockIdx.z
  int partial;               // 1: fp32 partial[z][K][T][C]; 0: bf16 dw[K][T][C] (single split)
  uint32_t dy_bytes, x_bytes;  // tensor sizes for the buffer descriptors
};

// rows = BMW output channels (k), columns = BNW input channels of ONE tap.
// Both operands hold 8 channels of one position per 16-byte chunk while LDS wants positions
// innermost, so chunks are transposed on their way in.  As in the gather kernel everything
// else a wavefront issues per tile is kept small, because a tile is only 8 matrix
// instructions per wavefront:
//  * chunk e = tid + kThreads*i of a tile is (position e % BK, channel group e / BK): all
//    chunks of a thread share ONE position, so one (image, p, q) tracker per thread, moved by
//    additions, serves them all, and consecutive lanes hold consecutive positions;
//  * dy is [position][K]: its byte offset is fixed for the whole kernel, the tile offset is the
//    load's scalar offset, and positions beyond the reduction lie beyond the buffer (read as
//    zero).  x gets one offset per tile (or one beyond the buffer outside the window);
//  * transposing store: a lane pair swaps halves (DPP) and one byte-permute builds the dword
//    of (channel, two positions): 2 vector instructions per 4-byte LDS store, no masks;
//  * two register sets keep the loads of tile t+2 in flight while tile t is multiplied.
// (3 waves per SIMD: the register allocator then keeps the accumulators in the unified file
// instead of 166 + 64 registers, which would leave room for two)
template <int BMW, int BNW>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(3, 3))) void wgrad_bf16_kernel(
    const WGradH g,
                                                              const bf16_t* __restrict__ dy,
                                                              const bf16_t* __restrict__ x,
                                                              void* __restrict__ out) {
  constexpr int TM = BMW / 64, TN = BNW / 64;
  constexpr int kAChunks = BMW * BK / 8 / kThreads;  // 16-byte chunks per thread and tile
  constexpr int kBChunks = BNW * BK / 8 / kThreads;
  constexpr int kGroupStep = kThreads / BK;          // channel groups between a thread's chunks
  constexpr uint32_t kBeyond = 0x80000000u;          // byte offset past any buffer (tensors < 2 GB)
  __shared__ __attribute__((aligned(16))) bf16_t lds_a[2][BMW][LDK];
  __shared__ __attribute__((aligned(16))) bf16_t lds_b[2][BNW][LDK];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave >> 1, wn = wave & 1;
  // XCD-aware order: whole slices of the reduction per XCD (their workgroups read the same
  // positions of dy and x)
  const uint32_t slot = xcd_slot();
  const uint32_t bz = slot / (gridDim.x * gridDim.y);
  const uint32_t in_z = slot - bz * (gridDim.x * gridDim.y);
  const uint32_t by = in_z / gridDim.x, bx = in_z - by * gridDim.x;
  const int m0 = by * BMW;
  const uint32_t ctiles = (uint32_t)g.C / BNW;
  const uint32_t tap = bx / ctiles;
  const uint32_t c0 = (bx - tap * ctiles) * BNW;
  const uint32_t r = tap / g.S, sx = tap - r * g.S;
  const int dh = (int)r * g.dH - g.pH, dw = (int)sx * g.dW - g.pW;
  const uint32_t PQ = (uint32_t)g.P * g.Q;

  const uint32_t total_tiles = (g.depth + BK - 1) / BK;
  const uint32_t t_begin = bz * g.tiles_per_split;
  const uint32_t t_end = min(t_begin + g.tiles_per_split, total_tiles);

  const __amdgpu_buffer_rsrc_t dy_buf =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(dy), 0, g.dy_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t x_buf =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(x), 0, g.x_bytes, 0x00020000);
  const uint32_t pos = tid % BK, group = tid / BK;
  // dy: element (d, m0 + 8*group) of [depth][K]; chunk i lies 8*kGroupStep channels further
  const uint32_t a_off = (pos * (uint32_t)g.K + m0 + group * 8) * 2u;
  const uint32_t a_tile = BK * (uint32_t)g.K * 2u;  // bytes per tile
  // x: this thread's position d = (image, p, q), carried from tile to tile
  uint32_t d = t_begin * BK + pos, bp, bq, img_off;
  {
    const uint32_t n = d / PQ, pq = d - n * PQ;
    bp = pq / g.Q;
    bq = pq - bp * g.Q;
    img_off = n * (uint32_t)g.H * g.W * (uint32_t)g.C * 2u;
  }
  const uint32_t kq = BK / (uint32_t)g.Q, rq = BK - kq * g.Q;
  const uint32_t img_bytes = (uint32_t)g.H * g.W * (uint32_t)g.C * 2u;
  const uint32_t b_chan = (c0 + group * 8) * 2u;

  uint32_t tile = t_begin;  // next tile to fetch (uniform)
  auto fetch = [&](uint4_t (&ra)[kAChunks], uint4_t (&rb)[kBChunks]) {
    const uint32_t a_so = tile * a_tile;
#pragma unroll
    for (int i = 0; i < kAChunks; ++i)
      ra[i] = __builtin_amdgcn_raw_buffer_load_b128(dy_buf, a_off + i * (8 * kGroupStep * 2), a_so, 0);
    const int hh = (int)__umul24(bp, (uint32_t)g.sH) + dh, ww = (int)__umul24(bq, (uint32_t)g.sW) + dw;
    const bool ok = d < g.depth && (unsigned)hh < (unsigned)g.H && (unsigned)ww < (unsigned)g.W;
    const uint32_t pix = __umul24((uint32_t)hh, (uint32_t)g.W) + (uint32_t)ww;
    const uint32_t b_off = ok ? img_off + pix * (uint32_t)g.C * 2u + b_chan : kBeyond;
#pragma unroll
    for (int i = 0; i < kBChunks; ++i)
      rb[i] = __builtin_amdgcn_raw_buffer_load_b128(x_buf, b_off + i * (8 * kGroupStep * 2), 0, 0);
    // next tile: position += BK
    ++tile;
    d += BK;
    bq += rq;
    bp += kq;
    if (bq >= (uint32_t)g.Q) {
      bq -= g.Q;
      ++bp;
    }
    while (bp >= (uint32_t)g.P) {
      bp -= g.P;
      img_off += img_bytes;
    }
  };
  // Transposing store of one chunk (8 channels of position `pos`): lane pairs hold positions
  // 2j and 2j+1; after the swap the even lane owns the even channels of both positions, the
  // odd lane the odd channels, each as whole dwords [channel][pos & ~1].
  const bool odd = tid & 1;
  const uint32_t sel = odd ? 0x03020706u : 0x05040100u;  // byte picks of (neighbour, own)
  auto scatter = [&](bf16_t (*dstp)[LDK], int grp, const uint4_t& v) {
#pragma unroll
    for (int j = 0; j < 4; ++j) {
      const uint32_t own = v[j];
      const uint32_t other = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)own, 0xB1, 0xF, 0xF, true);
      const uint32_t word = __builtin_amdgcn_perm(other, own, sel);
      *reinterpret_cast<uint32_t*>(&dstp[grp * 8 + 2 * j + (odd ? 1 : 0)][pos & ~1u]) = word;
    }
  };
  auto stage = [&](int buf, const uint4_t (&ra)[kAChunks], const uint4_t (&rb)[kBChunks]) {
#pragma unroll
    for (int i = 0; i < kAChunks; ++i) scatter(lds_a[buf], (int)group + kGroupStep * i, ra[i]);
#pragma unroll
    for (int i = 0; i < kBChunks; ++i) scatter(lds_b[buf], (int)group + kGroupStep * i, rb[i]);
  };

  float16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  if (t_begin < t_end) {
    const uint32_t ntiles = t_end - t_begin;
    uint4_t ra0[kAChunks], rb0[kBChunks], ra1[kAChunks], rb1[kBChunks];
    fetch(ra0, rb0);
    if (ntiles > 1) fetch(ra1, rb1);
    stage(0, ra0, rb0);
    __syncthreads();
    for (uint32_t kt = 0; kt + 1 < ntiles; kt += 2) {
      // tile kt is in LDS buffer 0, tile kt+1 in flight in set 1
      if (kt + 2 < ntiles) fetch(ra0, rb0);
      mma_tile<TM, TN, BMW, BNW>(lds_a[0], lds_b[0], wm, wn, lane, acc);
      stage(1, ra1, rb1);
      __syncthreads();
      // tile kt+1 is in LDS buffer 1, tile kt+2 in flight in set 0
      if (kt + 3 < ntiles) fetch(ra1, rb1);
      mma_tile<TM, TN, BMW, BNW>(lds_a[1], lds_b[1], wm, wn, lane, acc);
      if (kt + 2 < ntiles) stage(0, ra0, rb0);
      __syncthreads();
    }
    // an odd number of tiles: the last one was staged into buffer 0
    if (ntiles & 1) mma_tile<TM, TN, BMW, BNW>(lds_a[0], lds_b[0], wm, wn, lane, acc);
  }

  const size_t row_len = (size_t)g.T * g.C;
#pragma unroll
  for (int j = 0; j < TN; ++j) {
    const uint32_t c = c0 + wn * (BNW / 2) + 32 * j + (lane & 31);
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int m = m0 + wm * (BMW / 2) + 32 * i + acc_row(v, lane);
        const size_t o = (size_t)m * row_len + (size_t)tap * g.C + c;
        if (g.partial)
          reinterpret_cast<float*>(out)[(size_t)bz * g.K * row_len + o] = acc[i][j][v];
        else
          reinterpret_cast<bf16_t*>(out)[o] = f2bf(acc[i][j][v]);
      }
    }
  }
}

// dw[i] = bf16(sum over splits of partial[z][i]), fixed order
__global__ __launch_bounds__(kThreads) void wgrad_reduce_bf16_kernel(
    const float* __restrict__ partial, bf16_t* __restrict__ dw, size_t n, int splits) {
  const size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x;
  if (i >= n) return;
  float s = 0.f;
  for (int z = 0; z < splits; ++z) s += partial[(size_t)z * n + i];
  dw[i] = f2bf(s);
}

// The large-tile form of backward-weight: eight wavefronts with two roles, as in the gather kernel.
// A workgroup owns 64 TM output channels (rows, from dy) x 64 TN input channels (columns, from x) of
// ONE tap and a range of the positions; wavefronts 0-3 multiply (2 x 2 of them, TM x TN accumulator
// tiles of 32 x 32 each), wavefronts 4-7 feed.  Both tensors hold the channels of a position
// contiguously while the matrix instruction wants 8 consecutive positions per lane: the feeders
// copy 16-byte chunks into LDS unchanged ([position][channel], rows padded by 64 bytes: four lanes
// write the 64 bytes of a row piece, so consecutive rows must start 16 banks apart; with 32 bytes
// of padding the writes of two rows met in 8 banks) and the
// multiplying wavefronts read the operands with the transposing LDS load (ds_read_b64_tr_b16: 16
// lanes give the addresses of a 4-position x 16-channel block and lane i receives the 4 positions of
// channel i), two per operand fragment.  No shuffles, byte permutes or 4-byte LDS stores, which is
// what the kernel above spends its time on.  The partial sums of a workgroup go to the workspace in
// the order the accumulators lie in registers (16 bytes per lane, a whole KB per instruction) and
// `wgrad_roles_reduce_kernel` adds the ranges in a fixed order (reproducible).
constexpr int kWrDepth = 64;   // positions per stage

template <int TM, int TN>
__global__ __launch_bounds__(kRoleThreads) __attribute__((amdgpu_waves_per_eu(2, 2))) void wgrad_roles_kernel(
    const WGradH g, const bf16_t* __restrict__ dy, const bf16_t* __restrict__ x,
    float* __restrict__ partial, uint32_t tiles, uint32_t stages_per_split) {
  constexpr int BM = 64 * TM, BN = 64 * TN;
  constexpr int LDA = BM + 32, LDB = BN + 32;      // elements per LDS row (64 bytes of padding)
  constexpr int kLpr = 256 / kWrDepth;             // feeding threads per position
  constexpr int kA = BM / 8 / kLpr, kB = BN / 8 / kLpr;   // 16-byte chunks per feeding thread and stage
  constexpr uint32_t kBeyond = 0x80000000u;
  typedef short short4_t __attribute__((ext_vector_type(4)));
  typedef __attribute__((address_space(3))) short4_t* lds_frag_ptr;
  __shared__ __attribute__((aligned(16))) bf16_t lds_a[2][kWrDepth][LDA];
  __shared__ __attribute__((aligned(16))) bf16_t lds_b[2][kWrDepth][LDB];
  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  // a contiguous range of slots per XCD: the workgroups of one range of positions (they read the
  // same dy and x) lie under one L2
  const uint32_t slot = xcd_slot();
  const uint32_t split = slot / tiles, tile = slot - split * tiles;
  const uint32_t tiles_n = (uint32_t)g.C / BN, tiles_m = (uint32_t)g.K / BM;
  const uint32_t tn = tile % tiles_n, tm = (tile / tiles_n) % tiles_m, tap = tile / (tiles_n * tiles_m);
  const uint32_t total = (g.depth + kWrDepth - 1) / kWrDepth;
  const uint32_t t_begin = min(split * stages_per_split, total);
  const uint32_t t_end = min(t_begin + stages_per_split, total);
  const int stages = (int)(t_end - t_begin);

  if (wave >= 4) {
    // ------------------------------------------------------------------ feeding wavefronts
    if (stages == 0) return;
    const int ft = tid - 256;
    const uint32_t row = ft / kLpr, c8 = ft % kLpr;   // position of the stage, first 16-byte chunk
    const __amdgpu_buffer_rsrc_t dy_buf =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(dy), 0, g.dy_bytes, 0x00020000);
    const __amdgpu_buffer_rsrc_t x_buf =
        __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(x), 0, g.x_bytes, 0x00020000);
    const uint32_t r = tap / g.S, sx = tap - r * g.S;
    const int dh = (int)r * g.dH - g.pH, dw = (int)sx * g.dW - g.pW;
    const uint32_t PQ = (uint32_t)g.P * g.Q;
    // dy is [position][K]: a fixed byte offset per thread, the stage in the scalar offset;
    // positions past the end of the reduction lie past the buffer and read as zero
    const uint32_t a_off = (row * (uint32_t)g.K + tm * BM + c8 * 8) * 2u;
    const uint32_t a_stage = kWrDepth * (uint32_t)g.K * 2u;
    // x: this thread's position (image, p, q), carried from stage to stage by additions
    uint32_t d = t_begin * kWrDepth + row, bp, bq, img_off;
    {
      const uint32_t n = d / PQ, pq = d - n * PQ;
      bp = pq / g.Q;
      bq = pq - bp * g.Q;
      img_off = n * (uint32_t)g.H * g.W * (uint32_t)g.C * 2u;
    }
    const uint32_t kq = kWrDepth / (uint32_t)g.Q, rq = kWrDepth - kq * g.Q;
    const uint32_t img_bytes = (uint32_t)g.H * g.W * (uint32_t)g.C * 2u;
    const uint32_t b_chan = (tn * BN + c8 * 8) * 2u;
    uint32_t t = t_begin;
    constexpr int kSets = kWrDepth == 32 ? 4 : 2;   // register sets = stages the loads run ahead of the LDS writes
    uint4_t ra[kSets][kA], rb[kSets][kB];
    auto fetch = [&](uint4_t (&qa)[kA], uint4_t (&qb)[kB]) {
      const int so = __builtin_amdgcn_readfirstlane((int)(t * a_stage));
#pragma unroll
      for (int i = 0; i < kA; ++i)
        qa[i] = __builtin_amdgcn_raw_buffer_load_b128(dy_buf, a_off + i * (16 * kLpr), so, 0);
      const int hh = (int)__umul24(bp, (uint32_t)g.sH) + dh, ww = (int)__umul24(bq, (uint32_t)g.sW) + dw;
      const bool ok = d < g.depth && (unsigned)hh < (unsigned)g.H && (unsigned)ww < (unsigned)g.W;
      const uint32_t pix = __umul24((uint32_t)hh, (uint32_t)g.W) + (uint32_t)ww;
      const uint32_t b_off = ok ? img_off + pix * (uint32_t)g.C * 2u + b_chan : kBeyond;
#pragma unroll
      for (int i = 0; i < kB; ++i)
        qb[i] = __builtin_amdgcn_raw_buffer_load_b128(x_buf, b_off + i * (16 * kLpr), 0, 0);
      ++t;
      d += kWrDepth;
      bq += rq;
      bp += kq;
      if (bq >= (uint32_t)g.Q) {
        bq -= g.Q;
        ++bp;
      }
      while (bp >= (uint32_t)g.P) {
        bp -= g.P;
        img_off += img_bytes;
      }
    };
    auto stage = [&](int buf, const uint4_t (&qa)[kA], const uint4_t (&qb)[kB]) {
#pragma unroll
      for (int i = 0; i < kA; ++i)
        *reinterpret_cast<uint4_t*>(&lds_a[buf][row][(c8 + kLpr * i) * 8]) = qa[i];
#pragma unroll
      for (int i = 0; i < kB; ++i)
        *reinterpret_cast<uint4_t*>(&lds_b[buf][row][(c8 + kLpr * i) * 8]) = qb[i];
    };
#pragma unroll
    for (int k = 0; k < kSets; ++k)
      if (k < stages) fetch(ra[k], rb[k]);
    stage(0, ra[0], rb[0]);
    if (kSets < stages) fetch(ra[0], rb[0]);
    __syncthreads();
    for (int s2 = 0; s2 < stages; s2 += kSets) {
#pragma unroll
      for (int u = 0; u < kSets; ++u) {
        if (s2 + u >= stages) break;
        const int k = (u + 1) % kSets;   // register set of stage s2 + u + 1
        if (s2 + u + 1 < stages) stage((u + 1) & 1, ra[k], rb[k]);
        if (s2 + u + 1 + kSets < stages) fetch(ra[k], rb[k]);
        __syncthreads();
      }
    }
    return;
  }

  // -------------------------------------------------------------------- multiplying wavefronts
  const int wm = wave >> 1, wn = wave & 1;
  // the lane's address inside a 16-position x 32-channel fragment: 16 lanes cover 4 positions x 16
  // channels; lanes 32-63 hold the second half of the 16 positions of a matrix step
  const int l16 = lane & 15, grp = lane >> 4;
  const int pix0 = 8 * (grp >> 1) + (l16 >> 2), chan0 = 16 * (grp & 1) + 4 * (l16 & 3);
  const bf16_t* pa = &lds_a[0][pix0][wm * (TM * 32) + chan0];
  const bf16_t* pb = &lds_b[0][pix0][wn * (TN * 32) + chan0];
  float16_t acc[TM][TN];
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
  if (stages > 0) __syncthreads();   // stage 0 is in LDS
  for (int s2 = 0; s2 < stages; ++s2) {
    const bf16_t* qa = pa + (s2 & 1) * (kWrDepth * LDA);
    const bf16_t* qb = pb + (s2 & 1) * (kWrDepth * LDB);
#pragma unroll
    for (int ks = 0; ks < kWrDepth; ks += 16) {
      bf16x8 af[TM], bfr[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i) {
        const short4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_frag_ptr)(qa + ks * LDA + 32 * i));
        const short4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_frag_ptr)(qa + (ks + 4) * LDA + 32 * i));
        af[i] = __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
      }
#pragma unroll
      for (int j = 0; j < TN; ++j) {
        const short4_t lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_frag_ptr)(qb + ks * LDB + 32 * j));
        const short4_t hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_frag_ptr)(qb + (ks + 4) * LDB + 32 * j));
        bfr[j] = __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
      }
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(af[i], bfr[j], acc[i][j], 0, 0, 0);
    }
    __syncthreads();
  }
  // registers as they lie: unit ((slot * 4 + wave) * TM * TN * 4 + (i * TN + j) * 4 + a) * 64 + lane
  // holds acc[i][j][4a .. 4a + 3]
  float4* out = reinterpret_cast<float4*>(partial) +
                ((size_t)slot * 4 + wave) * (TM * TN * 4 * 64) + lane;
#pragma unroll
  for (int i = 0; i < TM; ++i)
#pragma unroll
    for (int j = 0; j < TN; ++j)
#pragma unroll
      for (int a = 0; a < 4; ++a)
        out[((i * TN + j) * 4 + a) * 64] =
            make_float4(acc[i][j][4 * a], acc[i][j][4 * a + 1], acc[i][j][4 * a + 2], acc[i][j][4 * a + 3]);
}

// dw[k][tap][c] = sum over the ranges of positions, in order; one thread per 16-byte unit of a
// range (four consecutive output channels k of one input channel c)
template <int TM, int TN>
__global__ __launch_bounds__(kThreads) void wgrad_roles_reduce_kernel(
    const float4* __restrict__ partial, bf16_t* __restrict__ dw, uint32_t units, int splits, int K,
    int C, int T) {
  constexpr int BM = 64 * TM, BN = 64 * TN;
  const uint32_t u = blockIdx.x * kThreads + threadIdx.x;
  if (u >= units) return;
  float4 s = partial[u];
  for (int z = 1; z < splits; ++z) {
    const float4 v = partial[(size_t)z * units + u];
    s.x += v.x;
    s.y += v.y;
    s.z += v.z;
    s.w += v.w;
  }
  const uint32_t lane = u & 63, a = (u >> 6) & 3, ij = (u >> 8) % (TM * TN);
  const uint32_t wave = (u / (256 * TM * TN)) & 3, tile = u / (1024 * TM * TN);
  const uint32_t i = ij / TN, j = ij - i * TN;
  const uint32_t tiles_n = (uint32_t)C / BN, tiles_m = (uint32_t)K / BM;
  const uint32_t tn = tile % tiles_n, tm = (tile / tiles_n) % tiles_m, tap = tile / (tiles_n * tiles_m);
  const uint32_t k = tm * BM + (wave >> 1) * (TM * 32) + 32 * i + 8 * a + 4 * (lane >> 5);
  const uint32_t c = tn * BN + (wave & 1) * (TN * 32) + 32 * j + (lane & 31);
  const size_t row = (size_t)T * C;
  bf16_t* o = dw + (size_t)k * row + (size_t)tap * C + c;
  o[0] = f2bf(s.x);
  o[row] = f2bf(s.y);
  o[2 * row] = f2bf(s.z);
  o[3 * row] = f2bf(s.w);
}

// ----------------------------------------------------------------------- host
static int check16(const mn_conv2d* g) {
  // every tensor is addressed with 32-bit element offsets
  const long long lim = 1ll << 31;
  if ((long long)g->N * g->C * g->H * g->W >= lim || (long long)g->N * g->K * g->P * g->Q >= lim ||
      (long long)g->K * g->C * g->R * g->S >= lim)
    return MN_EUNSUPPORTED;
  if (g->R * g->S > kMaxTaps) return MN_EUNSUPPORTED;
  return MN_OK;
}

// Shapes the large-tile kernel (feeding and multiplying wavefronts) takes, given weight rows in
// place: deep enough channel chunks, at least 128 output channels in whole 64s, enough positions
// to fill the device.
static bool roles_shape(int Cs, int Nout, unsigned long long npix) {
  return Cs % 64 == 0 && Nout % 64 == 0 && Nout >= 128 && npix >= 4096;
}

static int launch_gather16(GatherH q, const bf16_t* src, const bf16_t* w, const bf16_t* bias,
                           bf16_t* dst, hipStream_t s) {
  if (q.npix == 0 || q.Nout == 0) return MN_OK;
  // the kernel addresses its operands through buffer descriptors with byte offsets below 2^31
  const unsigned long long n_img = q.npix / ((unsigned long long)q.OH * q.OW);
  const unsigned long long src_bytes = n_img * q.Hs * q.Ws * q.Cs * 2ull;
  const unsigned long long w_rows = q.wstep == 1024 ? (q.Nout + 31) / 32 * 32ull : (unsigned long long)q.Nout;
  const unsigned long long w_bytes = w_rows * q.wrow * 2ull;
  if (src_bytes >= (1ull << 31) || w_bytes >= (1ull << 31)) return MN_EUNSUPPORTED;
  q.src_bytes = (uint32_t)src_bytes;
  q.w_bytes = (uint32_t)w_bytes;
  const bool deep = q.Cs % 64 == 0;
  if (roles_shape(q.Cs, q.Nout, q.npix)) {
    // large tiles, feeding and multiplying wavefronts.  256-channel tiles of 128 or 160 positions
    // (160 where it saves a round of the persistent, one-per-CU workgroups), 128-channel tiles of
    // 192 or 256 positions when that covers the channels with less padding.
    int dev = 0, cus = 256;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
      cus = 256;
    struct Cand { int bm, bp; };
    static const Cand cands[] = {{256, 160}, {256, 128}, {128, 256}, {128, 192}};
    int best = 0;
    double best_cost = 1e30;
    long long best_tiles = 0;
    for (int i = 0; i < 4; ++i) {
      const long long tiles = (long long)((q.npix + cands[i].bp - 1) / cands[i].bp) * ((q.Nout + cands[i].bm - 1) / cands[i].bm);
      // rounds x tile area; the narrower channel tile re-reads the pixels once more per 128 channels
      const double cost = (double)((tiles + cus - 1) / cus) * cands[i].bp * cands[i].bm * (cands[i].bm == 128 ? 1.1 : 1.0);
      if (cost < best_cost) {
        best_cost = cost;
        best = i;
        best_tiles = tiles;
      }
    }
    const dim3 grid((unsigned)(best_tiles < cus ? best_tiles : cus));
#define MN_ROLES(CMW, TN)                                                                   \
  do {                                                                                      \
    if (q.wstep == 1024)                                                                    \
      gather_roles_kernel<CMW, TN, true><<<grid, kRoleThreads, 0, s>>>(q, src, w, bias, dst);  \
    else                                                                                    \
      gather_roles_kernel<CMW, TN, false><<<grid, kRoleThreads, 0, s>>>(q, src, w, bias, dst); \
  } while (0)
    switch (best) {
      case 0: MN_ROLES(4, 5); break;
      case 1: MN_ROLES(4, 4); break;
      case 2: MN_ROLES(2, 4); break;
      default: MN_ROLES(2, 3); break;
    }
#undef MN_ROLES
    return MN_OK;
  }
  if (q.Nout % 128 == 0) {
    dim3 grid((q.npix + BM - 1) / BM, q.Nout / 128);
    if (deep)
      gather_bf16_kernel<128, 64><<<grid, kThreads, 0, s>>>(q, src, w, bias, dst);
    else
      gather_bf16_kernel<128, 32><<<grid, kThreads, 0, s>>>(q, src, w, bias, dst);
  } else {
    dim3 grid((q.npix + BM - 1) / BM, (q.Nout + 63) / 64);
    if (deep)
      gather_bf16_kernel<64, 64><<<grid, kThreads, 0, s>>>(q, src, w, bias, dst);
    else
      gather_bf16_kernel<64, 32><<<grid, kThreads, 0, s>>>(q, src, w, bias, dst);
  }
  return MN_OK;
}

// bytes of the fragment-packed weight operand of a gather direction
static size_t packed_weight_bytes(const mn_conv2d* g, bool transposed) {
  const size_t rows = transposed ? g->C : g->K, len = (size_t)g->R * g->S * (transposed ? g->K : g->C);
  return (rows + 31) / 32 * 32 * len * sizeof(bf16_t);
}

static void pack_weights(const mn_conv2d* g, const bf16_t* w, bf16_t* wp, bool transposed, hipStream_t s) {
  const size_t units = packed_weight_bytes(g, transposed) / 16;
  pack_weights_bf16_kernel<<<(unsigned)((units + kThreads - 1) / kThreads), kThreads, 0, s>>>(
      w, wp, g->K, g->C, g->R * g->S, transposed ? 1 : 0);
}

static void wgrad16_tiles(const mn_conv2d* g, int* bm, int* bn) {
  *bm = g->K % 128 == 0 ? 128 : 64;
  *bn = g->C % 128 == 0 ? 128 : 64;
}

static void wgrad16_split(const mn_conv2d* g, int* splits, int* tiles_per_split) {
  int bm, bn;
  wgrad16_tiles(g, &bm, &bn);
  const long long depth = (long long)g->N * g->P * g->Q;
  const long long total_tiles = (depth + BK - 1) / BK;
  const long long out_tiles = (long long)g->R * g->S * (g->C / bn) * (g->K / bm);
  long long want = (1024 + out_tiles - 1) / out_tiles;
  if (want > total_tiles) want = total_tiles;
  if (want > 128) want = 128;
  if (want < 1) want = 1;
  const long long tps = (total_tiles + want - 1) / want;
  *tiles_per_split = (int)(tps < 1 ? 1 : tps);
  *splits = (int)((total_tiles + *tiles_per_split - 1) / (*tiles_per_split));
  if (*splits < 1) *splits = 1;
}

// The large-tile backward-weight (variant 1): channel counts that are multiples of 128 and a
// reduction long enough to share out.  tm / tn = accumulator tiles per wavefront along K / C;
// splits = ranges of positions, one workgroup per (tile, range), about one workgroup per CU.
struct WgradRoles {
  int tm, tn;
  uint32_t tiles, splits, stages_per_split;
};

static bool wgrad16_roles(const mn_conv2d* g, WgradRoles* r) {
  if (g->K % 128 != 0 || g->C % 128 != 0) return false;
  const long long depth = (long long)g->N * g->P * g->Q;
  if (depth < 4096) return false;
  // 128 accumulation registers per lane: a wavefront has 256 registers in all at two per SIMD
  r->tm = g->K % 256 == 0 ? 4 : 2;
  r->tn = r->tm == 2 && g->C % 256 == 0 ? 4 : 2;
  const long long tiles = (long long)g->R * g->S * (g->K / (64 * r->tm)) * (g->C / (64 * r->tn));
  if (tiles > 65535) return false;
  int dev = 0, cus = 256;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
    cus = 256;
  const long long total = (depth + kWrDepth - 1) / kWrDepth;
  long long splits = cus / tiles;
  if (splits < 1) splits = 1;
  if (splits > total / 4) splits = total / 4 > 0 ? total / 4 : 1;
  const long long per = (total + splits - 1) / splits;
  r->tiles = (uint32_t)tiles;
  r->stages_per_split = (uint32_t)per;
  r->splits = (uint32_t)((total + per - 1) / per);
  return true;
}

}  // namespace mn_conv16

// Entry points used by the dtype dispatch in conv.hip.
int mn_conv16_ws_bytes(const mn_conv2d* g, int direction, int variant, size_t* bytes) {
  using namespace mn_conv16;
  *bytes = 0;
  const int st = check16(g);
  if (st != MN_OK) return st;
  if (variant < 0 || variant > 1) return MN_EUNSUPPORTED;
  if (direction == MN_CONV_FWD) {
    if (g->C % BK != 0) return MN_EUNSUPPORTED;
    if (variant == 1) *bytes = packed_weight_bytes(g, false);
    return MN_OK;
  }
  if (direction == MN_CONV_BWD_DATA) {
    if (g->K % BK != 0) return MN_EUNSUPPORTED;
    *bytes = variant == 1 ? packed_weight_bytes(g, true)
                          : (size_t)g->K * g->C * g->R * g->S * sizeof(bf16_t);
    return MN_OK;
  }
  if (g->K % 64 != 0 || g->C % 64 != 0) return MN_EUNSUPPORTED;
  WgradRoles wr;
  if (variant == 1 && wgrad16_roles(g, &wr)) {
    *bytes = (size_t)wr.splits * g->K * g->C * g->R * g->S * sizeof(float);
    return MN_OK;
  }
  int splits, tps;
  wgrad16_split(g, &splits, &tps);
  if (splits > 1) *bytes = (size_t)splits * g->K * g->C * g->R * g->S * sizeof(float);
  return MN_OK;
}

int mn_conv16_fwd(const mn_conv2d* g, const void* x, const void* w, const void* bias, void* y,
                  void* ws, size_t ws_bytes, int variant, hipStream_t s) {
  using namespace mn_conv16;
  const int st = check16(g);
  if (st != MN_OK) return st;
  if (g->C % BK != 0 || variant < 0 || variant > 1) return MN_EUNSUPPORTED;
  if (!mn_aligned(x, 16) || !mn_aligned(w, 16)) return MN_EINVAL;
  GatherH q = {};
  q.wstep = 32;
  // variant 1 packs the weights in fragment order for the kernels that load them straight into
  // registers
  if (variant == 1) {
    if (!ws || ws_bytes < packed_weight_bytes(g, false) || !mn_aligned(ws, 16)) return MN_EINVAL;
    pack_weights(g, (const bf16_t*)w, (bf16_t*)ws, false, s);
    w = ws;
    q.wstep = 1024;
  }
  q.npix = (uint32_t)((long long)g->N * g->P * g->Q);
  q.OH = g->P;
  q.OW = g->Q;
  q.Nout = g->K;
  q.Cs = g->C;
  q.Hs = g->H;
  q.Ws = g->W;
  q.ish = g->sH;
  q.isw = g->sW;
  q.DH = g->P;
  q.DW = g->Q;
  q.osh = q.osw = 1;
  q.T = g->R * g->S;
  q.wrow = (uint32_t)q.T * g->C;
  for (int r = 0; r < g->R; ++r)
    for (int sx = 0; sx < g->S; ++sx) {
      const int t = r * g->S + sx;
      q.dh[t] = (int16_t)(r * g->dH - g->pH);
      q.dw[t] = (int16_t)(sx * g->dW - g->pW);
      q.woff[t] = t * g->C;
    }
  const int lst = launch_gather16(q, (const bf16_t*)x, (const bf16_t*)w, (const bf16_t*)bias, (bf16_t*)y, s);
  if (lst != MN_OK) return lst;
  return mn_launch_status();
}

int mn_conv16_bwd_data(const mn_conv2d* g, const void* dy, const void* w, void* dx, void* ws,
                       size_t ws_bytes, int variant, hipStream_t s) {
  using namespace mn_conv16;
  const int st = check16(g);
  if (st != MN_OK) return st;
  if (g->K % BK != 0 || variant < 0 || variant > 1) return MN_EUNSUPPORTED;
  const int T = g->R * g->S;
  const size_t nw = (size_t)g->K * g->C * T;
  const size_t need = variant == 1 ? packed_weight_bytes(g, true) : nw * sizeof(bf16_t);
  if (!ws || ws_bytes < need || !mn_aligned(ws, 16) || !mn_aligned(dy, 16)) return MN_EINVAL;
  // variant 1: fragment-packed transposed weights
  const bool packed = variant == 1;
  if (packed)
    pack_weights(g, (const bf16_t*)w, (bf16_t*)ws, true, s);
  else
    transpose_weights_bf16_kernel<<<(unsigned)((nw + kThreads - 1) / kThreads), kThreads, 0, s>>>(
        (const bf16_t*)w, (bf16_t*)ws, g->K, g->C, T);
  bool empty_class = false;
  for (int ca = 0; ca < g->sH && !empty_class; ++ca) {
    bool any = false;
    for (int r = 0; r < g->R; ++r) any |= (r * g->dH) % g->sH == ca;
    empty_class |= !any;
  }
  for (int cb = 0; cb < g->sW && !empty_class; ++cb) {
    bool any = false;
    for (int sx = 0; sx < g->S; ++sx) any |= (sx * g->dW) % g->sW == cb;
    empty_class |= !any;
  }
  if (empty_class) {
    const size_t n = (size_t)g->N * g->C * g->H * g->W;
    fill_zero_bf16_kernel<<<2048, kThreads, 0, s>>>((bf16_t*)dx, n);
  }
  for (int ca = 0; ca < g->sH; ++ca) {
    for (int cb = 0; cb < g->sW; ++cb) {
      GatherH q = {};
      q.oh0 = ((ca - g->pH) % g->sH + g->sH) % g->sH;
      q.ow0 = ((cb - g->pW) % g->sW + g->sW) % g->sW;
      q.OH = q.oh0 < g->H ? (g->H - q.oh0 + g->sH - 1) / g->sH : 0;
      q.OW = q.ow0 < g->W ? (g->W - q.ow0 + g->sW - 1) / g->sW : 0;
      int Tc = 0;
      for (int r = 0; r < g->R; ++r) {
        if ((r * g->dH) % g->sH != ca) continue;
        for (int sx = 0; sx < g->S; ++sx) {
          if ((sx * g->dW) % g->sW != cb) continue;
          q.dh[Tc] = (int16_t)((q.oh0 + g->pH - r * g->dH) / g->sH);
          q.dw[Tc] = (int16_t)((q.ow0 + g->pW - sx * g->dW) / g->sW);
          q.woff[Tc] = (r * g->S + sx) * g->K;
          ++Tc;
        }
      }
      if (Tc == 0) continue;  // cleared above
      q.T = Tc;
      q.npix = (uint32_t)((long long)g->N * q.OH * q.OW);
      q.Nout = g->C;
      q.Cs = g->K;
      q.Hs = g->P;
      q.Ws = g->Q;
      q.ish = q.isw = 1;
      q.DH = g->H;
      q.DW = g->W;
      q.osh = g->sH;
      q.osw = g->sW;
      q.wrow = (uint32_t)T * g->K;
      q.wstep = packed ? 1024 : 32;
      const int lst = launch_gather16(q, (const bf16_t*)dy, (const bf16_t*)ws, nullptr, (bf16_t*)dx, s);
      if (lst != MN_OK) return lst;
    }
  }
  return mn_launch_status();
}

int mn_conv16_bwd_weight(const mn_conv2d* g, const void* dy, const void* x, void* dw, void* ws,
                         size_t ws_bytes, int variant, hipStream_t s) {
  using namespace mn_conv16;
  const int st = check16(g);
  if (st != MN_OK) return st;
  if (g->K % 64 != 0 || g->C % 64 != 0) return MN_EUNSUPPORTED;
  if (!mn_aligned(dy, 16) || !mn_aligned(x, 16)) return MN_EINVAL;
  WGradH q = {};
  q.K = g->K;
  q.C = g->C;
  q.T = g->R * g->S;
  q.S = g->S;
  q.H = g->H;
  q.W = g->W;
  q.P = g->P;
  q.Q = g->Q;
  q.sH = g->sH;
  q.sW = g->sW;
  q.pH = g->pH;
  q.pW = g->pW;
  q.dH = g->dH;
  q.dW = g->dW;
  q.depth = (uint32_t)((long long)g->N * g->P * g->Q);
  // the kernel addresses both tensors through buffer descriptors with byte offsets below 2^31
  const unsigned long long dy_bytes = (unsigned long long)q.depth * g->K * 2ull;
  const unsigned long long x_bytes = (unsigned long long)g->N * g->H * g->W * g->C * 2ull;
  if (dy_bytes >= (1ull << 31) || x_bytes >= (1ull << 31)) return MN_EUNSUPPORTED;
  q.dy_bytes = (uint32_t)dy_bytes;
  q.x_bytes = (uint32_t)x_bytes;
  WgradRoles wr;
  if (variant == 1 && wgrad16_roles(g, &wr)) {
    const size_t nw = (size_t)g->K * g->C * q.T;
    if (!ws || ws_bytes < nw * sizeof(float) * wr.splits || !mn_aligned(ws, 16)) return MN_EINVAL;
    const unsigned grid = wr.tiles * wr.splits;
    const uint32_t units = (uint32_t)(nw / 4);
    const unsigned rgrid = (units + kThreads - 1) / kThreads;
#define MN_WGRAD_ROLES(TM_, TN_)                                                                  \
  do {                                                                                            \
    wgrad_roles_kernel<TM_, TN_><<<grid, kRoleThreads, 0, s>>>(                                   \
        q, (const bf16_t*)dy, (const bf16_t*)x, (float*)ws, wr.tiles, wr.stages_per_split);       \
    wgrad_roles_reduce_kernel<TM_, TN_><<<rgrid, kThreads, 0, s>>>(                               \
        (const float4*)ws, (bf16_t*)dw, units, (int)wr.splits, g->K, g->C, q.T);                  \
  } while (0)
    if (wr.tm == 4) MN_WGRAD_ROLES(4, 2);
    else if (wr.tn == 4) MN_WGRAD_ROLES(2, 4);
    else MN_WGRAD_ROLES(2, 2);
#undef MN_WGRAD_ROLES
    return mn_launch_status();
  }
  int splits, tps, bm, bn;
  wgrad16_split(g, &splits, &tps);
  wgrad16_tiles(g, &bm, &bn);
  q.tiles_per_split = tps;
  q.partial = splits > 1;
  const size_t nw = (size_t)g->K * g->C * q.T;
  void* out = dw;
  if (q.partial) {
    if (!ws || ws_bytes < nw * sizeof(float) * splits || !mn_aligned(ws, 4)) return MN_EINVAL;
    out = ws;
  }
  dim3 grid(q.T * (g->C / bn), g->K / bm, splits);
  if (bm == 128 && bn == 128)
    wgrad_bf16_kernel<128, 128><<<grid, kThreads, 0, s>>>(q, (const bf16_t*)dy, (const bf16_t*)x, out);
  else if (bm == 128)
    wgrad_bf16_kernel<128, 64><<<grid, kThreads, 0, s>>>(q, (const bf16_t*)dy, (const bf16_t*)x, out);
  else if (bn == 128)
    wgrad_bf16_kernel<64, 128><<<grid, kThreads, 0, s>>>(q, (const bf16_t*)dy, (const bf16_t*)x, out);
  else
    wgrad_bf16_kernel<64, 64><<<grid, kThreads, 0, s>>>(q, (const bf16_t*)dy, (const bf16_t*)x, out);
  if (q.partial)
    wgrad_reduce_bf16_kernel<<<(unsigned)((nw + kThreads - 1) / kThreads), kThreads, 0, s>>>(
        (const float*)ws, (bf16_t*)dw, nw, splits);
  return mn_launch_status();
}
