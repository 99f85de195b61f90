// 2-D convolution as implicit GEMM on the fp32 matrix cores
// (v_mfma_f32_32x32x2_f32), NCHW tensors, no layout change in HBM.
//
// Forward and backward-data are the same "gather GEMM":
//     D[m][col] = sum over (ch, tap)  A(m, ch, tap) * src[n, ch, oh*ish + dh[tap], ow*isw + dw[tap]]
// with col = (n, oh, ow).  Forward: A = weights, src = x, taps = the R*S window.
// Backward-data: A = weights read through strides, src = dy; for stride > 1 the input positions are split by parity
// class so that every class is a dense stride-1 gather over the taps that can
// reach it (no multiplies by structural zeros).
//
// Variant 1 of both first repacks the weights into the workspace as
// A'[tap][ch][m] (m contiguous, padded), the order the kernel stages them in.
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
#include <type_traits>

// Winograd F(2x2, 3x3) tier of forward and backward-data (conv_wino.hip)
int mn_wino_ws_bytes(const mn_conv2d* g, bool backward_data, size_t* bytes);
int mn_wino_fwd(const mn_conv2d* g, const float* x, const float* w, const float* bias, float* y,
                void* ws, size_t ws_bytes, hipStream_t s);
int mn_wino_bwd_data(const mn_conv2d* g, const float* dy, const float* w, float* dx, bool accum,
                     void* ws, size_t ws_bytes, hipStream_t s);
int mn_wino_fused_ws_bytes(const mn_conv2d* g, bool backward_data, size_t* bytes);
int mn_wino_fused_fwd(const mn_conv2d* g, const float* x, const float* w, const float* bias, float* y,
                      void* ws, size_t ws_bytes, hipStream_t s);
int mn_wino_fused_bwd_data(const mn_conv2d* g, const float* dy, const float* w, float* dx, bool accum,
                           void* ws, size_t ws_bytes, hipStream_t s);
int mn_wino_bwd_weight_ws_bytes(const mn_conv2d* g, size_t* bytes);
int mn_wino_fused_bwd_weight_ws_bytes(const mn_conv2d* g, size_t* bytes);
int mn_wino_fused_bwd_weight(const mn_conv2d* g, const float* dy, const float* x, float* dw, float* db,
                             void* ws, size_t ws_bytes, hipStream_t s);
int mn_wino_bwd_weight(const mn_conv2d* g, const float* dy, const float* x, float* dw, float* db,
                       void* ws, size_t ws_bytes, hipStream_t s);

// bf16 / channels-last kernels (conv_bf16.hip)
int mn_conv16_ws_bytes(const mn_conv2d* g, int direction, int variant, size_t* bytes);
int mn_conv16_fwd(const mn_conv2d* g, const void* x, const void* w, const void* bias, void* y,
                  void* ws, size_t ws_bytes, int variant, hipStream_t s);
int mn_conv16_bwd_data(const mn_conv2d* g, const void* dy, const void* w, void* dx, void* ws,
                       size_t ws_bytes, int variant, hipStream_t s);
int mn_conv16_bwd_weight(const mn_conv2d* g, const void* dy, const void* x, void* dw, void* ws,
                         size_t ws_bytes, int variant, hipStream_t s);

// fp32 through three bf16 slices per operand (conv_split.hip)
int mn_stem_ws_bytes(const mn_conv2d* g, int direction, size_t* bytes);
int mn_stem_bwd_weight(const mn_conv2d* g, const float* dy, const float* x, float* dw, float* db,
                       void* ws, size_t ws_bytes, hipStream_t s);
int mn_stem_fwd(const mn_conv2d* g, const float* x, const float* w, const float* bias, float* y,
                void* ws, size_t ws_bytes, hipStream_t s);
int mn_split_ws_bytes(const mn_conv2d* g, int direction, size_t* bytes);
int mn_split_pointwise(const mn_conv2d* g, int direction, const float* in, const float* w,
                       const float* bias, float* out, bool accumulate, void* ws, size_t ws_bytes,
                       hipStream_t s);

namespace mn_conv {

typedef float float16_t __attribute__((ext_vector_type(16)));

constexpr int kThreads = 256;  // 4 wavefronts
constexpr int BK = 16;         // depth of a staged tile, gather GEMM
constexpr int WBK = 32;        // depth of a staged tile, backward-weight
constexpr int kPad = 1;        // LDS row padding (floats)
constexpr int kMaxTaps = 49;

// Workgroup tile BM x BN computed by WM x WN wavefronts; each wavefront owns
// TM x TN MFMA tiles of 32 x 32.
template <int BM_, int BN_, int WM_, int WN_>
struct Tile {
  static constexpr int BM = BM_, BN = BN_, WM = WM_, WN = WN_;
  static constexpr int TM = BM / WM / 32, TN = BN / WN / 32;
  static_assert(WM * WN * 64 == kThreads && TM >= 1 && TN >= 1, "bad tile");
};
typedef Tile<128, 128, 2, 2> T128x128;
typedef Tile<64, 256, 1, 4> T64x256;
typedef Tile<64, 128, 1, 4> T64x128;
typedef Tile<128, 64, 4, 1> T128x64;
typedef Tile<64, 64, 2, 2> T64x64;

// n / d, exact while n * d < 2^32 (mul = floor(2^32 / d) + 1): e.g. n < 2^20 and d < 4096.
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

// Multiply one staged k-tile (DEPTH deep, k-major in LDS) into the accumulators.
template <class TL, int DEPTH, int LDA = TL::BM + kPad, int LDB = TL::BN + kPad>
__device__ __forceinline__ void mma_tile(const float (*As)[LDA],
                                         const float (*Bs)[LDB], int wm, int wn,
                                         int lane, float16_t (&acc)[TL::TM][TL::TN]) {
  const int r = lane & 31, half = lane >> 5;
  const int arow = wm * (TL::TM * 32) + r, bcol = wn * (TL::TN * 32) + r;
#pragma unroll
  for (int ks = 0; ks < DEPTH; ks += 2) {
    const int k = ks + half;
    float af[TL::TM], bf[TL::TN];
#pragma unroll
    for (int i = 0; i < TL::TM; ++i) af[i] = As[k][arow + 32 * i];
#pragma unroll
    for (int j = 0; j < TL::TN; ++j) bf[j] = Bs[k][bcol + 32 * j];
#pragma unroll
    for (int i = 0; i < TL::TM; ++i)
#pragma unroll
      for (int j = 0; j < TL::TN; ++j)
        acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(af[i], bf[j], acc[i][j], 0, 0, 0);
  }
}

// Row of accumulator register v within a 32x32 MFMA tile, for this lane
// (the column is lane % 32).
__device__ __forceinline__ int acc_row(int v, int lane) {
  return 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
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
  int ksplit, tiles_per_split;  // split reduction (ksplit > 1): grid.z slices of k-tiles
  int chunk;  // tap-major kernels: the reduction visits all taps of `chunk` channels, then the next block
  int accum;                    // add to what dst already holds instead of overwriting it
  uint32_t src_bytes, a_bytes;  // sizes of the source tensor and of the repacked A (PACKED)
  // batch > 1: grid.z independent problems of this shape (no split reduction then); problem z
  // reads a + z*a_batch and src + z*src_batch and writes dst + z*dst_batch (floats)
  int batch;
  size_t a_batch, src_batch, dst_batch;
  FastDiv divOHW, divOW;        // column -> (image, row, column) by multiplication ...
  int exact_div;                // ... unless ncols * OH*OW is beyond FastDiv's exact range
};

// Column c of the GEMM = output pixel (n, oh, ow).
__device__ __forceinline__ void split_column(const Gather& g, uint32_t c, uint32_t& n, uint32_t& oh,
                                             uint32_t& ow) {
  const uint32_t ohw = (uint32_t)g.OH * g.OW;
  n = g.exact_div ? c / ohw : g.divOHW.div(c);
  const uint32_t rem = c - n * ohw;
  oh = g.exact_div ? rem / (uint32_t)g.OW : g.divOW.div(rem);
  ow = rem - oh * g.OW;
}

// FAST: the source has a multiple of BK channels.  Then the reduction index
// runs tap-major (kk = tap*Cs + ch): a k-tile lies inside one tap, so the
// window test and the spatial offset are computed once per tile and thread,
// every address is a 32-bit byte offset = per-thread constant + per-tile
// scalar, and little vector ALU work competes with the matrix cores.
// Otherwise (e.g. 3 input channels) kk = ch*T + tap and every element is
// decomposed on its own.  All tensors are < 4 GB (checked by the host).
// PACKED (with FAST): `a` is a repacked copy A'[tap][ch][m] with rows of g.lda
// floats (a multiple of 128, zero padded), so a k-tile of A is BK contiguous
// row pieces: one 16-byte load per lane and row piece, no masks, and 8 cache
// lines per wavefront load instead of the ~20 a strided gather touches.
// FAST kernels fetch through raw buffer descriptors: a thread's byte offset is fixed for a
// whole tap, an element outside the window or the tensor gets an offset beyond the buffer
// and reads as zero (no masks when staging), and the per-tile part of an address is the
// scalar offset of the load: no vector arithmetic per tile.  Both tensors must be < 2 GB.
// POINT (with PACKED): a 1x1 filter, stride 1, no padding - the gather is the identity, a
// k-tile of B is BK contiguous rows of pixels, loaded and staged as 16-byte vectors too.
constexpr int kPadPacked = 4;  // keeps LDS rows 16-byte aligned for the 128-bit stores
constexpr uint32_t kBeyond = 0x80000000u;  // a byte offset past the end of any buffer
template <class TL, bool FAST, bool PACKED = false, bool POINT = false>
__global__ __launch_bounds__(kThreads) void gather_gemm_kernel(const Gather g,
                                                               const float* __restrict__ a_in,
                                                               const float* __restrict__ src_in,
                                                               const float* __restrict__ bias,
                                                               float* __restrict__ dst_in) {
  const float* a = a_in;
  const float* src = src_in;
  float* dst = dst_in;
  static_assert(!PACKED || FAST, "the packed operand is only used with the tap-major path");
  static_assert(!POINT || PACKED, "the pointwise path is built on the packed one");
  constexpr int BM = TL::BM, BN = TL::BN;
  constexpr int LDA = BM + (PACKED ? kPadPacked : kPad);
  constexpr int LDB = BN + (POINT ? kPadPacked : kPad);
  __shared__ __attribute__((aligned(16))) float lds_a[2][BK][LDA];
  __shared__ __attribute__((aligned(16))) float lds_b[2][BK][LDB];
  __shared__ int tdh[kMaxTaps], tdw[kMaxTaps], taoff[kMaxTaps];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / TL::WN, wn = wave % TL::WN;
  // XCD-aware order: each XCD works on a contiguous range of column tiles, all row tiles of a
  // column tile one after the other, so the workgroups that gather the same pixels (other
  // output channels, overlapping windows) share one L2 (strided 1x1, 256 -> 512 channels at
  // batch 184: 0.71 -> 0.41 ms).
  const uint32_t slot = xcd_slot();
  const uint32_t bz = slot / (gridDim.x * gridDim.y);
  const uint32_t in_z = slot - bz * (gridDim.x * gridDim.y);
  const uint32_t bx = in_z / gridDim.y, by = in_z - bx * gridDim.y;
  const int m0 = by * BM;
  const uint32_t n0 = bx * BN;
  if (g.batch > 1) {  // uniform
    a += (size_t)bz * g.a_batch;
    src += (size_t)bz * g.src_batch;
    dst += (size_t)bz * g.dst_batch;
  }
  if (tid < g.T) {
    tdh[tid] = g.dh[tid];
    tdw[tid] = g.dw[tid];
    taoff[tid] = g.aoff[tid];
  }
  __syncthreads();

  // B loader: this thread always fetches column bcol, rows brow0 + kBStep*i
  constexpr int kBStep = kThreads / BN, kBRows = BK / kBStep;
  constexpr int kAStep = kThreads / BK, kARows = BM / kAStep;
  const int bcol = tid % BN, brow0 = tid / BN;
  const uint32_t col = n0 + bcol;
  const bool col_ok = col < g.ncols;
  int ohs = 0, ows = 0;
  uint32_t img = 0;
  {
    uint32_t oh, ow;
    split_column(g, col_ok ? col : 0, img, oh, ow);
    ohs = oh * g.ish;
    ows = ow * g.isw;
  }
  // A loader: this thread always fetches k-column ak, rows arow0 + kAStep*i
  const int ak = tid % BK, arow0 = tid / BK;

  // per-thread constant byte offsets
  const uint32_t plane_b = (uint32_t)g.Hs * g.Ws * 4u;
  const uint32_t img_b = img * (uint32_t)g.Cs * plane_b;
  const uint32_t pix_b = img_b + (uint32_t)(ohs * g.Ws + ows) * 4u + brow0 * plane_b;
  uint32_t am_b[kARows];
  uint32_t am_ok = 0;
  if (!PACKED) {
#pragma unroll
    for (int i = 0; i < kARows; ++i) {
      const int m = m0 + arow0 + kAStep * i;
      const bool ok = m < g.M;
      // tap-major path: rows past M get an offset beyond the buffer and read as zero
      am_b[i] = ok ? (uint32_t)(((long long)m * g.lda + (FAST ? (long long)ak * g.cha : 0)) * 4)
                   : (FAST ? kBeyond : 0u);
      am_ok |= (ok ? 1u : 0u) << i;
    }
  }
  // packed A loader: float4 number f = tid + kThreads*i of the k-tile, row f / (BM/4)
  constexpr int kA4 = BM * BK / 4 / kThreads;
  float4_t ra4[kA4 > 0 ? kA4 : 1];
  uint32_t ap_b[kA4 > 0 ? kA4 : 1];
  if (PACKED) {
#pragma unroll
    for (int i = 0; i < kA4; ++i) {
      const int f = tid + kThreads * i;
      ap_b[i] = (uint32_t)(((long long)(f / (BM / 4)) * g.lda + m0 + 4 * (f % (BM / 4))) * 4);
    }
  }

  // pointwise B loader: float4 number f = tid + kThreads*i of the k-tile, row f / (BN/4)
  constexpr int kB4 = BN * BK / 4 / kThreads;
  float4_t rb4[kB4 > 0 ? kB4 : 1];
  uint32_t bp_b[kB4 > 0 ? kB4 : 1];
  if (POINT) {
    const uint32_t PQ = (uint32_t)g.OH * g.OW;  // a multiple of 4: a float4 stays inside an image
#pragma unroll
    for (int i = 0; i < kB4; ++i) {
      const int f = tid + kThreads * i;
      const uint32_t krow = f / (BN / 4), c4 = n0 + 4 * (f % (BN / 4));
      const bool ok = c4 < g.ncols;
      const uint32_t im = ok ? (g.exact_div ? c4 / PQ : g.divOHW.div(c4)) : 0u;
      const uint32_t px = ok ? c4 - im * PQ : 0u;
      // columns past the end read as zero (an offset beyond the buffer)
      bp_b[i] = ok ? (im * (uint32_t)g.Cs + krow) * plane_b + px * 4u : kBeyond;
    }
  }

  const char* sp = reinterpret_cast<const char*>(src);
  const char* ap = reinterpret_cast<const char*>(a);
  float ra[kARows], rb[kBRows];
  uint32_t b_ok = 0;  // bit i: rb[i] holds a window element (else it is staged as zero)
  bool a_ok = true;
  // FAST: what only changes when the reduction enters a new tap.  tap_b: this thread's byte
  // offset of (pixel shifted by the tap, channel brow0) or, outside the window, of an
  // in-bounds dummy whose value is staged as zero; tap_in: inside the window; tap_a: byte
  // offset of the tap's block of A (uniform).
  uint32_t tap_b = 0, tap_a = 0;
  bool tap_in = false;
  bool b_in = false;  // tap_in at the time of the last fetch: what stage() masks with
  const __amdgpu_buffer_rsrc_t src_buf = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<float*>(src), 0, FAST ? g.src_bytes : 0u, 0x00020000);
  const __amdgpu_buffer_rsrc_t a_buf = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<float*>(a), 0, FAST ? g.a_bytes : 0u, 0x00020000);
  auto enter_tap = [&](int t) {  // t uniform
    const int dh = tdh[t], dw = tdw[t];
    const int hh = ohs + dh, ww = ows + dw;
    tap_in = col_ok && (unsigned)hh < (unsigned)g.Hs && (unsigned)ww < (unsigned)g.Ws;
    tap_b = tap_in ? pix_b + (uint32_t)((dh * g.Ws + dw) * 4) : kBeyond;
    const int ao = __builtin_amdgcn_readfirstlane(taoff[t]);  // uniform: keep it in a scalar register
    tap_a = PACKED ? (uint32_t)((long long)ao * g.Cs * g.lda * 4) : (uint32_t)(ao * 4);
  };
  // Only issues loads, so they stay in flight behind the matrix instructions of the current
  // tile.  The per-tile part of every address is uniform (c0) and goes into the scalar offset
  // of the load; the per-thread offsets stay put for a whole tap.
  auto fetch_fast = [&](int c0) {  // c0 uniform
    b_in = tap_in;
    if (POINT) {
      const uint32_t so = (uint32_t)c0 * plane_b;
#pragma unroll
      for (int i = 0; i < kB4; ++i)
        rb4[i] = __builtin_bit_cast(float4_t, __builtin_amdgcn_raw_buffer_load_b128(src_buf, bp_b[i], so, 0));
    } else {
#pragma unroll
      for (int i = 0; i < kBRows; ++i)
        rb[i] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(
            src_buf, tap_b, (uint32_t)(c0 + kBStep * i) * plane_b, 0));
    }
    if (PACKED) {
      const uint32_t so = tap_a + (uint32_t)c0 * (uint32_t)g.lda * 4u;
#pragma unroll
      for (int i = 0; i < kA4; ++i)
        ra4[i] = __builtin_bit_cast(float4_t, __builtin_amdgcn_raw_buffer_load_b128(a_buf, ap_b[i], so, 0));
    } else {
      const uint32_t so = tap_a + (uint32_t)c0 * (uint32_t)g.cha * 4u;
#pragma unroll
      for (int i = 0; i < kARows; ++i)
        ra[i] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(a_buf, am_b[i], so, 0));
    }
  };
  auto fetch_any = [&](int k0) {
    b_ok = 0;
#pragma unroll
    for (int i = 0; i < kBRows; ++i) {
      const uint32_t kk = k0 + brow0 + kBStep * i;
      uint32_t off = 0;
      if (col_ok && kk < (uint32_t)g.Kd) {
        const uint32_t ch = g.divT.div(kk);
        const uint32_t t = kk - ch * g.T;
        const int hh = ohs + tdh[t], ww = ows + tdw[t];
        if ((unsigned)hh < (unsigned)g.Hs && (unsigned)ww < (unsigned)g.Ws) {
          off = img_b + ch * plane_b + (uint32_t)(hh * g.Ws + ww) * 4u;
          b_ok |= 1u << i;
        }
      }
      rb[i] = *reinterpret_cast<const float*>(sp + off);
    }
    const uint32_t kk = k0 + ak;
    a_ok = kk < (uint32_t)g.Kd;
    uint32_t koff = 0;
    if (a_ok) {
      const uint32_t ch = g.divT.div(kk);
      koff = (uint32_t)(((long long)ch * g.cha + taoff[kk - ch * g.T]) * 4);
    }
#pragma unroll
    for (int i = 0; i < kARows; ++i) {
      const bool mok = a_ok && ((am_ok >> i) & 1u);
      ra[i] = *reinterpret_cast<const float*>(ap + (mok ? am_b[i] + koff : 0u));
    }
  };
  auto stage = [&](int buf) {
    if (POINT) {
#pragma unroll
      for (int i = 0; i < kB4; ++i) {
        const int f = tid + kThreads * i;
        *reinterpret_cast<float4_t*>(&lds_b[buf][f / (BN / 4)][4 * (f % (BN / 4))]) = rb4[i];
      }
    } else {
#pragma unroll
      for (int i = 0; i < kBRows; ++i) {
        // tap-major: what lies outside the window was fetched as zero already
        const bool in = FAST ? true : (((b_ok >> i) & 1u) != 0);
        lds_b[buf][brow0 + kBStep * i][bcol] = in ? rb[i] : 0.f;
      }
    }
    if (PACKED) {
#pragma unroll
      for (int i = 0; i < kA4; ++i) {
        const int f = tid + kThreads * i;
        *reinterpret_cast<float4_t*>(&lds_a[buf][f / (BM / 4)][4 * (f % (BM / 4))]) = ra4[i];
      }
    } else {
#pragma unroll
      for (int i = 0; i < kARows; ++i)
        lds_a[buf][ak][arow0 + kAStep * i] = (FAST || (a_ok && ((am_ok >> i) & 1u))) ? ra[i] : 0.f;
    }
  };

  float16_t acc[TL::TM][TL::TN];
#pragma unroll
  for (int i = 0; i < TL::TM; ++i)
#pragma unroll
    for (int j = 0; j < TL::TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  // reduction range of this workgroup: all k-tiles, or slice blockIdx.z of them (split
  // reduction: the slices are added into a cleared output with atomics)
  const int all_tiles = (g.Kd + BK - 1) / BK;
  const int kt_begin = g.ksplit > 1 ? (int)bz * g.tiles_per_split : 0;
  const int ktiles = g.ksplit > 1 ? min(kt_begin + g.tiles_per_split, all_tiles) : all_tiles;
  if (kt_begin < ktiles) {
    int t = 0, c0 = 0;  // FAST: position of the tile being fetched
    int c_lo = 0, c_hi = g.chunk;  // the block of channels the taps are cycled over
    if (FAST && kt_begin > 0) {
      const int per_tap = g.chunk / BK, per_chunk = per_tap * g.T;
      const int ch = kt_begin / per_chunk, r = kt_begin - ch * per_chunk;
      c_lo = ch * g.chunk;
      c_hi = c_lo + g.chunk;
      t = r / per_tap;
      c0 = c_lo + (r - t * per_tap) * BK;
    }
    if (FAST) enter_tap(t);
    auto fetch_next = [&](int kt) {
      if (FAST) {
        fetch_fast(c0);
        c0 += BK;
        if (c0 == c_hi) {
          ++t;
          if (t == g.T) {
            t = 0;
            c_lo = c_hi;
            c_hi += g.chunk;
          }
          c0 = c_lo;
          if (c_lo < g.Cs) enter_tap(t);
        }
      } else {
        fetch_any(kt * BK);
      }
    };
    fetch_next(kt_begin);
    stage(0);
    __syncthreads();
    for (int kt = kt_begin; kt < ktiles; ++kt) {
      const int buf = (kt - kt_begin) & 1;
      if (kt + 1 < ktiles) fetch_next(kt + 1);
      mma_tile<TL, BK, LDA, LDB>(lds_a[buf], lds_b[buf], wm, wn, lane, acc);
      if (kt + 1 < ktiles) stage(buf ^ 1);
      __syncthreads();
    }
  }

  // epilogue: lane owns columns (nj*32 + lane%32) and 16 rows per MFMA tile.  What kind of
  // store it is and whether the tile has rows beyond M are uniform, so they select one of a
  // few straight-line copies of the loop instead of being tested per element; an element's
  // address is a per-thread byte offset plus a compile-time multiple of the plane size.
  const uint32_t plane4 = (uint32_t)g.DH * g.DW * 4u;
  char* dstb = reinterpret_cast<char*>(dst);
  const bool add_bias = bias != nullptr && bz == 0;
  const int mbase = m0 + wm * (TL::TM * 32) + 4 * (lane >> 5);
  auto emit = [&](auto full_tag, auto how_tag) {
    constexpr bool kFull = decltype(full_tag)::value;
    constexpr int kHow = decltype(how_tag)::value;
#pragma unroll
    for (int nj = 0; nj < TL::TN; ++nj) {
      const uint32_t c = n0 + wn * (TL::TN * 32) + nj * 32 + (lane & 31);
      if (c >= g.ncols) continue;
      uint32_t n, oh, ow;
      split_column(g, c, n, oh, ow);
      const uint32_t col_b =
          ((n * (uint32_t)g.M * g.DH + (oh * g.osh + g.oh0)) * (uint32_t)g.DW + (ow * g.osw + g.ow0)) * 4u +
          (uint32_t)mbase * plane4;
#pragma unroll
      for (int mi = 0; mi < TL::TM; ++mi) {
#pragma unroll
        for (int v = 0; v < 16; ++v) {
          const int dm = mi * 32 + 8 * (v >> 2) + (v & 3);
          if (!kFull && mbase + dm >= g.M) continue;
          float r = acc[mi][nj][v];
          if (add_bias) r += bias[mbase + dm];
          float* o = reinterpret_cast<float*>(dstb + (col_b + (uint32_t)dm * plane4));
          if (kHow == 1)
            atomicAdd(o, r);  // split reduction: the slices meet in a cleared output
          else if (kHow == 2)
            *o += r;          // accumulate: every element belongs to one thread of the launch
          else if (kHow == 3)
            st_stream(o, r);  // dense output, written once and not read here: around the caches
          else
            *o = r;           // strided (parity-class) outputs share cache lines between launches
        }
      }
    }
  };
  using std::integral_constant;
  const int how = g.ksplit > 1 ? 1 : (g.accum ? 2 : ((g.osh == 1 && g.osw == 1) ? 3 : 0));
  if (m0 + BM <= g.M) {
    switch (how) {
      case 1: emit(integral_constant<bool, true>{}, integral_constant<int, 1>{}); break;
      case 2: emit(integral_constant<bool, true>{}, integral_constant<int, 2>{}); break;
      case 3: emit(integral_constant<bool, true>{}, integral_constant<int, 3>{}); break;
      default: emit(integral_constant<bool, true>{}, integral_constant<int, 0>{}); break;
    }
  } else {
    switch (how) {
      case 1: emit(integral_constant<bool, false>{}, integral_constant<int, 1>{}); break;
      case 2: emit(integral_constant<bool, false>{}, integral_constant<int, 2>{}); break;
      case 3: emit(integral_constant<bool, false>{}, integral_constant<int, 3>{}); break;
      default: emit(integral_constant<bool, false>{}, integral_constant<int, 0>{}); break;
    }
  }
}

// ------------------------------------------------------- backward weight --
// A thread's position d = n*PQ + pq in the (n, p, q) reduction, moved STEP at a time: the
// image index and the in-image offset are kept up to date by addition instead of two
// divisions per tile.
template <int STEP>
struct DepthPos {
  uint32_t d, n, pq;
  __device__ __forceinline__ DepthPos(uint32_t d0, uint32_t PQ) : d(d0), n(d0 / PQ) {
    pq = d0 - n * PQ;
  }
  __device__ __forceinline__ void advance(uint32_t PQ) {
    d += STEP;
    pq += STEP;
    if (PQ < STEP) {  // uniform: images smaller than a step (may cross several per step)
      const uint32_t k = pq / PQ;
      n += k;
      pq -= k * PQ;
    } else if (pq >= PQ) {
      pq -= PQ;
      ++n;
    }
  }
};

// dw[k][c][r][s] = sum over (n, p, q) dy[n,k,p,q] * x[n,c,p*sH + r*dH - pH, q*sW + s*dW - pW]
// GEMM: rows = k (M = K), columns = (c, r, s) (ncols = C*R*S), depth = (n, p, q).
struct WGrad {
  int K, C, R, S, H, W, P, Q, N;
  int sH, sW, pH, pW, dH, dW;
  uint32_t depth;       // N*P*Q
  uint32_t ncols;       // C*R*S
  FastDiv divRS, divS, divQ;
  int exact_div;             // P*Q or Q beyond FastDiv's range: divide the slow way
  uint32_t dy_bytes, x_bytes;  // tensor sizes, for the kernels that read through buffer descriptors
  uint32_t tiles_per_split;  // k-tiles handled by one blockIdx.z
  int mode;             // 0: store, 1: atomicAdd into dw, 2: store partial [z][K][ncols]
};

// Row sums of the dy tiles one workgroup has staged: LANES consecutive lanes (one per depth
// position) hold the partial sums of the same rows; they are added in a fixed order and lane 0
// of each group hands the result over the same way the tile itself is written (store, atomic
// add, or one partial per split).
template <int LANES, int ROWS>
__device__ __forceinline__ void store_row_sums(float (&row_sum)[ROWS], float* __restrict__ db,
                                               const WGrad& g, int first_row, int row_step,
                                               int depth_lane, uint32_t split = blockIdx.z) {
#pragma unroll
  for (int i = 0; i < ROWS; ++i) {
    float v = row_sum[i];
#pragma unroll
    for (int off = LANES / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    const int m = first_row + row_step * i;
    if (depth_lane == 0 && m < g.K) {
      if (g.mode == 1)
        atomicAdd(db + m, v);
      else
        db[(g.mode == 2 ? (size_t)split * g.K : 0) + m] = v;
    }
  }
}

// DB: the workgroups of the first column tile also reduce the rows of their dy tile (the values
// they fetch anyway) into the bias gradient db[k] = sum over (n, p, q) of dy[n,k,p,q].
template <class TL, bool DB = false>
__global__ __launch_bounds__(kThreads) void wgrad_kernel(const WGrad g,
                                                         const float* __restrict__ dy,
                                                         const float* __restrict__ x,
                                                         float* __restrict__ out,
                                                         float* __restrict__ db) {
  constexpr int BM = TL::BM, BN = TL::BN;
  __shared__ float lds_a[2][WBK][BM + kPad];
  __shared__ float lds_b[2][WBK][BN + kPad];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / TL::WN, wn = wave % TL::WN;
  // XCD-aware order: each XCD gets whole slices of the reduction, so the workgroups that read
  // the same positions of dy and x (other row and column tiles) share one L2
  const uint32_t slot = xcd_slot();
  const uint32_t bz = slot / (gridDim.x * gridDim.y);
  const uint32_t in_z = slot - bz * (gridDim.x * gridDim.y);
  const uint32_t by = in_z / gridDim.x, bx = in_z - by * gridDim.x;
  const int m0 = by * BM;
  const uint32_t n0 = bx * BN;
  const uint32_t PQ = (uint32_t)g.P * g.Q;

  // this thread always fetches depth lane kdl and rows row0 + kStep*i of both tiles
  constexpr int kStep = kThreads / WBK, kRowsA = BM / kStep, kRowsB = BN / kStep;
  const int kdl = tid % WBK, row0 = tid / WBK;

  // A rows: dy offset of row m (bytes), relative to the (n, p, q) of the tile
  uint32_t am_b[kRowsA];
  uint32_t am_ok = 0;
#pragma unroll
  for (int i = 0; i < kRowsA; ++i) {
    const int m = m0 + row0 + kStep * i;
    const bool ok = m < g.K;
    am_b[i] = ok ? (uint32_t)m * PQ * 4u : 0u;
    am_ok |= (ok ? 1u : 0u) << i;
  }
  // B rows: the (c, r, s) of a row never changes: byte offset inside an image and window shift
  uint32_t bo_b[kRowsB];
  int16_t bo_h[kRowsB], bo_w[kRowsB];
  uint32_t bo_ok = 0;
#pragma unroll
  for (int i = 0; i < kRowsB; ++i) {
    const uint32_t cc = n0 + row0 + kStep * i;
    bo_b[i] = 0;
    bo_h[i] = 0;
    bo_w[i] = 0;
    if (cc < g.ncols) {
      const uint32_t c = g.divRS.div(cc);
      const uint32_t rs = cc - c * (uint32_t)(g.R * g.S);
      const uint32_t r = g.divS.div(rs), s = rs - r * g.S;
      bo_h[i] = (int16_t)((int)r * g.dH - g.pH);
      bo_w[i] = (int16_t)((int)s * g.dW - g.pW);
      bo_b[i] = (uint32_t)(((int)(c * g.H) + bo_h[i]) * g.W + bo_w[i]) * 4u;
      bo_ok |= 1u << i;
    }
  }

  const char* dyp = reinterpret_cast<const char*>(dy);
  const char* xp = reinterpret_cast<const char*>(x);
  float ra[kRowsA], rb[kRowsB];
  float row_sum[DB ? kRowsA : 1] = {};
  const bool sums_rows = DB && bx == 0;
  uint32_t a_mask = 0, b_mask = 0;
  const uint32_t total_tiles = (g.depth + WBK - 1) / WBK;
  const uint32_t t_begin = bz * g.tiles_per_split;
  const uint32_t t_end = min(t_begin + g.tiles_per_split, total_tiles);
  DepthPos<WBK> pos(t_begin * WBK + kdl, PQ);
  // fetches the tile at the current depth position and moves on to the next one
  auto fetch = [&]() {
    const bool d_ok = pos.d < g.depth;
    const uint32_t n = d_ok ? pos.n : 0u, pq = d_ok ? pos.pq : 0u;
    const uint32_t p = g.exact_div ? pq / (uint32_t)g.Q : g.divQ.div(pq);
    const uint32_t q = pq - p * g.Q;
    pos.advance(PQ);
    const uint32_t abase = ((n * (uint32_t)g.K) * PQ + pq) * 4u;
    a_mask = d_ok ? am_ok : 0u;
#pragma unroll
    for (int i = 0; i < kRowsA; ++i)
      ra[i] = *reinterpret_cast<const float*>(dyp + (((a_mask >> i) & 1u) ? abase + am_b[i] : 0u));
    const int h0 = (int)p * g.sH, w0 = (int)q * g.sW;
    const uint32_t bbase = ((n * (uint32_t)g.C * g.H + h0) * (uint32_t)g.W + w0) * 4u;
    b_mask = 0;
#pragma unroll
    for (int i = 0; i < kRowsB; ++i) {
      const int hh = h0 + bo_h[i], ww = w0 + bo_w[i];
      const bool ok = d_ok && ((bo_ok >> i) & 1u) && (unsigned)hh < (unsigned)g.H &&
                      (unsigned)ww < (unsigned)g.W;
      b_mask |= (ok ? 1u : 0u) << i;
      rb[i] = *reinterpret_cast<const float*>(xp + (ok ? bbase + bo_b[i] : 0u));
    }
  };
  auto stage = [&](int buf) {
#pragma unroll
    for (int i = 0; i < kRowsA; ++i) {
      const float v = ((a_mask >> i) & 1u) ? ra[i] : 0.f;
      lds_a[buf][kdl][row0 + kStep * i] = v;
      if constexpr (DB) {
        if (sums_rows) row_sum[i] += v;
      }
    }
#pragma unroll
    for (int i = 0; i < kRowsB; ++i)
      lds_b[buf][kdl][row0 + kStep * i] = ((b_mask >> i) & 1u) ? rb[i] : 0.f;
  };

  float16_t acc[TL::TM][TL::TN];
#pragma unroll
  for (int i = 0; i < TL::TM; ++i)
#pragma unroll
    for (int j = 0; j < TL::TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  if (t_begin < t_end) {
    fetch();
    stage(0);
    __syncthreads();
    for (uint32_t kt = t_begin; kt < t_end; ++kt) {
      const int buf = (kt - t_begin) & 1;
      if (kt + 1 < t_end) fetch();
      mma_tile<TL, WBK>(lds_a[buf], lds_b[buf], wm, wn, lane, acc);
      if (kt + 1 < t_end) stage(buf ^ 1);
      __syncthreads();
    }
  }
  if constexpr (DB) {
    if (sums_rows) store_row_sums<WBK, kRowsA>(row_sum, db, g, m0 + row0, kStep, kdl, bz);
  }

  float* base = out;
  if (g.mode == 2) base += (size_t)bz * g.K * g.ncols;
#pragma unroll
  for (int nj = 0; nj < TL::TN; ++nj) {
    const uint32_t c = n0 + wn * (TL::TN * 32) + nj * 32 + (lane & 31);
    if (c >= g.ncols) continue;
#pragma unroll
    for (int mi = 0; mi < TL::TM; ++mi) {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int m = m0 + wm * (TL::TM * 32) + mi * 32 + acc_row(v, lane);
        if (m < g.K) {
          float* o = base + (size_t)m * g.ncols + c;
          if (g.mode == 1)
            atomicAdd(o, acc[mi][nj][v]);
          else
            *o = acc[mi][nj][v];
        }
      }
    }
  }
}


// Writes a workgroup's accumulators as the (m0.., c0.., tap) piece of dw (tap-major column
// tiles): plain store, atomic add, or the partial of split blockIdx.z.
template <class TL>
__device__ __forceinline__ void store_tap_tile(const WGrad& g, float16_t (&acc)[TL::TM][TL::TN],
                                               float* __restrict__ out, int m0, uint32_t c0,
                                               uint32_t tap, int wm, int wn, int lane,
                                               uint32_t split = blockIdx.z) {
  float* base = out;
  if (g.mode == 2) base += (size_t)split * g.K * g.ncols;
  const uint32_t RS = (uint32_t)g.R * g.S;
#pragma unroll
  for (int nj = 0; nj < TL::TN; ++nj) {
    const uint32_t c = c0 + wn * (TL::TN * 32) + nj * 32 + (lane & 31);
#pragma unroll
    for (int mi = 0; mi < TL::TM; ++mi) {
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int m = m0 + wm * (TL::TM * 32) + mi * 32 + acc_row(v, lane);
        float* o = base + (size_t)m * g.ncols + c * RS + tap;
        if (g.mode == 1)
          atomicAdd(o, acc[mi][nj][v]);
        else
          *o = acc[mi][nj][v];
      }
    }
  }
}

// The same GEMM with the columns ordered tap-major, for C % BN == 0 and K % BM == 0:
// blockIdx.x = tap * (C / BN) + channel tile, so a column tile lies inside ONE tap.
// Then the window shift is a per-workgroup scalar, a thread's window test is one
// comparison per k-tile (its depth lane fixes (p, q)), row addresses are arithmetic
// progressions instead of per-row tables, and no row needs a bounds mask: fewer
// vector registers (more resident waves) and far less address arithmetic between
// the matrix instructions.
template <class TL, int DEPTH, bool DB = false>
__global__ __launch_bounds__(kThreads) void wgrad_tap_kernel(const WGrad g,
                                                             const float* __restrict__ dy,
                                                             const float* __restrict__ x,
                                                             float* __restrict__ out,
                                                             float* __restrict__ db) {
  constexpr int BM = TL::BM, BN = TL::BN;
  __shared__ float lds_a[2][DEPTH][BM + kPad];
  __shared__ float lds_b[2][DEPTH][BN + kPad];
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / TL::WN, wn = wave % TL::WN;
  const int m0 = blockIdx.y * BM;
  const uint32_t ctiles = (uint32_t)g.C / BN;
  const uint32_t tap = blockIdx.x / ctiles;
  const uint32_t c0 = (blockIdx.x - tap * ctiles) * BN;
  const uint32_t r = g.divS.div(tap), sx = tap - r * g.S;
  const int dh = (int)r * g.dH - g.pH, dw = (int)sx * g.dW - g.pW;
  const uint32_t PQ = (uint32_t)g.P * g.Q;

  constexpr int kStep = kThreads / DEPTH, kRowsA = BM / kStep, kRowsB = BN / kStep;
  const int kdl = tid % DEPTH, row0 = tid / DEPTH;
  const uint32_t a_row0 = (uint32_t)(m0 + row0) * PQ * 4u, a_step = (uint32_t)kStep * PQ * 4u;
  const uint32_t HW4 = (uint32_t)g.H * g.W * 4u;
  const uint32_t b_row0 = (c0 + row0) * HW4 + (uint32_t)((dh * g.W + dw) * 4), b_step = kStep * HW4;

  const char* dyp = reinterpret_cast<const char*>(dy);
  const char* xp = reinterpret_cast<const char*>(x);
  float ra[kRowsA], rb[kRowsB];
  float row_sum[DB ? kRowsA : 1] = {};
  const bool sums_rows = DB && blockIdx.x == 0;
  bool a_ok = false, b_ok = false;
  const uint32_t total_tiles = (g.depth + DEPTH - 1) / DEPTH;
  const uint32_t t_begin = blockIdx.z * (g.tiles_per_split * (WBK / DEPTH));
  const uint32_t t_end = min(t_begin + g.tiles_per_split * (WBK / DEPTH), total_tiles);
  DepthPos<DEPTH> pos(t_begin * DEPTH + kdl, PQ);
  // fetches the tile at the current depth position and moves on to the next one
  auto fetch = [&]() {
    a_ok = pos.d < g.depth;
    const uint32_t n = a_ok ? pos.n : 0u, pq = a_ok ? pos.pq : 0u;
    const uint32_t p = g.exact_div ? pq / (uint32_t)g.Q : g.divQ.div(pq);
    const uint32_t q = pq - p * g.Q;
    pos.advance(PQ);
    const uint32_t abase = ((n * (uint32_t)g.K) * PQ + pq) * 4u + a_row0;
#pragma unroll
    for (int i = 0; i < kRowsA; ++i)
      ra[i] = *reinterpret_cast<const float*>(dyp + (abase + a_step * i));
    const int h0 = (int)p * g.sH, w0 = (int)q * g.sW;
    b_ok = a_ok && (unsigned)(h0 + dh) < (unsigned)g.H && (unsigned)(w0 + dw) < (unsigned)g.W;
    // an element outside the window is staged as zero; its load reads the row's first element
    const uint32_t bbase = b_ok ? ((n * (uint32_t)g.C * g.H + h0) * (uint32_t)g.W + w0) * 4u + b_row0
                                : (c0 + row0) * HW4;
#pragma unroll
    for (int i = 0; i < kRowsB; ++i)
      rb[i] = *reinterpret_cast<const float*>(xp + (bbase + b_step * i));
  };
  auto stage = [&](int buf) {
#pragma unroll
    for (int i = 0; i < kRowsA; ++i) {
      const float v = a_ok ? ra[i] : 0.f;
      lds_a[buf][kdl][row0 + kStep * i] = v;
      if constexpr (DB) {
        if (sums_rows) row_sum[i] += v;
      }
    }
#pragma unroll
    for (int i = 0; i < kRowsB; ++i) lds_b[buf][kdl][row0 + kStep * i] = b_ok ? rb[i] : 0.f;
  };

  float16_t acc[TL::TM][TL::TN];
#pragma unroll
  for (int i = 0; i < TL::TM; ++i)
#pragma unroll
    for (int j = 0; j < TL::TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  if (t_begin < t_end) {
    fetch();
    stage(0);
    __syncthreads();
    for (uint32_t kt = t_begin; kt < t_end; ++kt) {
      const int buf = (kt - t_begin) & 1;
      if (kt + 1 < t_end) fetch();
      mma_tile<TL, DEPTH>(lds_a[buf], lds_b[buf], wm, wn, lane, acc);
      if (kt + 1 < t_end) stage(buf ^ 1);
      __syncthreads();
    }
  }
  if constexpr (DB) {
    if (sums_rows) store_row_sums<DEPTH, kRowsA>(row_sum, db, g, m0 + row0, kStep, kdl);
  }

  store_tap_tile<TL>(g, acc, out, m0, c0, tap, wm, wn, lane);
}

// Tap-major backward-weight for images whose P*Q is a multiple of 4 (so is every depth tile
// boundary, and N*P*Q).  Vector instructions that are not matrix instructions take issue
// slots from the matrix pipe, so this variant is built to need few of them per tile:
//  * LDS tiles are ROW-major, [row][DEPTH], the 16-byte chunks of a row XOR-swizzled by the
//    row so that both the 128-bit fragment reads (8 rows at a time) and the staging writes are
//    bank-conflict free without padding.  A lane's operands for 8 matrix steps are 2 chunks.
//    The reduction index a lane feeds into step s is k = half * DEPTH/2 + s (any pairing of
//    the tile's depths is a valid order of summation, A and B use the same one).
//  * dy (and x for a 1x1, stride-1, unpadded filter: VECB) is contiguous along the depth, so
//    it is fetched as float4 and staged with one 128-bit write per fetch; byte offsets are
//    carried from tile to tile by addition (image wrap: one compare), the row part of an
//    address is the scalar offset of a buffer load, and what lies beyond the reduction or
//    outside the window is fetched as zero (an offset past the buffer): no staging masks.
//  * the gathered x of a windowed filter keeps one (p, q) position per thread, also carried
//    by addition.
// Without VECA (P*Q not a multiple of 4, or unaligned tensors) dy is fetched lane by lane
// like the gathered x, with the same carried addresses and the same LDS layout.
// Images so small that one tile could cross two of them go to wgrad_tap_kernel instead.
template <class TL, int DEPTH, bool DB, bool VECA, bool VECB_>
__global__ __launch_bounds__(kThreads) void wgrad_rows_kernel(const WGrad g,
                                                              const float* __restrict__ dy,
                                                              const float* __restrict__ x,
                                                              float* __restrict__ out,
                                                              float* __restrict__ db) {
  constexpr bool VECB = VECA && VECB_;  // without float4 alignment both operands go lane by lane
  constexpr int BM = TL::BM, BN = TL::BN;
  constexpr int CPR = DEPTH / 4;  // 16-byte chunks per staged row
  constexpr int RP = 32 / DEPTH;  // staged rows per 128 bytes of LDS
  static_assert(DEPTH == 16 || DEPTH == 32, "row-major staging is laid out for 16 or 32 deep tiles");
  __shared__ __attribute__((aligned(16))) float lds_a[2][BM * DEPTH];
  __shared__ __attribute__((aligned(16))) float lds_b[2][BN * DEPTH];
  auto swz = [](int row) { return (row / RP) & (CPR - 1); };  // chunk c of a row sits at c ^ swz(row)
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int wm = wave / TL::WN, wn = wave % TL::WN;
  // XCD-aware order: each XCD gets whole slices of the reduction, so all the (tap, channel
  // tile, row tile) workgroups that read the same positions of dy and x share one L2 (layer2
  // 3x3 stride 2 at batch 184: 0.54 -> 0.41 ms).
  const uint32_t slot = xcd_slot();
  const uint32_t bz = slot / (gridDim.x * gridDim.y);
  const uint32_t in_z = slot - bz * (gridDim.x * gridDim.y);
  const uint32_t by = in_z / gridDim.x, bx = in_z - by * gridDim.x;
  const int m0 = by * BM;
  const uint32_t ctiles = (uint32_t)g.C / BN;
  const uint32_t tap = bx / ctiles;
  const uint32_t c0 = (bx - tap * ctiles) * BN;
  const uint32_t r_tap = g.divS.div(tap), s_tap = tap - r_tap * g.S;
  const int dh = (int)r_tap * g.dH - g.pH, dw = (int)s_tap * g.dW - g.pW;
  const uint32_t PQ = (uint32_t)g.P * g.Q, PQ4 = PQ * 4u;
  const uint32_t HW4 = (uint32_t)g.H * g.W * 4u;

  const uint32_t total_tiles = (g.depth + DEPTH - 1) / DEPTH;
  const uint32_t t_begin = bz * (g.tiles_per_split * (WBK / DEPTH));
  const uint32_t t_end = min(t_begin + g.tiles_per_split * (WBK / DEPTH), total_tiles);

  // float4 loader: float4 number f = tid + kThreads*i of a tile is (row f / CPR, chunk f % CPR)
  constexpr int kRowsPass = kThreads / CPR;
  constexpr int kA4 = BM / kRowsPass, kB4 = BN / kRowsPass;
  const int chunk = tid % CPR, vrow0 = tid / CPR;
  // scalar loader of the gathered operand: depth lane kdl, rows row0 + kStep*i
  constexpr int kStep = kThreads / DEPTH, kRowsA = BM / kStep, kRowsB = BN / kStep;
  const int kdl = tid % DEPTH, row0 = tid / DEPTH;

  // depth position of this thread's float4 and the byte offsets that follow it
  uint32_t vd = t_begin * DEPTH + 4 * chunk;
  uint32_t vpq, a_off, bv_off = 0;
  {
    const uint32_t n = vd / PQ;
    vpq = vd - n * PQ;
    a_off = (n * (uint32_t)g.K * PQ + vpq) * 4u + (uint32_t)(m0 + vrow0) * PQ4;
    if (VECB) bv_off = (n * (uint32_t)g.C * PQ + vpq) * 4u + (c0 + vrow0) * PQ4;
  }
  const uint32_t a_wrap = (uint32_t)(g.K - 1) * PQ4, bv_wrap = (uint32_t)(g.C - 1) * PQ4;
  // (p, q) of this thread's gathered element, and the byte offset of its image
  uint32_t bd = t_begin * DEPTH + kdl, bp = 0, bq = 0, img_off = 0;
  // a step of DEPTH crosses kq whole rows of the image and rq pixels; the host only sends
  // images here that a step cannot cross twice (P*Q >= DEPTH and kq + 1 <= P)
  const uint32_t kq = DEPTH / (uint32_t)g.Q, rq = DEPTH - kq * g.Q;
  const uint32_t chw4 = (uint32_t)g.C * HW4;
  const uint32_t b_row0 = (c0 + row0) * HW4 + (uint32_t)((dh * g.W + dw) * 4), b_step = kStep * HW4;
  uint32_t as_off = 0;  // scalar dy loader (!VECA): byte offset of (image, pixel, row m0 + row0)
  if (!VECB) {
    const uint32_t n = bd / PQ, pq = bd - n * PQ;
    bp = pq / g.Q;
    bq = pq - bp * g.Q;
    img_off = n * chw4;
    as_off = (n * (uint32_t)g.K * PQ + pq) * 4u + (uint32_t)(m0 + row0) * PQ4;
  }

  // Both tensors are read through buffer descriptors: the per-thread part of an address is one
  // 32-bit byte offset, the row part the load's scalar offset, and an element that is not to
  // be read (beyond the reduction, outside the window) gets an offset past the buffer and
  // arrives as zero, so staging has no masks.
  const __amdgpu_buffer_rsrc_t dy_buf =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(dy), 0, g.dy_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t x_buf =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(x), 0, g.x_bytes, 0x00020000);
  const uint32_t a_row_step = (VECA ? kRowsPass : kStep) * PQ4;
  const uint32_t b_row_step = VECB ? kRowsPass * PQ4 : b_step;
  float4_t ra4[VECA ? kA4 : 1], rb4[VECB ? kB4 : 1];
  float ra[VECA ? 1 : kRowsA], rb[VECB ? 1 : kRowsB];
  float row_sum[DB ? (VECA ? kA4 : kRowsA) : 1] = {};
  const bool sums_rows = DB && bx == 0;
  bool a_ok = false, b_ok = false;
  auto fetch = [&]() {
    if (VECA) {
      a_ok = vd < g.depth;
      const uint32_t ao = a_ok ? a_off : kBeyond;
#pragma unroll
      for (int i = 0; i < kA4; ++i)
        ra4[i] = __builtin_bit_cast(float4_t, __builtin_amdgcn_raw_buffer_load_b128(dy_buf, ao, i * a_row_step, 0));
    } else {
      a_ok = bd < g.depth;
      const uint32_t ao = a_ok ? as_off : kBeyond;
#pragma unroll
      for (int i = 0; i < kRowsA; ++i)
        ra[i] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(dy_buf, ao, i * a_row_step, 0));
    }
    if (VECB) {
      const uint32_t bo = a_ok ? bv_off : kBeyond;
#pragma unroll
      for (int i = 0; i < kB4; ++i)
        rb4[i] = __builtin_bit_cast(float4_t, __builtin_amdgcn_raw_buffer_load_b128(x_buf, bo, i * b_row_step, 0));
    } else {
      const int h0 = (int)__umul24(bp, (uint32_t)g.sH), w0 = (int)__umul24(bq, (uint32_t)g.sW);
      b_ok = bd < g.depth && (unsigned)(h0 + dh) < (unsigned)g.H && (unsigned)(w0 + dw) < (unsigned)g.W;
      const uint32_t bbase = b_ok ? img_off + (uint32_t)(h0 * g.W + w0) * 4u + b_row0 : kBeyond;
#pragma unroll
      for (int i = 0; i < kRowsB; ++i)
        rb[i] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(x_buf, bbase, i * b_row_step, 0));
      // next tile
      bd += DEPTH;
      bq += rq;
      bp += kq;
      if (!VECA) as_off += DEPTH * 4;
      if (bq >= (uint32_t)g.Q) {
        bq -= g.Q;
        ++bp;
      }
      if (bp >= (uint32_t)g.P) {  // next image
        bp -= g.P;
        img_off += chw4;
        if (!VECA) as_off += a_wrap;
      }
    }
    if (VECA) {
      vd += DEPTH;
      vpq += DEPTH;
      a_off += DEPTH * 4;
      if (VECB) bv_off += DEPTH * 4;
      if (vpq >= PQ) {
        vpq -= PQ;
        a_off += a_wrap;
        if (VECB) bv_off += bv_wrap;
      }
    }
  };
  // LDS byte offsets of this thread's staging writes (the swizzle is the same for all its rows)
  const uint32_t va_w = (uint32_t)(vrow0 * DEPTH + ((chunk ^ swz(vrow0)) << 2));
  const uint32_t sb_w = (uint32_t)(row0 * DEPTH + ((((kdl >> 2) ^ swz(row0)) << 2) | (kdl & 3)));
  auto stage = [&](int buf) {
    if constexpr (VECA) {
#pragma unroll
      for (int i = 0; i < kA4; ++i) {
        const float4_t v = ra4[i];
        *reinterpret_cast<float4_t*>(&lds_a[buf][va_w + i * kRowsPass * DEPTH]) = v;
        if constexpr (DB) {
          if (sums_rows) row_sum[i] += (v[0] + v[1]) + (v[2] + v[3]);
        }
      }
    } else {
#pragma unroll
      for (int i = 0; i < kRowsA; ++i) {
        lds_a[buf][sb_w + i * kStep * DEPTH] = ra[i];
        if constexpr (DB) {
          if (sums_rows) row_sum[i] += ra[i];
        }
      }
    }
    if (VECB) {
#pragma unroll
      for (int i = 0; i < kB4; ++i)
        *reinterpret_cast<float4_t*>(&lds_b[buf][va_w + i * kRowsPass * DEPTH]) = rb4[i];
    } else {
#pragma unroll
      for (int i = 0; i < kRowsB; ++i) lds_b[buf][sb_w + i * kStep * DEPTH] = rb[i];
    }
  };

  float16_t acc[TL::TM][TL::TN];
#pragma unroll
  for (int i = 0; i < TL::TM; ++i)
#pragma unroll
    for (int j = 0; j < TL::TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;

  // fragment reads: lane (r, half) owns rows r of each 32-row block and depths half*DEPTH/2 ...
  const int r = lane & 31, half = lane >> 5;
  const int fa_row = wm * (TL::TM * 32) + r, fb_row = wn * (TL::TN * 32) + r;
  const int f_swz = swz(r);  // block bases are multiples of 32: the swizzle only depends on r
  auto multiply = [&](int buf) {
#pragma unroll
    for (int g8 = 0; g8 < DEPTH / 16; ++g8) {
      const int cb = half * (CPR / 2) + 2 * g8;
      float4_t a4[TL::TM][2], b4[TL::TN][2];
#pragma unroll
      for (int i = 0; i < TL::TM; ++i)
#pragma unroll
        for (int h = 0; h < 2; ++h)
          a4[i][h] = *reinterpret_cast<const float4_t*>(
              &lds_a[buf][(fa_row + 32 * i) * DEPTH + (((cb + h) ^ f_swz) << 2)]);
#pragma unroll
      for (int j = 0; j < TL::TN; ++j)
#pragma unroll
        for (int h = 0; h < 2; ++h)
          b4[j][h] = *reinterpret_cast<const float4_t*>(
              &lds_b[buf][(fb_row + 32 * j) * DEPTH + (((cb + h) ^ f_swz) << 2)]);
#pragma unroll
      for (int st = 0; st < 8; ++st)
#pragma unroll
        for (int i = 0; i < TL::TM; ++i)
#pragma unroll
          for (int j = 0; j < TL::TN; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(a4[i][st >> 2][st & 3], b4[j][st >> 2][st & 3],
                                                             acc[i][j], 0, 0, 0);
    }
  };

  if (t_begin < t_end) {
    fetch();
    stage(0);
    __syncthreads();
    for (uint32_t kt = t_begin; kt < t_end; ++kt) {
      const int buf = (kt - t_begin) & 1;
      if (kt + 1 < t_end) fetch();
      multiply(buf);
      if (kt + 1 < t_end) stage(buf ^ 1);
      __syncthreads();
    }
  }
  if constexpr (DB) {
    if (sums_rows) {
      if constexpr (VECA)
        store_row_sums<CPR, kA4>(row_sum, db, g, m0 + vrow0, kRowsPass, chunk, bz);
      else
        store_row_sums<DEPTH, kRowsA>(row_sum, db, g, m0 + row0, kStep, kdl, bz);
    }
  }
  store_tap_tile<TL>(g, acc, out, m0, c0, tap, wm, wn, lane, bz);
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

// Clears n floats; float4 stores where the pointer allows.
__global__ __launch_bounds__(kThreads) void fill_zero_kernel(float* p, size_t n) {
  const size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x;
  const size_t n4 = (reinterpret_cast<uintptr_t>(p) & 15) == 0 ? n / 4 : 0;
  if (i < n4) {
    const float4_t z = {0.f, 0.f, 0.f, 0.f};
    reinterpret_cast<float4_t*>(p)[i] = z;
  }
  // tail (or everything, if unaligned): grid covers at least n/4 + 1 threads
  for (size_t j = n4 * 4 + i; j < n; j += (size_t)gridDim.x * kThreads) p[j] = 0.f;
}

// out[(t*Cs + ch)*Mp + m] = A(m, ch, t) = a[m*lda + ch*cha + t] for m < M, else 0
__global__ __launch_bounds__(kThreads) void pack_weights_kernel(const float* __restrict__ a,
                                                                float* __restrict__ out, int M,
                                                                int Mp, int Cs, int T,
                                                                long long lda, long long cha) {
  const size_t i = (size_t)blockIdx.x * kThreads + threadIdx.x;
  const size_t n = (size_t)T * Cs * Mp;
  if (i >= n) return;
  const int m = (int)(i % Mp);
  const size_t row = i / Mp;
  const int ch = (int)(row % Cs), t = (int)(row / Cs);
  out[i] = m < M ? a[(size_t)m * lda + (size_t)ch * cha + t] : 0.f;
}

static long long packed_rows(long long M) { return (M + 127) / 128 * 128; }
// The repacked-weight kernels address both operands through buffer descriptors with byte
// offsets below 2^31; larger tensors run variant 1 with the variant-0 kernel.
// Bytes of the weight tensor, or 0 if it cannot be addressed with 31-bit byte offsets.
static uint32_t weight_bytes(const mn_conv2d* g) {
  const unsigned long long b = (unsigned long long)g->K * g->C * g->R * g->S * sizeof(float);
  return b < (1ull << 31) ? (uint32_t)b : 0u;
}
static bool buffers_fit(size_t src_floats, size_t a_floats) {
  return src_floats < (1ull << 29) && a_floats < (1ull << 29);
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
  // the kernels address every tensor with 32-bit byte offsets
  const long long lim = 1ll << 30;  // elements
  if ((long long)g->N * g->C * g->H * g->W >= lim || (long long)g->N * g->K * g->P * g->Q >= lim ||
      (long long)g->K * g->C * g->R * g->S >= lim)
    return MN_EUNSUPPORTED;
  return MN_OK;
}

// Tile choice, from sweeps over the ResNet-50 shapes at batch 184 on MI355X.
// Weights read in place: 64 x 128 is within a few percent of the best tile everywhere
// (its 6 waves per SIMD hide the staging latency better than the larger tiles' 3), GEMMs
// with at most 64 rows want all four wavefronts side by side on the columns, and the
// element-wise path (channels not a multiple of 16) always takes 64 x 128: the wider
// tiles spill there.  Repacked weights: the A tile costs one load per lane, so 128 rows
// per workgroup (each gathered column element reused twice as often) wins from 128 rows
// up, most of all for strided gathers (stride-2 forward: 51 -> 81, 75 -> 102 TFLOP/s).
static int pick_tile(long long M, long long ncols, bool fast, bool packed) {
  (void)ncols;
  if (!fast) return 2;
  if (packed) return M <= 64 ? 2 : 3;
  return M <= 64 ? 1 : 2;
}

// The tap-major kernels address both operands through buffer descriptors with byte offsets
// below 2^31 (g.a_bytes is set by the callers, 0 if the operand is too large).
static bool fast_path(const Gather& g) {
  const unsigned long long src_bytes = (unsigned long long)g.N * g.Cs * g.Hs * g.Ws * sizeof(float);
  return g.T > 0 && g.Cs % BK == 0 && src_bytes < (1ull << 31) && g.a_bytes > 0 && g.a_bytes < (1u << 31);
}

template <class TL>
static void launch_gather_t(const Gather& g, const float* a, const float* src, const float* bias,
                            float* dst, hipStream_t s, bool packed) {
  dim3 grid((g.ncols + TL::BN - 1) / TL::BN, (g.M + TL::BM - 1) / TL::BM,
            g.batch > 1 ? g.batch : (g.ksplit > 1 ? g.ksplit : 1));
  // pointwise: the gather is the identity and pixels come in whole float4
  const bool point = packed && g.T == 1 && g.dh[0] == 0 && g.dw[0] == 0 && g.ish == 1 &&
                     g.isw == 1 && g.Hs == g.OH && g.Ws == g.OW && (g.OH * g.OW) % 4 == 0 &&
                     mn_aligned(src, 16);
  if (point)
    gather_gemm_kernel<TL, true, true, true><<<grid, kThreads, 0, s>>>(g, a, src, bias, dst);
  else if (packed)
    gather_gemm_kernel<TL, true, true><<<grid, kThreads, 0, s>>>(g, a, src, bias, dst);
  else if (fast_path(g))
    gather_gemm_kernel<TL, true><<<grid, kThreads, 0, s>>>(g, a, src, bias, dst);
  else if constexpr (TL::BN <= 128)
    gather_gemm_kernel<TL, false><<<grid, kThreads, 0, s>>>(g, a, src, bias, dst);
  else  // the element-wise path only exists for tiles up to 128 columns: wider ones would spill
    launch_gather_t<T64x128>(g, a, src, bias, dst, s, packed);
}

static void tile_dims(int tile, int* bm, int* bn);

// Few, long workgroups quantise badly over 256 CUs (2.2 per CU run as 3 rounds): when a
// launch has fewer than ~6 workgroups per CU, a long reduction and a dense output, slice the
// reduction so that there are ~8 per CU and add the slices into a cleared output.
static void plan_split(Gather& g, int tile, bool allow, int max_split) {
  g.ksplit = 1;
  g.tiles_per_split = 0;
  if (!allow || g.osh != 1 || g.osw != 1) return;
  int bm, bn;
  tile_dims(tile, &bm, &bn);
  const long long wgs = ((long long)(g.ncols + bn - 1) / bn) * ((g.M + bm - 1) / bm);
  const int ktiles = (g.Kd + BK - 1) / BK;
  if (wgs >= 6 * 256 || ktiles < 32) return;
  int want = (int)((8 * 256 + wgs - 1) / wgs);
  if (want > ktiles / 16) want = ktiles / 16;  // at least 16 k-tiles per slice
  if (want > max_split) want = max_split;
  if (want <= 1) return;
  g.tiles_per_split = (ktiles + want - 1) / want;
  g.ksplit = (ktiles + g.tiles_per_split - 1) / g.tiles_per_split;
  if (g.ksplit <= 1) g.ksplit = 1;
}

// `packed`: a = the repacked operand (pack_weights_kernel) with rows of g.lda floats.
// `split_ok`: the caller allows a split reduction (dst is then cleared here first).
static void launch_gather(Gather g, const float* a, const float* src, const float* bias,
                          float* dst, hipStream_t s, bool packed = false, bool split_ok = false,
                          int max_split = 8, int tile = -1) {
  if (g.ncols == 0 || g.M == 0) return;
  if (fast_path(g)) g.src_bytes = (uint32_t)((size_t)g.N * g.Cs * g.Hs * g.Ws * sizeof(float));
  g.divOHW = make_fastdiv((uint32_t)(g.OH * g.OW));
  g.divOW = make_fastdiv((uint32_t)g.OW);
  // multiplication by the reciprocal is exact while dividend * divisor < 2^32
  g.exact_div = ((unsigned long long)(g.ncols + 256) * (unsigned long long)(g.OH * g.OW) >= (1ull << 32)) ? 1 : 0;
  if (tile < 0) tile = pick_tile(g.M, g.ncols, fast_path(g), packed);
  plan_split(g, tile, split_ok && packed && g.batch <= 1, max_split);
  // Tap after tap over ALL channels re-reads each pixel once per tap with the whole channel
  // range in between, far more than an L2 holds across the workgroups of an XCD.  Cycling the
  // taps over a block of 2-4 k-tiles keeps the re-reads in cache; shorter blocks re-enter taps
  // (a few vector instructions each) more often.
  g.chunk = g.Cs;
  if (g.T > 1 && fast_path(g)) {
    const int want = g.Cs >= 256 ? 64 : 32;
    if (g.Cs % want == 0) g.chunk = want;
  }
  if (g.ksplit > 1 && !g.accum) {
    const size_t n = (size_t)g.N * g.M * g.DH * g.DW;
    fill_zero_kernel<<<(unsigned)((n / 4 + kThreads) / kThreads), kThreads, 0, s>>>(dst, n);
  }
  switch (tile) {
    case 1: launch_gather_t<T64x256>(g, a, src, bias, dst, s, packed); break;
    case 2: launch_gather_t<T64x128>(g, a, src, bias, dst, s, packed); break;
    case 3: launch_gather_t<T128x64>(g, a, src, bias, dst, s, packed); break;
    case 4: launch_gather_t<T64x64>(g, a, src, bias, dst, s, packed); break;
    default: launch_gather_t<T128x128>(g, a, src, bias, dst, s, packed); break;
  }
}

// Split of the (n, p, q) reduction: enough workgroups for ~2 per CU.
static int wgrad_tile(const mn_conv2d* g, int variant) {
  // from the same sweeps: 128 x 128 for windows, 128 x 64 for 1x1 filters, 64 rows for K <= 64
  const long long ncols = (long long)g->C * g->R * g->S;
  int tile;
  if (g->K <= 64) {
    // 64 columns per tile when 128 would mostly pad (the 3-channel stem: 147 columns)
    const long long pad128 = (ncols + 127) / 128 * 128, pad64 = (ncols + 63) / 64 * 64;
    tile = (ncols <= 64 || 4 * pad128 >= 5 * pad64) ? 4 : 2;
  }
  else
    tile = (g->R * g->S == 1 || ncols <= 64) ? 3 : 0;
  // a 64-wide column tile where it lets the tap-major kernel run (C a multiple of 64, not 128)
  if (variant == 1 && g->C % 128 != 0 && g->C % 64 == 0 && g->R * g->S > 1) {
    if (tile == 2) tile = 4;
    if (tile == 0) tile = 3;
  }
  return tile;
}
static bool wgrad_tap_major(const mn_conv2d* g, int bm, int bn) {
  return g->C % bn == 0 && g->K % bm == 0;
}
static void tile_dims(int tile, int* bm, int* bn) {
  switch (tile) {
    case 1: *bm = 64; *bn = 256; break;
    case 2: *bm = 64; *bn = 128; break;
    case 3: *bm = 128; *bn = 64; break;
    case 4: *bm = 64; *bn = 64; break;
    default: *bm = 128; *bn = 128; break;
  }
}
// Split of the (n, p, q) reduction: enough workgroups for ~3 per CU.
static void wgrad_split(const mn_conv2d* g, int variant, int* splits, int* tiles_per_split) {
  int bm, bn;
  tile_dims(wgrad_tile(g, variant), &bm, &bn);
  const long long depth = (long long)g->N * g->P * g->Q;
  const long long total_tiles = (depth + WBK - 1) / WBK;
  const long long out_tiles =
      (((long long)g->C * g->R * g->S + bn - 1) / bn) * (((long long)g->K + bm - 1) / bm);
  // All workgroups of the launch should be resident at once: one more than the CUs can hold
  // runs as a second round on its own and nearly doubles the time.  Resident workgroups per
  // CU by tile (LDS / register footprint): 128x128 2 (3 in the 16-deep tap-major kernel),
  // 128x64 and 64x128 3, 64x64 4.
  const int tile = wgrad_tile(g, variant);
  const bool tap = wgrad_tap_major(g, bm, bn) && (variant == 1 || g->R * g->S == 1);
  const int per_cu = tile == 0 ? (tap ? 3 : 2) : (tile == 4 ? 4 : 3);
  long long slots = 256ll * per_cu;
  long long want = slots / out_tiles;  // rounded down: never a partial extra round
  if (want > total_tiles) want = total_tiles;
  if (want > 256) want = 256;
  if (want < 1) want = 1;
  const long long tps = (total_tiles + want - 1) / want;
  *tiles_per_split = (int)(tps < 1 ? 1 : tps);
  *splits = (int)((total_tiles + *tiles_per_split - 1) / (*tiles_per_split));
  if (*splits < 1) *splits = 1;
}

}  // namespace mn_conv

// `batch` independent GEMMs in one launch (used by the Winograd variant, conv_wino.hip):
// dst[b][m][col] = sum over ch of a[b][ch][m] * src[b][ch][col], with a = [batch][Cs][Mp]
// (rows of Mp floats, Mp a multiple of 128 and >= M, zero padded), src = [batch][Cs][cols],
// dst = [batch][M][cols]; Cs a multiple of 16, cols a multiple of 4, 16-byte aligned pointers,
// every slice below 2 GB.  Runs the pointwise path of the gather GEMM (both operands fetched
// as 16-byte vectors through buffer descriptors).
int mn_conv_batched_gemm(const float* a, const float* src, float* dst, int M, int Mp, int Cs,
                         uint32_t cols, int batch, hipStream_t s) {
  using namespace mn_conv;
  if (M <= 0 || Cs <= 0 || cols == 0 || batch <= 0) return MN_EINVAL;
  if (Cs % BK != 0 || cols % 4 != 0 || Mp % 128 != 0 || Mp < M) return MN_EUNSUPPORTED;
  if (!mn_aligned(a, 16) || !mn_aligned(src, 16) || !mn_aligned(dst, 16)) return MN_EINVAL;
  if (!buffers_fit((size_t)Cs * cols, (size_t)Cs * Mp) || (size_t)M * cols >= (1ull << 30))
    return MN_EUNSUPPORTED;
  Gather q = {};
  q.M = M;
  q.T = 1;
  q.Kd = Cs;
  q.divT = make_fastdiv(1);
  q.N = 1;
  q.OH = 1;
  q.OW = (int)cols;
  q.ncols = cols;
  q.Cs = Cs;
  q.Hs = 1;
  q.Ws = (int)cols;
  q.ish = q.isw = 1;
  q.DH = 1;
  q.DW = (int)cols;
  q.osh = q.osw = 1;
  q.lda = Mp;
  q.cha = 1;
  q.a_bytes = (uint32_t)((size_t)Cs * Mp * sizeof(float));
  q.batch = batch;
  q.a_batch = (size_t)Cs * Mp;
  q.src_batch = (size_t)Cs * cols;
  q.dst_batch = (size_t)M * cols;
  launch_gather(q, a, src, nullptr, dst, s, true, false);
  return mn_launch_status();
}

extern "C" {

int mn_conv_n_variants(int direction) {
  switch (direction) {
    case MN_CONV_FWD:
      return 5;
    case MN_CONV_BWD_DATA:
      return 5;
    case MN_CONV_BWD_WEIGHT:
      return 4;
    default:
      return 0;
  }
}

int mn_conv_n_variants_for(int direction, int dtype) {
  if (dtype == MN_F32) return mn_conv_n_variants(direction);
  // bf16: two tiers per direction (conv_bf16.hip)
  if (dtype == MN_BF16) return mn_conv_n_variants(direction) > 0 ? 2 : 0;
  return 0;
}

int mn_conv_ws_bytes(const mn_conv2d* g, int direction, int variant, int dtype, size_t* bytes) {
  using namespace mn_conv;
  if (!bytes) return MN_EINVAL;
  *bytes = 0;
  const int st = check(g);
  if (st != MN_OK) return st;
  if (variant < 0 || variant >= mn_conv_n_variants(direction)) return MN_EUNSUPPORTED;
  if (dtype == MN_BF16)  // there is no bf16 Winograd tier
    return variant <= 1 ? mn_conv16_ws_bytes(g, direction, variant, bytes) : MN_EUNSUPPORTED;
  if (dtype != MN_F32) return MN_EUNSUPPORTED;
  if (variant == 2)
    return direction == MN_CONV_BWD_WEIGHT ? mn_wino_bwd_weight_ws_bytes(g, bytes)
                                           : mn_wino_ws_bytes(g, direction == MN_CONV_BWD_DATA, bytes);
  if (variant == 3)
    return direction == MN_CONV_BWD_WEIGHT ? mn_wino_fused_bwd_weight_ws_bytes(g, bytes)
                                           : mn_wino_fused_ws_bytes(g, direction == MN_CONV_BWD_DATA, bytes);
  if (variant == 4) return mn_split_ws_bytes(g, direction, bytes);
  const size_t wsize = (size_t)g->K * g->C * g->R * g->S * sizeof(float);
  // variant 1 of the gather directions: the repacked weight operand (rows padded to 128); the
  // 3 -> 64 channel 7x7 / 2 stem runs a kernel of its own with transposed weights
  if (direction == MN_CONV_FWD && variant == 1) {
    if (mn_stem_ws_bytes(g, direction, bytes) == MN_OK) return MN_OK;
    *bytes = (size_t)g->R * g->S * g->C * packed_rows(g->K) * sizeof(float);
  }
  if (direction == MN_CONV_BWD_DATA && variant == 1)
    *bytes = (size_t)g->R * g->S * g->K * packed_rows(g->C) * sizeof(float);
  if (direction == MN_CONV_BWD_WEIGHT && variant == 1) {
    int splits, tiles;
    wgrad_split(g, 1, &splits, &tiles);
    // one partial weight gradient and one partial bias gradient (K floats) per split
    *bytes = splits > 1 ? (wsize + (size_t)g->K * sizeof(float)) * splits : 0;
    // the stem runs a kernel of its own (one partial result per workgroup)
    size_t stem_bytes = 0;
    if (mn_stem_ws_bytes(g, direction, &stem_bytes) == MN_OK && stem_bytes > *bytes) *bytes = stem_bytes;
  }
  return MN_OK;
}

int mn_conv_fwd(const mn_conv2d* g, const void* x, const void* w, const void* bias, void* y,
                void* ws, size_t ws_bytes, int variant, int dtype, mn_stream_t stream) {
  using namespace mn_conv;
  const int st = check(g);
  if (st != MN_OK) return st;
  if (variant < 0 || variant > 4 || (variant >= 2 && dtype != MN_F32)) return MN_EUNSUPPORTED;
  if (g->N == 0) return MN_OK;
  if (!x || !w || !y) return MN_EINVAL;
  if (dtype == MN_BF16) return mn_conv16_fwd(g, x, w, bias, y, ws, ws_bytes, variant, mn_stream(stream));
  if (dtype != MN_F32) return MN_EUNSUPPORTED;
  if (variant == 2)
    return mn_wino_fwd(g, (const float*)x, (const float*)w, (const float*)bias, (float*)y, ws,
                       ws_bytes, mn_stream(stream));
  if (variant == 3)
    return mn_wino_fused_fwd(g, (const float*)x, (const float*)w, (const float*)bias, (float*)y, ws,
                             ws_bytes, mn_stream(stream));
  if (variant == 4)
    return mn_split_pointwise(g, MN_CONV_FWD, (const float*)x, (const float*)w, (const float*)bias,
                              (float*)y, false, ws, ws_bytes, mn_stream(stream));
  if (variant == 1) {
    size_t stem_bytes;
    if (mn_stem_ws_bytes(g, MN_CONV_FWD, &stem_bytes) == MN_OK)
      return mn_stem_fwd(g, (const float*)x, (const float*)w, (const float*)bias, (float*)y, ws,
                         ws_bytes, mn_stream(stream));
  }
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
  hipStream_t s = mn_stream(stream);
  const float* a = (const float*)w;
  q.a_bytes = weight_bytes(g);  // weights read in place
  // the repacked operand needs the tap-major path; other shapes run variant 1 like variant 0
  const bool packed = variant == 1 && fast_path(q) &&
                      buffers_fit((size_t)g->N * g->C * g->H * g->W, (size_t)q.T * q.Cs * packed_rows(q.M));
  if (packed) {
    const long long Mp = packed_rows(q.M);
    const size_t n = (size_t)q.T * q.Cs * Mp;
    if (!ws || ws_bytes < n * sizeof(float) || !mn_aligned(ws, 16)) return MN_EINVAL;
    pack_weights_kernel<<<(unsigned)((n + kThreads - 1) / kThreads), kThreads, 0, s>>>(
        a, (float*)ws, q.M, (int)Mp, q.Cs, q.T, q.lda, q.cha);
    a = (const float*)ws;
    q.lda = Mp;
    q.a_bytes = (uint32_t)(n * sizeof(float));
  }
  // A forward may be run again by a schedule that recomputes it, and what follows (a ReLU mask,
  // max-pool indices) must then come out bit for bit the same.  With two slices the atomic
  // additions into the cleared output give the same bits in either order (0 + a + b and
  // 0 + b + a round identically); with more they would not.
  launch_gather(q, a, (const float*)x, (const float*)bias, (float*)y, s, packed, packed, 2);
  return mn_launch_status();
}

static int conv_bwd_data(const mn_conv2d* g, const void* dy, const void* w, void* dx, void* ws,
                         size_t ws_bytes, int variant, int dtype, mn_stream_t stream, bool accum) {
  using namespace mn_conv;
  const int st = check(g);
  if (st != MN_OK) return st;
  if (variant < 0 || variant > 4 || (variant >= 2 && dtype != MN_F32)) return MN_EUNSUPPORTED;
  if (g->N == 0) return MN_OK;
  if (!dy || !w || !dx) return MN_EINVAL;
  hipStream_t s = mn_stream(stream);
  if (dtype == MN_BF16)
    return accum ? MN_EUNSUPPORTED : mn_conv16_bwd_data(g, dy, w, dx, ws, ws_bytes, variant, s);
  if (dtype != MN_F32) return MN_EUNSUPPORTED;
  if (variant == 2)
    return mn_wino_bwd_data(g, (const float*)dy, (const float*)w, (float*)dx, accum, ws, ws_bytes, s);
  if (variant == 3)
    return mn_wino_fused_bwd_data(g, (const float*)dy, (const float*)w, (float*)dx, accum, ws, ws_bytes, s);
  if (variant == 4)
    return mn_split_pointwise(g, MN_CONV_BWD_DATA, (const float*)dy, (const float*)w, nullptr,
                              (float*)dx, accum, ws, ws_bytes, s);
  const int RS = g->R * g->S;
  const float* a = (const float*)w;
  uint32_t a_bytes = weight_bytes(g);  // size of the A operand: the weights, or their repacked copy
  long long lda = RS, cha = (long long)g->C * RS;  // read w[k][c][r][s] as A(c, k, rs)
  const bool packed = variant == 1 && g->K % BK == 0 &&
                      buffers_fit((size_t)g->N * g->K * g->P * g->Q, (size_t)RS * g->K * packed_rows(g->C));
  if (packed) {  // A'[rs][k][c], rows of Cp floats
    const long long Cp = packed_rows(g->C);
    const size_t n = (size_t)RS * g->K * Cp;
    if (!ws || ws_bytes < n * sizeof(float) || !mn_aligned(ws, 16)) return MN_EINVAL;
    pack_weights_kernel<<<(unsigned)((n + kThreads - 1) / kThreads), kThreads, 0, s>>>(
        a, (float*)ws, g->C, (int)Cp, g->K, RS, lda, cha);
    a = (const float*)ws;
    lda = Cp;
    a_bytes = (uint32_t)(n * sizeof(float));
  }
  // Classes no tap can reach (e.g. 1x1 filters with stride 2) are plain zeros: clear dx once
  // with full-width stores instead of scattering zeros class by class.
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
  if (empty_class && !accum) {  // (accumulating: those positions simply keep their values)
    const size_t n = (size_t)g->N * g->C * g->H * g->W;
    fill_zero_kernel<<<(unsigned)((n / 4 + kThreads) / kThreads), kThreads, 0, s>>>((float*)dx, n);
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
      if (T == 0) continue;  // already cleared above
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
      q.a_bytes = a_bytes;
      q.cha = cha;
      q.accum = accum ? 1 : 0;
      launch_gather(q, a, (const float*)dy, nullptr, (float*)dx, s, packed,
                    packed && g->sH == 1 && g->sW == 1);
    }
  }
  return mn_launch_status();
}

int mn_conv_bwd_data(const mn_conv2d* g, const void* dy, const void* w, void* dx, void* ws,
                     size_t ws_bytes, int variant, int dtype, mn_stream_t stream) {
  return conv_bwd_data(g, dy, w, dx, ws, ws_bytes, variant, dtype, stream, false);
}

int mn_conv_bwd_data_accumulate(const mn_conv2d* g, const void* dy, const void* w, void* dx,
                                void* ws, size_t ws_bytes, int variant, int dtype,
                                mn_stream_t stream) {
  return conv_bwd_data(g, dy, w, dx, ws, ws_bytes, variant, dtype, stream, true);
}

// db_out: where the bias gradient goes (fp32, K elements), or null for the weight gradient alone.
static int conv_bwd_weight(const mn_conv2d* g, const void* dy, const void* x, void* dw, void* db_out,
                           void* ws, size_t ws_bytes, int variant, int dtype, mn_stream_t stream) {
  using namespace mn_conv;
  const int st = check(g);
  if (st != MN_OK) return st;
  if (dtype != MN_F32 && dtype != MN_BF16) return MN_EUNSUPPORTED;
  if (variant < 0 || variant > 3 || (variant >= 2 && dtype != MN_F32)) return MN_EUNSUPPORTED;
  if (!dw) return MN_EINVAL;
  hipStream_t s = mn_stream(stream);
  if (variant == 3) {
    if (g->N == 0) return MN_EUNSUPPORTED;
    if (!dy || !x) return MN_EINVAL;
    return mn_wino_fused_bwd_weight(g, (const float*)dy, (const float*)x, (float*)dw, (float*)db_out,
                                    ws, ws_bytes, s);
  }
  if (variant == 2) {
    if (g->N == 0) return MN_EUNSUPPORTED;  // nothing to reduce: variants 0 and 1 clear dw
    if (!dy || !x) return MN_EINVAL;
    return mn_wino_bwd_weight(g, (const float*)dy, (const float*)x, (float*)dw, (float*)db_out, ws,
                              ws_bytes, s);
  }
  if (dtype == MN_BF16) {
    if (db_out) return MN_EUNSUPPORTED;     // the bf16 kernel has no bias-gradient epilogue
    if (g->N == 0) return MN_EUNSUPPORTED;  // nothing to reduce: the caller clears dw itself
    if (!dy || !x) return MN_EINVAL;
    return mn_conv16_bwd_weight(g, dy, x, dw, ws, ws_bytes, variant, s);
  }
  if (db_out && !mn_aligned(db_out, 4)) return MN_EINVAL;
  const size_t nw = (size_t)g->K * g->C * g->R * g->S;
  const size_t nb = (size_t)g->K;
  float* db = (float*)db_out;
  if (g->N == 0) {
    fill_zero_kernel<<<(unsigned)((nw / 4 + kThreads) / kThreads), kThreads, 0, s>>>((float*)dw, nw);
    if (db) fill_zero_kernel<<<(unsigned)((nb / 4 + kThreads) / kThreads), kThreads, 0, s>>>(db, nb);
    return mn_launch_status();
  }
  if (!dy || !x) return MN_EINVAL;
  if (variant == 1) {
    size_t stem_bytes = 0;
    if (mn_stem_ws_bytes(g, MN_CONV_BWD_WEIGHT, &stem_bytes) == MN_OK && ws && ws_bytes >= stem_bytes &&
        mn_aligned(ws, 16))
      return mn_stem_bwd_weight(g, (const float*)dy, (const float*)x, (float*)dw, db, ws, ws_bytes, s);
  }
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
  q.divQ = make_fastdiv(g->Q);
  const unsigned long long dy_bytes = (unsigned long long)g->N * g->K * g->P * g->Q * sizeof(float);
  const unsigned long long x_bytes = (unsigned long long)g->N * g->C * g->H * g->W * sizeof(float);
  q.dy_bytes = (uint32_t)dy_bytes;
  q.x_bytes = (uint32_t)x_bytes;
  q.exact_div = ((long long)g->P * g->Q > (1ll << 20) || g->Q >= 4096) ? 1 : 0;
  int splits, tps;
  wgrad_split(g, variant, &splits, &tps);
  q.tiles_per_split = tps;
  float* out = (float*)dw;
  float* db_dst = db;  // where the kernel leaves its row sums
  if (splits == 1) {
    q.mode = 0;
  } else if (variant == 0) {
    q.mode = 1;
    fill_zero_kernel<<<(unsigned)((nw / 4 + kThreads) / kThreads), kThreads, 0, s>>>((float*)dw, nw);
    if (db) fill_zero_kernel<<<(unsigned)((nb / 4 + kThreads) / kThreads), kThreads, 0, s>>>(db, nb);
  } else {
    q.mode = 2;
    // partial weight gradients, then (always reserved) one partial bias gradient per split
    if (!ws || ws_bytes < (nw + nb) * sizeof(float) * splits || !mn_aligned(ws, 4)) return MN_EINVAL;
    out = (float*)ws;
    if (db) db_dst = (float*)ws + nw * splits;
  }
  const int tile = wgrad_tile(g, variant);
  int bm, bn;
  tile_dims(tile, &bm, &bn);
  // with atomics, a tap-major tile would scatter them R*S floats apart: only for 1x1 filters
  if (wgrad_tap_major(g, bm, bn) && (q.mode != 1 || g->R * g->S == 1)) {
    dim3 grid(g->R * g->S * (g->C / bn), g->K / bm, splits);
    // row-major staging; float4 fetches of dy for images of a multiple of 4 pixels and 16-byte
    // aligned tensors, of x too where the filter is a plain 1x1
    const bool vecb = g->R * g->S == 1 && g->sH == 1 && g->sW == 1 && g->pH == 0 && g->pW == 0;
    const bool veca = ((long long)g->P * g->Q) % 4 == 0 && mn_aligned(dy, 16) && (!vecb || mn_aligned(x, 16));
    bool rows = (long long)g->P * g->Q >= 32 && 32 / g->Q + 1 <= g->P &&
                dy_bytes < (1ull << 31) && x_bytes < (1ull << 31);  // buffer offsets below 2^31
    if (rows) {
#define MN_ROWS_V(TL, D, B, V)                                                                   \
  if (veca)                                                                                      \
    wgrad_rows_kernel<TL, D, B, true, V><<<grid, kThreads, 0, s>>>(q, (const float*)dy,          \
                                                                   (const float*)x, out, db_dst); \
  else                                                                                           \
    wgrad_rows_kernel<TL, D, B, false, false><<<grid, kThreads, 0, s>>>(                         \
        q, (const float*)dy, (const float*)x, out, db_dst)
#define MN_ROWS(TL, D)              \
  if (db) {                         \
    if (vecb) {                     \
      MN_ROWS_V(TL, D, true, true); \
    } else {                        \
      MN_ROWS_V(TL, D, true, false); \
    }                               \
  } else {                          \
    if (vecb) {                     \
      MN_ROWS_V(TL, D, false, true); \
    } else {                        \
      MN_ROWS_V(TL, D, false, false); \
    }                               \
  }
      switch (tile) {
        case 2: MN_ROWS(T64x128, 32); break;
        case 3: MN_ROWS(T128x64, 32); break;
        case 4: MN_ROWS(T64x64, 32); break;
        default: MN_ROWS(T128x128, 16); break;
      }
#undef MN_ROWS
#undef MN_ROWS_V
    } else {
    int deep = tile == 0 ? 16 : 32;  // 128 x 128 at depth 32 leaves LDS for 2 workgroups per CU only
#define MN_TAP_D(TL, D)                                                                           \
  if (db)                                                                                         \
    wgrad_tap_kernel<TL, D, true><<<grid, kThreads, 0, s>>>(q, (const float*)dy, (const float*)x, \
                                                            out, db_dst);                         \
  else                                                                                            \
    wgrad_tap_kernel<TL, D><<<grid, kThreads, 0, s>>>(q, (const float*)dy, (const float*)x, out,  \
                                                      nullptr)
#define MN_TAP(TL)       \
  if (deep == 16) {      \
    MN_TAP_D(TL, 16);    \
  } else {               \
    MN_TAP_D(TL, 32);    \
  }
    switch (tile) {
      case 2: MN_TAP(T64x128); break;
      case 3: MN_TAP(T128x64); break;
      case 4: MN_TAP(T64x64); break;
      default: MN_TAP(T128x128); break;
    }
#undef MN_TAP
#undef MN_TAP_D
    }
  } else {
    dim3 grid((q.ncols + bn - 1) / bn, (g->K + bm - 1) / bm, splits);
#define MN_GEN(TL)                                                                              \
  if (db)                                                                                       \
    wgrad_kernel<TL, true><<<grid, kThreads, 0, s>>>(q, (const float*)dy, (const float*)x, out, \
                                                     db_dst);                                   \
  else                                                                                          \
    wgrad_kernel<TL><<<grid, kThreads, 0, s>>>(q, (const float*)dy, (const float*)x, out, nullptr)
    switch (tile) {
      case 2: MN_GEN(T64x128); break;
      case 3: MN_GEN(T128x64); break;
      case 4: MN_GEN(T64x64); break;
      default: MN_GEN(T128x128); break;
    }
#undef MN_GEN
  }
  if (q.mode == 2) {
    wgrad_reduce_kernel<<<(unsigned)((nw + kThreads - 1) / kThreads), kThreads, 0, s>>>(
        (const float*)ws, (float*)dw, nw, splits);
    if (db)
      wgrad_reduce_kernel<<<(unsigned)((nb + kThreads - 1) / kThreads), kThreads, 0, s>>>(
          db_dst, db, nb, splits);
  }
  return mn_launch_status();
}

int mn_conv_bwd_weight(const mn_conv2d* g, const void* dy, const void* x, void* dw, void* ws,
                       size_t ws_bytes, int variant, int dtype, mn_stream_t stream) {
  return conv_bwd_weight(g, dy, x, dw, nullptr, ws, ws_bytes, variant, dtype, stream);
}

int mn_conv_bwd_weight_bias(const mn_conv2d* g, const void* dy, const void* x, void* dw, void* db,
                            void* ws, size_t ws_bytes, int variant, int dtype,
                            mn_stream_t stream) {
  if (!db) return MN_EINVAL;
  return conv_bwd_weight(g, dy, x, dw, db, ws, ws_bytes, variant, dtype, stream);
}

}  // extern "C"
