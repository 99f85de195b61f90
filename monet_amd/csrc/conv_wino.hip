// Winograd F(2x2, 3x3) convolution, fp32: the memory-for-arithmetic tier of the forward and
// backward-data directions (3x3 filters, stride 1, dilation 1).
//
//   Y = A^T [ (G g G^T) .* (B^T d B) ] A          per 4x4 input tile d -> 2x2 output tile Y
//
// with the element-wise product summed over the input channels.  Written per transform-domain
// position (xi, nu) in 0..15 that sum is a plain matrix product
//   Mt[pos][m][tile] = sum over ch of U[pos][ch][m] * V[pos][ch][tile]
// so the arithmetic is 16 GEMMs of (output channels) x (tiles) x (input channels): 16 multiplies
// per 2x2 outputs and channel pair instead of 36, i.e. 2.25 times fewer than the direct form.
// The price is the workspace: V and Mt hold 16 floats per tile and channel where the tensors
// themselves hold 4.
//
// Four launches: weights -> U, source -> V, one batched GEMM (the pointwise path of the gather
// GEMM in conv.hip), Mt -> destination (+ bias, or added to what the destination holds).
// Backward-data is the same computation on dy with the filter rotated by 180 degrees, the two
// channel roles swapped and padding 2 - pad.
#include <mutex>

#include "common.h"

int mn_conv_batched_gemm(const float* a, const float* src, float* dst, int M, int Mp, int Cs,
                         uint32_t cols, int batch, hipStream_t s);

namespace mn_wino {

constexpr int kThreads = 256;
constexpr int FK = 64, FT = 64, FC = 4;  // fused kernel: outputs, tiles per workgroup; channels per chunk
constexpr unsigned long long kSliceBytes = 512ull << 20;  // cap of the transformed source + product buffers

struct Plan {
  int N, Cs, Hs, Ws;   // source tensor [N, Cs, Hs, Ws]
  int M, OH, OW;       // destination tensor [N, M, OH, OW]
  int pad;             // source coordinate of tile element (i, j) = (2*th - pad + i, 2*tw - pad + j)
  int TH, TW;          // tiles per image
  uint32_t T, Tp;      // tiles; row capacity of V and Mt (tiles of the largest slice, multiple of 4)
  uint32_t slice;      // tiles per slice: the transforms and the GEMM run slice after slice
  uint32_t t0, Ts, Tsp;  // the current slice: first tile, tiles, row length (multiple of 4)
  uint32_t src_bytes, u_bytes;  // fused kernel: sizes of the source tensor and of U (0: 2 GB or more)
  int Mp;              // rows of U padded to a multiple of 128
};

static size_t u_floats(const Plan& p) { return (size_t)16 * p.Cs * p.Mp; }
static size_t v_floats(const Plan& p) { return (size_t)16 * p.Cs * p.Tp; }
static size_t m_floats(const Plan& p) { return (size_t)16 * p.M * p.Tp; }

// U[pos][ch][m] = (G g G^T)[pos] for the 3x3 filter g of (m, ch).
// FLIP = false (forward):      g[r][s] = w[m][ch][r][s]       (w is [M][Cs][3][3])
// FLIP = true (backward-data): g[r][s] = w[ch][m][2-r][2-s]   (w is [Cs][M][3][3])
// BLOCKED (for the fused kernel): U[m / FK][ch / FC][ch % FC][m % FK][pos], so that what one
// workgroup stages per chunk is 16 KB in one piece (with rows of Mp floats every workgroup
// reads 64 rows Mp * 4 bytes apart at the same moment as all the others) and the 16 positions
// of one (channel, output) pair are 64 bytes in a row, as the kernel's LDS layout wants them.
template <bool FLIP, bool BLOCKED = false>
__global__ __launch_bounds__(kThreads) void weight_kernel(const float* __restrict__ w,
                                                          float* __restrict__ U, int M, int Mp,
                                                          int Cs) {
  const uint32_t i = blockIdx.x * kThreads + threadIdx.x;
  if (i >= (uint32_t)Cs * Mp) return;
  const int m = i % Mp, ch = i / Mp;
  float g[3][3];
#pragma unroll
  for (int r = 0; r < 3; ++r)
#pragma unroll
    for (int s = 0; s < 3; ++s) {
      float v = 0.f;
      if (m < M)
        v = FLIP ? w[(((size_t)ch * M + m) * 3 + (2 - r)) * 3 + (2 - s)]
                 : w[(((size_t)m * Cs + ch) * 3 + r) * 3 + s];
      g[r][s] = v;
    }
  // t = G g (4x3), then u = t G^T (4x4); G = [1 0 0; .5 .5 .5; .5 -.5 .5; 0 0 1]
  float t[4][3];
#pragma unroll
  for (int s = 0; s < 3; ++s) {
    t[0][s] = g[0][s];
    t[1][s] = 0.5f * (g[0][s] + g[1][s] + g[2][s]);
    t[2][s] = 0.5f * (g[0][s] - g[1][s] + g[2][s]);
    t[3][s] = g[2][s];
  }
  const size_t stride = BLOCKED ? (size_t)1 : (size_t)Cs * Mp;
  const size_t at = BLOCKED ? ((((size_t)(m / FK) * (Cs / FC) + ch / FC) * FC + ch % FC) * FK + m % FK) * 16
                            : (size_t)i;
#pragma unroll
  for (int r = 0; r < 4; ++r) {
    const float u0 = t[r][0];
    const float u1 = 0.5f * (t[r][0] + t[r][1] + t[r][2]);
    const float u2 = 0.5f * (t[r][0] - t[r][1] + t[r][2]);
    const float u3 = t[r][2];
    U[(size_t)(4 * r + 0) * stride + at] = u0;
    U[(size_t)(4 * r + 1) * stride + at] = u1;
    U[(size_t)(4 * r + 2) * stride + at] = u2;
    U[(size_t)(4 * r + 3) * stride + at] = u3;
  }
}

// V[pos][ch][tile] = (B^T d B)[pos], d = the 4x4 source patch of the tile (zero outside the
// image).  One thread per (ch, tile); tiles run fastest, so the 16 stores are coalesced.
// B^T = [1 0 -1 0; 0 1 1 0; 0 -1 1 0; 0 1 0 -1]
__global__ __launch_bounds__(kThreads) void input_kernel(const Plan p, const float* __restrict__ src,
                                                         float* __restrict__ V) {
  const uint32_t i = blockIdx.x * kThreads + threadIdx.x;
  const uint32_t row = i / p.Tsp, col = i - row * p.Tsp;  // row = ch
  if (row >= (uint32_t)p.Cs) return;
  const uint32_t tile = p.t0 + col;
  const size_t stride = (size_t)p.Cs * p.Tsp;
  float d[4][4];
  if (col < p.Ts) {
    const uint32_t per_img = (uint32_t)p.TH * p.TW;
    const uint32_t n = tile / per_img, r = tile - n * per_img;
    const int th = r / p.TW, tw = r - th * p.TW;
    const int h0 = 2 * th - p.pad, w0 = 2 * tw - p.pad;
    const float* plane = src + ((size_t)n * p.Cs + row) * p.Hs * p.Ws;
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      const int h = h0 + a;
      const bool hok = (unsigned)h < (unsigned)p.Hs;
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        const int w = w0 + b;
        d[a][b] = (hok && (unsigned)w < (unsigned)p.Ws) ? plane[(size_t)h * p.Ws + w] : 0.f;
      }
    }
  } else {
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int b = 0; b < 4; ++b) d[a][b] = 0.f;  // padding columns of V: defined, never used
  }
  float t[4][4];  // t = B^T d
#pragma unroll
  for (int b = 0; b < 4; ++b) {
    t[0][b] = d[0][b] - d[2][b];
    t[1][b] = d[1][b] + d[2][b];
    t[2][b] = d[2][b] - d[1][b];
    t[3][b] = d[1][b] - d[3][b];
  }
#pragma unroll
  for (int a = 0; a < 4; ++a) {  // v = t B
    st_stream(V + (size_t)(4 * a + 0) * stride + i, t[a][0] - t[a][2]);
    st_stream(V + (size_t)(4 * a + 1) * stride + i, t[a][1] + t[a][2]);
    st_stream(V + (size_t)(4 * a + 2) * stride + i, t[a][2] - t[a][1]);
    st_stream(V + (size_t)(4 * a + 3) * stride + i, t[a][1] - t[a][3]);
  }
}

// dst 2x2 tile = A^T m A with m = Mt[.][row][tile]; A^T = [1 1 1 0; 0 1 -1 -1].
// One thread per (row, tile).  ACCUM: dst += result.
template <bool ACCUM>
__global__ __launch_bounds__(kThreads) void output_kernel(const Plan p, const float* __restrict__ Mt,
                                                          const float* __restrict__ bias,
                                                          float* __restrict__ dst) {
  const uint32_t i = blockIdx.x * kThreads + threadIdx.x;
  const uint32_t row = i / p.Tsp, col = i - row * p.Tsp;
  if (row >= (uint32_t)p.M || col >= p.Ts) return;
  const uint32_t tile = p.t0 + col;
  const size_t stride = (size_t)p.M * p.Tsp;
  float m[4][4];
#pragma unroll
  for (int a = 0; a < 4; ++a)
#pragma unroll
    for (int b = 0; b < 4; ++b) m[a][b] = ld_stream(Mt + (size_t)(4 * a + b) * stride + i);
  float t[2][4];  // t = A^T m
#pragma unroll
  for (int b = 0; b < 4; ++b) {
    t[0][b] = m[0][b] + m[1][b] + m[2][b];
    t[1][b] = m[1][b] - m[2][b] - m[3][b];
  }
  const float bv = bias ? bias[row] : 0.f;
  float y[2][2];
#pragma unroll
  for (int a = 0; a < 2; ++a) {
    y[a][0] = t[a][0] + t[a][1] + t[a][2] + bv;
    y[a][1] = t[a][1] - t[a][2] - t[a][3] + bv;
  }
  const uint32_t per_img = (uint32_t)p.TH * p.TW;
  const uint32_t n = tile / per_img, r = tile - n * per_img;
  const int th = r / p.TW, tw = r - th * p.TW;
  const int oh = 2 * th, ow = 2 * tw;
  float* o = dst + (((size_t)n * p.M + row) * p.OH + oh) * p.OW + ow;
#pragma unroll
  for (int a = 0; a < 2; ++a) {
    if (oh + a >= p.OH) break;
    float* q = o + (size_t)a * p.OW;
    if (ACCUM) {
      q[0] += y[a][0];
      if (ow + 1 < p.OW) q[1] += y[a][1];
    } else {
      q[0] = y[a][0];
      if (ow + 1 < p.OW) q[1] = y[a][1];
    }
  }
}

// ------------------------------------------------------------------- fused --
// The same algorithm in ONE kernel, with no transformed tensors in HBM (workspace = U only):
// a workgroup owns 64 outputs x 64 tiles and keeps all 16 transform-domain products of that
// block in registers (16 accumulator tiles of 32x32 per wavefront = 256 registers, one
// wavefront per SIMD).  Per chunk of 4 channels it stages U[4][64][16] (copied) and
// V[4][64][16] (each thread loads one 4x4 source patch and applies B^T . B) in LDS, double
// buffered, the 16 positions of a (channel, output) or (channel, tile) pair next to each other
// so that a lane fetches its operands of 16 MFMAs with four 16-byte reads and a patch is staged
// with four 16-byte writes (rows padded from 16 to 20 floats: 16 consecutive lanes then cover
// all 64 banks once).  Every wavefront issues 16 positions x 2 steps of
// v_mfma_f32_32x32x2_f32 per chunk.
// At the end each lane holds, for its 16 (output, tile) pairs, the 16 values A^T . A needs.
// It pays where the transforms of the unfused form dominate (few channels, large planes).
constexpr int LP = 20;                                  // floats per LDS row of 16 positions
constexpr int kFusedHalf = FC * FK * LP;                // floats of U (or V) in one buffer
constexpr size_t kFusedLds = (size_t)4 * kFusedHalf * sizeof(float);  // U and V, two buffers: 80 KB
typedef float float16_t __attribute__((ext_vector_type(16)));

__device__ __forceinline__ void input_transform(const float (&d)[4][4], float (&v)[16]) {
  float t[4][4];  // t = B^T d
#pragma unroll
  for (int b = 0; b < 4; ++b) {
    t[0][b] = d[0][b] - d[2][b];
    t[1][b] = d[1][b] + d[2][b];
    t[2][b] = d[2][b] - d[1][b];
    t[3][b] = d[1][b] - d[3][b];
  }
#pragma unroll
  for (int a = 0; a < 4; ++a) {  // v = t B
    v[4 * a + 0] = t[a][0] - t[a][2];
    v[4 * a + 1] = t[a][1] + t[a][2];
    v[4 * a + 2] = t[a][2] - t[a][1];
    v[4 * a + 3] = t[a][1] - t[a][3];
  }
}

template <bool ACCUM>
__global__ __launch_bounds__(kThreads) void fused_kernel(const Plan p, const float* __restrict__ src,
                                                         const float* __restrict__ U,
                                                         const float* __restrict__ bias,
                                                         float* __restrict__ dst, uint32_t nkb) {
  extern __shared__ float4_t fused_lds[];  // [buffer][U | V][channel][output | tile][LP]
  float* const lds = reinterpret_cast<float*>(fused_lds);
  const uint32_t slot = xcd_slot();
  const uint32_t kb = slot % nkb, tb = slot / nkb;  // neighbours share the source patches
  const int k0 = (int)kb * FK;
  const uint32_t t0 = tb * FT;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const uint32_t per_img = (uint32_t)p.TH * p.TW;
  const size_t plane = (size_t)p.Hs * p.Ws;

  // loader role: the patch of tile t0 + lane in channel `wave` of every chunk
  const uint32_t ltile = t0 + lane;
  const bool lt_ok = ltile < p.T;
  const uint32_t ln = lt_ok ? ltile / per_img : 0u, lr = lt_ok ? ltile - ln * per_img : 0u;
  const int lth = lr / p.TW, ltw = lr - lth * p.TW;
  const int h0 = 2 * lth - p.pad, w0 = 2 * ltw - p.pad;
  // Every load is issued unconditionally (straight-line code the scheduler can interleave with
  // the MFMAs) through a buffer descriptor: the per-lane part of an address is a byte offset
  // that stays the same for all chunks, the per-chunk part is uniform and travels in the
  // scalar offset of the load, so a load costs no address arithmetic; a patch element outside
  // the image gets an offset beyond the buffer, which the hardware answers with zero.
  constexpr uint32_t kBeyond = 0x80000000u;
  const __amdgpu_buffer_rsrc_t src_buf =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(src), 0, p.src_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t u_buf =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(U), 0, p.u_bytes, 0x00020000);
  uint32_t eoff[4][4];
  const uint32_t pbase = (uint32_t)(((size_t)ln * p.Cs + wave) * plane);
#pragma unroll
  for (int a = 0; a < 4; ++a)
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      const bool ok = lt_ok && (unsigned)(h0 + a) < (unsigned)p.Hs && (unsigned)(w0 + b) < (unsigned)p.Ws;
      eoff[a][b] = ok ? (pbase + (uint32_t)((h0 + a) * p.Ws + (w0 + b))) * 4u : kBeyond;
    }
  // U loader: four 16-byte pieces per thread and chunk, piece j = 16 bytes number tid + 256 j of
  // the chunk's [16][FC][FK] block, which is contiguous in the blocked U
  const uint32_t uoff = 16u * tid;
  uint32_t u_so = kb * (uint32_t)(p.Cs / FC) * (16u * FC * FK * 4u);  // byte offset of the next chunk of U
  uint32_t p_so = 0;                                                    // ... and of the source planes
  const uint32_t ustep = 16u * FC * FK * 4u, pstep = (uint32_t)(FC * plane * 4);

  // four register sets: the loads of chunks ch + 1 .. ch + 4 are in flight while chunk ch is
  // multiplied (with a single wavefront per SIMD nothing else covers a trip to HBM, and the
  // patch loads of a chunk were measured to take longer than two chunks of MFMAs)
  float d0[4][4], d1[4][4], d2[4][4], d3[4][4];
  float4_t u0[4], u1[4], u2[4], u3[4];
  // `advance` = 0 near the end: the loop body has no branch (a conditional load would make the
  // compiler wait for every load in flight at the join), so the last iterations load the last
  // chunk again and nobody uses it
  auto fetch = [&](float (&d)[4][4], float4_t (&uq)[4], bool advance) {
#pragma unroll
    for (int j = 0; j < 4; ++j)
      uq[j] = __builtin_bit_cast(
          float4_t, __builtin_amdgcn_raw_buffer_load_b128(u_buf, uoff, u_so + 16u * kThreads * j, 0));
    u_so += advance ? ustep : 0u;
#pragma unroll
    for (int a = 0; a < 4; ++a)
#pragma unroll
      for (int b = 0; b < 4; ++b)
        d[a][b] = __uint_as_float(__builtin_amdgcn_raw_buffer_load_b32(src_buf, eoff[a][b], p_so, 0));
    p_so += advance ? pstep : 0u;
  };
  // this thread's patch goes to row (channel = wave, tile = lane) of V; piece j of U (16 bytes
  // number tid + 256 j of the chunk) is positions 4 (tid & 3) .. + 3 of row (tid >> 2) + 64 j
  float* const vrow = lds + kFusedHalf + (wave * FT + lane) * LP;
  float* const urow = lds + (tid >> 2) * LP + 4 * (tid & 3);
  auto stage = [&](int buf, float (&d)[4][4], const float4_t (&uq)[4]) {
    float v[16];
    input_transform(d, v);
#pragma unroll
    for (int q = 0; q < 4; ++q)
      *reinterpret_cast<float4_t*>(vrow + buf * 2 * kFusedHalf + 4 * q) =
          float4_t{v[4 * q], v[4 * q + 1], v[4 * q + 2], v[4 * q + 3]};
#pragma unroll
    for (int j = 0; j < 4; ++j)
      *reinterpret_cast<float4_t*>(urow + buf * 2 * kFusedHalf + 64 * j * LP) = uq[j];
  };

  float16_t acc[16];
#pragma unroll
  for (int pos = 0; pos < 16; ++pos)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[pos][v] = 0.f;

  const int wk = (wave >> 1) * 32, wt = (wave & 1) * 32;
  const int r = lane & 31, half = lane >> 5;
  // operands: row (channel 2 s + half, output wk + r) of U and (channel 2 s + half, tile wt + r)
  // of V, 16 positions each, for the two steps s of a chunk
  const float* const arow = lds + (half * FK + wk + r) * LP;
  const float* const brow = lds + kFusedHalf + (half * FT + wt + r) * LP;
  // The last 8 MFMAs of a chunk (second step, positions 8..15) are issued at the START of the
  // next step, from operands that wait in registers across the barrier: the new chunk's first
  // LDS reads then travel while the matrix pipe is busy, instead of every step beginning with an
  // idle pipe until the first operands arrive.
  float4_t ca[2], cb[2];
#pragma unroll
  for (int q = 0; q < 2; ++q) ca[q] = cb[q] = float4_t{0.f, 0.f, 0.f, 0.f};
  auto tail = [&]() {
#pragma unroll
    for (int q = 0; q < 2; ++q)
#pragma unroll
      for (int e = 0; e < 4; ++e)
        acc[8 + 4 * q + e] = __builtin_amdgcn_mfma_f32_32x32x2f32(ca[q][e], cb[q][e], acc[8 + 4 * q + e], 0, 0, 0);
  };
  auto head = [&](int buf) {
    float4_t av[FC / 2][4], bv[FC / 2][4];
#pragma unroll
    for (int cs = 0; cs < FC / 2; ++cs)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        av[cs][q] = *reinterpret_cast<const float4_t*>(arow + buf * 2 * kFusedHalf + 2 * cs * FK * LP + 4 * q);
        bv[cs][q] = *reinterpret_cast<const float4_t*>(brow + buf * 2 * kFusedHalf + 2 * cs * FT * LP + 4 * q);
      }
#pragma unroll
    for (int i = 0; i < 24; ++i) {  // step 0: 16 positions, step 1: positions 0..7
      const int cs = i >> 4, pos = i & 15;
      acc[pos] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[cs][pos >> 2][pos & 3], bv[cs][pos >> 2][pos & 3],
                                                      acc[pos], 0, 0, 0);
    }
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      ca[q] = av[1][2 + q];
      cb[q] = bv[1][2 + q];
    }
  };
  // Order of one step, for the instruction scheduler: the MFMA of a 32x32x2 tile keeps the matrix
  // pipe busy for 64 cycles after its issue, and this wavefront is alone on its SIMD, so
  // everything else of the step (LDS reads of the operands, the global loads of a later chunk,
  // the transform and the LDS writes of the next one) goes into the gaps between two MFMAs
  // instead of before and after all 32 of them.
  auto interleave = [&]() {
#pragma unroll
    for (int i = 0; i < 32; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);              // one MFMA
      if (i < 8) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);   // two LDS reads
      if (i >= 4 && i < 24) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);  // one global load
      __builtin_amdgcn_sched_group_barrier(0x002, 2, 0);              // VALU
      if (i >= 24) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0); // one LDS write
    }
  };
  // the channel count is a multiple of 16, so the number of chunks is a multiple of 4
  const int nchunks = p.Cs / FC;
  fetch(d0, u0, 1 < nchunks);
  fetch(d1, u1, 2 < nchunks);
  fetch(d2, u2, 3 < nchunks);
  fetch(d3, u3, 4 < nchunks);  // the pointers now stand at chunk 4, or stay at the last one
  stage(0, d0, u0);
  __syncthreads();
  // one step: load chunk c + 4 into the set chunk c came from, multiply chunk c, stage chunk c + 1
#define MN_WINO_STEP(c, buf, dk, uk, dn, un)  \
  fetch(dk, uk, (c) + 5 < nchunks);           \
  tail();                                     \
  head(buf);                                  \
  stage((buf) ^ 1, dn, un);                   \
  interleave();                               \
  __syncthreads();
  for (int ch = 0; ch < nchunks; ch += 4) {
    MN_WINO_STEP(ch, 0, d0, u0, d1, u1)
    MN_WINO_STEP(ch + 1, 1, d1, u1, d2, u2)
    MN_WINO_STEP(ch + 2, 0, d2, u2, d3, u3)
    MN_WINO_STEP(ch + 3, 1, d3, u3, d0, u0)
  }
#undef MN_WINO_STEP
  tail();

  // output transform: this lane's tile is t0 + wt + r, its outputs k0 + wk + row(v)
  const uint32_t etile = t0 + wt + r;
  const bool e_ok = etile < p.T;
  const uint32_t en = e_ok ? etile / per_img : 0u, er = e_ok ? etile - en * per_img : 0u;
  const int eth = er / p.TW, etw = er - eth * p.TW;
  const int oh = 2 * eth, ow = 2 * etw;
  const bool row1 = oh + 1 < p.OH, col1 = ow + 1 < p.OW;
  // output k0 + wk + 4 half + kofs(v), kofs(v) = 8 (v / 4) + v % 4: the lane's part of the address
  // once, the rest a compile-time multiple of the plane size
  const int kl = k0 + wk + 4 * half;
  const size_t oplane = (size_t)p.OH * p.OW;
  float* const obase = dst + ((size_t)en * p.M + kl) * oplane + (size_t)oh * p.OW + ow;
  // the bias values of this lane's 16 outputs in one go (a load per output inside the loop below
  // waited for each before it went on)
  float bvs[16];
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const int k = kl + 8 * (v >> 2) + (v & 3);
    bvs[v] = bias ? bias[k < p.M ? k : p.M - 1] : 0.f;
  }
  // Interior blocks (every lane has a whole 2x2 tile and all 64 outputs exist) store without
  // predicates: four stores per output behind no branch.
  const bool whole = __all(e_ok && row1 && col1) && k0 + FK <= p.M;
  if (whole) {
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      float t[2][4];  // t = A^T m, m[a][b] = acc[4a + b][v]
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        t[0][b] = acc[b][v] + acc[4 + b][v] + acc[8 + b][v];
        t[1][b] = acc[4 + b][v] - acc[8 + b][v] - acc[12 + b][v];
      }
      float* o = obase + (size_t)(8 * (v >> 2) + (v & 3)) * oplane;
#pragma unroll
      for (int a = 0; a < 2; ++a) {
        float* q = o + (size_t)a * p.OW;
        const float y0 = t[a][0] + t[a][1] + t[a][2] + bvs[v];
        const float y1 = t[a][1] - t[a][2] - t[a][3] + bvs[v];
        q[0] = ACCUM ? q[0] + y0 : y0;
        q[1] = ACCUM ? q[1] + y1 : y1;
      }
    }
    return;
  }
  if (!e_ok) return;
#pragma unroll
  for (int v = 0; v < 16; ++v) {
    const int k = kl + 8 * (v >> 2) + (v & 3);
    if (k >= p.M) continue;
    float t[2][4];
#pragma unroll
    for (int b = 0; b < 4; ++b) {
      t[0][b] = acc[b][v] + acc[4 + b][v] + acc[8 + b][v];
      t[1][b] = acc[4 + b][v] - acc[8 + b][v] - acc[12 + b][v];
    }
    float* o = obase + (size_t)(8 * (v >> 2) + (v & 3)) * oplane;
#pragma unroll
    for (int a = 0; a < 2; ++a) {
      if (a == 1 && !row1) break;
      float* q = o + (size_t)a * p.OW;
      const float y0 = t[a][0] + t[a][1] + t[a][2] + bvs[v];
      const float y1 = t[a][1] - t[a][2] - t[a][3] + bvs[v];
      q[0] = ACCUM ? q[0] + y0 : y0;
      if (col1) q[1] = ACCUM ? q[1] + y1 : y1;
    }
  }
}

// ------------------------------------------ backward weight in one kernel --
// dW = G^T [ sum over tiles of (A dY A^T) .* (B^T X B) ] G without the transformed tensors in HBM:
// Z[pos][k][c] = sum_t Ud[pos][t][k] Vx[pos][t][c] is a product over the TILES, so a workgroup owns
// 64 outputs x 64 inputs x 16 positions (the accumulator shape of the forward kernel above, 256
// registers per lane) and walks a range of tile rows, four tiles of a row per chunk: per chunk a
// thread transforms one 4x4 patch of x and one 2x2 patch of dy and writes one row of Vx and of Ud
// (the LDS layout, the operand reads and the 32 matrix instructions per chunk are the forward
// kernel's with "channel of the chunk" read as "tile of the chunk"; a tile's block of 64 rows is
// padded by 16 floats: the four tiles of a channel are written by neighbouring lanes, and 64 * LP
// is a multiple of the 64 banks, a 4-way conflict on every staging write otherwise).
// The result of a range of tile rows goes to Z[pos][range][k][c]; wgrad_output_kernel adds the
// ranges in order and applies G^T . G (reproducible).
// Needs: 3x3, stride 1, padding 1, H even, W % 4 == 0 (16-byte pieces of a row; a last chunk with
// fewer than four tiles multiplies zeros), K % 64 == 0, C % 64 == 0.
constexpr int kWgTile = FK * LP + 16;                   // floats of one tile's 64 rows (FK == FT), padded
constexpr int kWgHalf = FC * kWgTile;                   // floats of Ud (or Vx) in one buffer
static_assert(FK == FT, "one row count for both operands");
struct FWPlan {
  int N, C, K, H, W;
  int TH, TW;                 // tiles per image
  uint32_t rows;              // N * TH tile rows
  uint32_t rows_per_range;
  int S;                      // ranges
  uint32_t x_bytes, dy_bytes;
};

// The source rows are staged RAW in LDS first.  Loading one 4x4 patch per lane straight from
// memory costs 14 load instructions per chunk that each touch 16 cache lines for 4 to 8 bytes per
// lane (430 million L1 lookups per call at 128 -> 128 channels, 208 x 304), and a chunk only uses
// 32 bytes of every 128-byte line it touches while the CU's lines of one chunk (48 KB) do not fit
// its L1: every line came from L2 four times (1.44 ms; 1.32 ms with the loads of four chunks
// issued together; 0.94 ms with the same instructions on cache-resident addresses).  Here the
// workgroup copies, for a GROUP of four chunks (32 output columns of one tile row), the 64
// channels x 4 rows x 40 columns of x and the 64 outputs x 2 rows x 32 columns of dy into LDS with
// 16-byte loads along the rows (14 per thread and group instead of 56, whole lines: 1.15 ms, of
// which the loads are 1 %), and every lane then reads its patches from LDS.  Out-of-image rows and
// columns are written as zeros at that point (a load whose offset is beyond the buffer), so
// staging a chunk has no masks.  A tile row whose chunk count is no multiple of 4 is padded with
// chunks of zeros.  The raw rows are single-buffered (59 KB beside the 81 KB of transformed
// operands): the group's registers are written to LDS in the step that stages the group's first
// chunk, with one more barrier in the middle of that step.
// BIAS: the workgroups of input block 0 also add up the gradient tiles they stage; their sums per
// (range, output) go to dbp[range][k] and bias_ranges_kernel adds the ranges in order.
constexpr int kRawXRow = 40;                  // floats of an input row piece: columns 32 Q - 4 .. 32 Q + 35
constexpr int kRawXCh = 4 * kRawXRow + 4;     // per channel, padded: 16 channels start in 16 different banks
constexpr int kRawDyRow = 32;
constexpr int kRawDyCh = 2 * kRawDyRow + 4;
constexpr int kRawX = FT * kRawXCh, kRawDy = FK * kRawDyCh;
constexpr int kRawXItems = FT * 4 * (kRawXRow / 4) / kThreads;   // 16-byte pieces per thread: 10
constexpr int kRawDyItems = FK * 2 * (kRawDyRow / 4) / kThreads;  // 4
constexpr size_t kWgRowsLds = (size_t)(4 * kWgHalf + kRawX + kRawDy) * sizeof(float);  // 139 KB
static_assert(FT * 4 * (kRawXRow / 4) % kThreads == 0 && FK * 2 * (kRawDyRow / 4) % kThreads == 0, "whole items");

template <bool BIAS>
__global__ __launch_bounds__(kThreads) void fused_wgrad_kernel(const FWPlan p, const float* __restrict__ x,
                                                                    const float* __restrict__ dy,
                                                                    float* __restrict__ Z,
                                                                    float* __restrict__ dbp) {
  extern __shared__ float4_t fused_lds[];  // [buffer][Ud | Vx][tile of the chunk][channel][LP], raw x, raw dy
  float* const lds = reinterpret_cast<float*>(fused_lds);
  float* const raw_x = lds + 4 * kWgHalf;
  float* const raw_dy = raw_x + kRawX;
  const uint32_t slot = xcd_slot();
  const uint32_t ncb = (uint32_t)p.C / FT, blocks = ((uint32_t)p.K / FK) * ncb;
  const uint32_t blk = slot % blocks, range = slot / blocks;  // neighbours read the same tile rows
  const uint32_t kb = blk / ncb, cb = blk - kb * ncb;
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int ci = 16 * wave + (lane >> 2), ti = lane & 3;   // staging role: channel, tile of the chunk
  const uint32_t r_begin = range * p.rows_per_range;
  const uint32_t r_end = min(r_begin + p.rows_per_range, p.rows);
  const int cpr = (p.TW + 3) >> 2;                         // chunks per tile row (the last may be ragged)
  const int gpr = (cpr + 3) >> 2;                          // groups per tile row
  const int ngroups = (int)(r_end - r_begin) * gpr;
  const uint32_t plane = (uint32_t)p.H * p.W;
  constexpr uint32_t kBeyond = 0x80000000u;

  const __amdgpu_buffer_rsrc_t x_buf =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(x), 0, p.x_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t dy_buf =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<float*>(dy), 0, p.dy_bytes, 0x00020000);
  // copier role: piece i = tid + 256 u of [channel][row][16-byte piece]; what never changes
  uint32_t x_const[kRawXItems], x_af[kRawXItems], d_const[kRawDyItems], d_f[kRawDyItems];
  int x_lds[kRawXItems], d_lds[kRawDyItems];
#pragma unroll
  for (int u = 0; u < kRawXItems; ++u) {
    const int i = tid + u * kThreads, ch = i / 40, rem = i - ch * 40, a = rem / 10, f = rem - a * 10;
    x_const[u] = ((cb * FT + ch) * plane + a * p.W + 4 * f) * 4u;
    x_af[u] = a | (f << 8);
    x_lds[u] = ch * kRawXCh + a * kRawXRow + 4 * f;
  }
#pragma unroll
  for (int u = 0; u < kRawDyItems; ++u) {
    const int i = tid + u * kThreads, k = i >> 4, rem = i & 15, a = rem >> 3, f = rem & 7;
    d_const[u] = ((kb * FK + k) * plane + a * p.W + 4 * f) * 4u;
    d_f[u] = f;
    d_lds[u] = k * kRawDyCh + a * kRawDyRow + 4 * f;
  }
  // the next group to copy (scalar): image, tile row, group of the row
  int gn = (int)(r_begin / (uint32_t)p.TH), gth = (int)(r_begin - (uint32_t)gn * p.TH), gq = 0, copied = 0;
  float4_t rx[kRawXItems], rd[kRawDyItems];
  auto fetch_group = [&]() {
    const bool real = copied < ngroups;  // past the end: every piece reads as zeros
    // byte offset of (row 2 th - 1, column 32 Q - 4) of channel 0 / (row 2 th, column 32 Q) of
    // output 0; pieces outside the image are the only ones whose sum with it is negative
    const uint32_t x_term = (uint32_t)(((gn * p.C * p.H + 2 * gth - 1) * p.W + 32 * gq - 4) * 4);
    const uint32_t d_term = (uint32_t)(((gn * p.K * p.H + 2 * gth) * p.W + 32 * gq) * 4);
    const bool top = gth == 0, bottom = gth == p.TH - 1;
    const int f_first = gq == 0 ? 1 : 0;                 // piece 0 of the first group is columns -4 .. -1
    const int f_end = (p.W - 32 * gq + 4) >> 2;          // first piece that starts at or beyond column W
#pragma unroll
    for (int u = 0; u < kRawXItems; ++u) {
      const int a = x_af[u] & 255, f = x_af[u] >> 8;
      const bool ok = real && !(top && a == 0) && !(bottom && a == 3) && f >= f_first && f < f_end;
      rx[u] = __builtin_bit_cast(
          float4_t, __builtin_amdgcn_raw_buffer_load_b128(x_buf, ok ? x_const[u] + x_term : kBeyond, 0, 0));
    }
#pragma unroll
    for (int u = 0; u < kRawDyItems; ++u) {
      const bool ok = real && (int)d_f[u] < f_end - 1;   // columns 32 Q + 4 f < W
      rd[u] = __builtin_bit_cast(
          float4_t, __builtin_amdgcn_raw_buffer_load_b128(dy_buf, ok ? d_const[u] + d_term : kBeyond, 0, 0));
    }
    ++copied;
    if (++gq == gpr) {
      gq = 0;
      if (++gth == p.TH) {
        gth = 0;
        ++gn;
      }
    }
  };
  auto write_raw = [&]() {
#pragma unroll
    for (int u = 0; u < kRawXItems; ++u) *reinterpret_cast<float4_t*>(raw_x + x_lds[u]) = rx[u];
#pragma unroll
    for (int u = 0; u < kRawDyItems; ++u) *reinterpret_cast<float4_t*>(raw_dy + d_lds[u]) = rd[u];
  };
  float bsum = 0.f;
  // this lane's patches of chunk j of the group in LDS: columns 8 j + 2 ti - 1 .. + 2 of the rows
  // (the staged piece starts at column - 4), and its 2x2 gradient tile
  const float* const px = raw_x + ci * kRawXCh + 3 + 2 * ti;
  const float* const pd = raw_dy + ci * kRawDyCh + 2 * ti;
  float* const vrow = lds + kWgHalf + ti * kWgTile + ci * LP;
  float* const urow = lds + ti * kWgTile + ci * LP;
  auto stage = [&](int buf, int j) {
    float d[4][4];
    typedef float f2 __attribute__((ext_vector_type(2)));
#pragma unroll
    for (int a = 0; a < 4; ++a) {
      const float* row = px + a * kRawXRow + 8 * j;
      d[a][0] = row[0];
      const f2 mid = *reinterpret_cast<const f2*>(row + 1);
      d[a][1] = mid[0];
      d[a][2] = mid[1];
      d[a][3] = row[3];
    }
    const f2 ea = *reinterpret_cast<const f2*>(pd + 8 * j), eb = *reinterpret_cast<const f2*>(pd + kRawDyRow + 8 * j);
    float v[16];
    input_transform(d, v);
#pragma unroll
    for (int q = 0; q < 4; ++q)
      *reinterpret_cast<float4_t*>(vrow + buf * 2 * kWgHalf + 4 * q) =
          float4_t{v[4 * q], v[4 * q + 1], v[4 * q + 2], v[4 * q + 3]};
    // A e A^T, A = [1 0; 1 1; 1 -1; 0 -1]
    const float e00 = ea[0], e01 = ea[1], e10 = eb[0], e11 = eb[1];
    const float t0[2] = {e00, e01}, t1[2] = {e00 + e10, e01 + e11}, t2[2] = {e00 - e10, e01 - e11},
                t3[2] = {-e10, -e11};
    if (BIAS) bsum += t1[0] + t1[1];
    *reinterpret_cast<float4_t*>(urow + buf * 2 * kWgHalf + 0) = float4_t{t0[0], t0[0] + t0[1], t0[0] - t0[1], -t0[1]};
    *reinterpret_cast<float4_t*>(urow + buf * 2 * kWgHalf + 4) = float4_t{t1[0], t1[0] + t1[1], t1[0] - t1[1], -t1[1]};
    *reinterpret_cast<float4_t*>(urow + buf * 2 * kWgHalf + 8) = float4_t{t2[0], t2[0] + t2[1], t2[0] - t2[1], -t2[1]};
    *reinterpret_cast<float4_t*>(urow + buf * 2 * kWgHalf + 12) = float4_t{t3[0], t3[0] + t3[1], t3[0] - t3[1], -t3[1]};
  };

  float16_t acc[16];
#pragma unroll
  for (int pos = 0; pos < 16; ++pos)
#pragma unroll
    for (int v = 0; v < 16; ++v) acc[pos][v] = 0.f;
  const int wk = (wave >> 1) * 32, wc = (wave & 1) * 32;
  const int r = lane & 31, half = lane >> 5;
  // operands: row (tile 2 s + half, output wk + r) of Ud and (tile 2 s + half, input wc + r) of Vx
  const float* const arow = lds + half * kWgTile + (wk + r) * LP;
  const float* const brow = lds + kWgHalf + half * kWgTile + (wc + r) * LP;
  float4_t ca[2], cbv[2];
#pragma unroll
  for (int q = 0; q < 2; ++q) ca[q] = cbv[q] = float4_t{0.f, 0.f, 0.f, 0.f};
  auto tail = [&]() {
#pragma unroll
    for (int q = 0; q < 2; ++q)
#pragma unroll
      for (int e = 0; e < 4; ++e)
        acc[8 + 4 * q + e] = __builtin_amdgcn_mfma_f32_32x32x2f32(ca[q][e], cbv[q][e], acc[8 + 4 * q + e], 0, 0, 0);
  };
  float4_t av[FC / 2][4], bv[FC / 2][4];
  auto head_read = [&](int buf) {
#pragma unroll
    for (int s2 = 0; s2 < FC / 2; ++s2)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        av[s2][q] = *reinterpret_cast<const float4_t*>(arow + buf * 2 * kWgHalf + 2 * s2 * kWgTile + 4 * q);
        bv[s2][q] = *reinterpret_cast<const float4_t*>(brow + buf * 2 * kWgHalf + 2 * s2 * kWgTile + 4 * q);
      }
  };
  auto head_mul = [&](int from, int to) {  // step 0: 16 positions, step 1: positions 0..7
#pragma unroll
    for (int i = from; i < to; ++i) {
      const int s2 = i >> 4, pos = i & 15;
      acc[pos] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[s2][pos >> 2][pos & 3], bv[s2][pos >> 2][pos & 3],
                                                      acc[pos], 0, 0, 0);
    }
  };
  auto head_keep = [&]() {
#pragma unroll
    for (int q = 0; q < 2; ++q) {
      ca[q] = av[1][2 + q];
      cbv[q] = bv[1][2 + q];
    }
  };
  auto interleave = [&](int nloads) {
#pragma unroll
    for (int i = 0; i < 32; ++i) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);              // one MFMA
      if (i < 11) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);  // two LDS reads (16 operand, 14 patch... the rest follows)
      if (i >= 4 && i < 4 + nloads) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);  // one global load
      __builtin_amdgcn_sched_group_barrier(0x002, 2, 0);              // VALU
      if (i >= 24) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0); // one LDS write
    }
  };
  fetch_group();
  write_raw();
  __syncthreads();
  stage(0, 0);
  __syncthreads();
  for (int g = 0; g < ngroups; ++g) {
    // step 0 of the group: request the next group's rows; chunks 1..3 are staged in steps 0..2
    fetch_group();
    tail();
    head_read(0);
    head_mul(0, 24);
    head_keep();
    stage(1, 1);
    interleave(kRawXItems + kRawDyItems);
    __syncthreads();
    tail();
    head_read(1);
    head_mul(0, 24);
    head_keep();
    stage(0, 2);
    interleave(0);
    __syncthreads();
    tail();
    head_read(0);
    head_mul(0, 24);
    head_keep();
    stage(1, 3);
    interleave(0);
    __syncthreads();
    // step 3: the next group's rows go to LDS (the barrier above was the last reader's), and after
    // one more barrier its first chunk is staged
    write_raw();
    tail();
    head_read(1);
    head_mul(0, 12);
    __syncthreads();
    head_mul(12, 24);
    head_keep();
    stage(0, 0);
    __syncthreads();
  }
  tail();

  if (BIAS && cb == 0) {
    float t = bsum;  // this lane: output ci, tile ti of every chunk
    t += __shfl_xor(t, 1);
    t += __shfl_xor(t, 2);
    if (ti == 0) dbp[(size_t)range * p.K + kb * FK + ci] = t;
  }
  // Z[pos][range][k][c]: a register holds one output for 32 consecutive inputs
  const size_t kc = (size_t)p.K * p.C;
  float* zb = Z + (size_t)range * kc + (size_t)(kb * FK + wk) * p.C + cb * FT + wc + r;
#pragma unroll
  for (int pos = 0; pos < 16; ++pos)
#pragma unroll
    for (int v = 0; v < 16; ++v) {
      const int k = 8 * (v >> 2) + 4 * half + (v & 3);
      zb[(size_t)pos * p.S * kc + (size_t)k * p.C] = acc[pos][v];
    }
}

// db[k] = sum over the ranges of dbp[range][k], in order
__global__ __launch_bounds__(kThreads) void bias_ranges_kernel(const float* __restrict__ dbp,
                                                               float* __restrict__ db, int K, int S) {
  const int k = blockIdx.x * kThreads + threadIdx.x;
  if (k >= K) return;
  float s = 0.f;
  for (int r = 0; r < S; ++r) s += dbp[(size_t)r * K + k];
  db[k] = s;
}

// ------------------------------------------------------------ backward weight --
// dW (3x3) = sum over tiles of G^T [ (A dY A^T) .* (B^T X B) ] G, with dY the 2x2 tile of the
// output gradient and X the 4x4 input tile the forward used for it (the transposed form of the
// forward algorithm).  Per transform-domain position that is a matrix product over the TILES,
//   Z[pos][k][c] = sum over t of Ud[pos][t][k] * Vx[pos][t][c],
// 16 multiplies per tile and (k, c) pair instead of 36.  The reduction is long (all tiles) and
// the result small (K x C), so it is cut into S slices that run as 16 * S independent GEMMs
// of the same batched launch the forward uses; their partial results are added in a fixed order
// by the kernel that applies G^T . G (reproducible run to run).
//
// Both transforms write [pos][tile][channel], channel fastest, which is the reduction-major
// layout the GEMM wants; the tensors have the pixel fastest, so a workgroup transposes a block
// of 32 tiles x 32 channels through LDS (8 positions at a time).
template <bool DY>
__global__ __launch_bounds__(kThreads) void wgrad_transform_kernel(const Plan p, int channels,
                                                                   const float* __restrict__ src,
                                                                   float* __restrict__ out,
                                                                   int row_len, uint32_t Tpad) {
  __shared__ float lds[8][32][33];
  const int lane_t = threadIdx.x & 31, cg = threadIdx.x >> 5;
  const uint32_t t0 = blockIdx.x * 32u;
  const int c0 = blockIdx.y * 32;
  const uint32_t tile = p.t0 + t0 + lane_t;  // p.t0: first tile of this pass
  const bool t_ok = tile < p.T;
  const uint32_t per_img = (uint32_t)p.TH * p.TW;
  const uint32_t n = t_ok ? tile / per_img : 0u, r = t_ok ? tile - n * per_img : 0u;
  const int th = r / p.TW, tw = r - th * p.TW;
  float v[4][16];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int ch = c0 + cg + 8 * i;
    const bool ok = t_ok && ch < channels;
    if (DY) {
      // 2x2 tile of dy [N, channels, OH, OW] at (2 th, 2 tw), zero beyond the edge
      float d[2][2];
      const float* plane = src + ((size_t)n * channels + (ok ? ch : 0)) * p.OH * p.OW;
#pragma unroll
      for (int a = 0; a < 2; ++a)
#pragma unroll
        for (int b = 0; b < 2; ++b) {
          const int h = 2 * th + a, w = 2 * tw + b;
          d[a][b] = (ok && h < p.OH && w < p.OW) ? plane[(size_t)h * p.OW + w] : 0.f;
        }
      // A d A^T, A = [1 0; 1 1; 1 -1; 0 -1]
      float t[4][2];
#pragma unroll
      for (int b = 0; b < 2; ++b) {
        t[0][b] = d[0][b];
        t[1][b] = d[0][b] + d[1][b];
        t[2][b] = d[0][b] - d[1][b];
        t[3][b] = -d[1][b];
      }
#pragma unroll
      for (int a = 0; a < 4; ++a) {
        v[i][4 * a + 0] = t[a][0];
        v[i][4 * a + 1] = t[a][0] + t[a][1];
        v[i][4 * a + 2] = t[a][0] - t[a][1];
        v[i][4 * a + 3] = -t[a][1];
      }
    } else {
      // 4x4 tile of x [N, channels, Hs, Ws] at (2 th - pad, 2 tw - pad), zero outside the image
      float d[4][4];
      const float* plane = src + ((size_t)n * channels + (ok ? ch : 0)) * p.Hs * p.Ws;
      const int h0 = 2 * th - p.pad, w0 = 2 * tw - p.pad;
#pragma unroll
      for (int a = 0; a < 4; ++a) {
        const int h = h0 + a;
        const bool hok = ok && (unsigned)h < (unsigned)p.Hs;
#pragma unroll
        for (int b = 0; b < 4; ++b) {
          const int w = w0 + b;
          d[a][b] = (hok && (unsigned)w < (unsigned)p.Ws) ? plane[(size_t)h * p.Ws + w] : 0.f;
        }
      }
      float t[4][4];  // B^T d
#pragma unroll
      for (int b = 0; b < 4; ++b) {
        t[0][b] = d[0][b] - d[2][b];
        t[1][b] = d[1][b] + d[2][b];
        t[2][b] = d[2][b] - d[1][b];
        t[3][b] = d[1][b] - d[3][b];
      }
#pragma unroll
      for (int a = 0; a < 4; ++a) {  // (B^T d) B
        v[i][4 * a + 0] = t[a][0] - t[a][2];
        v[i][4 * a + 1] = t[a][1] + t[a][2];
        v[i][4 * a + 2] = t[a][2] - t[a][1];
        v[i][4 * a + 3] = t[a][1] - t[a][3];
      }
    }
  }
#pragma unroll
  for (int half = 0; half < 2; ++half) {
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
      for (int pp = 0; pp < 8; ++pp) lds[pp][lane_t][cg + 8 * i] = v[i][8 * half + pp];
    __syncthreads();
    // rows of 32 channels leave as eight 16-byte stores (row_len is a multiple of 4)
    for (int idx = threadIdx.x; idx < 8 * 32 * 8; idx += kThreads) {
      const int pp = idx >> 8, rem = idx & 255, tl = rem >> 3, ch = (rem & 7) * 4;
      if (c0 + ch < row_len && t0 + tl < Tpad) {
        const float4_t q = {lds[pp][tl][ch], lds[pp][tl][ch + 1], lds[pp][tl][ch + 2],
                            lds[pp][tl][ch + 3]};
        st_stream(reinterpret_cast<float4_t*>(
                      out + ((size_t)(8 * half + pp) * Tpad + t0 + tl) * row_len + c0 + ch), q);
      }
    }
    __syncthreads();
  }
}

// dw[k][c] (3x3) = G^T (sum over the S slices of Z[pos][s][k][c]) G; G^T = [1 .5 .5 0; 0 .5 -.5 0; 0 .5 .5 1].
// A workgroup takes 64 consecutive (k, c) pairs: each wavefront adds up the slices of four
// positions for them (64 lanes = 64 consecutive floats per load), the sums meet in LDS and the
// first wavefront applies G^T . G and writes the nine taps.
// ACCUM: dw += (a later pass over the tiles; the passes run in order, so the sum is reproducible).
template <bool ACCUM>
__global__ __launch_bounds__(kThreads) void wgrad_output_kernel(const float* __restrict__ Z,
                                                                float* __restrict__ dw, int K, int C,
                                                                int S) {
  __shared__ float lds[16][64];
  const size_t kc = (size_t)K * C;
  const int lane = threadIdx.x & 63, pg = threadIdx.x >> 6;
  const size_t i = (size_t)blockIdx.x * 64 + lane;
  const bool ok = i < kc;
#pragma unroll
  for (int q = 0; q < 4; ++q) {
    const int pos = 4 * pg + q;
    const float* base = Z + (size_t)pos * S * kc + (ok ? i : 0);
    float acc = 0.f;
    int s = 0;
    for (; s + 4 <= S; s += 4) {  // four loads in flight, added in slice order
      const float a0 = base[(size_t)s * kc], a1 = base[(size_t)(s + 1) * kc];
      const float a2 = base[(size_t)(s + 2) * kc], a3 = base[(size_t)(s + 3) * kc];
      acc = (((acc + a0) + a1) + a2) + a3;
    }
    for (; s < S; ++s) acc += base[(size_t)s * kc];
    lds[pos][lane] = acc;
  }
  __syncthreads();
  if (pg != 0 || !ok) return;
  float z[4][4];
#pragma unroll
  for (int pos = 0; pos < 16; ++pos) z[pos >> 2][pos & 3] = lds[pos][lane];
  float t[3][4];
#pragma unroll
  for (int b = 0; b < 4; ++b) {
    t[0][b] = z[0][b] + 0.5f * (z[1][b] + z[2][b]);
    t[1][b] = 0.5f * (z[1][b] - z[2][b]);
    t[2][b] = 0.5f * (z[1][b] + z[2][b]) + z[3][b];
  }
  float* o = dw + i * 9;
#pragma unroll
  for (int a = 0; a < 3; ++a) {
    const float r0 = t[a][0] + 0.5f * (t[a][1] + t[a][2]);
    const float r1 = 0.5f * (t[a][1] - t[a][2]);
    const float r2 = 0.5f * (t[a][1] + t[a][2]) + t[a][3];
    o[3 * a + 0] = ACCUM ? o[3 * a + 0] + r0 : r0;
    o[3 * a + 1] = ACCUM ? o[3 * a + 1] + r1 : r1;
    o[3 * a + 2] = ACCUM ? o[3 * a + 2] + r2 : r2;
  }
}

// db[k] = sum over (n, p, q) of dy[n][k][p][q], one workgroup per k, fixed order.  A plane is
// read as 16-byte vectors, eight per thread in flight (a loop of one 4-byte load per trip is
// bound by the latency of a load: 4.3 ms for 64 channels of 11 x 416 x 608, 0.15 ms this way).
__global__ __launch_bounds__(kThreads) void bias_grad_kernel(const float* __restrict__ dy,
                                                             float* __restrict__ db, int N, int K,
                                                             int PQ) {
  __shared__ float lds[2 * (kThreads / 64)];
  constexpr int kInFlight = 8;
  const int k = blockIdx.x;
  float4_t acc[kInFlight];
#pragma unroll
  for (int u = 0; u < kInFlight; ++u) acc[u] = float4_t{0.f, 0.f, 0.f, 0.f};
  float s = 0.f, unused = 0.f;
  const bool vec = (PQ & 3) == 0 && (reinterpret_cast<uintptr_t>(dy) & 15) == 0;
  for (int n = 0; n < N; ++n) {
    const float* plane = dy + ((size_t)n * K + k) * PQ;
    if (vec) {
      const float4_t* p4 = reinterpret_cast<const float4_t*>(plane);
      const int nvec = PQ >> 2;
      int i = threadIdx.x;
      for (; i + (kInFlight - 1) * kThreads < nvec; i += kInFlight * kThreads) {
#pragma unroll
        for (int u = 0; u < kInFlight; ++u) acc[u] += __builtin_nontemporal_load(p4 + i + u * kThreads);
      }
      for (; i < nvec; i += kThreads) acc[0] += __builtin_nontemporal_load(p4 + i);
    } else {
      for (int i = threadIdx.x; i < PQ; i += kThreads) s += plane[i];
    }
  }
#pragma unroll
  for (int u = 0; u < kInFlight; ++u) s += (acc[u][0] + acc[u][1]) + (acc[u][2] + acc[u][3]);
  block_sum2<kThreads / 64>(s, unused, lds);
  if (threadIdx.x == 0) db[k] = s;
}

struct WPlan {
  Plan p;          // tiles over the OUTPUT of the forward (dy), source = x
  int K, C, S;     // S slices of the reduction over the tiles of one pass
  uint32_t Tc, Tpad;  // tiles per slice, tiles per pass (= S * Tc)
  uint32_t passes;    // the tiles are taken Tpad at a time so that the transforms fit kSliceBytes
  int Kp;
};
static size_t wu_floats(const WPlan& w) { return (size_t)16 * w.Tpad * w.Kp; }
static size_t wv_floats(const WPlan& w) { return (size_t)16 * w.Tpad * w.C; }
static size_t wz_floats(const WPlan& w) { return (size_t)16 * w.S * w.K * w.C; }

static bool make_wplan(const mn_conv2d* g, WPlan& w) {
  Plan& p = w.p;
  p.N = g->N;
  p.Cs = g->C;
  p.Hs = g->H;
  p.Ws = g->W;
  p.M = g->K;
  p.OH = g->P;
  p.OW = g->Q;
  p.pad = g->pH;
  p.TH = (g->P + 1) / 2;
  p.TW = (g->Q + 1) / 2;
  const unsigned long long T = (unsigned long long)g->N * p.TH * p.TW;
  if (T == 0 || T >= (1ull << 28) || g->C % 4 != 0) return false;
  p.T = (uint32_t)T;
  p.Tp = p.T;
  p.Mp = 0;
  w.K = g->K;
  w.C = g->C;
  w.Kp = (g->K + 127) / 128 * 128;
  // tiles per pass: both transforms together under kSliceBytes
  const unsigned long long per_tile = 64ull * ((unsigned long long)w.Kp + g->C);
  unsigned long long Tpass = T;
  if (per_tile * T > kSliceBytes) {
    Tpass = kSliceBytes / per_tile / 2048 * 2048;
    if (Tpass < 2048) Tpass = 2048;
    if (Tpass > T) Tpass = T;
  }
  // enough independent GEMMs for ~8 workgroups per CU, at least 64 tiles per slice
  const long long per_batch = (long long)((g->C + 63) / 64) * ((g->K + 127) / 128);
  long long S = (2048 + 16 * per_batch - 1) / (16 * per_batch);
  if (S > (long long)(Tpass / 64)) S = (long long)(Tpass / 64);
  if (S > 64) S = 64;
  if (S < 1) S = 1;
  w.S = (int)S;
  w.Tc = (uint32_t)(((Tpass + S - 1) / S + 31) / 32 * 32);
  w.Tpad = w.Tc * (uint32_t)S;
  w.passes = (uint32_t)((T + w.Tpad - 1) / w.Tpad);
  p.t0 = 0;
  if ((unsigned long long)w.Tc * w.Kp >= (1ull << 29) || (unsigned long long)w.Tc * w.C >= (1ull << 29) ||
      (unsigned long long)16 * w.Tpad * w.Kp >= (1ull << 36))
    return false;
  return true;
}

static bool make_plan(int N, int Cs, int Hs, int Ws, int M, int OH, int OW, int pad, Plan& p) {
  p.N = N;
  p.Cs = Cs;
  p.Hs = Hs;
  p.Ws = Ws;
  p.M = M;
  p.OH = OH;
  p.OW = OW;
  p.pad = pad;
  p.TH = (OH + 1) / 2;
  p.TW = (OW + 1) / 2;
  const unsigned long long T = (unsigned long long)N * p.TH * p.TW;
  if (T == 0 || T >= (1ull << 28)) return false;
  p.T = (uint32_t)T;
  p.Mp = (M + 127) / 128 * 128;
  // V and Mt together stay under kSliceBytes: larger problems run slice after slice through the
  // same two buffers (measured at 512 MB: within 1 % of the unsliced time from 256 channels up,
  // where this variant is the fastest; 192 MB costs 4-10 %, 48 MB 25-35 %)
  p.slice = p.T;
  const unsigned long long per_tile = 64ull * ((unsigned long long)Cs + M);
  if (per_tile * p.T > kSliceBytes) {
    const unsigned long long t = kSliceBytes / per_tile / 256 * 256;
    p.slice = (uint32_t)(t < 256 ? 256 : t);
    if (p.slice > p.T) p.slice = p.T;
  }
  // the fused kernel addresses its operands through buffer descriptors with 31-bit byte offsets
  const unsigned long long sb = (unsigned long long)N * Cs * Hs * Ws * 4ull, ub = 64ull * Cs * p.Mp;
  p.src_bytes = sb < (1ull << 31) ? (uint32_t)sb : 0u;
  p.u_bytes = ub < (1ull << 31) ? (uint32_t)ub : 0u;
  p.Tp = (p.slice + 3u) & ~3u;
  p.t0 = 0;
  p.Ts = p.slice;
  p.Tsp = p.Tp;
  // one thread per (channel, tile) with 32-bit indices; every GEMM slice below 2 GB
  if ((unsigned long long)Cs * p.Tp >= (1ull << 29) || (unsigned long long)M * p.Tp >= (1ull << 29) ||
      (unsigned long long)Cs * p.Mp >= (1ull << 29))
    return false;
  return Cs % 16 == 0;
}

static int run(Plan p, const float* src, const float* w, bool flip, const float* bias,
               float* dst, bool accum, void* ws, size_t ws_bytes, hipStream_t s) {
  const size_t need = (u_floats(p) + v_floats(p) + m_floats(p)) * sizeof(float);
  if (!ws || ws_bytes < need || !mn_aligned(ws, 16)) return MN_EINVAL;
  float* U = static_cast<float*>(ws);
  float* V = U + u_floats(p);
  float* Mt = V + v_floats(p);
  const uint32_t nu = (uint32_t)p.Cs * p.Mp;
  if (flip)
    weight_kernel<true><<<(nu + kThreads - 1) / kThreads, kThreads, 0, s>>>(w, U, p.M, p.Mp, p.Cs);
  else
    weight_kernel<false><<<(nu + kThreads - 1) / kThreads, kThreads, 0, s>>>(w, U, p.M, p.Mp, p.Cs);
  for (uint32_t t0 = 0; t0 < p.T; t0 += p.slice) {
    p.t0 = t0;
    p.Ts = p.T - t0 < p.slice ? p.T - t0 : p.slice;
    p.Tsp = (p.Ts + 3u) & ~3u;
    const uint32_t nv = (uint32_t)p.Cs * p.Tsp;
    input_kernel<<<(nv + kThreads - 1) / kThreads, kThreads, 0, s>>>(p, src, V);
    const int st = mn_conv_batched_gemm(U, V, Mt, p.M, p.Mp, p.Cs, p.Tsp, 16, s);
    if (st != MN_OK) return st;
    const uint32_t no = (uint32_t)p.M * p.Tsp;
    if (accum)
      output_kernel<true><<<(no + kThreads - 1) / kThreads, kThreads, 0, s>>>(p, Mt, bias, dst);
    else
      output_kernel<false><<<(no + kThreads - 1) / kThreads, kThreads, 0, s>>>(p, Mt, bias, dst);
  }
  return mn_launch_status();
}

// The fused kernels use 80 KB (forward, backward-data) and 139 KB (backward-weight) of LDS per
// workgroup, more than a kernel gets without asking:
// raise its limit once per device (gfx950 has 160 KB per CU).
static bool fused_lds_allowed() {
  static std::mutex lock;
  static bool done[64] = {};
  int dev = 0;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return false;
  std::lock_guard<std::mutex> hold(lock);
  if (done[dev]) return true;
  const bool ok =
      hipFuncSetAttribute(reinterpret_cast<const void*>(&fused_kernel<true>),
                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)kFusedLds) == hipSuccess &&
      hipFuncSetAttribute(reinterpret_cast<const void*>(&fused_kernel<false>),
                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)kFusedLds) == hipSuccess &&
      hipFuncSetAttribute(reinterpret_cast<const void*>(&fused_wgrad_kernel<true>),
                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)kWgRowsLds) == hipSuccess &&
      hipFuncSetAttribute(reinterpret_cast<const void*>(&fused_wgrad_kernel<false>),
                          hipFuncAttributeMaxDynamicSharedMemorySize, (int)kWgRowsLds) == hipSuccess;
  done[dev] = ok;
  return ok;
}

static int run_fused(const Plan& p, const float* src, const float* w, bool flip, const float* bias,
                     float* dst, bool accum, void* ws, size_t ws_bytes, hipStream_t s) {
  // every refusal comes before the first launch: a caller that falls back to another variant
  // (and one that accumulates into dst) must find nothing done
  const uint32_t nkb = (uint32_t)(p.M + FK - 1) / FK, ntb = (p.T + FT - 1) / FT;
  if ((unsigned long long)nkb * ntb >= (1ull << 31) || !p.src_bytes || !p.u_bytes) return MN_EUNSUPPORTED;
  if (!fused_lds_allowed()) return MN_EUNSUPPORTED;  // this device does not grant 80 KB of LDS to a workgroup
  const size_t need = u_floats(p) * sizeof(float);
  if (!ws || ws_bytes < need || !mn_aligned(ws, 16)) return MN_EINVAL;
  float* U = static_cast<float*>(ws);
  const uint32_t nu = (uint32_t)p.Cs * p.Mp;
  if (flip)
    weight_kernel<true, true><<<(nu + kThreads - 1) / kThreads, kThreads, 0, s>>>(w, U, p.M, p.Mp, p.Cs);
  else
    weight_kernel<false, true><<<(nu + kThreads - 1) / kThreads, kThreads, 0, s>>>(w, U, p.M, p.Mp, p.Cs);
  if (accum)
    fused_kernel<true><<<nkb * ntb, kThreads, kFusedLds, s>>>(p, src, U, bias, dst, nkb);
  else
    fused_kernel<false><<<nkb * ntb, kThreads, kFusedLds, s>>>(p, src, U, bias, dst, nkb);
  return mn_launch_status();
}

static bool shape_ok(const mn_conv2d* g) {
  return g->R == 3 && g->S == 3 && g->sH == 1 && g->sW == 1 && g->dH == 1 && g->dW == 1 &&
         g->pH == g->pW && g->pH <= 2 && g->groups == 1;
}

}  // namespace mn_wino

// Part of mn_init(): the LDS limit of the one-kernel form, for the current device.
bool mn_wino_init() { return mn_wino::fused_lds_allowed(); }

// Entry points used by conv.hip (all fp32).  `bytes` = 0 and MN_EUNSUPPORTED when the shape is
// not a 3x3 / stride 1 / dilation 1 convolution with a reduction over a multiple of 16 channels.
int mn_wino_ws_bytes(const mn_conv2d* g, bool backward_data, size_t* bytes) {
  using namespace mn_wino;
  *bytes = 0;
  if (!shape_ok(g)) return MN_EUNSUPPORTED;
  Plan p;
  const bool ok = backward_data
                      ? make_plan(g->N, g->K, g->P, g->Q, g->C, g->H, g->W, 2 - g->pH, p)
                      : make_plan(g->N, g->C, g->H, g->W, g->K, g->P, g->Q, g->pH, p);
  if (!ok) return MN_EUNSUPPORTED;
  *bytes = (u_floats(p) + v_floats(p) + m_floats(p)) * sizeof(float);
  return MN_OK;
}

int mn_wino_fwd(const mn_conv2d* g, const float* x, const float* w, const float* bias, float* y,
                void* ws, size_t ws_bytes, hipStream_t s) {
  using namespace mn_wino;
  Plan p;
  if (!shape_ok(g) || !make_plan(g->N, g->C, g->H, g->W, g->K, g->P, g->Q, g->pH, p))
    return MN_EUNSUPPORTED;
  return run(p, x, w, false, bias, y, false, ws, ws_bytes, s);
}

int mn_wino_bwd_data(const mn_conv2d* g, const float* dy, const float* w, float* dx, bool accum,
                     void* ws, size_t ws_bytes, hipStream_t s) {
  using namespace mn_wino;
  Plan p;
  if (!shape_ok(g) || !make_plan(g->N, g->K, g->P, g->Q, g->C, g->H, g->W, 2 - g->pH, p))
    return MN_EUNSUPPORTED;
  return run(p, dy, w, true, nullptr, dx, accum, ws, ws_bytes, s);
}

// The fused kernel: workspace = the transformed weights only.
int mn_wino_fused_ws_bytes(const mn_conv2d* g, bool backward_data, size_t* bytes) {
  using namespace mn_wino;
  *bytes = 0;
  if (!shape_ok(g)) return MN_EUNSUPPORTED;
  Plan p;
  const bool ok = backward_data
                      ? make_plan(g->N, g->K, g->P, g->Q, g->C, g->H, g->W, 2 - g->pH, p)
                      : make_plan(g->N, g->C, g->H, g->W, g->K, g->P, g->Q, g->pH, p);
  if (!ok || !p.src_bytes || !p.u_bytes) return MN_EUNSUPPORTED;  // 2 GB or more: not through this kernel
  *bytes = u_floats(p) * sizeof(float);
  return MN_OK;
}

int mn_wino_fused_fwd(const mn_conv2d* g, const float* x, const float* w, const float* bias, float* y,
                      void* ws, size_t ws_bytes, hipStream_t s) {
  using namespace mn_wino;
  Plan p;
  if (!shape_ok(g) || !make_plan(g->N, g->C, g->H, g->W, g->K, g->P, g->Q, g->pH, p))
    return MN_EUNSUPPORTED;
  return run_fused(p, x, w, false, bias, y, false, ws, ws_bytes, s);
}

int mn_wino_fused_bwd_data(const mn_conv2d* g, const float* dy, const float* w, float* dx, bool accum,
                           void* ws, size_t ws_bytes, hipStream_t s) {
  using namespace mn_wino;
  Plan p;
  if (!shape_ok(g) || !make_plan(g->N, g->K, g->P, g->Q, g->C, g->H, g->W, 2 - g->pH, p))
    return MN_EUNSUPPORTED;
  return run_fused(p, dy, w, true, nullptr, dx, accum, ws, ws_bytes, s);
}

// Weight gradient (fp32) through the Winograd form above; db (optional): the bias gradient.
namespace mn_wino {
static bool make_fwplan(const mn_conv2d* g, FWPlan& f) {
  if (!shape_ok(g) || g->pH != 1 || g->pW != 1) return false;
  if (g->H != g->P || g->W != g->Q || (g->H & 1) || (g->W & 3) || g->K % FK != 0 || g->C % FT != 0)
    return false;
  const unsigned long long xb = (unsigned long long)g->N * g->C * g->H * g->W * 4ull;
  const unsigned long long yb = (unsigned long long)g->N * g->K * g->H * g->W * 4ull;
  if (xb >= (1ull << 31) || yb >= (1ull << 31) || g->N == 0) return false;
  f.N = g->N;
  f.C = g->C;
  f.K = g->K;
  f.H = g->H;
  f.W = g->W;
  f.TH = g->H / 2;
  f.TW = g->W / 2;
  f.rows = (uint32_t)g->N * f.TH;
  f.x_bytes = (uint32_t)xb;
  f.dy_bytes = (uint32_t)yb;
  // one workgroup per CU (256 accumulation registers per lane, 139 KB of LDS): as many ranges of
  // tile rows as that leaves per (output, input) block
  int dev = 0, cus = 256;
  if (hipGetDevice(&dev) != hipSuccess ||
      hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
    cus = 256;
  const long long blocks = (long long)(g->K / FK) * (g->C / FT);
  long long S = cus / blocks;
  if (S < 1) S = 1;
  if (S > f.rows) S = f.rows;
  f.rows_per_range = (uint32_t)((f.rows + S - 1) / S);
  f.S = (int)((f.rows + f.rows_per_range - 1) / f.rows_per_range);
  return true;
}
}  // namespace mn_wino

// Backward-weight variant 3: Z (16 * ranges * K * C floats) and the bias sums per range.
int mn_wino_fused_bwd_weight_ws_bytes(const mn_conv2d* g, size_t* bytes) {
  using namespace mn_wino;
  *bytes = 0;
  FWPlan f;
  if (!make_fwplan(g, f)) return MN_EUNSUPPORTED;
  *bytes = ((size_t)16 * f.S * f.K * f.C + (size_t)f.S * f.K) * sizeof(float);
  return MN_OK;
}

int mn_wino_fused_bwd_weight(const mn_conv2d* g, const float* dy, const float* x, float* dw, float* db,
                             void* ws, size_t ws_bytes, hipStream_t s) {
  using namespace mn_wino;
  FWPlan f;
  if (!make_fwplan(g, f)) return MN_EUNSUPPORTED;
  if (!fused_lds_allowed()) return MN_EUNSUPPORTED;
  const size_t zf = (size_t)16 * f.S * f.K * f.C;
  const size_t need = (zf + (size_t)f.S * f.K) * sizeof(float);
  if (!ws || ws_bytes < need || !mn_aligned(ws, 16) || !mn_aligned(x, 8) || !mn_aligned(dy, 8))
    return MN_EINVAL;
  float* Z = static_cast<float*>(ws);
  float* dbp = Z + zf;
  const uint32_t grid = (uint32_t)(f.K / FK) * (f.C / FT) * f.S;
  if (db)
    fused_wgrad_kernel<true><<<grid, kThreads, kWgRowsLds, s>>>(f, x, dy, Z, dbp);
  else
    fused_wgrad_kernel<false><<<grid, kThreads, kWgRowsLds, s>>>(f, x, dy, Z, dbp);
  const uint32_t n = (uint32_t)f.K * f.C;
  wgrad_output_kernel<false><<<(n + 63) / 64, kThreads, 0, s>>>(Z, dw, f.K, f.C, f.S);
  if (db) bias_ranges_kernel<<<(f.K + kThreads - 1) / kThreads, kThreads, 0, s>>>(dbp, db, f.K, f.S);
  return mn_launch_status();
}

int mn_wino_bwd_weight_ws_bytes(const mn_conv2d* g, size_t* bytes) {
  using namespace mn_wino;
  *bytes = 0;
  WPlan w;
  if (!shape_ok(g) || !make_wplan(g, w)) return MN_EUNSUPPORTED;
  *bytes = (wu_floats(w) + wv_floats(w) + wz_floats(w)) * sizeof(float);
  return MN_OK;
}

int mn_wino_bwd_weight(const mn_conv2d* g, const float* dy, const float* x, float* dw, float* db,
                       void* ws, size_t ws_bytes, hipStream_t s) {
  using namespace mn_wino;
  WPlan w;
  if (!shape_ok(g) || !make_wplan(g, w)) return MN_EUNSUPPORTED;
  const size_t need = (wu_floats(w) + wv_floats(w) + wz_floats(w)) * sizeof(float);
  if (!ws || ws_bytes < need || !mn_aligned(ws, 16)) return MN_EINVAL;
  float* U = static_cast<float*>(ws);
  float* V = U + wu_floats(w);
  float* Z = V + wv_floats(w);
  const dim3 gu(w.Tpad / 32, w.Kp / 32), gv(w.Tpad / 32, (w.C + 31) / 32);
  const uint32_t n = (uint32_t)w.K * w.C;
  for (uint32_t pass = 0; pass < w.passes; ++pass) {
    w.p.t0 = pass * w.Tpad;
    wgrad_transform_kernel<true><<<gu, kThreads, 0, s>>>(w.p, w.K, dy, U, w.Kp, w.Tpad);
    wgrad_transform_kernel<false><<<gv, kThreads, 0, s>>>(w.p, w.C, x, V, w.C, w.Tpad);
    const int st = mn_conv_batched_gemm(U, V, Z, w.K, w.Kp, (int)w.Tc, (uint32_t)w.C, 16 * w.S, s);
    if (st != MN_OK) return st;
    if (pass == 0)
      wgrad_output_kernel<false><<<(n + 63) / 64, kThreads, 0, s>>>(Z, dw, w.K, w.C, w.S);
    else
      wgrad_output_kernel<true><<<(n + 63) / 64, kThreads, 0, s>>>(Z, dw, w.K, w.C, w.S);
  }
  if (db) bias_grad_kernel<<<w.K, kThreads, 0, s>>>(dy, db, g->N, g->K, g->P * g->Q);
  return mn_launch_status();
}
