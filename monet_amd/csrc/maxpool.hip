// Max-pool forward with 4-bit window-relative argmax indices, and the
// backward that gathers from them.  Index of a window element =
// ch*kW + cw, where (ch, cw) count rows / columns from the UNCLIPPED window
// origin (ph*sH - pH, pw*sW - pW) in steps of the dilation.
#include "common.h"

namespace {

constexpr int kThreads = 256;

// Geometry with compile-time constants (K == kernel, S == stride, P == pad,
// dilation 1) or, for the generic case, run-time fields.
template <int K, int S, int P>
struct CtGeo {
  __device__ __forceinline__ int kH() const { return K; }
  __device__ __forceinline__ int kW() const { return K; }
  __device__ __forceinline__ int sH() const { return S; }
  __device__ __forceinline__ int sW() const { return S; }
  __device__ __forceinline__ int pH() const { return P; }
  __device__ __forceinline__ int pW() const { return P; }
  __device__ __forceinline__ int dH() const { return 1; }
  __device__ __forceinline__ int dW() const { return 1; }
};
struct RtGeo {
  int kh, kw, sh, sw, ph, pw, dh, dw;
  __device__ __forceinline__ int kH() const { return kh; }
  __device__ __forceinline__ int kW() const { return kw; }
  __device__ __forceinline__ int sH() const { return sh; }
  __device__ __forceinline__ int sW() const { return sw; }
  __device__ __forceinline__ int pH() const { return ph; }
  __device__ __forceinline__ int pW() const { return pw; }
  __device__ __forceinline__ int dH() const { return dh; }
  __device__ __forceinline__ int dW() const { return dw; }
};

// One output element: scan the window row-major; a strictly larger value or a
// NaN takes over.  If nothing does (window of -inf) the first valid element
// is reported.
template <class G>
__device__ __forceinline__ void pool_one(const G g, const float* __restrict__ xp, int H, int W,
                                         int ph, int pw, float& best, uint32_t& bidx) {
  int hstart = ph * g.sH() - g.pH();
  int wstart = pw * g.sW() - g.pW();
  const int hend = min(hstart + (g.kH() - 1) * g.dH() + 1, H);
  const int wend = min(wstart + (g.kW() - 1) * g.dW() + 1, W);
  int ch0 = 0, cw0 = 0;
  while (hstart < 0) {
    hstart += g.dH();
    ++ch0;
  }
  while (wstart < 0) {
    wstart += g.dW();
    ++cw0;
  }
  float maxval = -INFINITY;
  uint32_t maxidx = ch0 * g.kW() + cw0;
  int ch = ch0;
  for (int h = hstart; h < hend; h += g.dH(), ++ch) {
    int cw = cw0;
    for (int w = wstart; w < wend; w += g.dW(), ++cw) {
      const float val = xp[(size_t)h * W + w];
      if (val > maxval || val != val) {
        maxidx = ch * g.kW() + cw;
        maxval = val;
      }
    }
  }
  best = maxval;
  bidx = maxidx;
}

// One thread per PAIR of consecutive outputs in flat NCHW order = one index
// byte.  `total` = N*C*PH*PW.
template <class G>
__global__ __launch_bounds__(kThreads) void maxpool_fwd_idx_kernel(
    const G g, const float* __restrict__ x, float* __restrict__ y, uint8_t* __restrict__ idx4,
    int H, int W, int PH, int PW, size_t total) {
  const size_t j = (size_t)blockIdx.x * kThreads + threadIdx.x;
  const size_t o0 = 2 * j;
  if (o0 >= total) return;
  const uint32_t plane_sz = (uint32_t)PH * PW;
  size_t plane = o0 / plane_sz;
  uint32_t r = (uint32_t)(o0 - plane * plane_sz);
  int ph = r / PW;
  int pw = r - ph * PW;
  float v0, v1 = 0.f;
  uint32_t i0, i1 = 0;
  pool_one(g, x + plane * (size_t)H * W, H, W, ph, pw, v0, i0);
  y[o0] = v0;
  if (o0 + 1 < total) {
    if (++pw == PW) {
      pw = 0;
      if (++ph == PH) {
        ph = 0;
        ++plane;
      }
    }
    pool_one(g, x + plane * (size_t)H * W, H, W, ph, pw, v1, i1);
    y[o0 + 1] = v1;
  }
  idx4[j] = (uint8_t)(((i0 & 15u) << 4) | (i1 & 15u));
}

// Forward for kernel 3, stride 2, pad 1, dilation 1 with even H and W % 4 == 0
// (PH = H/2, PW = W/2): one workgroup per (n, c) plane, one thread per pair of
// horizontally adjacent outputs = one index byte.  The pair's two windows span
// input columns 4q-1 .. 4q+3 of rows 2ph-1 .. 2ph+1: per row one aligned
// 16-byte load plus the left neighbour.  Scan order and tie rules are those of
// pool_one, so values and indices are identical to the generic kernel's.
__global__ __launch_bounds__(kThreads) void maxpool_fwd_k3s2p1_kernel(
    const float* __restrict__ x, float* __restrict__ y, uint8_t* __restrict__ idx4, int H, int W) {
  const int PH = H >> 1, PW = W >> 1, QW = W >> 2;
  const size_t plane = blockIdx.x;
  const float* xp = x + plane * (size_t)H * W;
  float* yp = y + plane * (size_t)PH * PW;
  uint8_t* ip = idx4 + ((plane * (size_t)PH * PW) >> 1);  // PH*PW is even
  const int items = PH * QW;
  const int qstep = kThreads / QW, rstep = kThreads - qstep * QW;
  int ph = threadIdx.x / QW;
  int q = threadIdx.x - ph * QW;
  for (int it = threadIdx.x; it < items; it += kThreads) {
    const bool top = ph > 0, left = q > 0;
    float m0 = -INFINITY, m1 = -INFINITY;
    uint32_t i0 = (top ? 0u : 3u) + (left ? 0u : 1u), i1 = top ? 0u : 3u;
#pragma unroll
    for (int ch = 0; ch < 3; ++ch) {
      if (ch == 0 && !top) continue;
      const float* row = xp + (size_t)(2 * ph - 1 + ch) * W + 4 * q;
      const float4_t v = *reinterpret_cast<const float4_t*>(row);
      if (left) {
        const float l = row[-1];
        if (l > m0 || l != l) { m0 = l; i0 = ch * 3; }
      }
      if (v.x > m0 || v.x != v.x) { m0 = v.x; i0 = ch * 3 + 1; }
      if (v.y > m0 || v.y != v.y) { m0 = v.y; i0 = ch * 3 + 2; }
      if (v.y > m1 || v.y != v.y) { m1 = v.y; i1 = ch * 3; }
      if (v.z > m1 || v.z != v.z) { m1 = v.z; i1 = ch * 3 + 1; }
      if (v.w > m1 || v.w != v.w) { m1 = v.w; i1 = ch * 3 + 2; }
    }
    const int o = ph * PW + 2 * q;  // even
    float2_t out = {m0, m1};
    *reinterpret_cast<float2_t*>(yp + o) = out;
    ip[o >> 1] = (uint8_t)((i0 << 4) | i1);
    ph += qstep;
    q += rstep;
    if (q >= QW) {
      q -= QW;
      ++ph;
    }
  }
}

// The two windows of an output pair over one input row: `l` = the column left of the aligned
// four in `v` (only read when `left`).  Same scan order as pool_one.
__device__ __forceinline__ void k3_row(const float4_t v, float l, bool left, uint32_t ch, float& m0,
                                       uint32_t& i0, float& m1, uint32_t& i1) {
  if (left && (l > m0 || l != l)) { m0 = l; i0 = ch * 3; }
  if (v.x > m0 || v.x != v.x) { m0 = v.x; i0 = ch * 3 + 1; }
  if (v.y > m0 || v.y != v.y) { m0 = v.y; i0 = ch * 3 + 2; }
  if (v.y > m1 || v.y != v.y) { m1 = v.y; i1 = ch * 3; }
  if (v.z > m1 || v.z != v.z) { m1 = v.z; i1 = ch * 3 + 1; }
  if (v.w > m1 || v.w != v.w) { m1 = v.w; i1 = ch * 3 + 2; }
}

// The same geometry with H % 4 == 0 as well: one thread per 2 x 2 block of outputs (two
// index bytes), blocks numbered flat over all planes in memory order.  The block's
// windows span input rows 4*ph2-1 .. 4*ph2+3, the middle one shared by both output rows: five
// aligned 16-byte loads per four outputs instead of six plus six scalar ones, and the left
// neighbour column comes from the lane to the left (the previous item of the same rows)
// instead of from memory.  Values and indices are those of pool_one.
__global__ __launch_bounds__(kThreads) void maxpool_fwd_k3s2p1_2x2_kernel(
    const float* __restrict__ x, float* __restrict__ y, uint8_t* __restrict__ idx4, int H, int W,
    uint32_t total) {
  const uint32_t PW = W >> 1, QW = W >> 2, PH2 = H >> 2;
  const uint32_t per_plane = PH2 * QW;
  const size_t in_plane = (size_t)H * W, out_plane = in_plane >> 2;
  const uint32_t lane = threadIdx.x & 63u;
  for (uint32_t base = blockIdx.x * kThreads; base < total; base += gridDim.x * kThreads) {
    const uint32_t it = base + threadIdx.x;
    const bool active = it < total;
    const uint32_t item = active ? it : total - 1;
    const uint32_t plane = item / per_plane;
    const uint32_t rem = item - plane * per_plane;
    const uint32_t ph2 = rem / QW, q = rem - ph2 * QW;
    const bool top = ph2 > 0, left = q > 0;
    const float* xp = x + plane * in_plane + (size_t)(4 * ph2) * W + 4 * q;  // row 4*ph2
    float4_t v[5];
    float l[5];
#pragma unroll
    for (int r = 0; r < 5; ++r) {
      v[r] = float4_t{0.f, 0.f, 0.f, 0.f};
      if (active && (r > 0 || top))
        v[r] = *reinterpret_cast<const float4_t*>(xp + (ptrdiff_t)(r - 1) * W);
    }
#pragma unroll
    for (int r = 0; r < 5; ++r) l[r] = __shfl_up(v[r].w, 1, MN_WAVE);
    if (lane == 0 && left && active) {
#pragma unroll
      for (int r = 0; r < 5; ++r)
        if (r > 0 || top) l[r] = xp[(ptrdiff_t)(r - 1) * W - 1];
    }
    if (!active) continue;
    float* yp = y + plane * out_plane + (size_t)(2 * ph2) * PW + 2 * q;
    uint8_t* ip = idx4 + ((plane * out_plane + (size_t)(2 * ph2) * PW + 2 * q) >> 1);
    {
      float m0 = -INFINITY, m1 = -INFINITY;
      uint32_t i0 = (top ? 0u : 3u) + (left ? 0u : 1u), i1 = top ? 0u : 3u;
      if (top) k3_row(v[0], l[0], left, 0, m0, i0, m1, i1);
      k3_row(v[1], l[1], left, 1, m0, i0, m1, i1);
      k3_row(v[2], l[2], left, 2, m0, i0, m1, i1);
      *reinterpret_cast<float2_t*>(yp) = float2_t{m0, m1};
      ip[0] = (uint8_t)((i0 << 4) | i1);
    }
    {
      float m0 = -INFINITY, m1 = -INFINITY;
      uint32_t i0 = left ? 0u : 1u, i1 = 0u;
      k3_row(v[2], l[2], left, 0, m0, i0, m1, i1);
      k3_row(v[3], l[3], left, 1, m0, i0, m1, i1);
      k3_row(v[4], l[4], left, 2, m0, i0, m1, i1);
      *reinterpret_cast<float2_t*>(yp + PW) = float2_t{m0, m1};
      ip[PW >> 1] = (uint8_t)((i0 << 4) | i1);
    }
  }
}

// Range of windows along one axis that cover input coordinate `c`.
template <class G>
__device__ __forceinline__ void cover(int c, int pad, int k, int dil, int stride, int pooled,
                                      int& lo, int& hi) {
  const int ext = (k - 1) * dil + 1;
  lo = (c + pad < ext) ? 0 : (c + pad - ext) / stride + 1;
  hi = min((c + pad) / stride + 1, pooled);
}

template <class G>
__device__ __forceinline__ float pool_bwd_one(const G g, const float* __restrict__ dyp,
                                              const uint8_t* __restrict__ idx4, size_t obase,
                                              int PH, int PW, int h, int w) {
  int ph0, ph1, pw0, pw1;
  cover<G>(h, g.pH(), g.kH(), g.dH(), g.sH(), PH, ph0, ph1);
  cover<G>(w, g.pW(), g.kW(), g.dW(), g.sW(), PW, pw0, pw1);
  float grad = 0.f;
  for (int ph = ph0; ph < ph1; ++ph) {
    const int oh = h - ph * g.sH() + g.pH();
    if (g.dH() != 1 && oh % g.dH() != 0) continue;
    for (int pw = pw0; pw < pw1; ++pw) {
      const int ow = w - pw * g.sW() + g.pW();
      if (g.dW() != 1 && ow % g.dW() != 0) continue;
      const uint32_t rel = (oh / g.dH()) * g.kW() + ow / g.dW();
      const size_t o = obase + (size_t)ph * PW + pw;
      const uint32_t b = idx4[o >> 1];
      const uint32_t stored = (o & 1) ? (b & 15u) : (b >> 4);
      if (stored == rel) grad += dyp[(size_t)ph * PW + pw];
    }
  }
  return grad;
}

// grid = (chunks of a plane, planes); VEC consecutive w per thread.
template <class G, int VEC>
__global__ __launch_bounds__(kThreads) void maxpool_bwd_idx_kernel(
    const G g, const float* __restrict__ dy, const uint8_t* __restrict__ idx4,
    float* __restrict__ dx, int H, int W, int PH, int PW, uint32_t planes) {
  const int WV = W / VEC;
  const uint32_t per_plane = (uint32_t)H * WV;
  const uint32_t t = blockIdx.x * kThreads + threadIdx.x;
  if (t >= per_plane) return;
  const int h = t / WV;
  const int w0 = (t - h * WV) * VEC;
  for (uint32_t plane = blockIdx.y; plane < planes; plane += gridDim.y) {
    const size_t obase = (size_t)plane * PH * PW;
    const float* dyp = dy + obase;
    float r[VEC];
#pragma unroll
    for (int v = 0; v < VEC; ++v) r[v] = pool_bwd_one(g, dyp, idx4, obase, PH, PW, h, w0 + v);
    float* out = dx + ((size_t)plane * H + h) * W + w0;
    if (VEC == 4) {
      float4_t q = {r[0], r[1], r[2], r[3]};
      st_stream(reinterpret_cast<float4_t*>(out), q);
    } else {
#pragma unroll
      for (int v = 0; v < VEC; ++v) out[v] = r[v];
    }
  }
}

// Backward for kernel 3, stride 2, pad 1, dilation 1 with even H, W % 4 == 0
// (so PH = H/2, PW = W/2).  One workgroup per (n, c) plane; a thread produces a
// 2-row x 4-column patch of dx from the 2 x 3 windows that can reach it, so
// every dy / index element is fetched by at most two threads and every dx
// element is written once with 16-byte stores.  Window (ph, pw) covers rows
// 2ph-1..2ph+1 and columns 2pw-1..2pw+1; index k = ch*3 + cw.
__global__ __launch_bounds__(kThreads) void maxpool_bwd_k3s2p1_kernel(
    const float* __restrict__ dy, const uint8_t* __restrict__ idx4, float* __restrict__ dx, int H,
    int W) {
  const int PH = H >> 1, PW = W >> 1, QW = W >> 2, RH = H >> 1;
  const size_t plane = blockIdx.x;
  const float* dyp = dy + plane * (size_t)PH * PW;
  const uint8_t* ip = idx4 + ((plane * (size_t)PH * PW) >> 1);  // PH*PW is even
  float* dxp = dx + plane * (size_t)H * W;
  const int items = RH * QW;
  const int qstep = kThreads / QW, rstep = kThreads - qstep * QW;
  int r = threadIdx.x / QW;
  int q = threadIdx.x - r * QW;
  for (int it = threadIdx.x; it < items; it += kThreads) {
    // windows: rows r (A) and r+1 (B); columns 2q, 2q+1, 2q+2
    const bool rowB = r + 1 < PH;
    const bool col2 = 2 * q + 2 < PW;
    const int oA = r * PW + 2 * q;  // even
    const int oB = oA + PW;
    const uint32_t a01 = ip[oA >> 1];
    const uint32_t a2 = col2 ? ip[(oA >> 1) + 1] : 0xFFu;
    const uint32_t b01 = rowB ? ip[oB >> 1] : 0xFFu;
    const uint32_t b2 = (rowB && col2) ? ip[(oB >> 1) + 1] : 0xFFu;
    const float2_t ga = *reinterpret_cast<const float2_t*>(dyp + oA);
    const float ga2 = col2 ? dyp[oA + 2] : 0.f;
    float2_t gb = {0.f, 0.f};
    if (rowB) gb = *reinterpret_cast<const float2_t*>(dyp + oB);
    const float gb2 = (rowB && col2) ? dyp[oB + 2] : 0.f;
    const uint32_t iA0 = a01 >> 4, iA1 = a01 & 15u, iA2 = a2 >> 4;
    const uint32_t iB0 = b01 >> 4, iB1 = b01 & 15u, iB2 = b2 >> 4;  // 0xFF >> 4 = 15: never a k < 9
#define MN_M(i, k, g) ((i) == (k) ? (g) : 0.f)
    float4_t top, bot;
    // row 2r: only window row A, ch = 1
    top.x = 0.f + MN_M(iA0, 4u, ga.x);
    top.y = 0.f + MN_M(iA0, 5u, ga.x) + MN_M(iA1, 3u, ga.y);
    top.z = 0.f + MN_M(iA1, 4u, ga.y);
    top.w = 0.f + MN_M(iA1, 5u, ga.y) + MN_M(iA2, 3u, ga2);
    // row 2r+1: window row A with ch = 2, then window row B with ch = 0
    bot.x = 0.f + MN_M(iA0, 7u, ga.x) + MN_M(iB0, 1u, gb.x);
    bot.y = 0.f + MN_M(iA0, 8u, ga.x) + MN_M(iA1, 6u, ga.y) + MN_M(iB0, 2u, gb.x) +
            MN_M(iB1, 0u, gb.y);
    bot.z = 0.f + MN_M(iA1, 7u, ga.y) + MN_M(iB1, 1u, gb.y);
    bot.w = 0.f + MN_M(iA1, 8u, ga.y) + MN_M(iA2, 6u, ga2) + MN_M(iB1, 2u, gb.y) +
            MN_M(iB2, 0u, gb2);
#undef MN_M
    float* o = dxp + (size_t)(2 * r) * W + 4 * q;
    st_stream(reinterpret_cast<float4_t*>(o), top);
    st_stream(reinterpret_cast<float4_t*>(o + W), bot);
    r += qstep;
    q += rstep;
    if (q >= QW) {
      q -= QW;
      ++r;
    }
  }
}

// The same patches, one per thread, numbered in memory order over the whole tensor with no loop:
// every load of a thread is in flight at once and a CU holds 2048 such threads, which is what a
// cold dy / index tensor needs (one workgroup per plane, above, walks its plane in seven dependent
// rounds of small loads: 188 us at [184,64,112,112] when dy comes from memory, against 122 us when
// a benchmark loop keeps it in the memory-side cache).  The third window column of a patch is
// the first column of the next thread's windows and comes from that lane instead of from memory
// (the last lane of a wavefront loads it).  Same sums in the same order as the kernel above.
__global__ __launch_bounds__(kThreads) void maxpool_bwd_k3s2p1_flat_kernel(
    const float* __restrict__ dy, const uint8_t* __restrict__ idx4, float* __restrict__ dx, int H,
    int W, uint32_t total) {
  const uint32_t PH = (uint32_t)H >> 1, PW = (uint32_t)W >> 1, QW = (uint32_t)W >> 2;
  const uint32_t t = blockIdx.x * kThreads + threadIdx.x;
  const bool live = t < total;
  const uint32_t tt = live ? t : total - 1;
  const uint32_t per_plane = PH * QW;
  const uint32_t plane = tt / per_plane, rem = tt - plane * per_plane;
  const uint32_t r = rem / QW, q = rem - r * QW;
  const bool rowB = r + 1 < PH;
  const bool col2 = 2 * q + 2 < PW;
  const size_t oA = (size_t)plane * PH * PW + (size_t)r * PW + 2 * q;  // even: PH*PW is even
  const size_t oB = oA + PW;
  // Streaming loads for dy and the indices, although a pooled row is read twice (as row B of
  // patch row r - 1 and as row A of patch row r, one plane row of threads later): an ordinary
  // load for the first read saves 7 % of the HBM traffic and measured 7 % SLOWER (0.159
  // against 0.148 ms at [184,64,112,112]).  dx is written with ordinary stores, which measured
  // 8 % faster here than streaming ones (0.147 against 0.160 ms with operands from memory)
  const uint32_t a01 = ld_stream(idx4 + (oA >> 1));
  const uint32_t b01 = rowB ? ld_stream(idx4 + (oB >> 1)) : 0xFFu;
  const float2_t ga = ld_stream(reinterpret_cast<const float2_t*>(dy + oA));
  float2_t gb = {0.f, 0.f};
  if (rowB) gb = ld_stream(reinterpret_cast<const float2_t*>(dy + oB));
  // next thread = next patch of the same row whenever col2 holds
  uint32_t a2 = (uint32_t)__shfl_down((int)a01, 1, MN_WAVE);
  uint32_t b2 = (uint32_t)__shfl_down((int)b01, 1, MN_WAVE);
  float ga2 = __shfl_down(ga.x, 1, MN_WAVE);
  float gb2 = __shfl_down(gb.x, 1, MN_WAVE);
  if ((threadIdx.x & (MN_WAVE - 1)) == MN_WAVE - 1 && col2) {
    a2 = idx4[(oA >> 1) + 1];
    ga2 = dy[oA + 2];
    b2 = rowB ? idx4[(oB >> 1) + 1] : 0xFFu;
    gb2 = rowB ? dy[oB + 2] : 0.f;
  }
  if (!col2) {
    a2 = 0xFFu;
    b2 = 0xFFu;
    ga2 = 0.f;
    gb2 = 0.f;
  }
  const uint32_t iA0 = a01 >> 4, iA1 = a01 & 15u, iA2 = a2 >> 4;
  const uint32_t iB0 = b01 >> 4, iB1 = b01 & 15u, iB2 = b2 >> 4;  // 0xFF >> 4 = 15: never a k < 9
#define MN_M(i, k, g) ((i) == (k) ? (g) : 0.f)
  float4_t top, bot;
  top.x = 0.f + MN_M(iA0, 4u, ga.x);
  top.y = 0.f + MN_M(iA0, 5u, ga.x) + MN_M(iA1, 3u, ga.y);
  top.z = 0.f + MN_M(iA1, 4u, ga.y);
  top.w = 0.f + MN_M(iA1, 5u, ga.y) + MN_M(iA2, 3u, ga2);
  bot.x = 0.f + MN_M(iA0, 7u, ga.x) + MN_M(iB0, 1u, gb.x);
  bot.y = 0.f + MN_M(iA0, 8u, ga.x) + MN_M(iA1, 6u, ga.y) + MN_M(iB0, 2u, gb.x) +
          MN_M(iB1, 0u, gb.y);
  bot.z = 0.f + MN_M(iA1, 7u, ga.y) + MN_M(iB1, 1u, gb.y);
  bot.w = 0.f + MN_M(iA1, 8u, ga.y) + MN_M(iA2, 6u, ga2) + MN_M(iB1, 2u, gb.y) +
          MN_M(iB2, 0u, gb2);
#undef MN_M
  if (!live) return;
  float* o = dx + (size_t)plane * H * W + (size_t)(2 * r) * W + 4 * q;
  *reinterpret_cast<float4_t*>(o) = top;
  *reinterpret_cast<float4_t*>(o + W) = bot;
}

// NR patch rows per thread (H % (2 NR) == 0): a thread owns 2 NR rows x 4 columns of dx and reads
// pooled rows NR rp .. NR rp + NR.  With one patch row per thread every pooled row is read twice
// (as row B of one patch row and row A of the next); here only every NR-th one is.
template <int NR>
__global__ __launch_bounds__(kThreads) void maxpool_bwd_k3s2p1_flatn_kernel(
    const float* __restrict__ dy, const uint8_t* __restrict__ idx4, float* __restrict__ dx, int H,
    int W, uint32_t total) {
  const uint32_t PH = (uint32_t)H >> 1, PW = (uint32_t)W >> 1, QW = (uint32_t)W >> 2, RP = PH / NR;
  const uint32_t t = blockIdx.x * kThreads + threadIdx.x;
  const bool live = t < total;
  const uint32_t tt = live ? t : total - 1;
  const uint32_t per_plane = RP * QW;
  const uint32_t plane = tt / per_plane, rem = tt - plane * per_plane;
  const uint32_t rp = rem / QW, q = rem - rp * QW;
  const uint32_t r = NR * rp;
  const bool row_last = r + NR < PH;  // the pooled row below the last patch row exists
  const bool col2 = 2 * q + 2 < PW;
  const size_t o0 = (size_t)plane * PH * PW + (size_t)r * PW + 2 * q;  // even: PH*PW is even
  uint32_t i01[NR + 1], i2[NR + 1];
  float2_t g01[NR + 1];
  float g2[NR + 1];
#pragma unroll
  for (int k = 0; k <= NR; ++k) {
    const bool ok = k < NR || row_last;
    const size_t o = o0 + (size_t)(ok ? k : 0) * PW;
    const uint32_t i = ld_stream(idx4 + (o >> 1));
    const float2_t g = ld_stream(reinterpret_cast<const float2_t*>(dy + o));
    i01[k] = ok ? i : 0xFFu;
    g01[k] = ok ? g : float2_t{0.f, 0.f};
  }
  // next thread = next patch of the same rows whenever col2 holds
#pragma unroll
  for (int k = 0; k <= NR; ++k) {
    i2[k] = (uint32_t)__shfl_down((int)i01[k], 1, MN_WAVE);
    g2[k] = __shfl_down(g01[k].x, 1, MN_WAVE);
  }
  if ((threadIdx.x & (MN_WAVE - 1)) == MN_WAVE - 1 && col2) {
#pragma unroll
    for (int k = 0; k <= NR; ++k) {
      const bool ok = k < NR || row_last;
      const size_t o = o0 + (size_t)(ok ? k : 0) * PW;
      i2[k] = ok ? idx4[(o >> 1) + 1] : 0xFFu;
      g2[k] = ok ? dy[o + 2] : 0.f;
    }
  }
  if (!col2) {
#pragma unroll
    for (int k = 0; k <= NR; ++k) {
      i2[k] = 0xFFu;
      g2[k] = 0.f;
    }
  }
  if (!live) return;
  float* o = dx + (size_t)plane * H * W + (size_t)(2 * r) * W + 4 * q;
#define MN_M(i, k, g) ((i) == (k) ? (g) : 0.f)
  // the two dx rows under pooled row A (its windows' rows 1 and 2) with pooled row B's row 0;
  // same sums in the same order as the one-row kernel
#pragma unroll
  for (int k = 0; k < NR; ++k) {
    const uint32_t iA0 = i01[k] >> 4, iA1 = i01[k] & 15u, iA2 = i2[k] >> 4;
    const uint32_t iB0 = i01[k + 1] >> 4, iB1 = i01[k + 1] & 15u, iB2 = i2[k + 1] >> 4;
    const float2_t ga = g01[k], gb = g01[k + 1];
    const float ga2 = g2[k], gb2 = g2[k + 1];
    float4_t top, bot;
    top.x = 0.f + MN_M(iA0, 4u, ga.x);
    top.y = 0.f + MN_M(iA0, 5u, ga.x) + MN_M(iA1, 3u, ga.y);
    top.z = 0.f + MN_M(iA1, 4u, ga.y);
    top.w = 0.f + MN_M(iA1, 5u, ga.y) + MN_M(iA2, 3u, ga2);
    bot.x = 0.f + MN_M(iA0, 7u, ga.x) + MN_M(iB0, 1u, gb.x);
    bot.y = 0.f + MN_M(iA0, 8u, ga.x) + MN_M(iA1, 6u, ga.y) + MN_M(iB0, 2u, gb.x) + MN_M(iB1, 0u, gb.y);
    bot.z = 0.f + MN_M(iA1, 7u, ga.y) + MN_M(iB1, 1u, gb.y);
    bot.w = 0.f + MN_M(iA1, 8u, ga.y) + MN_M(iA2, 6u, ga2) + MN_M(iB1, 2u, gb.y) + MN_M(iB2, 0u, gb2);
    *reinterpret_cast<float4_t*>(o + (size_t)(2 * k) * W) = top;
    *reinterpret_cast<float4_t*>(o + (size_t)(2 * k + 1) * W) = bot;
  }
#undef MN_M
}

int check_geo(const mn_pool2d* g) {
  if (!g) return MN_EINVAL;
  if (g->N < 0 || g->C < 0 || g->H <= 0 || g->W <= 0 || g->PH <= 0 || g->PW <= 0) return MN_EINVAL;
  if (g->kH <= 0 || g->kW <= 0 || g->sH <= 0 || g->sW <= 0 || g->dH <= 0 || g->dW <= 0)
    return MN_EINVAL;
  if (g->pH < 0 || g->pW < 0 || 2 * g->pH > g->kH || 2 * g->pW > g->kW) return MN_EINVAL;
  if (g->kH * g->kW > 16) return MN_EUNSUPPORTED;  // index must fit a nibble
  // every window must start inside the padded image and hold >= 1 real element
  if ((int64_t)(g->PH - 1) * g->sH >= (int64_t)g->H + g->pH) return MN_EINVAL;
  if ((int64_t)(g->PW - 1) * g->sW >= (int64_t)g->W + g->pW) return MN_EINVAL;
  if ((int64_t)g->H * g->W >= (1ll << 31) || (int64_t)g->PH * g->PW >= (1ll << 31))
    return MN_EUNSUPPORTED;
  return MN_OK;
}

template <class G>
void launch_fwd(const G geo, const mn_pool2d* g, const float* x, float* y, uint8_t* idx4,
                hipStream_t s) {
  const size_t total = (size_t)g->N * g->C * g->PH * g->PW;
  const size_t pairs = (total + 1) / 2;
  const unsigned blocks = (unsigned)((pairs + kThreads - 1) / kThreads);
  maxpool_fwd_idx_kernel<G><<<blocks, kThreads, 0, s>>>(geo, x, y, idx4, g->H, g->W, g->PH, g->PW,
                                                        total);
}

template <class G>
void launch_bwd(const G geo, const mn_pool2d* g, const float* dy, const uint8_t* idx4, float* dx,
                hipStream_t s) {
  const uint32_t planes = (uint32_t)g->N * g->C;
  const bool vec = (g->W % 4 == 0) && mn_aligned(dx, 16);
  const uint32_t per_plane = (uint32_t)g->H * (vec ? g->W / 4 : g->W);
  dim3 grid((per_plane + kThreads - 1) / kThreads, planes < 65535u ? planes : 65535u);
  if (vec)
    maxpool_bwd_idx_kernel<G, 4><<<grid, kThreads, 0, s>>>(geo, dy, idx4, dx, g->H, g->W, g->PH,
                                                           g->PW, planes);
  else
    maxpool_bwd_idx_kernel<G, 1><<<grid, kThreads, 0, s>>>(geo, dy, idx4, dx, g->H, g->W, g->PH,
                                                           g->PW, planes);
}

bool is_ct(const mn_pool2d* g, int k, int s, int p) {
  return g->kH == k && g->kW == k && g->sH == s && g->sW == s && g->pH == p && g->pW == p &&
         g->dH == 1 && g->dW == 1;
}

RtGeo rt(const mn_pool2d* g) {
  return RtGeo{g->kH, g->kW, g->sH, g->sW, g->pH, g->pW, g->dH, g->dW};
}

}  // namespace

extern "C" {

int64_t mn_pool_out_size(int64_t in, int64_t k, int64_t pad, int64_t stride, int64_t dil,
                         int ceil_mode) {
  if (in <= 0 || k <= 0 || stride <= 0 || dil <= 0 || pad < 0) return -1;
  const int64_t num = in + 2 * pad - dil * (k - 1) - 1 + (ceil_mode ? stride - 1 : 0);
  // floor division (num may be negative)
  int64_t q = num / stride;
  if ((num % stride != 0) && ((num < 0) != (stride < 0))) --q;
  int64_t out = q + 1;
  if (pad && (out - 1) * stride >= in + pad) --out;  // last window must start inside the image
  return out;
}

int mn_maxpool_fwd_idx_f32(const mn_pool2d* g, const float* x, float* y, uint8_t* idx4,
                           mn_stream_t stream) {
  const int st = check_geo(g);
  if (st != MN_OK) return st;
  if ((size_t)g->N * g->C == 0) return MN_OK;
  if (!x || !y || !idx4) return MN_EINVAL;
  hipStream_t s = mn_stream(stream);
  const uint64_t blocks2x2 = (uint64_t)g->N * g->C * (uint64_t)(g->H / 4) * (uint64_t)(g->W / 4);
  if (is_ct(g, 3, 2, 1) && g->H % 4 == 0 && g->W % 4 == 0 && g->PH == g->H / 2 &&
      g->PW == g->W / 2 && mn_aligned(x, 16) && mn_aligned(y, 8) && blocks2x2 < (1ull << 31)) {
    // one block per thread, workgroups in memory order: the workgroups that run at the same
    // time then read neighbouring rows (a fixed grid striding over the planes measured 0.157 ms
    // against 0.138 ms at [184,64,112,112]; non-temporal stores cost another 0.01 ms)
    const unsigned grid = (unsigned)((blocks2x2 + kThreads - 1) / kThreads);
    maxpool_fwd_k3s2p1_2x2_kernel<<<grid, kThreads, 0, s>>>(x, y, idx4, g->H, g->W,
                                                            (uint32_t)blocks2x2);
  } else if (is_ct(g, 3, 2, 1) && g->H % 2 == 0 && g->W % 4 == 0 && g->PH == g->H / 2 &&
      g->PW == g->W / 2 && mn_aligned(x, 16) && mn_aligned(y, 8) && g->W / 4 <= kThreads)
    maxpool_fwd_k3s2p1_kernel<<<(unsigned)g->N * g->C, kThreads, 0, s>>>(x, y, idx4, g->H, g->W);
  else if (is_ct(g, 3, 2, 1))
    launch_fwd(CtGeo<3, 2, 1>{}, g, x, y, idx4, s);
  else if (is_ct(g, 2, 2, 0))
    launch_fwd(CtGeo<2, 2, 0>{}, g, x, y, idx4, s);
  else
    launch_fwd(rt(g), g, x, y, idx4, s);
  return mn_launch_status();
}

int mn_maxpool_bwd_idx_f32(const mn_pool2d* g, const float* dy, const uint8_t* idx4, float* dx,
                           mn_stream_t stream) {
  const int st = check_geo(g);
  if (st != MN_OK) return st;
  if ((size_t)g->N * g->C == 0) return MN_OK;
  if (!dy || !dx || !idx4) return MN_EINVAL;
  hipStream_t s = mn_stream(stream);
  // the fast kernel assumes pooled planes of exactly H/2 x W/2 (ceil_mode can add a row)
  if (is_ct(g, 3, 2, 1) && g->H % 2 == 0 && g->W % 4 == 0 && g->PH == g->H / 2 &&
      g->PW == g->W / 2 && mn_aligned(dx, 16) && mn_aligned(dy, 8) && g->W / 4 <= kThreads)
  {
    // one thread per 2 x 4 patch (per two or four of them, one below the other, when H % 4 == 0 or
    // H % 8 == 0: 0.148 -> 0.142 -> 0.140 ms at [184,64,112,112]) over the whole tensor when the patch count fits 32 bits of
    // thread index, else one workgroup per plane
    const unsigned long long patches = (unsigned long long)g->N * g->C * (g->H / 2) * (g->W / 4);
    if (g->H % 8 == 0 && patches / 4 < (1ull << 32) - kThreads)
      maxpool_bwd_k3s2p1_flatn_kernel<4><<<(unsigned)((patches / 4 + kThreads - 1) / kThreads), kThreads, 0, s>>>(
          dy, idx4, dx, g->H, g->W, (uint32_t)(patches / 4));
    else if (g->H % 4 == 0 && patches / 2 < (1ull << 32) - kThreads)
      maxpool_bwd_k3s2p1_flatn_kernel<2><<<(unsigned)((patches / 2 + kThreads - 1) / kThreads), kThreads, 0, s>>>(
          dy, idx4, dx, g->H, g->W, (uint32_t)(patches / 2));
    else if (patches < (1ull << 32) - kThreads)
      maxpool_bwd_k3s2p1_flat_kernel<<<(unsigned)((patches + kThreads - 1) / kThreads), kThreads, 0, s>>>(
          dy, idx4, dx, g->H, g->W, (uint32_t)patches);
    else
      maxpool_bwd_k3s2p1_kernel<<<(unsigned)g->N * g->C, kThreads, 0, s>>>(dy, idx4, dx, g->H, g->W);
  }
  else if (is_ct(g, 3, 2, 1))
    launch_bwd(CtGeo<3, 2, 1>{}, g, dy, idx4, dx, s);
  else if (is_ct(g, 2, 2, 0))
    launch_bwd(CtGeo<2, 2, 0>{}, g, dy, idx4, dx, s);
  else
    launch_bwd(rt(g), g, dy, idx4, dx, s);
  return mn_launch_status();
}

}  // extern "C"
