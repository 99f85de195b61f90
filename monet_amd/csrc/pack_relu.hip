// 1-bit / 4-bit packing and the ReLU kernels that use the 1-bit mask.
//
// Bit order (all kernels): element i lives in byte i/8, bit 7-(i%8); nibble
// order: element 2j in the high nibble of byte j.  Every kernel is a single
// streaming pass: each HBM byte is read once and written once.
#include "common.h"

namespace {

constexpr int kThreads = 256;

// OR of `v` over each aligned group of 8 lanes, via DPP (no LDS traffic).
__device__ __forceinline__ uint32_t or_reduce8(uint32_t v) {
  v |= (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0xB1, 0xF, 0xF, true);   // lane ^ 1
  v |= (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x4E, 0xF, 0xF, true);   // lane ^ 2
  v |= (uint32_t)__builtin_amdgcn_update_dpp(0, (int)v, 0x141, 0xF, 0xF, true);  // 7 - lane
  return v;
}

__device__ __forceinline__ float relu1(float x) {
  // x > 0 keeps x; NaN is kept; everything else (incl. -0.0) becomes +0.0
  return x > 0.f ? x : (x != x ? x : 0.f);
}

// ---------------------------------------------------------------- forward --
// Vector body: lane l of each aligned group of 8 lanes owns 4 consecutive
// floats; the group owns 32 consecutive floats = one 32-bit mask word.  `ng4`
// (number of float4 in the body) is a multiple of 8, so a group is either
// fully inside or fully outside the body.  Tail (< 32 elements) is done by
// the first threads of workgroup 0, one mask byte each.
template <int U, bool WRITE_Y>
__global__ __launch_bounds__(kThreads) void relu_fwd_mask_vec(const float* x, float* y,
                                                              uint8_t* __restrict__ mask,
                                                              size_t ng4, size_t n) {
  const size_t base = (size_t)blockIdx.x * (U * kThreads) + threadIdx.x;
  const float4_t* x4 = reinterpret_cast<const float4_t*>(x);
  float4_t* y4 = reinterpret_cast<float4_t*>(y);
  uint32_t* m32 = reinterpret_cast<uint32_t*>(mask);
  float4_t v[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const size_t g = base + (size_t)u * kThreads;
    if (g < ng4) v[u] = ld_stream(x4 + g);
  }
  const uint32_t m = threadIdx.x & 7;
  const uint32_t shift = 8 * (m >> 1) + ((m & 1) ? 0 : 4);
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const size_t g = base + (size_t)u * kThreads;
    if (g < ng4) {
      const float4_t a = v[u];
      uint32_t nib = ((a.x > 0.f) ? 8u : 0u) | ((a.y > 0.f) ? 4u : 0u) | ((a.z > 0.f) ? 2u : 0u) |
                     ((a.w > 0.f) ? 1u : 0u);
      if (WRITE_Y) {
        float4_t r;
        r.x = relu1(a.x);
        r.y = relu1(a.y);
        r.z = relu1(a.z);
        r.w = relu1(a.w);
        st_stream(y4 + g, r);
      }
      const uint32_t word = or_reduce8(nib << shift);
      if (m == 0) st_stream(m32 + (g >> 3), word);
    }
  }
  if (blockIdx.x == 0) {
    const size_t e0 = ng4 * 4 + (size_t)threadIdx.x * 8;
    if (e0 < n) {
      uint32_t b = 0;
      for (int k = 0; k < 8 && e0 + k < n; ++k) {
        const float a = x[e0 + k];
        if (a > 0.f) b |= 0x80u >> k;
        if (WRITE_Y) y[e0 + k] = relu1(a);
      }
      mask[e0 >> 3] = (uint8_t)b;
    }
  }
}

// Fallback for operands that are not 16-byte (x, y) / 4-byte (mask) aligned:
// one thread per mask byte.
template <bool WRITE_Y>
__global__ __launch_bounds__(kThreads) void relu_fwd_mask_scalar(const float* x, float* y,
                                                                 uint8_t* mask, size_t n) {
  const size_t j = (size_t)blockIdx.x * kThreads + threadIdx.x;
  const size_t e0 = j * 8;
  if (e0 >= n) return;
  uint32_t b = 0;
  for (int k = 0; k < 8 && e0 + k < n; ++k) {
    const float a = x[e0 + k];
    if (a > 0.f) b |= 0x80u >> k;
    if (WRITE_Y) y[e0 + k] = relu1(a);
  }
  mask[j] = (uint8_t)b;
}

// y = max(a + alpha*b, 0), optionally with the 1-bit mask of (a + alpha*b > 0): the residual
// add and the ReLU behind it in one pass (2 reads + 1 write instead of 3 reads + 2 writes).
// Same work split and mask layout as relu_fwd_mask_vec; y may alias a.
template <int U, bool WRITE_MASK>
__global__ __launch_bounds__(kThreads) void add_relu_fwd_vec(const float* a, const float* b,
                                                             float alpha, float* y,
                                                             uint8_t* __restrict__ mask, size_t ng4,
                                                             size_t n) {
  const size_t base = (size_t)blockIdx.x * (U * kThreads) + threadIdx.x;
  const float4_t* a4 = reinterpret_cast<const float4_t*>(a);
  const float4_t* b4 = reinterpret_cast<const float4_t*>(b);
  float4_t* y4 = reinterpret_cast<float4_t*>(y);
  uint32_t* m32 = reinterpret_cast<uint32_t*>(mask);
  float4_t va[U], vb[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const size_t g = base + (size_t)u * kThreads;
    if (g < ng4) {
      va[u] = ld_stream(a4 + g);
      vb[u] = ld_stream(b4 + g);
    }
  }
  const uint32_t m = threadIdx.x & 7;
  const uint32_t shift = 8 * (m >> 1) + ((m & 1) ? 0 : 4);
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const size_t g = base + (size_t)u * kThreads;
    if (g < ng4) {
      float4_t t;
      t.x = va[u].x + alpha * vb[u].x;
      t.y = va[u].y + alpha * vb[u].y;
      t.z = va[u].z + alpha * vb[u].z;
      t.w = va[u].w + alpha * vb[u].w;
      float4_t r;
      r.x = relu1(t.x);
      r.y = relu1(t.y);
      r.z = relu1(t.z);
      r.w = relu1(t.w);
      st_stream(y4 + g, r);
      if (WRITE_MASK) {
        const uint32_t nib = ((t.x > 0.f) ? 8u : 0u) | ((t.y > 0.f) ? 4u : 0u) |
                             ((t.z > 0.f) ? 2u : 0u) | ((t.w > 0.f) ? 1u : 0u);
        const uint32_t word = or_reduce8(nib << shift);
        if (m == 0) st_stream(m32 + (g >> 3), word);
      }
    }
  }
  if (blockIdx.x == 0) {  // tail (< 32 elements), one mask byte per thread
    const size_t e0 = ng4 * 4 + (size_t)threadIdx.x * 8;
    if (e0 < n) {
      uint32_t bits = 0;
      for (int k = 0; k < 8 && e0 + k < n; ++k) {
        const float t = a[e0 + k] + alpha * b[e0 + k];
        if (t > 0.f) bits |= 0x80u >> k;
        y[e0 + k] = relu1(t);
      }
      if (WRITE_MASK) mask[e0 >> 3] = (uint8_t)bits;
    }
  }
}

// Fallback for unaligned operands: one thread per mask byte.
__global__ __launch_bounds__(kThreads) void add_relu_fwd_scalar(const float* a, const float* b,
                                                                float alpha, float* y,
                                                                uint8_t* mask, size_t n) {
  const size_t j = (size_t)blockIdx.x * kThreads + threadIdx.x;
  const size_t e0 = j * 8;
  if (e0 >= n) return;
  uint32_t bits = 0;
  for (int k = 0; k < 8 && e0 + k < n; ++k) {
    const float t = a[e0 + k] + alpha * b[e0 + k];
    if (t > 0.f) bits |= 0x80u >> k;
    y[e0 + k] = relu1(t);
  }
  if (mask) mask[j] = (uint8_t)bits;
}

// --------------------------------------------------------------- backward --
__device__ __forceinline__ float mask_mul(float g, uint32_t bit) { return bit ? g : g * 0.f; }

template <int U>
__global__ __launch_bounds__(kThreads) void relu_bwd_mask_vec(const float* grad,
                                                              const uint8_t* __restrict__ mask,
                                                              float* dx, size_t ng4, size_t n) {
  const size_t base = (size_t)blockIdx.x * (U * kThreads) + threadIdx.x;
  const float4_t* g4 = reinterpret_cast<const float4_t*>(grad);
  float4_t* d4 = reinterpret_cast<float4_t*>(dx);
  float4_t v[U];
  uint32_t mb[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const size_t g = base + (size_t)u * kThreads;
    if (g < ng4) {
      v[u] = ld_stream(g4 + g);
      mb[u] = mask[g >> 1];
    }
  }
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const size_t g = base + (size_t)u * kThreads;
    if (g < ng4) {
      const uint32_t nib = (g & 1) ? (mb[u] & 15u) : (mb[u] >> 4);
      float4_t r;
      r.x = mask_mul(v[u].x, nib & 8u);
      r.y = mask_mul(v[u].y, nib & 4u);
      r.z = mask_mul(v[u].z, nib & 2u);
      r.w = mask_mul(v[u].w, nib & 1u);
      st_stream(d4 + g, r);
    }
  }
  if (blockIdx.x == 0) {
    const size_t e = ng4 * 4 + threadIdx.x;
    if (e < n) dx[e] = mask_mul(grad[e], (mask[e >> 3] >> (7 - (e & 7))) & 1u);
  }
}

__global__ __launch_bounds__(kThreads) void relu_bwd_mask_scalar(const float* grad,
                                                                 const uint8_t* mask, float* dx,
                                                                 size_t n) {
  const size_t e = (size_t)blockIdx.x * kThreads + threadIdx.x;
  if (e < n) dx[e] = mask_mul(grad[e], (mask[e >> 3] >> (7 - (e & 7))) & 1u);
}

template <int U>
__global__ __launch_bounds__(kThreads) void relu_bwd_ref_vec(const float* grad, const float* ref,
                                                             float threshold, float* dx,
                                                             size_t ng4, size_t n) {
  const size_t base = (size_t)blockIdx.x * (U * kThreads) + threadIdx.x;
  const float4_t* g4 = reinterpret_cast<const float4_t*>(grad);
  const float4_t* r4 = reinterpret_cast<const float4_t*>(ref);
  float4_t* d4 = reinterpret_cast<float4_t*>(dx);
  float4_t v[U], s[U];
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const size_t g = base + (size_t)u * kThreads;
    if (g < ng4) {
      v[u] = ld_stream(g4 + g);
      s[u] = ld_stream(r4 + g);
    }
  }
#pragma unroll
  for (int u = 0; u < U; ++u) {
    const size_t g = base + (size_t)u * kThreads;
    if (g < ng4) {
      float4_t r;
      r.x = s[u].x > threshold ? v[u].x : 0.f;
      r.y = s[u].y > threshold ? v[u].y : 0.f;
      r.z = s[u].z > threshold ? v[u].z : 0.f;
      r.w = s[u].w > threshold ? v[u].w : 0.f;
      st_stream(d4 + g, r);
    }
  }
  if (blockIdx.x == 0) {
    const size_t e = ng4 * 4 + threadIdx.x;
    if (e < n) dx[e] = ref[e] > threshold ? grad[e] : 0.f;
  }
}

__global__ __launch_bounds__(kThreads) void relu_bwd_ref_scalar(const float* grad, const float* ref,
                                                                float threshold, float* dx,
                                                                size_t n) {
  const size_t e = (size_t)blockIdx.x * kThreads + threadIdx.x;
  if (e < n) dx[e] = ref[e] > threshold ? grad[e] : 0.f;
}

// ------------------------------------------------------- standalone packs --
// 8 bytes of 0/1 -> one byte, first byte in bit 7 (multiply gathers the low
// bit of byte i into bit 63-i; distinct (i, j) never collide, so no carries).
__device__ __forceinline__ uint32_t gather8(uint64_t w) {
  return (uint32_t)(((w & 0x0101010101010101ull) * 0x8040201008040201ull) >> 56);
}
// One byte -> 8 bytes of 0/1, bit 7 first.
__device__ __forceinline__ uint64_t spread8(uint32_t b) {
  const uint64_t t = ((uint64_t)b * 0x0101010101010101ull) & 0x0102040810204080ull;
  return ((t + 0x7F7F7F7F7F7F7F7Full) >> 7) & 0x0101010101010101ull;
}

// one thread per output byte; `vec` says the bool array is 8-byte aligned
__global__ __launch_bounds__(kThreads) void pack_bits_kernel(const uint8_t* __restrict__ in,
                                                             uint8_t* __restrict__ out, size_t n,
                                                             bool vec) {
  const size_t j = (size_t)blockIdx.x * kThreads + threadIdx.x;
  const size_t e0 = j * 8;
  if (e0 >= n) return;
  uint32_t b;
  if (vec && e0 + 8 <= n) {
    b = gather8(ld_stream(reinterpret_cast<const uint64_t*>(in) + j));
  } else {
    b = 0;
    for (int k = 0; k < 8 && e0 + k < n; ++k) b |= (uint32_t)(in[e0 + k] & 1u) << (7 - k);
  }
  out[j] = (uint8_t)b;
}

__global__ __launch_bounds__(kThreads) void unpack_bits_kernel(const uint8_t* __restrict__ in,
                                                               uint8_t* __restrict__ out, size_t n,
                                                               bool vec) {
  const size_t j = (size_t)blockIdx.x * kThreads + threadIdx.x;
  const size_t e0 = j * 8;
  if (e0 >= n) return;
  const uint32_t b = in[j];
  if (vec && e0 + 8 <= n) {
    st_stream(reinterpret_cast<uint64_t*>(out) + j, spread8(b));
  } else {
    for (int k = 0; k < 8 && e0 + k < n; ++k) out[e0 + k] = (uint8_t)((b >> (7 - k)) & 1u);
  }
}

// one thread per 4 output bytes (8 inputs)
__global__ __launch_bounds__(kThreads) void pack_nibbles_kernel(const uint8_t* __restrict__ in,
                                                                uint8_t* __restrict__ out, size_t n,
                                                                bool vec) {
  const size_t j = (size_t)blockIdx.x * kThreads + threadIdx.x;
  const size_t e0 = j * 8;
  if (e0 >= n) return;
  if (vec && e0 + 8 <= n) {
    const uint64_t w = ld_stream(reinterpret_cast<const uint64_t*>(in) + j);
    const uint64_t hi = w & 0x000F000F000F000Full;
    const uint64_t lo = (w >> 8) & 0x000F000F000F000Full;
    const uint64_t t = (hi << 4) | lo;
    const uint32_t r = (uint32_t)(t & 0xFF) | (uint32_t)((t >> 8) & 0xFF00) |
                       (uint32_t)((t >> 16) & 0xFF0000) | (uint32_t)((t >> 24) & 0xFF000000);
    st_stream(reinterpret_cast<uint32_t*>(out) + j, r);
  } else {
    for (size_t e = e0; e < n && e < e0 + 8; e += 2) {
      uint32_t b = (uint32_t)(in[e] & 15u) << 4;
      if (e + 1 < n) b |= in[e + 1] & 15u;
      out[e >> 1] = (uint8_t)b;
    }
  }
}

__global__ __launch_bounds__(kThreads) void unpack_nibbles_kernel(const uint8_t* __restrict__ in,
                                                                  uint8_t* __restrict__ out,
                                                                  size_t n, bool vec) {
  const size_t j = (size_t)blockIdx.x * kThreads + threadIdx.x;
  const size_t e0 = j * 8;
  if (e0 >= n) return;
  if (vec && e0 + 8 <= n) {
    const uint32_t r = ld_stream(reinterpret_cast<const uint32_t*>(in) + j);
    uint64_t w = 0;
#pragma unroll
    for (int k = 0; k < 4; ++k) {
      const uint64_t b = (r >> (8 * k)) & 0xFFu;
      w |= ((b >> 4) | ((b & 15u) << 8)) << (16 * k);
    }
    st_stream(reinterpret_cast<uint64_t*>(out) + j, w);
  } else {
    for (size_t e = e0; e < n && e < e0 + 8; ++e) {
      const uint32_t b = in[e >> 1];
      out[e] = (uint8_t)((e & 1) ? (b & 15u) : (b >> 4));
    }
  }
}

inline unsigned blocks_for(size_t work, size_t per_block) {
  return (unsigned)((work + per_block - 1) / per_block);
}

}  // namespace

extern "C" {

int mn_pack_bits(const uint8_t* bools, uint8_t* packed, size_t n, mn_stream_t stream) {
  if (n == 0) return MN_OK;
  if (!bools || !packed) return MN_EINVAL;
  const size_t nb = (n + 7) / 8;
  pack_bits_kernel<<<blocks_for(nb, kThreads), kThreads, 0, mn_stream(stream)>>>(
      bools, packed, n, mn_aligned(bools, 8));
  return mn_launch_status();
}

int mn_unpack_bits(const uint8_t* packed, uint8_t* bools, size_t n, mn_stream_t stream) {
  if (n == 0) return MN_OK;
  if (!bools || !packed) return MN_EINVAL;
  const size_t nb = (n + 7) / 8;
  unpack_bits_kernel<<<blocks_for(nb, kThreads), kThreads, 0, mn_stream(stream)>>>(
      packed, bools, n, mn_aligned(bools, 8));
  return mn_launch_status();
}

int mn_unpack_bits_mul_f32(const uint8_t* packed, const float* v, float* r, size_t n,
                           mn_stream_t stream) {
  return mn_relu_bwd_mask_f32(v, packed, r, n, stream);
}

int mn_pack_nibbles(const uint8_t* u, uint8_t* packed, size_t n, mn_stream_t stream) {
  if (n == 0) return MN_OK;
  if (!u || !packed) return MN_EINVAL;
  const size_t nt = (n + 7) / 8;
  pack_nibbles_kernel<<<blocks_for(nt, kThreads), kThreads, 0, mn_stream(stream)>>>(
      u, packed, n, mn_aligned(u, 8) && mn_aligned(packed, 4));
  return mn_launch_status();
}

int mn_unpack_nibbles(const uint8_t* packed, uint8_t* u, size_t n, mn_stream_t stream) {
  if (n == 0) return MN_OK;
  if (!u || !packed) return MN_EINVAL;
  const size_t nt = (n + 7) / 8;
  unpack_nibbles_kernel<<<blocks_for(nt, kThreads), kThreads, 0, mn_stream(stream)>>>(
      packed, u, n, mn_aligned(u, 8) && mn_aligned(packed, 4));
  return mn_launch_status();
}

int mn_relu_fwd_mask_f32(const float* x, float* y, uint8_t* mask, size_t n, mn_stream_t stream) {
  if (n == 0) return MN_OK;
  if (!x || !mask) return MN_EINVAL;
  hipStream_t s = mn_stream(stream);
  const bool vec = mn_aligned(x, 16) && (!y || mn_aligned(y, 16)) && mn_aligned(mask, 4);
  if (vec) {
    constexpr int U = 4;
    const size_t ng4 = (n / 32) * 8;
    const unsigned blocks = ng4 ? blocks_for(ng4, (size_t)U * kThreads) : 1u;
    if (y)
      relu_fwd_mask_vec<U, true><<<blocks, kThreads, 0, s>>>(x, y, mask, ng4, n);
    else
      relu_fwd_mask_vec<U, false><<<blocks, kThreads, 0, s>>>(x, nullptr, mask, ng4, n);
  } else {
    const unsigned blocks = blocks_for((n + 7) / 8, kThreads);
    if (y)
      relu_fwd_mask_scalar<true><<<blocks, kThreads, 0, s>>>(x, y, mask, n);
    else
      relu_fwd_mask_scalar<false><<<blocks, kThreads, 0, s>>>(x, nullptr, mask, n);
  }
  return mn_launch_status();
}

int mn_add_relu_fwd_f32(const float* a, const float* b, float alpha, float* y, uint8_t* mask,
                        size_t n, mn_stream_t stream) {
  if (n == 0) return MN_OK;
  if (!a || !b || !y) return MN_EINVAL;
  hipStream_t s = mn_stream(stream);
  const bool vec = mn_aligned(a, 16) && mn_aligned(b, 16) && mn_aligned(y, 16) &&
                   (!mask || mn_aligned(mask, 4));
  if (vec) {
    constexpr int U = 4;
    const size_t ng4 = (n / 32) * 8;
    const unsigned blocks = ng4 ? blocks_for(ng4, (size_t)U * kThreads) : 1u;
    if (mask)
      add_relu_fwd_vec<U, true><<<blocks, kThreads, 0, s>>>(a, b, alpha, y, mask, ng4, n);
    else
      add_relu_fwd_vec<U, false><<<blocks, kThreads, 0, s>>>(a, b, alpha, y, nullptr, ng4, n);
  } else {
    add_relu_fwd_scalar<<<blocks_for((n + 7) / 8, kThreads), kThreads, 0, s>>>(a, b, alpha, y, mask,
                                                                              n);
  }
  return mn_launch_status();
}

int mn_relu_bwd_mask_f32(const float* grad, const uint8_t* mask, float* dx, size_t n,
                         mn_stream_t stream) {
  if (n == 0) return MN_OK;
  if (!grad || !mask || !dx) return MN_EINVAL;
  hipStream_t s = mn_stream(stream);
  if (mn_aligned(grad, 16) && mn_aligned(dx, 16)) {
    constexpr int U = 4;
    const size_t ng4 = n / 4;
    const unsigned blocks = ng4 ? blocks_for(ng4, (size_t)U * kThreads) : 1u;
    relu_bwd_mask_vec<U><<<blocks, kThreads, 0, s>>>(grad, mask, dx, ng4, n);
  } else {
    relu_bwd_mask_scalar<<<blocks_for(n, kThreads), kThreads, 0, s>>>(grad, mask, dx, n);
  }
  return mn_launch_status();
}

int mn_relu_bwd_ref_f32(const float* grad, const float* ref, float threshold, float* dx, size_t n,
                        mn_stream_t stream) {
  if (n == 0) return MN_OK;
  if (!grad || !ref || !dx) return MN_EINVAL;
  hipStream_t s = mn_stream(stream);
  if (mn_aligned(grad, 16) && mn_aligned(dx, 16) && mn_aligned(ref, 16)) {
    constexpr int U = 4;
    const size_t ng4 = n / 4;
    const unsigned blocks = ng4 ? blocks_for(ng4, (size_t)U * kThreads) : 1u;
    relu_bwd_ref_vec<U><<<blocks, kThreads, 0, s>>>(grad, ref, threshold, dx, ng4, n);
  } else {
    relu_bwd_ref_scalar<<<blocks_for(n, kThreads), kThreads, 0, s>>>(grad, ref, threshold, dx, n);
  }
  return mn_launch_status();
}

}  // extern "C"
