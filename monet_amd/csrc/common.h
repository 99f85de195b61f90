// Shared device/host helpers for the gfx950 kernels of libmonet_hip.so.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>
#include "../../include/monet_hip.h"

typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float2_t __attribute__((ext_vector_type(2)));
typedef uint32_t uint4_t __attribute__((ext_vector_type(4)));

#define MN_WAVE 64

static inline int mn_launch_status() {
  return hipGetLastError() == hipSuccess ? MN_OK : MN_ELAUNCH;
}

static inline bool mn_aligned(const void* p, size_t a) {
  return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0;
}

static inline hipStream_t mn_stream(mn_stream_t s) { return reinterpret_cast<hipStream_t>(s); }

// Streaming (read-once / write-once) accesses: the tensors on this path are
// far larger than the caches, so loads and stores are marked non-temporal.
template <typename T>
__device__ __forceinline__ T ld_stream(const T* p) {
  return __builtin_nontemporal_load(p);
}
template <typename T>
__device__ __forceinline__ void st_stream(T* p, T v) {
  __builtin_nontemporal_store(v, p);
}

// Sum across the 64 lanes of a wavefront; every lane gets the total.
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, MN_WAVE);
  return v;
}

// Per-device set-up that is not a stream operation (see mn_init); defined in bn.hip and
// conv_wino.hip.  Both are idempotent and also run lazily from the entry points that need them.
bool mn_bn_static_init();
bool mn_wino_init();

// Workgroups are handed to the 8 XCDs (each with its own L2) round-robin in launch order.
// xcd_slot() turns a workgroup's launch index into a position in a LOGICAL order in which each
// XCD runs one contiguous range: a kernel that decodes its tile from the slot, neighbours
// first, lets the workgroups that read the same data share one L2 instead of pulling it into
// eight.  A bijection on [0, total) for any total.
__device__ __forceinline__ uint32_t xcd_slot() {
  const uint32_t total = gridDim.x * gridDim.y * gridDim.z;
  const uint32_t lin = blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z);
  const uint32_t xcd = lin & 7u, j = lin >> 3, rem = total & 7u;
  return xcd * (total >> 3) + (xcd < rem ? xcd : rem) + j;
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v = fmaxf(v, __shfl_xor(v, o, MN_WAVE));
  return v;
}

// Sum of two values across a workgroup of NW wavefronts. `lds` holds 2*NW
// floats. Every thread gets both totals. Summation order is fixed (lane tree,
// then wave 0..NW-1), so results are reproducible run to run.
template <int NW>
__device__ __forceinline__ void block_sum2(float& a, float& b, float* lds) {
  a = wave_sum(a);
  b = wave_sum(b);
  const int wave = threadIdx.x / MN_WAVE;
  const int lane = threadIdx.x % MN_WAVE;
  __syncthreads();  // lds may still be read from a previous call
  if (lane == 0) {
    lds[2 * wave] = a;
    lds[2 * wave + 1] = b;
  }
  __syncthreads();
  float sa = 0.f, sb = 0.f;
#pragma unroll
  for (int w = 0; w < NW; ++w) {
    sa += lds[2 * w];
    sb += lds[2 * w + 1];
  }
  a = sa;
  b = sb;
}
