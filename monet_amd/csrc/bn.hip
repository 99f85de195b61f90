// BatchNorm kernels over an [N, C, HW] view (NCHW): training forward, forward
// from saved statistics, backward from the input and backward from the output.
//
// Work decomposition: channel c owns N*HW elements, visited as the flat
// sequence j = n*HWV + i (HWV = HW / VEC vectors per image slab).  That
// sequence is cut into S equal pieces, one workgroup each.  Reductions are
// two-level and free of floating-point atomics: every workgroup writes one
// partial pair to the workspace and the S partials of a channel are re-added
// in a fixed order, so results are reproducible.
//
// The statistics-then-apply operators (training forward, both backwards) need
// every element twice.  Re-reading it costs a second trip through the memory
// fabric whether or not a cache holds it, so the main formulation keeps it ON
// CHIP: a piece is sized to fit the registers of one workgroup (kKeep vectors
// per thread and tensor).  A workgroup loads its piece once, reduces it,
// publishes the partial, waits until the other workgroups of its channel have
// published theirs, then computes the result from the registers it still
// holds.  HBM traffic is the algorithmic minimum: each operand read once, the
// result written once.
//
// Why the wait always ends: workgroups take their work item from a ticket
// counter when they start, so the items of a channel are held by workgroups
// that are all running or about to be started in ticket order; the lowest
// unfinished channel can always complete because at most S <= 256 workgroups
// are needed at once and the device holds more than that.  If that guarantee
// is lost (fewer workgroups resident than a channel has pieces: a partitioned
// or CU-masked device, another stream's kernel beside this one) a bounded wait
// gives up: the totals of that piece become NaN, so every result derived from
// them is NaN, and an error word in the workspace is set, which
// mn_bn_ws_status() reports as MN_ELAUNCH.  Every workgroup still exits.
//
// Channels too large for S <= 256 resident pieces fall back to two launches
// (reduce, then apply) that read the operands twice.
#include "common.h"

#include <mutex>

namespace mn_bn {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / MN_WAVE;
constexpr int kMaxSplit = 64;
constexpr int kU = 4;  // vectors in flight per thread per tensor


template <int VEC>
struct Vec;
template <>
struct Vec<4> {
  typedef float4_t type;
};
template <>
struct Vec<1> {
  typedef float type;
};

struct Shape {
  int C;
  int S;         // pieces per channel
  int G;         // resident launch: channels whose pieces are handed out interleaved
  uint32_t HWV;  // vectors per (n, c) slab
  uint32_t HW;   // elements per slab
  uint64_t L;    // vectors per piece
  uint64_t tot;  // vectors per channel = N * HWV
};

// Walks the vectors of one piece with a stride of STRIDE (= workgroup size), keeping (n, i)
// without a division per step.
template <int STRIDE>
struct CursorT {
  uint64_t j, jend;
  uint32_t n, i, qstep, rstep, HWV;
  __device__ __forceinline__ CursorT(const Shape& sh, int piece) {
    HWV = sh.HWV;
    const uint64_t j0 = (uint64_t)piece * sh.L;
    jend = min(j0 + sh.L, sh.tot);
    j = j0 + threadIdx.x;
    n = (uint32_t)(j / HWV);
    i = (uint32_t)(j - (uint64_t)n * HWV);
    qstep = STRIDE / HWV;
    rstep = STRIDE - qstep * HWV;
  }
  __device__ __forceinline__ bool valid() const { return j < jend; }
  __device__ __forceinline__ void next() {
    j += STRIDE;
    n += qstep;
    i += rstep;
    if (i >= HWV) {
      i -= HWV;
      ++n;
    }
  }
  // element offset of the current vector for channel c
  template <int VEC>
  __device__ __forceinline__ size_t off(int C, int c, uint32_t HW) const {
    return ((size_t)n * C + c) * HW + (size_t)i * VEC;
  }
};

typedef CursorT<kThreads> Cursor;

// H: cache hints of the tensor accesses, bit 0 = loads non-temporal, bit 1 = stores non-temporal
// (around the caches).  Right for planes that are whole cache lines, where every line is
// touched once; wrong for planes that are not, where the first and last line of a plane are
// shared with the neighbouring channel's plane: a non-temporal load fetches such a line once per
// sharer and a non-temporal store writes it to memory in parts ([184,2048,7,7] forward: 2.2 TB/s
// with both hints, 5.0 without).  A compile-time choice: a run-time one folds into plain accesses.
constexpr int kNtLoad = 1, kNtStore = 2;
template <int VEC, int H>
__device__ __forceinline__ typename Vec<VEC>::type ldv(const float* p) {
  const typename Vec<VEC>::type* q = reinterpret_cast<const typename Vec<VEC>::type*>(p);
  if (H & kNtLoad) return ld_stream(q);
  return *q;
}
template <int VEC, int H>
__device__ __forceinline__ void stv(float* p, typename Vec<VEC>::type v) {
  typename Vec<VEC>::type* q = reinterpret_cast<typename Vec<VEC>::type*>(p);
  if (H & kNtStore)
    st_stream(q, v);
  else
    *q = v;
}
__device__ __forceinline__ float comp(const float4_t& v, int k) { return v[k]; }
__device__ __forceinline__ float comp(const float& v, int) { return v; }
__device__ __forceinline__ void setc(float4_t& v, int k, float a) { v[k] = a; }
__device__ __forceinline__ void setc(float& v, int, float a) { v = a; }

// FWD_TRAIN_ADD: the forward with a second activation added before the (optional) ReLU,
// out = max((b - mean) * scale + bias + ralpha * a, 0): the end of a residual block in one pass.
// BWD_FROM_X_GATED: its backward from x and the output y: the incoming gradient only counts
// where y > 0; the gated gradient (times ralpha) is also written out, as the gradient of the
// added tensor.
// BWD_FROM_X_MASKED: the same with the gate read from a 1-bit mask (bit 7 of a byte = first
// element) that the forward wrote.
enum Mode {
  BWD_FROM_X = 0, BWD_FROM_Y = 1, FWD_TRAIN = 2, FWD_TRAIN_ADD = 3, BWD_FROM_X_GATED = 4,
  BWD_FROM_X_MASKED = 5
};
constexpr bool hands_on_gradient(int mode) {
  return mode == BWD_FROM_X_GATED || mode == BWD_FROM_X_MASKED;
}
constexpr bool is_fwd(int mode) { return mode == FWD_TRAIN || mode == FWD_TRAIN_ADD; }

// Everything a statistics-then-apply operator needs.
//   backward: a = dy, b = x or y, shift = mean or beta, out = dx
//   forward : b = x, out = y (FWD_TRAIN_ADD: a = the tensor added to the normalised value)
struct Args {
  Shape sh;
  const float* a;
  const float* b;
  const float* gamma;
  const float* shift;   // backward: mean (from x) / beta (from y); forward: beta
  const float* invstd;  // backward only
  float* out;
  float* vec0;          // backward: dgamma; forward: save_mean
  float* vec1;          // backward: dbeta;  forward: save_invstd
  float* running_mean;  // forward only
  float* running_var;
  float* partial;       // [C][S][2]
  float* pivot;         // [C], forward only
  uint32_t* ticket;     // resident launch only
  uint32_t* error;      // set to 1 by a wait that gave up; cleared by every launch
  uint32_t* sticky;     // the device's own word, set with it and only cleared by mn_bn_wait_status
  uint32_t spin_limit;  // polls of one slot before the wait gives up
  float inv_m, unbias, momentum, eps;
  // Fused ReLU.  Forward: out = max(out, 0).  Backward from the input: the incoming gradient
  // is that of the ReLU output, so it only counts where the recomputed pre-activation
  // (b - mean) * (invstd * gamma) + rbeta is positive.
  int relu;
  const float* rbeta;
  float ralpha;         // FWD_TRAIN_ADD: factor of the added tensor; BWD_FROM_X_GATED: of gated_out
  const float* gate_ref;  // BWD_FROM_X_GATED: y
  float* gated_out;       // BWD_FROM_X_GATED / _MASKED: ralpha * (gate ? dy : 0); may alias a
  const uint8_t* mask_in; // BWD_FROM_X_MASKED: packed sign bits of y over the flat tensor
  uint8_t* mask_out;      // FWD_TRAIN_ADD, optional: packed y > 0 (vector kernels whose lane pairs
                          // hold the two halves of a byte: HW % 8 == 0, even piece lengths)
};

// g where ref > 0, else 0 (a NaN reference passes nothing, like the ReLU backward from a
// stored activation)
__device__ __forceinline__ float4_t gate_by(float4_t g, float4_t ref) {
  float4_t r;
#pragma unroll
  for (int k = 0; k < 4; ++k) r[k] = ref[k] > 0.f ? g[k] : 0.f;
  return r;
}
__device__ __forceinline__ float gate_by(float g, float ref) { return ref > 0.f ? g : 0.f; }
// The same from the packed mask; `o` = flat element offset of the vector / element.
__device__ __forceinline__ float4_t gate_by_mask(float4_t g, const uint8_t* mask, size_t o) {
  const uint32_t byte = mask[o >> 3];
  const uint32_t nib = (o & 4) ? (byte & 15u) : (byte >> 4);
  float4_t r;
#pragma unroll
  for (int k = 0; k < 4; ++k) r[k] = (nib & (8u >> k)) ? g[k] : 0.f;
  return r;
}
__device__ __forceinline__ float gate_by_mask(float g, const uint8_t* mask, size_t o) {
  return ((mask[o >> 3] >> (7 - (o & 7))) & 1u) ? g : 0.f;
}
// Forward: the four sign bits of a result vector, joined with the neighbouring lane's into one
// mask byte (the even lane of a pair holds the even vector, i.e. the high nibble, and stores).
__device__ __forceinline__ void put_mask(uint8_t* mask, size_t o, float4_t y) {
  const uint32_t nib = (y[0] > 0.f ? 8u : 0u) | (y[1] > 0.f ? 4u : 0u) | (y[2] > 0.f ? 2u : 0u) |
                       (y[3] > 0.f ? 1u : 0u);
  const uint32_t other = __shfl_xor(nib, 1, MN_WAVE);
  if (!(threadIdx.x & 1u)) mask[o >> 3] = (uint8_t)((nib << 4) | other);
}
__device__ __forceinline__ void put_mask(uint8_t*, size_t, float) {}

// The ReLU gate of the fused backward, per channel.
struct Gate {
  bool on;
  float k1, beta;
  __device__ __forceinline__ float operator()(float g, float d) const {
    return (!on || k1 * d + beta > 0.f) ? g : 0.f;
  }
};
template <int MODE>
__device__ __forceinline__ Gate make_gate(const Args& A, int c) {
  Gate r;
  r.on = MODE == BWD_FROM_X && A.relu;
  r.k1 = r.on ? A.invstd[c] * (A.gamma ? A.gamma[c] : 1.f) : 0.f;
  r.beta = (r.on && A.rbeta) ? A.rbeta[c] : 0.f;
  return r;
}

// ---------------------------------------------------------------- reduce --
// (s0, s1) = ( sum a , sum a*(b - shift) )   backward
//          = ( sum (b - K) , sum (b - K)^2 ) forward, K = first element of the channel
template <int VEC, int MODE, int H>
__device__ __forceinline__ void reduce_piece(const Args& A, int c, int piece, float sft, float& s0,
                                             float& s1) {
  typedef typename Vec<VEC>::type V;
  const Shape& sh = A.sh;
  s0 = 0.f;
  s1 = 0.f;
  const Gate gate = make_gate<MODE>(A, c);
  Cursor cur(sh, piece);
  while (cur.valid()) {
    V va[kU], vb[kU];
    bool ok[kU];
#pragma unroll
    for (int u = 0; u < kU; ++u) {
      ok[u] = cur.valid();
      if (ok[u]) {
        const size_t o = cur.off<VEC>(sh.C, c, sh.HW);
        vb[u] = ldv<VEC, H>(A.b + o);
        if (!is_fwd(MODE)) va[u] = ldv<VEC, H>(A.a + o);
        if (MODE == BWD_FROM_X_GATED) va[u] = gate_by(va[u], ldv<VEC, H>(A.gate_ref + o));
        if (MODE == BWD_FROM_X_MASKED) va[u] = gate_by_mask(va[u], A.mask_in, o);
      }
      cur.next();
    }
#pragma unroll
    for (int u = 0; u < kU; ++u) {
      if (ok[u]) {
#pragma unroll
        for (int k = 0; k < VEC; ++k) {
          const float d = comp(vb[u], k) - sft;
          if (is_fwd(MODE)) {
            s0 += d;
            s1 += d * d;
          } else {
            const float g = gate(comp(va[u], k), d);
            s0 += g;
            s1 += g * d;
          }
        }
      }
    }
  }
}

template <int MODE>
__device__ __forceinline__ float reduce_shift(const Args& A, int c) {
  if (is_fwd(MODE)) return A.b[(size_t)c * A.sh.HW];
  return A.shift ? A.shift[c] : 0.f;
}

// ----------------------------------------------------------------- apply --
// out = (a - (b - sft)*proj - gmean) * gscale     backward
// out = (b - mean) * scale + bias                 forward (proj = mean, gmean = bias, gscale = scale)
template <int VEC, int MODE, int H>
__device__ __forceinline__ void apply_piece(const Args& A, int c, int piece, float sft, float proj,
                                            float gmean, float gscale) {
  typedef typename Vec<VEC>::type V;
  const Shape& sh = A.sh;
  const Gate gate = make_gate<MODE>(A, c);
  const bool relu = is_fwd(MODE) && A.relu;
  Cursor cur(sh, piece);
  while (cur.valid()) {
    V va[kU], vb[kU];
    size_t o[kU];
    bool ok[kU];
#pragma unroll
    for (int u = 0; u < kU; ++u) {
      ok[u] = cur.valid();
      if (ok[u]) {
        o[u] = cur.off<VEC>(sh.C, c, sh.HW);
        vb[u] = ldv<VEC, H>(A.b + o[u]);
        if (MODE != FWD_TRAIN) va[u] = ldv<VEC, H>(A.a + o[u]);
        if (MODE == BWD_FROM_X_GATED) va[u] = gate_by(va[u], ldv<VEC, H>(A.gate_ref + o[u]));
        if (MODE == BWD_FROM_X_MASKED) va[u] = gate_by_mask(va[u], A.mask_in, o[u]);
      }
      cur.next();
    }
#pragma unroll
    for (int u = 0; u < kU; ++u) {
      if (ok[u]) {
        V r;
#pragma unroll
        for (int k = 0; k < VEC; ++k) {
          if (is_fwd(MODE)) {
            float y = (comp(vb[u], k) - proj) * gscale + gmean;
            if (MODE == FWD_TRAIN_ADD) y += A.ralpha * comp(va[u], k);
            setc(r, k, relu ? fmaxf(y, 0.f) : y);
          } else {
            const float d = comp(vb[u], k) - sft;
            setc(r, k, (gate(comp(va[u], k), d) - d * proj - gmean) * gscale);
          }
        }
        stv<VEC, H>(A.out + o[u], r);
        if (hands_on_gradient(MODE)) stv<VEC, H>(A.gated_out + o[u], va[u] * A.ralpha);
        if (MODE == FWD_TRAIN_ADD && VEC == 4 && A.mask_out) put_mask(A.mask_out, o[u], r);
      }
    }
  }
}

// Turn the channel totals into the apply coefficients; piece 0 also writes
// the per-channel outputs.
template <int MODE>
__device__ __forceinline__ void coefficients(const Args& A, int c, int piece, float t0, float t1,
                                             float pivot, float& sft, float& proj, float& gmean,
                                             float& gscale) {
  const float w = A.gamma ? A.gamma[c] : 1.f;
  const bool writer = piece == 0 && threadIdx.x == 0;
  if (is_fwd(MODE)) {
    const float dm = t0 * A.inv_m;
    const float mean = pivot + dm;
    const float var = fmaxf(t1 * A.inv_m - dm * dm, 0.f);
    const float istd = 1.f / sqrtf(var + A.eps);
    if (writer) {
      A.vec0[c] = mean;
      A.vec1[c] = istd;
      if (A.running_mean)
        A.running_mean[c] = (1.f - A.momentum) * A.running_mean[c] + A.momentum * mean;
      if (A.running_var)
        A.running_var[c] = (1.f - A.momentum) * A.running_var[c] + A.momentum * (var * A.unbias);
    }
    sft = 0.f;
    proj = mean;
    gscale = istd * w;
    gmean = A.shift ? A.shift[c] : 0.f;
  } else {
    sft = A.shift ? A.shift[c] : 0.f;
    const float istd = A.invstd[c];
    float dg;
    if (MODE == BWD_FROM_Y) {
      const float inv_w = 1.f / w;
      proj = t1 * A.inv_m * inv_w * inv_w;
      dg = t1 * inv_w;
    } else {
      proj = t1 * A.inv_m * istd * istd;
      dg = t1 * istd;
    }
    gmean = t0 * A.inv_m;
    gscale = istd * w;
    if (writer) {
      if (A.vec0) A.vec0[c] = dg;
      if (A.vec1) A.vec1[c] = t0;
    }
  }
}

// Re-add the S (<= 64) partial pairs of channel c in a fixed order; every
// thread gets the totals.  COHERENT: read past the caches of this XCD, for
// partials written by other workgroups of the same launch.
template <bool COHERENT>
__device__ __forceinline__ void channel_totals(const float* partial, int c, int S, float& t0,
                                               float& t1) {
  const int lane = threadIdx.x % MN_WAVE;
  float p0 = 0.f, p1 = 0.f;
  if (lane < S) {
    const float* p = partial + 2 * ((size_t)c * S + lane);
    if (COHERENT) {
      p0 = __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      p1 = __hip_atomic_load(p + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    } else {
      p0 = p[0];
      p1 = p[1];
    }
  }
  t0 = wave_sum(p0);
  t1 = wave_sum(p1);
}

// ------------------------------------------------- two-launch formulation --
template <int VEC, int MODE, int H>
__global__ __launch_bounds__(kThreads) void bn_reduce_kernel(const Args A) {
  __shared__ float lds[2 * kWaves];
  const int c = blockIdx.x / A.sh.S;
  const int piece = blockIdx.x - c * A.sh.S;
  const float sft = reduce_shift<MODE>(A, c);
  if (is_fwd(MODE) && piece == 0 && threadIdx.x == 0) A.pivot[c] = sft;
  if (blockIdx.x == 0 && threadIdx.x == 0) *A.error = 0u;  // this formulation never waits
  float s0, s1;
  reduce_piece<VEC, MODE, H>(A, c, piece, sft, s0, s1);
  block_sum2<kWaves>(s0, s1, lds);
  if (threadIdx.x == 0) {
    A.partial[2 * (size_t)blockIdx.x] = s0;
    A.partial[2 * (size_t)blockIdx.x + 1] = s1;
  }
}

template <int VEC, int MODE, int H>
__global__ __launch_bounds__(kThreads) void bn_apply_kernel(const Args A) {
  const int c = blockIdx.x / A.sh.S;
  const int piece = blockIdx.x - c * A.sh.S;
  float t0, t1, sft, proj, gmean, gscale;
  channel_totals<false>(A.partial, c, A.sh.S, t0, t1);
  coefficients<MODE>(A, c, piece, t0, t1, is_fwd(MODE) ? A.pivot[c] : 0.f, sft, proj, gmean,
                     gscale);
  if (!A.out) return;
  apply_piece<VEC, MODE, H>(A, c, piece, sft, proj, gmean, gscale);
}

// Forward from saved statistics (no reduction).
template <int VEC, int MODE, int H>
__global__ __launch_bounds__(kThreads) void bn_fwd_saved_kernel(const Args A, const float* mean,
                                                                const float* invstd) {
  const int c = blockIdx.x / A.sh.S;
  const int piece = blockIdx.x - c * A.sh.S;
  const float scale = invstd[c] * (A.gamma ? A.gamma[c] : 1.f);
  const float bias = A.shift ? A.shift[c] : 0.f;
  apply_piece<VEC, MODE, H>(A, c, piece, 0.f, mean[c], bias, scale);
}

// ------------------------------------------------- one-launch formulation --
// A published partial pair is ONE 64-bit word (low = s0, high = s1) written
// and read with relaxed device-scope atomics, so the word itself is the
// "ready" flag and no cache flush / invalidate is ever needed.  Unpublished
// slots hold kEmptySlot, which publish() never writes.
constexpr uint64_t kEmptySlot = 0xFFFFFFFFFFFFFFFFull;

__global__ void bn_prepare_kernel(uint64_t* slots, uint32_t nslots, uint32_t* ticket,
                                  uint32_t* error) {
  const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < nslots) slots[i] = kEmptySlot;
  if (i == 0) {
    *ticket = 0u;
    *error = 0u;
  }
}

__device__ __forceinline__ void publish(uint64_t* slot, float s0, float s1) {
  uint64_t w = (uint64_t)__float_as_uint(s0) | ((uint64_t)__float_as_uint(s1) << 32);
  if (w == kEmptySlot) w = 0x7FC000007FC00000ull;  // same meaning (NaN, NaN), different bits
  __hip_atomic_store(slot, w, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}

constexpr int kMaxResident = 256;  // most pieces per channel in the resident formulation

// Wave 0 polls the S slots of a channel until all are published, adds them in
// a fixed order (lane l takes slots l, l+64, ..; then a lane tree) and hands
// the totals to the workgroup through `lds`.
__device__ __forceinline__ void gather_totals(const uint64_t* slots, int S, float* lds, float& t0,
                                              float& t1, uint32_t spin_limit, uint32_t* error,
                                              uint32_t* sticky) {
  if (threadIdx.x < MN_WAVE) {
    const int lane = threadIdx.x;
    float p0 = 0.f, p1 = 0.f;
    for (int k = lane; k < S; k += MN_WAVE) {  // at most kMaxResident / 64 rounds
      uint64_t w;
      uint32_t spins = 0;
      // The pieces polled here are published or held by running workgroups that publish
      // before they wait, so this ends.  Should that guarantee ever be lost, the bound ends
      // the wait anyway: the slot then counts as (NaN, NaN), which poisons everything computed
      // from these totals, and the workspace's error word is raised.
      while ((w = __hip_atomic_load(slots + k, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)) ==
                 kEmptySlot &&
             ++spins < spin_limit)
        __builtin_amdgcn_s_sleep(1);
      if (w == kEmptySlot) {
        w = 0x7FC000007FC00000ull;
        __hip_atomic_store(error, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (sticky) __hip_atomic_store(sticky, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
      p0 += __uint_as_float((uint32_t)w);
      p1 += __uint_as_float((uint32_t)(w >> 32));
    }
    p0 = wave_sum(p0);
    p1 = wave_sum(p1);
    if (lane == 0) {
      lds[0] = p0;
      lds[1] = p1;
    }
  }
  __syncthreads();
  t0 = lds[0];
  t1 = lds[1];
}

// One piece held in registers: thread t owns vectors p*L + t + k*THREADS, k < KEEP
// (sh.L must be THREADS * KEEP).
template <int VEC, int KEEP>
struct Held {
  typename Vec<VEC>::type a[KEEP], b[KEEP];
  int c, piece;
  float sft;
  float t0, t1;  // SOLO: the piece is the whole channel, these are its totals
};

// Load a piece, reduce it and publish its partial pair.  Never waits for
// another workgroup.
template <int VEC, int MODE, int KEEP, int THREADS, int H, bool SOLO = false>
__device__ __forceinline__ void hold_piece(const Args& A, uint32_t item, Held<VEC, KEEP>& h,
                                           float* lds) {
  typedef CursorT<THREADS> Cursor;
  const Shape& sh = A.sh;
  const int S = sh.S;
  if (SOLO || sh.G <= 1) {
    h.c = item / S;
    h.piece = item - h.c * S;
  } else {
    // tickets run over groups of G neighbouring channels, inside a group piece by piece with
    // the channels of a piece next to each other: workgroups that run at the same time read
    // neighbouring planes of the same images
    const uint32_t per_group = (uint32_t)sh.G * S;
    const uint32_t grp = item / per_group, within = item - grp * per_group;
    const uint32_t c0 = grp * sh.G;
    const uint32_t gc = min((uint32_t)sh.G, (uint32_t)sh.C - c0);
    h.piece = within / gc;
    h.c = c0 + (within - h.piece * gc);
  }
  h.sft = reduce_shift<MODE>(A, h.c);  // forward: the pivot, read before any store to the channel
  {
    Cursor cur(sh, h.piece);
#pragma unroll
    for (int k = 0; k < KEEP; ++k) {
      if (cur.valid()) {
        const size_t o = cur.template off<VEC>(sh.C, h.c, sh.HW);
        h.b[k] = ldv<VEC, H>(A.b + o);
        if (MODE != FWD_TRAIN) h.a[k] = ldv<VEC, H>(A.a + o);
      }
      cur.next();
    }
  }
  if (MODE == BWD_FROM_X_GATED) {
    // the gate needs y only now: gate the gradient in its registers and hand it on
    Cursor cur(sh, h.piece);
    typename Vec<VEC>::type ref[KEEP];
#pragma unroll
    for (int k = 0; k < KEEP; ++k) {
      if (cur.valid()) ref[k] = ldv<VEC, H>(A.gate_ref + cur.template off<VEC>(sh.C, h.c, sh.HW));
      cur.next();
    }
    Cursor cur2(sh, h.piece);
#pragma unroll
    for (int k = 0; k < KEEP; ++k) {
      if (cur2.valid()) {
        h.a[k] = gate_by(h.a[k], ref[k]);
        stv<VEC, H>(A.gated_out + cur2.template off<VEC>(sh.C, h.c, sh.HW), h.a[k] * A.ralpha);
      }
      cur2.next();
    }
  }
  if (MODE == BWD_FROM_X_MASKED) {
    Cursor cur(sh, h.piece);
#pragma unroll
    for (int k = 0; k < KEEP; ++k) {
      if (cur.valid()) {
        const size_t o = cur.template off<VEC>(sh.C, h.c, sh.HW);
        h.a[k] = gate_by_mask(h.a[k], A.mask_in, o);
        stv<VEC, H>(A.gated_out + o, h.a[k] * A.ralpha);
      }
      cur.next();
    }
  }
  float s0 = 0.f, s1 = 0.f;
  {
    const Gate gate = make_gate<MODE>(A, h.c);
    Cursor cur(sh, h.piece);
#pragma unroll
    for (int k = 0; k < KEEP; ++k) {
      if (cur.valid()) {
#pragma unroll
        for (int e = 0; e < VEC; ++e) {
          const float d = comp(h.b[k], e) - h.sft;
          if (is_fwd(MODE)) {
            s0 += d;
            s1 += d * d;
          } else {
            const float g = gate(comp(h.a[k], e), d);
            s0 += g;
            s1 += g * d;
          }
        }
      }
      cur.next();
    }
  }
  block_sum2<THREADS / MN_WAVE>(s0, s1, lds);
  if (SOLO) {
    h.t0 = s0;
    h.t1 = s1;
  } else if (threadIdx.x == 0) {
    publish(reinterpret_cast<uint64_t*>(A.partial) + (size_t)h.c * S + h.piece, s0, s1);
  }
}

// Wait for the channel totals of a held piece and write its result.
template <int VEC, int MODE, int KEEP, int THREADS, int H, bool SOLO = false>
__device__ __forceinline__ void finish_piece(const Args& A, const Held<VEC, KEEP>& h, float* lds) {
  typedef typename Vec<VEC>::type V;
  typedef CursorT<THREADS> Cursor;
  const Shape& sh = A.sh;
  float t0 = h.t0, t1 = h.t1;
  if (!SOLO) {
    __syncthreads();  // lds is free again
    gather_totals(reinterpret_cast<uint64_t*>(A.partial) + (size_t)h.c * sh.S, sh.S, lds, t0, t1,
                  A.spin_limit, A.error, A.sticky);
  }
  float s_, proj, gmean, gscale;
  coefficients<MODE>(A, h.c, h.piece, t0, t1, h.sft, s_, proj, gmean, gscale);
  if (!A.out) return;
  const Gate gate = make_gate<MODE>(A, h.c);
  const bool relu = is_fwd(MODE) && A.relu;
  Cursor cur(sh, h.piece);
#pragma unroll
  for (int k = 0; k < KEEP; ++k) {
    if (cur.valid()) {
      V r;
#pragma unroll
      for (int e = 0; e < VEC; ++e) {
        if (is_fwd(MODE)) {
          float y = (comp(h.b[k], e) - proj) * gscale + gmean;
          if (MODE == FWD_TRAIN_ADD) y += A.ralpha * comp(h.a[k], e);
          setc(r, e, relu ? fmaxf(y, 0.f) : y);
        } else {
          const float d = comp(h.b[k], e) - s_;
          setc(r, e, (gate(comp(h.a[k], e), d) - d * proj - gmean) * gscale);
        }
      }
      const size_t o = cur.template off<VEC>(sh.C, h.c, sh.HW);
      stv<VEC, H>(A.out + o, r);
      if (MODE == FWD_TRAIN_ADD && VEC == 4 && A.mask_out) put_mask(A.mask_out, o, r);
    }
    cur.next();
  }
}

// Persistent workgroups: each keeps two pieces in flight, so the wait for the
// other workgroups of one piece's channel is spent loading the next piece.
// Every piece is published before its holder waits for anything, and pieces
// are handed out in ticket order, so the lowest unfinished channel always has
// all its pieces either published or about to be taken by a running workgroup
// (at least kMaxResident workgroups run at once).
template <int VEC, int MODE, int KEEP, int THREADS, int H>
__global__ __launch_bounds__(THREADS) void bn_resident_kernel(const Args A, uint32_t items) {
  __shared__ float lds[2 * (THREADS / MN_WAVE)];
  __shared__ uint32_t s_ticket;
  Held<VEC, KEEP> h0, h1;
  auto take = [&]() -> uint32_t {
    __syncthreads();  // s_ticket of the previous round has been read by everyone
    if (threadIdx.x == 0)
      s_ticket = __hip_atomic_fetch_add(A.ticket, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    __syncthreads();
    return s_ticket;
  };
  uint32_t i0 = take();
  if (i0 >= items) return;
  hold_piece<VEC, MODE, KEEP, THREADS, H>(A, i0, h0, lds);
  for (;;) {
    const uint32_t i1 = take();
    if (i1 < items) hold_piece<VEC, MODE, KEEP, THREADS, H>(A, i1, h1, lds);
    finish_piece<VEC, MODE, KEEP, THREADS, H>(A, h0, lds);
    if (i1 >= items) break;
    i0 = take();
    if (i0 < items) hold_piece<VEC, MODE, KEEP, THREADS, H>(A, i0, h0, lds);
    finish_piece<VEC, MODE, KEEP, THREADS, H>(A, h1, lds);
    if (i0 >= items) break;
  }
}

// Channels short enough for ONE workgroup's registers (N*HW <= THREADS * KEEP vectors, e.g.
// 14 x 14 and 7 x 7 planes at batch 184): a workgroup takes whole channels, so there is nothing
// to publish, poll or prepare - one launch, no workspace traffic, no atomics.
template <int VEC, int MODE, int KEEP, int THREADS, int H>
__global__ __launch_bounds__(THREADS) void bn_solo_kernel(const Args A) {
  __shared__ float lds[2 * (THREADS / MN_WAVE)];
  Held<VEC, KEEP> h;
  if (blockIdx.x == 0 && threadIdx.x == 0) *A.error = 0u;  // nothing here ever waits
  // Planes this short do not end on cache-line boundaries: neighbouring channels share their
  // first and last lines.  Each XCD takes a contiguous range of channels, so the shared lines
  // meet in one L2 instead of being fetched (and written back in parts) by two.
  for (uint32_t c = xcd_slot(); c < (uint32_t)A.sh.C; c += gridDim.x) {
    hold_piece<VEC, MODE, KEEP, THREADS, H, true>(A, c, h, lds);
    finish_piece<VEC, MODE, KEEP, THREADS, H, true>(A, h, lds);
  }
}

// ------------------------------------------------------------------ host --
// Launch choices.  `resident`: 1 = one launch keeping the operands in
// registers (falls back when a channel needs more than kMaxResident pieces),
// 0 = always reduce launch + apply launch.
struct Tuning {
  int target_blocks = 2048;  // two-launch formulation: aim for C*S workgroups
  int resident = 1;
  int keep = 8;              // vectors kept per thread, tensor and piece (two pieces in flight)
  int threads = 256;         // workgroup size of the resident kernel
  int grid = 768;            // persistent workgroups of the resident kernel (3 per CU)
  uint32_t spin_limit = 1u << 22;  // polls of one slot (seconds) before a wait gives up
  int group = 0;             // channels whose pieces are handed out interleaved (0: chosen here)
  int hints = 0;             // 0: chosen from the plane size; else 4 | kNtLoad and / or kNtStore
};

static bool shape_limits(int64_t N, int64_t C, int64_t HW) {
  return N > 0 && C > 0 && HW > 0 && C <= (1 << 22) && HW < (1ll << 31) && N < (1ll << 31);
}
static int64_t resident_pieces(int64_t N, int64_t HW, int vec, int keep) {
  const int64_t tot = N * (HW / vec);
  return (tot + kThreads * keep - 1) / (kThreads * keep);
}
// Vectors per resident piece in product builds: (keep 8 x 256 threads) float4, or
// (keep 16 x 256 threads) scalars when the shape / alignment rules out float4.
static int64_t product_pieces(int64_t N, int64_t HW, int vec) {
  return resident_pieces(N, HW, vec, vec == 4 ? 8 : 16);
}
// Workspace: partial pairs [C][P][2] floats, pivot [C] floats, ticket word; P covers both the
// resident formulation (if the channel qualifies) and the two-launch one.
static size_t ws_floats(int64_t N, int64_t C, int64_t HW) {
  int64_t P = kMaxSplit;
  const int64_t p1 = product_pieces(N, HW, 1);
  if (p1 <= kMaxResident && p1 > P) P = p1;
  if (HW % 4 == 0) {
    int64_t p4 = product_pieces(N, HW, 4);
    if (p4 > kMaxResident) p4 = resident_pieces(N, HW, 4, 16);  // 512-thread workgroups
    if (p4 <= kMaxResident && p4 > P) P = p4;
  }
  return (size_t)C * (2 * (size_t)P + 1);
}
static size_t ws_bytes_for(int64_t N, int64_t C, int64_t HW) {
  return ws_floats(N, C, HW) * sizeof(float) + 2 * sizeof(uint32_t);
}

static void fill_shape(int64_t N, int64_t C, int64_t HW, int vec, int64_t S, uint64_t L,
                       Shape& sh) {
  sh.C = (int)C;
  sh.S = (int)S;
  sh.HWV = (uint32_t)(HW / vec);
  sh.HW = (uint32_t)HW;
  sh.tot = (uint64_t)N * sh.HWV;
  sh.L = L + (L & 1);  // even: a lane pair never straddles two pieces (put_mask)
  sh.G = 1;
}

// Cache hints by plane size, from measurements at batch 184: planes of whole cache lines stream
// fastest around the caches (56 x 56, 112 x 112); planes that share their end lines with the
// neighbouring channel want ordinary stores, so that the parts of a line meet in L2 (14 x 14:
// 4.4 -> 5.1 TB/s), and below a few lines per plane ordinary loads as well (7 x 7: 2.4 ->
// 5.3 TB/s).  With both plain at 14 x 14 the two streams evict each other; from 28 x 28 up the
// shared lines are too few to matter and ordinary stores cost the three-tensor backward of the
// fused operators a fifth of its rate.
static int cache_hints(int64_t HW, int forced = 0) {
  const int64_t plane = HW * (int64_t)sizeof(float);
  if (forced) return forced & (kNtLoad | kNtStore);
  if (plane % 128 == 0 || plane >= 2048) return kNtLoad | kNtStore;
  if (plane < 512) return 0;
  return kNtLoad;
}
// Runs `CALL(H)` with the compile-time constant H equal to the run-time `hints`.
#define MN_BN_WITH_HINTS(hints, CALL)        \
  do {                                       \
    switch (hints) {                         \
      case 0: CALL(0); break;                \
      case kNtLoad: CALL(kNtLoad); break;    \
      case kNtStore: CALL(kNtStore); break;  \
      default: CALL(kNtLoad | kNtStore);     \
    }                                        \
  } while (0)

// One word per device that every wait that gives up raises besides the word in its workspace
// (workspaces are usually freed right after the call): mn_bn_wait_status reads and clears it.
// In host code the name is a handle for hipGetSymbolAddress, not a device address.
static __device__ uint32_t gave_up_word;

static uint32_t* sticky_word() {
  constexpr int kMaxDevices = 64;
  static std::mutex lock;
  static uint32_t* address[kMaxDevices] = {};
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
  std::lock_guard<std::mutex> hold(lock);
  if (!address[dev]) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(gave_up_word)) != hipSuccess) return nullptr;
    address[dev] = static_cast<uint32_t*>(p);
  }
  return address[dev];
}

template <int MODE>
static int run(Args& A, int64_t N, int64_t C, int64_t HW, bool aligned16, void* ws,
               const Tuning& t, hipStream_t s) {
  const int vec = (HW % 4 == 0 && aligned16) ? 4 : 1;
  const int hints = cache_hints(HW, t.hints);
  A.partial = static_cast<float*>(ws);
  uint32_t* counters = reinterpret_cast<uint32_t*>(A.partial + ws_floats(N, C, HW));
  A.pivot = reinterpret_cast<float*>(counters) - C;  // last C floats of the float area
  A.ticket = counters;
  A.error = counters + 1;
  A.sticky = sticky_word();
  A.spin_limit = t.spin_limit ? t.spin_limit : 1u;
  int keep = t.keep > 0 ? t.keep : 8, threads = t.threads > 0 ? t.threads : kThreads;
  // The forward holds one tensor per piece: 512-thread workgroups (pieces twice as long, half as
  // many partials to publish and poll) measured 7-20 % faster on every ResNet-50 shape at batch
  // 184; the backward kernels hold two tensors per piece and gain nothing from it.
  const bool long_pieces = MODE == FWD_TRAIN && vec == 4 && keep == 8 && threads == kThreads;
  if (long_pieces) threads = 512;
  int64_t rp = resident_pieces(N, HW, vec, (vec == 4 ? keep * threads : 16 * kThreads) / kThreads);
  // channels too long for 256 pieces of 256 x 8 vectors (e.g. 64 x 112 x 112 at batch 184):
  // twice the workgroup size doubles the piece and keeps them in the one-pass kernel
  bool wide = false;
  if (vec == 4 && keep == 8 && threads == kThreads && rp > kMaxResident &&
      resident_pieces(N, HW, 4, 16) <= kMaxResident) {
    wide = true;
    threads = 512;
    rp = resident_pieces(N, HW, 4, 16);
  }
  // whole channels in one workgroup's registers
  const uint64_t chan = (uint64_t)N * (HW / vec);
  bool solo = t.resident && t.keep == 8 && t.threads == kThreads;
  if (solo) {
    const unsigned grid = (unsigned)(C < 65535 ? C : 65535);
#define MN_BN_SOLO(V, K, T)                                              \
  do {                                                                   \
    fill_shape(N, C, HW, V, 1, (uint64_t)(T) * (K), A.sh);               \
    if (hints == 0) bn_solo_kernel<V, MODE, K, T, 0><<<grid, T, 0, s>>>(A);                         \
    else if (hints == kNtLoad) bn_solo_kernel<V, MODE, K, T, kNtLoad><<<grid, T, 0, s>>>(A);        \
    else if (hints == kNtStore) bn_solo_kernel<V, MODE, K, T, kNtStore><<<grid, T, 0, s>>>(A);      \
    else bn_solo_kernel<V, MODE, K, T, kNtLoad | kNtStore><<<grid, T, 0, s>>>(A);                   \
    return mn_launch_status();                                           \
  } while (0)
    if (vec == 4 && chan <= 256u * 9u) MN_BN_SOLO(4, 9, 256);
    // (a third tensor - the gate of BWD_FROM_X_GATED - does not fit beside 2 x 18 vectors per
    // thread: that mode takes the multi-piece kernel for such channels)
    if constexpr (MODE != BWD_FROM_X_GATED) {
      if (vec == 4 && chan <= 1024u * 9u) MN_BN_SOLO(4, 18, 512);
    }
    if (vec == 1 && chan <= 256u * 36u) MN_BN_SOLO(1, 36, 256);
#undef MN_BN_SOLO
  }
  if (t.resident && rp <= kMaxResident) {
    fill_shape(N, C, HW, vec, rp, vec == 4 ? (uint64_t)threads * keep : (uint64_t)kThreads * 16, A.sh);
    const unsigned blocks = (unsigned)(C * rp);
    // Interleave the pieces of up to 8 neighbouring channels (the workgroups of the moment then
    // read neighbouring planes of the same images: 1-2 % at [184,256,56,56]).  A workgroup only
    // waits while it holds two published pieces, both inside the lowest unfinished group or
    // later, so with at least kMaxResident workgroups running nobody can be left waiting as
    // long as a group has fewer than 2 * kMaxResident pieces.
    // Not with one workgroup per CU (`wide`): a channel then completes G times later and nothing
    // else on the CU covers the wait (64 x 112 x 112 at batch 184: 0.377 -> 0.454 ms with G = 3).
    A.sh.G = wide ? 1 : (int)(448 / rp < 1 ? 1 : (448 / rp > 8 ? 8 : 448 / rp));
    if (t.group > 0) A.sh.G = t.group;
    bn_prepare_kernel<<<(blocks + 255) / 256, 256, 0, s>>>(
          reinterpret_cast<uint64_t*>(A.partial), blocks, A.ticket, A.error);
    // persistent grid: enough workgroups to fill 256 CUs at this register footprint
    // (512-thread workgroups: one per CU at this register footprint)
    const unsigned want = (wide && t.grid > 256) ? 256u : (unsigned)t.grid;
    const unsigned grid = blocks < want ? blocks : want;
#define MN_BN_RES(V, K, T)                                                                          \
  do {                                                                                              \
    if (hints == 0) bn_resident_kernel<V, MODE, K, T, 0><<<grid, T, 0, s>>>(A, blocks);             \
    else if (hints == kNtLoad) bn_resident_kernel<V, MODE, K, T, kNtLoad><<<grid, T, 0, s>>>(A, blocks); \
    else if (hints == kNtStore) bn_resident_kernel<V, MODE, K, T, kNtStore><<<grid, T, 0, s>>>(A, blocks); \
    else bn_resident_kernel<V, MODE, K, T, kNtLoad | kNtStore><<<grid, T, 0, s>>>(A, blocks);       \
  } while (0)
    if (vec == 4) {
      if (wide || long_pieces) MN_BN_RES(4, 8, 512);
      else MN_BN_RES(4, 8, 256);
    } else {
      MN_BN_RES(1, 16, 256);
    }
#undef MN_BN_RES
    return mn_launch_status();
  }
  const uint64_t tot = (uint64_t)N * (HW / vec);
  int64_t S = (t.target_blocks + C - 1) / C;
  const int64_t cap = (int64_t)((tot + kThreads * kU - 1) / (kThreads * kU));
  if (S > cap) S = cap;
  if (S > kMaxSplit) S = kMaxSplit;
  if (S < 1) S = 1;
  fill_shape(N, C, HW, vec, S, (tot + S - 1) / S, A.sh);
  const unsigned blocks = (unsigned)(C * S);
#define MN_BN_TWO(H)                                              \
  do {                                                            \
    if (vec == 4) {                                               \
      bn_reduce_kernel<4, MODE, H><<<blocks, kThreads, 0, s>>>(A); \
      bn_apply_kernel<4, MODE, H><<<blocks, kThreads, 0, s>>>(A);  \
    } else {                                                      \
      bn_reduce_kernel<1, MODE, H><<<blocks, kThreads, 0, s>>>(A); \
      bn_apply_kernel<1, MODE, H><<<blocks, kThreads, 0, s>>>(A);  \
    }                                                             \
  } while (0)
  MN_BN_WITH_HINTS(hints, MN_BN_TWO);
#undef MN_BN_TWO
  return mn_launch_status();
}

int bwd_launch(bool from_y, const float* dy, const float* t, const float* gamma, const float* shift,
               const float* invstd, float* dx, float* dgamma, float* dbeta, int64_t N, int64_t C,
               int64_t HW, void* ws, size_t ws_bytes, hipStream_t s, const Tuning& tune,
               bool relu = false, const float* relu_beta = nullptr,
               const float* gate_ref = nullptr, float* gated_out = nullptr, float alpha = 1.f,
               const uint8_t* mask_in = nullptr) {
  if (N < 0 || C < 0 || HW < 0) return MN_EINVAL;
  if (N == 0 || C == 0 || HW == 0) return MN_OK;
  if (!dy || !t || !invstd || !ws) return MN_EINVAL;
  if (gate_ref && mask_in) return MN_EINVAL;
  if ((gate_ref != nullptr || mask_in != nullptr) != (gated_out != nullptr)) return MN_EINVAL;
  if (gated_out && (from_y || relu || !dx)) return MN_EUNSUPPORTED;
  if (!shape_limits(N, C, HW)) return MN_EUNSUPPORTED;
  if (ws_bytes < ws_bytes_for(N, C, HW) || !mn_aligned(ws, 8)) return MN_EINVAL;
  Args A = {};
  const bool al = mn_aligned(dy, 16) && mn_aligned(t, 16) && (!dx || mn_aligned(dx, 16)) &&
                  mn_aligned(gate_ref, 16) && mn_aligned(gated_out, 16);
  A.gate_ref = gate_ref;
  A.mask_in = mask_in;
  A.gated_out = gated_out;
  A.ralpha = alpha;
  A.a = dy;
  A.b = t;
  A.gamma = gamma;
  A.shift = shift;
  A.invstd = invstd;
  A.out = dx;
  A.vec0 = dgamma;
  A.vec1 = dbeta;
  A.inv_m = 1.f / (float)((double)N * (double)HW);
  A.relu = relu ? 1 : 0;
  A.rbeta = relu_beta;
  if (relu && from_y) return MN_EUNSUPPORTED;
  if (gate_ref) return run<BWD_FROM_X_GATED>(A, N, C, HW, al, ws, tune, s);
  if (mask_in) return run<BWD_FROM_X_MASKED>(A, N, C, HW, al, ws, tune, s);
  return from_y ? run<BWD_FROM_Y>(A, N, C, HW, al, ws, tune, s)
                : run<BWD_FROM_X>(A, N, C, HW, al, ws, tune, s);
}

int fwd_train_launch(const float* x, const float* gamma, const float* beta, float* running_mean,
                     float* running_var, float* y, float* save_mean, float* save_invstd, int64_t N,
                     int64_t C, int64_t HW, double momentum, double eps, void* ws, size_t ws_bytes,
                     hipStream_t s, const Tuning& tune, bool relu = false,
                     const float* added = nullptr, float alpha = 1.f, uint8_t* mask = nullptr) {
  if (N < 0 || C < 0 || HW < 0) return MN_EINVAL;
  if (N == 0 || C == 0 || HW == 0) return MN_OK;
  if (!x || !y || !save_mean || !save_invstd || !ws) return MN_EINVAL;
  if (!shape_limits(N, C, HW)) return MN_EUNSUPPORTED;
  if (ws_bytes < ws_bytes_for(N, C, HW) || !mn_aligned(ws, 8)) return MN_EINVAL;
  Args A = {};
  const bool al = mn_aligned(x, 16) && mn_aligned(y, 16) && mn_aligned(added, 16);
  const double M = (double)N * (double)HW;
  A.a = added;
  A.ralpha = alpha;
  A.mask_out = (al && HW % 8 == 0) ? mask : nullptr;  // else the caller packs y afterwards
  A.b = x;
  A.gamma = gamma;
  A.shift = beta;
  A.out = y;
  A.vec0 = save_mean;
  A.vec1 = save_invstd;
  A.running_mean = running_mean;
  A.running_var = running_var;
  A.inv_m = (float)(1.0 / M);
  A.unbias = M > 1.0 ? (float)(M / (M - 1.0)) : 1.f;
  A.momentum = (float)momentum;
  A.eps = (float)eps;
  A.relu = relu ? 1 : 0;
  if (added) return run<FWD_TRAIN_ADD>(A, N, C, HW, al, ws, tune, s);
  return run<FWD_TRAIN>(A, N, C, HW, al, ws, tune, s);
}

}  // namespace mn_bn

extern "C" {

size_t mn_bn_ws_bytes(int64_t N, int64_t C, int64_t HW) {
  return (N > 0 && C > 0 && HW > 0) ? mn_bn::ws_bytes_for(N, C, HW) : 0;
}

int mn_bn_fwd_train_f32(const float* x, const float* gamma, const float* beta, float* running_mean,
                        float* running_var, float* y, float* save_mean, float* save_invstd,
                        int64_t N, int64_t C, int64_t HW, double momentum, double eps, void* ws,
                        size_t ws_bytes, mn_stream_t stream) {
  return mn_bn::fwd_train_launch(x, gamma, beta, running_mean, running_var, y, save_mean,
                                 save_invstd, N, C, HW, momentum, eps, ws, ws_bytes,
                                 mn_stream(stream), mn_bn::Tuning());
}

static int bn_fwd_apply(const float* x, const float* mean, const float* invstd, const float* gamma,
                        const float* beta, float* y, int64_t N, int64_t C, int64_t HW,
                        mn_stream_t stream, bool relu, const float* added = nullptr,
                        float alpha = 1.f, uint8_t* mask = nullptr) {
  using namespace mn_bn;
  if (N < 0 || C < 0 || HW < 0) return MN_EINVAL;
  if (N == 0 || C == 0 || HW == 0) return MN_OK;
  if (!x || !y || !mean || !invstd) return MN_EINVAL;
  if (!shape_limits(N, C, HW)) return MN_EUNSUPPORTED;
  Args A = {};
  const int vec =
      (HW % 4 == 0 && mn_aligned(x, 16) && mn_aligned(y, 16) && mn_aligned(added, 16)) ? 4 : 1;
  {
    const uint64_t tot = (uint64_t)N * (HW / vec);
    int64_t S = (4096 + C - 1) / C;
    const int64_t cap = (int64_t)((tot + kThreads * kU - 1) / (kThreads * kU));
    if (S > cap) S = cap;
    if (S < 1) S = 1;
    fill_shape(N, C, HW, vec, S, (tot + S - 1) / S, A.sh);
  }
  A.b = x;
  A.gamma = gamma;
  A.shift = beta;
  A.out = y;
  A.relu = relu ? 1 : 0;
  A.a = added;
  A.ralpha = alpha;
  A.mask_out = (vec == 4 && HW % 8 == 0) ? mask : nullptr;
  const int hints = cache_hints(HW);
  const unsigned blocks = (unsigned)C * A.sh.S;
  hipStream_t s = mn_stream(stream);
#define MN_BN_SAVED(H)                                                                        \
  do {                                                                                        \
    if (added) {                                                                              \
      if (vec == 4)                                                                           \
        bn_fwd_saved_kernel<4, FWD_TRAIN_ADD, H><<<blocks, kThreads, 0, s>>>(A, mean, invstd); \
      else                                                                                    \
        bn_fwd_saved_kernel<1, FWD_TRAIN_ADD, H><<<blocks, kThreads, 0, s>>>(A, mean, invstd); \
    } else if (vec == 4) {                                                                    \
      bn_fwd_saved_kernel<4, FWD_TRAIN, H><<<blocks, kThreads, 0, s>>>(A, mean, invstd);      \
    } else {                                                                                  \
      bn_fwd_saved_kernel<1, FWD_TRAIN, H><<<blocks, kThreads, 0, s>>>(A, mean, invstd);      \
    }                                                                                         \
  } while (0)
  MN_BN_WITH_HINTS(hints, MN_BN_SAVED);
#undef MN_BN_SAVED
  return mn_launch_status();
}

int mn_bn_fwd_apply_f32(const float* x, const float* mean, const float* invstd, const float* gamma,
                        const float* beta, float* y, int64_t N, int64_t C, int64_t HW,
                        mn_stream_t stream) {
  return bn_fwd_apply(x, mean, invstd, gamma, beta, y, N, C, HW, stream, false);
}

int mn_bn_relu_fwd_train_f32(const float* x, const float* gamma, const float* beta,
                             float* running_mean, float* running_var, float* y, float* save_mean,
                             float* save_invstd, int64_t N, int64_t C, int64_t HW, double momentum,
                             double eps, void* ws, size_t ws_bytes, mn_stream_t stream) {
  return mn_bn::fwd_train_launch(x, gamma, beta, running_mean, running_var, y, save_mean,
                                 save_invstd, N, C, HW, momentum, eps, ws, ws_bytes,
                                 mn_stream(stream), mn_bn::Tuning(), true);
}

int mn_bn_relu_fwd_apply_f32(const float* x, const float* mean, const float* invstd,
                             const float* gamma, const float* beta, float* y, int64_t N, int64_t C,
                             int64_t HW, mn_stream_t stream) {
  return bn_fwd_apply(x, mean, invstd, gamma, beta, y, N, C, HW, stream, true);
}

int mn_bn_add_relu_fwd_train_f32(const float* x, const float* gamma, const float* beta,
                                 float* running_mean, float* running_var, const float* added,
                                 double alpha, float* y, float* save_mean, float* save_invstd,
                                 int64_t N, int64_t C, int64_t HW, double momentum, double eps,
                                 void* ws, size_t ws_bytes, mn_stream_t stream) {
  if (!added && N > 0 && C > 0 && HW > 0) return MN_EINVAL;
  return mn_bn::fwd_train_launch(x, gamma, beta, running_mean, running_var, y, save_mean,
                                 save_invstd, N, C, HW, momentum, eps, ws, ws_bytes,
                                 mn_stream(stream), mn_bn::Tuning(), true, added, (float)alpha);
}

int mn_bn_add_relu_fwd_apply_f32(const float* x, const float* mean, const float* invstd,
                                 const float* gamma, const float* beta, const float* added,
                                 double alpha, float* y, int64_t N, int64_t C, int64_t HW,
                                 mn_stream_t stream) {
  if (!added && N > 0 && C > 0 && HW > 0) return MN_EINVAL;
  return bn_fwd_apply(x, mean, invstd, gamma, beta, y, N, C, HW, stream, true, added,
                      (float)alpha);
}

int mn_bn_add_relu_bwd_f32(const float* dy, const float* x, const float* y, const float* gamma,
                           const float* mean, const float* invstd, double alpha, float* dx,
                           float* dadded, float* dgamma, float* dbeta, int64_t N, int64_t C,
                           int64_t HW, void* ws, size_t ws_bytes, mn_stream_t stream) {
  if (N > 0 && C > 0 && HW > 0 && (!mean || !y || !dadded || !dx)) return MN_EINVAL;
  // Channels short enough for one workgroup's registers hold two tensors per thread already; a
  // third does not fit beside them, and the ReLU backward as a launch of its own in front of
  // the plain backward measured faster there ([184,1024,14,14]: 0.199 ms against 0.229 ms).
  const uint64_t chan = (uint64_t)N * (uint64_t)(HW % 4 == 0 ? HW / 4 : HW);
  const bool one_workgroup = HW % 4 == 0 ? chan <= 1024u * 9u : chan <= 256u * 36u;
  if (one_workgroup && alpha == 1.0 && N > 0 && C > 0 && HW > 0) {
    const int st = mn_relu_bwd_ref_f32(dy, y, 0.f, dadded, (size_t)N * C * HW, stream);
    if (st != MN_OK) return st;
    return mn_bn::bwd_launch(false, dadded, x, gamma, mean, invstd, dx, dgamma, dbeta, N, C, HW,
                             ws, ws_bytes, mn_stream(stream), mn_bn::Tuning());
  }
  return mn_bn::bwd_launch(false, dy, x, gamma, mean, invstd, dx, dgamma, dbeta, N, C, HW, ws,
                           ws_bytes, mn_stream(stream), mn_bn::Tuning(), false, nullptr, y, dadded,
                           (float)alpha);
}

// Whether the forward kernels write the mask themselves (else mn_relu_fwd_mask_f32 packs y).
static bool mask_in_kernel(const float* x, const float* y, const float* added, int64_t HW) {
  return HW % 8 == 0 && mn_aligned(x, 16) && mn_aligned(y, 16) && mn_aligned(added, 16);
}

int mn_bn_add_relu_mask_fwd_train_f32(const float* x, const float* gamma, const float* beta,
                                      float* running_mean, float* running_var, const float* added,
                                      double alpha, float* y, uint8_t* mask, float* save_mean,
                                      float* save_invstd, int64_t N, int64_t C, int64_t HW,
                                      double momentum, double eps, void* ws, size_t ws_bytes,
                                      mn_stream_t stream) {
  if (N <= 0 || C <= 0 || HW <= 0) return (N < 0 || C < 0 || HW < 0) ? MN_EINVAL : MN_OK;
  if (!added || !mask) return MN_EINVAL;
  const int st = mn_bn::fwd_train_launch(x, gamma, beta, running_mean, running_var, y, save_mean,
                                         save_invstd, N, C, HW, momentum, eps, ws, ws_bytes,
                                         mn_stream(stream), mn_bn::Tuning(), true, added,
                                         (float)alpha, mask);
  if (st != MN_OK || mask_in_kernel(x, y, added, HW)) return st;
  return mn_relu_fwd_mask_f32(y, nullptr, mask, (size_t)N * C * HW, stream);
}

int mn_bn_add_relu_mask_fwd_apply_f32(const float* x, const float* mean, const float* invstd,
                                      const float* gamma, const float* beta, const float* added,
                                      double alpha, float* y, uint8_t* mask, int64_t N, int64_t C,
                                      int64_t HW, mn_stream_t stream) {
  if (N <= 0 || C <= 0 || HW <= 0) return (N < 0 || C < 0 || HW < 0) ? MN_EINVAL : MN_OK;
  if (!added || !mask) return MN_EINVAL;
  const int st = bn_fwd_apply(x, mean, invstd, gamma, beta, y, N, C, HW, stream, true, added,
                              (float)alpha, mask);
  if (st != MN_OK || mask_in_kernel(x, y, added, HW)) return st;
  return mn_relu_fwd_mask_f32(y, nullptr, mask, (size_t)N * C * HW, stream);
}

int mn_bn_add_relu_mask_bwd_f32(const float* dy, const float* x, const uint8_t* mask,
                                const float* gamma, const float* mean, const float* invstd,
                                double alpha, float* dx, float* dadded, float* dgamma,
                                float* dbeta, int64_t N, int64_t C, int64_t HW, void* ws,
                                size_t ws_bytes, mn_stream_t stream) {
  if (N > 0 && C > 0 && HW > 0 && (!mean || !mask || !dadded || !dx)) return MN_EINVAL;
  return mn_bn::bwd_launch(false, dy, x, gamma, mean, invstd, dx, dgamma, dbeta, N, C, HW, ws,
                           ws_bytes, mn_stream(stream), mn_bn::Tuning(), false, nullptr, nullptr,
                           dadded, (float)alpha, mask);
}

int mn_bn_relu_bwd_from_x_f32(const float* dy, const float* x, const float* gamma,
                              const float* beta, const float* mean, const float* invstd, float* dx,
                              float* dgamma, float* dbeta, int64_t N, int64_t C, int64_t HW,
                              void* ws, size_t ws_bytes, mn_stream_t stream) {
  if (!mean) return MN_EINVAL;
  return mn_bn::bwd_launch(false, dy, x, gamma, mean, invstd, dx, dgamma, dbeta, N, C, HW, ws,
                           ws_bytes, mn_stream(stream), mn_bn::Tuning(), true, beta);
}

int mn_bn_bwd_from_x_f32(const float* dy, const float* x, const float* gamma, const float* mean,
                         const float* invstd, float* dx, float* dgamma, float* dbeta, int64_t N,
                         int64_t C, int64_t HW, void* ws, size_t ws_bytes, mn_stream_t stream) {
  if (!mean) return MN_EINVAL;
  return mn_bn::bwd_launch(false, dy, x, gamma, mean, invstd, dx, dgamma, dbeta, N, C, HW, ws,
                           ws_bytes, mn_stream(stream), mn_bn::Tuning());
}

int mn_bn_bwd_from_y_f32(const float* dy, const float* y, const float* gamma, const float* beta,
                         const float* invstd, float* dx, float* dgamma, float* dbeta, int64_t N,
                         int64_t C, int64_t HW, void* ws, size_t ws_bytes, mn_stream_t stream) {
  return mn_bn::bwd_launch(true, dy, y, gamma, beta, invstd, dx, dgamma, dbeta, N, C, HW, ws,
                           ws_bytes, mn_stream(stream), mn_bn::Tuning());
}

int mn_bn_bwd_from_y_f32_limits(const float* dy, const float* y, const float* gamma,
                                const float* beta, const float* invstd, float* dx, float* dgamma,
                                float* dbeta, int64_t N, int64_t C, int64_t HW, void* ws,
                                size_t ws_bytes, uint32_t spin_limit, uint32_t max_workgroups,
                                uint32_t channel_group, uint32_t cache_hints, mn_stream_t stream) {
  mn_bn::Tuning t;
  t.hints = (int)(cache_hints & 7u);
  t.group = (int)(channel_group < 4096u ? channel_group : 4096u);
  if (spin_limit) t.spin_limit = spin_limit;
  if (max_workgroups) t.grid = (int)(max_workgroups < 65535u ? max_workgroups : 65535u);
  return mn_bn::bwd_launch(true, dy, y, gamma, beta, invstd, dx, dgamma, dbeta, N, C, HW, ws,
                           ws_bytes, mn_stream(stream), t);
}

// The workspace of mn_bn_bwd_from_y_static_f32.  In host code this name is only a handle for
// hipGetSymbolAddress, not a device address: kernels are given the address looked up below.
static __device__ __align__(256) unsigned char scratch[MN_BN_STATIC_WS_BYTES];

// Device address of `scratch` on the current device (every GPU holds its own copy at its own
// address); looked up once per device.  Null if the lookup fails.
static void* static_workspace() {
  constexpr int kMaxDevices = 64;
  static std::mutex lock;
  static void* address[kMaxDevices] = {};
  int dev = -1;
  if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kMaxDevices) return nullptr;
  std::lock_guard<std::mutex> hold(lock);
  if (!address[dev]) {
    void* p = nullptr;
    if (hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)) != hipSuccess) return nullptr;
    address[dev] = p;
  }
  return address[dev];
}

int mn_bn_bwd_from_y_static_f32(const float* dy, const float* y, const float* gamma,
                                const float* beta, const float* invstd, float* dx, float* dgamma,
                                float* dbeta, int64_t N, int64_t C, int64_t HW,
                                mn_stream_t stream) {
  if (N < 0 || C < 0 || HW < 0) return MN_EINVAL;
  if (N == 0 || C == 0 || HW == 0) return MN_OK;
  if (!mn_bn::shape_limits(N, C, HW)) return MN_EUNSUPPORTED;
  const size_t need = mn_bn::ws_bytes_for(N, C, HW);
  if (need > (size_t)MN_BN_STATIC_WS_BYTES) return MN_ELIMIT;
  void* ws = static_workspace();
  if (!ws) return MN_ELAUNCH;
  // every formulation initialises what it reads of the workspace (slots, ticket and error word
  // by the prepare launch; partial sums are written before they are read), so whatever the
  // previous call left there does not matter
  return mn_bn::bwd_launch(true, dy, y, gamma, beta, invstd, dx, dgamma, dbeta, N, C, HW, ws, need,
                           mn_stream(stream), mn_bn::Tuning());
}

int mn_bn_ws_status(const void* ws, size_t ws_bytes, int64_t N, int64_t C, int64_t HW,
                    mn_stream_t stream) {
  if (N <= 0 || C <= 0 || HW <= 0) return (N < 0 || C < 0 || HW < 0) ? MN_EINVAL : MN_OK;
  if (!mn_bn::shape_limits(N, C, HW)) return MN_EINVAL;
  if (!ws) {   // the array of mn_bn_bwd_from_y_static_f32
    if (mn_bn::ws_bytes_for(N, C, HW) > (size_t)MN_BN_STATIC_WS_BYTES) return MN_EINVAL;
    ws = static_workspace();
    if (!ws) return MN_ELAUNCH;
  } else if (ws_bytes < mn_bn::ws_bytes_for(N, C, HW)) {
    return MN_EINVAL;
  }
  const char* word = static_cast<const char*>(ws) + mn_bn::ws_floats(N, C, HW) * sizeof(float) +
                     sizeof(uint32_t);
  uint32_t raised = 0;
  hipStream_t s = mn_stream(stream);
  if (hipMemcpyAsync(&raised, word, sizeof(raised), hipMemcpyDeviceToHost, s) != hipSuccess ||
      hipStreamSynchronize(s) != hipSuccess)
    return MN_ELAUNCH;
  return raised ? MN_ELAUNCH : MN_OK;
}

int mn_bn_wait_status(uint32_t* host_word, mn_stream_t stream) {
  uint32_t* word = mn_bn::sticky_word();
  if (!word) return MN_ELAUNCH;
  hipStream_t s = mn_stream(stream);
  if (host_word)
    return hipMemcpyAsync(host_word, word, sizeof(uint32_t), hipMemcpyDeviceToHost, s) == hipSuccess
               ? MN_OK
               : MN_ELAUNCH;
  uint32_t raised = 0;
  if (hipMemcpyAsync(&raised, word, sizeof(raised), hipMemcpyDeviceToHost, s) != hipSuccess ||
      hipStreamSynchronize(s) != hipSuccess)
    return MN_ELAUNCH;
  if (raised && (hipMemsetAsync(word, 0, sizeof(uint32_t), s) != hipSuccess ||
                 hipStreamSynchronize(s) != hipSuccess))
    return MN_ELAUNCH;
  return raised ? MN_ELAUNCH : MN_OK;
}

}  // extern "C"

// Part of mn_init(): the address lookups of the static workspace and of the word
// mn_bn_wait_status reads, for the current device.
bool mn_bn_static_init() { return static_workspace() != nullptr && mn_bn::sticky_word() != nullptr; }
