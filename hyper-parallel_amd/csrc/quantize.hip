// Quantize / dequantize kernels for the FP8 linear path (gfx950).
//
// All of them are HBM-bound streaming kernels: 128-bit coalesced loads, |x| compared as packed
// 16-bit integers (exact for bf16), amax reduced across lanes with DPP, scale = 448/amax by a
// full IEEE division, E4M3 conversion with the hardware packed converter after an explicit
// clamp to +-448, 64/128-bit stores.
#include <atomic>
#include <mutex>

#include "hpfp8_device.h"
#include "hpfp8_host.h"

namespace hpfp8 {

// ---------------------------------------------------------------------------------------------
// device memory for the entry point that allocates nothing
// ---------------------------------------------------------------------------------------------
// hpfp8_quantize_per_tensor_noalloc_bf16 keeps its amax word here instead of taking it from the caller.  Every
// GPU holds its own copy of this array for the life of the process.  In host code the array's name is only a
// handle: the address kernels can use is asked for once per device (scratch_for_current_device) and that pointer is
// what is passed on; the array keeps the previous call's contents, so a call clears the word it uses first.
constexpr int kScratchWords = 64;
static __device__ __align__(256) uint32_t scratch[kScratchWords];

constexpr int kMaxDevices = 64;
static std::mutex g_scratch_mutex;
static uint32_t* g_scratch_ptr[kMaxDevices] = {nullptr};

// The scratch array's device address on the current device (resolved on the first call per device); nullptr
// with the error text set if HIP refuses.
static uint32_t* scratch_for_current_device() {
  int dev = 0;
  hipError_t e = hipGetDevice(&dev);
  if (e != hipSuccess || dev < 0 || dev >= kMaxDevices) {
    fail(HPFP8_ERR_DEVICE, "scratch: no usable current device (%s)", e != hipSuccess ? hipGetErrorString(e) : "index beyond 63");
    return nullptr;
  }
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    uint32_t* p = nullptr;
    e = hipGetSymbolAddress((void**)&p, HIP_SYMBOL(scratch));
    if (e != hipSuccess || !p) {
      fail(HPFP8_ERR_DEVICE, "scratch: hipGetSymbolAddress failed on device %d: %s", dev, hipGetErrorString(e));
      return nullptr;
    }
    g_scratch_ptr[dev] = p;
  }
  return g_scratch_ptr[dev];
}

int prepare_scratch() { return scratch_for_current_device() ? HPFP8_OK : HPFP8_ERR_DEVICE; }

// ---------------------------------------------------------------------------------------------
// per-tensor amax
// ---------------------------------------------------------------------------------------------
__global__ void fill_u32_kernel(uint32_t* p, uint32_t v, int n) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = v;
}
__global__ void fill2_u32_kernel(uint32_t* a, uint32_t* b) {
  if (threadIdx.x == 0) *a = 0u;
  if (threadIdx.x == 1) *b = 0u;
}

// amax_bits receives the fp32 bit pattern of max|x| (non-negative floats order like integers).
__global__ __launch_bounds__(256) void amax_bf16_kernel(const uint16_t* __restrict__ x, int64_t n,
                                                        uint32_t* __restrict__ amax_bits) {
  const uint4* xv = reinterpret_cast<const uint4*>(x);
  const int64_t nvec = n >> 3;
  uint32_t m = 0;
  int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  const int64_t stride = (int64_t)gridDim.x * 256;
  for (; i + 7 * stride < nvec; i += 8 * stride) {     // eight 128-bit loads in flight per thread
    uint4 v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) v[u] = nt_load16(&xv[i + u * stride]);
#pragma unroll
    for (int u = 0; u < 8; ++u) m = umax(m, mag8(v[u]));
  }
  for (; i < nvec; i += stride) m = umax(m, mag8(nt_load16(&xv[i])));
  if (blockIdx.x == 0 && threadIdx.x < (n & 7)) m = umax(m, x[(nvec << 3) + threadIdx.x] & 0x7FFFu);
  m = row16_max_u32(m);
  __shared__ uint32_t part[16];
  if ((threadIdx.x & 15) == 0) part[threadIdx.x >> 4] = m;
  __syncthreads();
  if (threadIdx.x < 16) {
    m = row16_max_u32(part[threadIdx.x]);
    // The result only grows, so a block whose maximum does not exceed a (possibly stale) reading of
    // it has nothing to add; this keeps most of the same-address atomics out of the L2.
    if (threadIdx.x == 0 &&
        (m << 16) > __hip_atomic_load(amax_bits, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))
      atomicMax(amax_bits, m << 16);
  }
}

// Cast with one scale for the whole tensor; the scale is derived from *amax on the device.
__global__ __launch_bounds__(256) void cast_per_tensor_kernel(const uint16_t* __restrict__ x, int64_t n,
                                                              const float* __restrict__ amax,
                                                              uint8_t* __restrict__ q,
                                                              float* __restrict__ scale_out,
                                                              float* __restrict__ scale_inv_out) {
  float scale, scale_inv;
  scales_from_amax(*amax, scale, scale_inv);
  if (blockIdx.x == 0 && threadIdx.x == 0) {
    if (scale_out) *scale_out = scale;
    if (scale_inv_out) *scale_inv_out = scale_inv;
  }
  const uint4* xv = reinterpret_cast<const uint4*>(x);
  uint2* qv = reinterpret_cast<uint2*>(q);
  const int64_t nvec = n >> 3;
  const int64_t stride = (int64_t)gridDim.x * 256;
  int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  for (; i + 3 * stride < nvec; i += 4 * stride) {     // four 128-bit loads in flight per thread
    uint4 v[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) v[u] = nt_load16(&xv[i + u * stride]);
#pragma unroll
    for (int u = 0; u < 4; ++u) nt_store8(&qv[i + u * stride], cvt8<true>(v[u], scale));
  }
  for (; i < nvec; i += stride) nt_store8(&qv[i], cvt8<true>(nt_load16(&xv[i]), scale));
  if (blockIdx.x == 0 && threadIdx.x < (n & 7)) {
    int64_t j = (nvec << 3) + threadIdx.x;
    uint32_t r = cvt2<false, true>(0u, x[j], scale);
    q[j] = (uint8_t)(r & 0xFF);
  }
}


// ---------------------------------------------------------------------------------------------
// per-tensor amax + cast in one launch, for tensors small enough that the grid holds them in registers
// ---------------------------------------------------------------------------------------------
// Each workgroup loads its slice once (VEC 128-bit vectors per thread), the grid agrees on the maximum through
// two 32-bit words, and every workgroup then casts the slice it still holds: 3 bytes per element instead of the
// 5 of the two-pass form, one pass instead of two.
//   amax word : raised with an atomic maximum by the workgroups whose own maximum exceeds a (possibly stale)
//               reading of it -- a handful of atomics, as in amax_bf16_kernel; a clean fp32 value at all times
//   count word: every workgroup adds 1 once its maximum is published (release), then polls it (acquire) until it
//               has reached the grid size; it is never decremented.  Both words must be zero at launch.
// The count word is the caller's scale_inv output: when the first workgroup finally stores scale_inv there, every
// value it can take (amax_c / 448 >= 2e-15, Inf, NaN) reads as an integer far above the grid size, so a
// workgroup still polling sees "everyone has arrived" either way.
// Every wait is bounded: a workgroup whose polls run out (the grid was not resident together for that long)
// computes the maximum of the whole tensor by itself and publishes it, so the result does not depend on how the
// wait ended.  A workgroup that arrives only after scale_inv has been stored (possible only after such a
// time-out) finds a count above the grid size: its own + 1 has disturbed the stored value, and it stores the value
// again at its end (the amax word is final by then: the store is ordered after the maximum that justified it).
// The grid is at most 64 workgroups of 1024 threads: few and large, because every arrival is an atomic on one word,
// and those serialise across the chip at tens of nanoseconds each (256 arrivals cost more than the second pass
// they save).  On an otherwise idle chip of 256 CUs they are resident together and the wait is a few polls; when
// they are not (a persistent kernel of another stream holds the CUs, or the device is a partition with fewer CUs than
// the grid has workgroups) the bounded wait below runs out and the workgroups fall back to the solo maximum, with
// the same bits.
constexpr int kFusedMaxBlocks = 64;
constexpr int kFusedThreads = 1024;
constexpr int kFusedMaxVec = 8;
constexpr int64_t kFusedMaxElems = (int64_t)kFusedMaxBlocks * kFusedThreads * kFusedMaxVec * 8;   // 4 Mi elements

// maximum over a workgroup of 1024 threads; part: 16 words of LDS
__device__ __forceinline__ uint32_t block_max_u32(uint32_t m, uint32_t* part) {
  m = row16_max_u32(m);
  m = umax(m, (uint32_t)__shfl_xor((int)m, 16));
  m = umax(m, (uint32_t)__shfl_xor((int)m, 32));
  if ((threadIdx.x & 63) == 0) part[threadIdx.x >> 6] = m;
  __syncthreads();
  m = row16_max_u32(part[threadIdx.x & 15]);
  __syncthreads();
  return m;                       // the same in every thread
}

// SYNC3: the grid agrees through a block of the caller's that is zero at launch and zero again when the kernel ends:
// 64 slots, one per workgroup (amax_word points at them), and a departure count (count_word).  A workgroup STORES
// its own maximum, tagged valid, into its slot -- no read-modify-write on a shared word, whose 64 arrivals would
// queue up behind each other across the chip -- and its first wave then polls all slots with one 256-byte load per
// poll until every slot of the grid is valid; the maximum over the slots is the tensor's.  After its last read of
// the slots a workgroup adds to the departure count (behind the cast's stores, off the critical path), and the last
// one to leave clears slots and count.  No word needs clearing before the launch, and the results go to their own
// outputs (amax_out, scale_out, scale_inv_out).  (A workgroup whose wait ran out computes the maximum alone.)
constexpr uint32_t kSlotValid = 0x80000000u;
template <int VEC, bool SYNC3 = false>
__global__ __launch_bounds__(kFusedThreads) void quant_per_tensor_fused_kernel(const uint16_t* __restrict__ x, int64_t n,
                                                                     uint32_t* __restrict__ amax_word,
                                                                     uint32_t* __restrict__ count_word,
                                                                     uint8_t* __restrict__ q,
                                                                     float* __restrict__ scale_out,
                                                                     uint32_t spin_limit,
                                                                     float* __restrict__ amax_out = nullptr,
                                                                     float* __restrict__ scale_inv_out = nullptr) {
  __shared__ uint32_t part[16];
  __shared__ uint32_t s_amax, s_alone, s_repair;
  const uint4* xv = reinterpret_cast<const uint4*>(x);
  const int64_t nvec = n >> 3;
  const int64_t base = (int64_t)blockIdx.x * (kFusedThreads * VEC) + threadIdx.x;
  uint4 v[VEC];
  uint32_t m = 0;
#pragma unroll
  for (int u = 0; u < VEC; ++u) {
    const int64_t i = base + u * kFusedThreads;
    v[u] = i < nvec ? nt_load16(&xv[i]) : make_uint4(0, 0, 0, 0);
  }
#pragma unroll
  for (int u = 0; u < VEC; ++u) m = umax(m, mag8(v[u]));
  uint32_t tail = 0;              // the last n % 8 elements, one per thread of workgroup 0
  const bool has_tail = blockIdx.x == 0 && threadIdx.x < (n & 7);
  if (has_tail) {
    tail = x[(nvec << 3) + threadIdx.x];
    m = umax(m, tail & 0x7FFFu);
  }
  m = block_max_u32(m, part);
  const uint32_t grid = gridDim.x;
  if (SYNC3) {
    if (threadIdx.x < 64) {              // the first wave: lane l watches slot l
      const uint32_t lane = threadIdx.x;
      // (Relaxed accesses: a slot's value is all that is communicated -- nothing else is published with it, nothing
      // else of another workgroup's is read after it -- so no cache needs writing back or invalidating; a release or
      // an acquire at device scope does that to the XCD's whole L2.)
      if (lane == 0) __hip_atomic_store(amax_word + blockIdx.x, kSlotValid | m, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      uint32_t spins = 0, slot = 0;
      bool all = false;
      while (true) {
        slot = lane < grid ? __hip_atomic_load(amax_word + lane, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) : kSlotValid;
        all = __ballot((slot & kSlotValid) != 0) == ~0ull;
        if (all || spins++ >= spin_limit) break;
        __builtin_amdgcn_s_sleep(1);
      }
      uint32_t mx = (slot & kSlotValid) ? (slot & 0xFFFFu) : 0u;
      mx = row16_max_u32(mx);
      mx = umax(mx, (uint32_t)__shfl_xor((int)mx, 16));
      mx = umax(mx, (uint32_t)__shfl_xor((int)mx, 32));
      if (lane == 0) {
        s_amax = mx;
        s_alone = all ? 0u : 1u;
        s_repair = 0u;
      }
    }
  } else if (threadIdx.x == 0) {
    if ((m << 16) > __hip_atomic_load(amax_word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT))
      __hip_atomic_fetch_max(amax_word, m << 16, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    uint32_t seen = __hip_atomic_fetch_add(count_word, 1u, __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT) + 1u;
    s_repair = seen > grid ? 1u : 0u;
    uint32_t spins = 0;
    while (seen < grid && spins++ < spin_limit) {
      __builtin_amdgcn_s_sleep(1);
      seen = __hip_atomic_load(count_word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    }
    __atomic_thread_fence(__ATOMIC_ACQUIRE);          // (agent scope and wider)
    s_amax = __hip_atomic_load(amax_word, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) >> 16;
    s_alone = seen < grid ? 1u : 0u;
  }
  __syncthreads();
  uint32_t amax16 = s_amax;
  if (s_alone) {                  // (uniform over the workgroup) the wait ran out: the whole tensor's maximum, alone
    uint32_t mm = m;
    for (int64_t i = threadIdx.x; i < nvec; i += kFusedThreads) mm = umax(mm, mag8(xv[i]));
    if (threadIdx.x < (n & 7)) mm = umax(mm, x[(nvec << 3) + threadIdx.x] & 0x7FFFu);
    amax16 = block_max_u32(mm, part);
    if (!SYNC3 && threadIdx.x == 0) __hip_atomic_fetch_max(amax_word, amax16 << 16, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
  }
  float scale, scale_inv;
  scales_from_amax(__uint_as_float(amax16 << 16), scale, scale_inv);
  uint2* qv = reinterpret_cast<uint2*>(q);
#pragma unroll
  for (int u = 0; u < VEC; ++u) {
    const int64_t i = base + u * kFusedThreads;
    if (i < nvec) nt_store8(&qv[i], cvt8<true>(v[u], scale));
  }
  if (has_tail) q[(nvec << 3) + threadIdx.x] = (uint8_t)(cvt2<false, true>(0u, tail, scale) & 0xFFu);
  if (SYNC3) {
    if (threadIdx.x == 0 && blockIdx.x == 0) {
      if (amax_out) *amax_out = __uint_as_float(amax16 << 16);
      if (scale_out) *scale_out = scale;
      if (scale_inv_out) *scale_inv_out = scale_inv;
    }
    // this workgroup has read the slots for the last time (before the barrier above: the values had arrived, they
    // were used); the last one to say so clears them for the next launch
    if (threadIdx.x < 64) {
      uint32_t last = 0;
      if (threadIdx.x == 0)
        last = __hip_atomic_fetch_add(count_word, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1u == grid ? 1u : 0u;
      last = (uint32_t)__shfl((int)last, 0);
      if (last) {
        __hip_atomic_store(amax_word + threadIdx.x, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        if (threadIdx.x == 0) __hip_atomic_store(count_word, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
      }
    }
    return;
  }
  if (threadIdx.x == 0 && (blockIdx.x == 0 || s_repair)) {
    if (scale_out) *scale_out = scale;
    // scale_inv takes the place of the count (ordered after the maximum this workgroup may have published)
    __hip_atomic_store(count_word, __float_as_uint(scale_inv), __ATOMIC_RELEASE, __HIP_MEMORY_SCOPE_AGENT);
  }
}

// (SYNC3: the `seen > grid` repair of the two-word form cannot occur -- every workgroup arrives exactly once
// between two clearings.)
// Polls a waiting workgroup makes before it stops relying on the others (about a microsecond each): a few hundred
// microseconds at most, two orders of magnitude above what a resident grid needs.  The fallback gives the same
// bits, so a short wait loses nothing but time in the rare case.  (Atomic: the test hook below may be called from
// any thread.)
static std::atomic<uint32_t> g_spin_limit{1u << 8};

// Launches fill + fused kernel; the two words (device, 4 bytes each: amax, and scale_inv as the count) are zeroed
// first by a kernel (not a memset node, so the sequence can be captured in a graph).  n in (0, kFusedMaxElems].
static int launch_per_tensor_fused(const void* x, int64_t n, void* q, uint32_t* word, float* scale, float* scale_inv,
                                   hipStream_t s) {
  fill2_u32_kernel<<<1, 64, 0, s>>>(word, reinterpret_cast<uint32_t*>(scale_inv));
  const int64_t nvec = (n >> 3) > 0 ? (n >> 3) : 1;
  const int64_t per_thread = (nvec + (int64_t)kFusedMaxBlocks * kFusedThreads - 1) / ((int64_t)kFusedMaxBlocks * kFusedThreads);
  const int vec = per_thread <= 1 ? 1 : (per_thread <= 2 ? 2 : (per_thread <= 4 ? 4 : 8));
  const unsigned grid = (unsigned)((nvec + kFusedThreads * vec - 1) / (kFusedThreads * vec));
  const uint16_t* xs = (const uint16_t*)x;
  uint8_t* q8 = (uint8_t*)q;
  switch (vec) {
    case 1: quant_per_tensor_fused_kernel<1><<<grid, kFusedThreads, 0, s>>>(xs, n, word, reinterpret_cast<uint32_t*>(scale_inv), q8, scale, g_spin_limit.load(std::memory_order_relaxed)); break;
    case 2: quant_per_tensor_fused_kernel<2><<<grid, kFusedThreads, 0, s>>>(xs, n, word, reinterpret_cast<uint32_t*>(scale_inv), q8, scale, g_spin_limit.load(std::memory_order_relaxed)); break;
    case 4: quant_per_tensor_fused_kernel<4><<<grid, kFusedThreads, 0, s>>>(xs, n, word, reinterpret_cast<uint32_t*>(scale_inv), q8, scale, g_spin_limit.load(std::memory_order_relaxed)); break;
    default: quant_per_tensor_fused_kernel<8><<<grid, kFusedThreads, 0, s>>>(xs, n, word, reinterpret_cast<uint32_t*>(scale_inv), q8, scale, g_spin_limit.load(std::memory_order_relaxed)); break;
  }
  return check_launch("quantize_per_tensor");
}

// ---------------------------------------------------------------------------------------------
// 1x128 groups along the contiguous dim (activations, gradient buckets)
// ---------------------------------------------------------------------------------------------
// One group = 128 bf16 = 16 lanes x 16 B.  A thread handles UNROLL groups-slices so several
// 128-bit loads are in flight before the first reduction.
template <int UNROLL>
__global__ __launch_bounds__(256) void quant_1x128_kernel(const uint4* __restrict__ x,
                                                          uint2* __restrict__ q,
                                                          float* __restrict__ scale,
                                                          float* __restrict__ scale_inv,
                                                          int64_t nvec) {
  const int64_t base = (int64_t)blockIdx.x * (256 * UNROLL) + threadIdx.x;
  uint4 v[UNROLL];
#pragma unroll
  for (int u = 0; u < UNROLL; ++u) {
    int64_t i = base + u * 256;
    v[u] = i < nvec ? nt_load16(&x[i]) : make_uint4(0, 0, 0, 0);
  }
  static_assert(UNROLL == 4, "scales4_from_amax serves four groups per 16-lane row");
  uint32_t m[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) m[u] = row16_max_u32(mag8(v[u]));
  const int l16 = threadIdx.x & 15;
  float s[4], mine, mine_inv;
  scales4_from_amax(m, l16, 0, s, mine, mine_inv);
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    int64_t i = base + u * 256;
    if (i < nvec) nt_store8(&q[i], cvt8<false>(v[u], s[u]));
  }
  const int64_t i_mine = base - l16 + l16 * 256;      // first vector of the group whose scales this lane holds
  if (l16 < 4 && i_mine < nvec) {
    if (scale) scale[i_mine >> 4] = mine;
    scale_inv[i_mine >> 4] = mine_inv;
  }
}

// Same arithmetic, scales written k-block-major: scale[g * rows + row] for group g of a row.  This
// is the layout the GEMM reads with unit stride across the 16 rows of a fragment.  A workgroup owns
// 16 rows x 4 consecutive groups so that its 64 scales leave as four 64-byte runs.
__global__ __launch_bounds__(256) void quant_1x128_kmajor_kernel(const uint16_t* __restrict__ x,
                                                                 uint8_t* __restrict__ q,
                                                                 float* __restrict__ scale,
                                                                 float* __restrict__ scale_inv, int rows,
                                                                 int cols, int pow2) {
  const int groups = cols >> 7;
  const int gtiles = (groups + 3) >> 2;
  const int g0 = (blockIdx.x % gtiles) * 4, row0 = (blockIdx.x / gtiles) * 16;
  const int r = threadIdx.x >> 4, l16 = threadIdx.x & 15;
  const int row = row0 + r;
  __shared__ float s_s[4][16], s_si[4][16];
  uint4 v[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const bool ok = row < rows && g0 + u < groups;
    v[u] = ok ? nt_load16(x + (int64_t)row * cols + (g0 + u) * 128 + l16 * 8) : make_uint4(0, 0, 0, 0);
  }
  uint32_t m[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) m[u] = row16_max_u32(mag8(v[u]));
  float s[4], mine, mine_inv;
  scales4_from_amax(m, l16, pow2, s, mine, mine_inv);
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const bool ok = row < rows && g0 + u < groups;
    if (ok) nt_store8(q + (int64_t)row * cols + (g0 + u) * 128 + l16 * 8, cvt8<false>(v[u], s[u]));
  }
  if (l16 < 4) {
    s_s[l16][r] = mine;
    s_si[l16][r] = mine_inv;
  }
  __syncthreads();
  if (threadIdx.x < 64) {
    const int u = threadIdx.x >> 4, rr = threadIdx.x & 15;
    if (row0 + rr < rows && g0 + u < groups) {
      const int64_t o = (int64_t)(g0 + u) * rows + row0 + rr;
      if (scale) scale[o] = s_s[u][rr];
      scale_inv[o] = s_si[u][rr];
    }
  }
}

// ---------------------------------------------------------------------------------------------
// SwiGLU fused with the 1x128 quantization of its result (input of the down projection)
// ---------------------------------------------------------------------------------------------
// (exp_spec, silu_f32 and swiglu2 are in hpfp8_device.h: the GEMM's SwiGLU epilogue uses them too)
// h[rows, 2 * inter] (row stride ld elements): gate = columns [0, inter), up = [inter, 2 inter).
// q[rows, inter] = codes of act = silu(gate) * up in 1x128 groups; scales [rows, inter/128], or
// [inter/128, rows] with KMAJOR.  Work split as in quant_1x128_kmajor_kernel.
template <bool KMAJOR, bool FAST>
__global__ __launch_bounds__(256) void swiglu_quant_1x128_kernel(const uint16_t* __restrict__ h, int64_t ld,
                                                                 uint8_t* __restrict__ q, float* __restrict__ scale,
                                                                 float* __restrict__ scale_inv,
                                                                 uint16_t* __restrict__ act, int rows, int inter,
                                                                 int pow2) {
  const int groups = inter >> 7;
  const int gtiles = (groups + 3) >> 2;
  const int g0 = (blockIdx.x % gtiles) * 4, row0 = (blockIdx.x / gtiles) * 16;
  const int r = threadIdx.x >> 4, l16 = threadIdx.x & 15;
  const int row = row0 + r;
  __shared__ float s_s[4][16], s_si[4][16];
  uint4 vg[4], vu[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    const bool ok = row < rows && g0 + u < groups;
    const uint16_t* src = h + (int64_t)row * ld + (g0 + u) * 128 + l16 * 8;
    vg[u] = ok ? nt_load16(src) : make_uint4(0, 0, 0, 0);
    vu[u] = ok ? nt_load16(src + inter) : make_uint4(0, 0, 0, 0);
  }
  uint4 a[4];
  uint32_t m[4];
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    a[u].x = swiglu2<FAST>(vg[u].x, vu[u].x);
    a[u].y = swiglu2<FAST>(vg[u].y, vu[u].y);
    a[u].z = swiglu2<FAST>(vg[u].z, vu[u].z);
    a[u].w = swiglu2<FAST>(vg[u].w, vu[u].w);
    m[u] = row16_max_u32(mag8(a[u]));
  }
  float s[4], mine, mine_inv;
  scales4_from_amax(m, l16, pow2, s, mine, mine_inv);
#pragma unroll
  for (int u = 0; u < 4; ++u) {
    if (row < rows && g0 + u < groups) {
      const int64_t o = (int64_t)row * inter + (g0 + u) * 128 + l16 * 8;
      nt_store8(q + o, cvt8<false>(a[u], s[u]));
      if (act) nt_store16(act + o, a[u]);
    }
  }
  if (l16 < 4) {
    s_s[l16][r] = mine;
    s_si[l16][r] = mine_inv;
  }
  __syncthreads();
  if (threadIdx.x < 64) {
    const int u = KMAJOR ? threadIdx.x >> 4 : threadIdx.x & 3, rr = KMAJOR ? threadIdx.x & 15 : threadIdx.x >> 2;
    if (row0 + rr < rows && g0 + u < groups) {
      const int64_t o = KMAJOR ? (int64_t)(g0 + u) * rows + row0 + rr : (int64_t)(row0 + rr) * groups + g0 + u;
      if (scale) scale[o] = s_s[u][rr];
      scale_inv[o] = s_si[u][rr];
    }
  }
}

// Backward of act = silu(gate) * up for two (gate, up, d act) triples packed like their sources:
//   d up   = d act * bf16(silu(g))                (the rounded silu is what forward multiplied with)
//   d gate = d act * up * (sig + silu * (1 - sig)),  sig = 1 / (1 + exp(-g)), silu = g * sig
// in fp32 with the hardware's base-2 exponential and reciprocal, each result rounded to bf16 once.
__device__ __forceinline__ void swiglu_bwd2(uint32_t gw, uint32_t uw, uint32_t dw, uint32_t& dgw, uint32_t& duw) {
  typedef float f32x2 __attribute__((ext_vector_type(2)));
  typedef __bf16 bf16x2 __attribute__((ext_vector_type(2)));
  const float g[2] = {bf16lo(gw), bf16hi(gw)}, u[2] = {bf16lo(uw), bf16hi(uw)}, d[2] = {bf16lo(dw), bf16hi(dw)};
  float sig[2], silu[2];
#pragma unroll
  for (int t = 0; t < 2; ++t) {
    sig[t] = __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(g[t] * -1.44269504f));
    silu[t] = g[t] * sig[t];
  }
  const f32x2 sf = {silu[0], silu[1]};
  const uint32_t sw = __builtin_bit_cast(uint32_t, __builtin_convertvector(sf, bf16x2));
  const f32x2 du = {d[0] * bf16lo(sw), d[1] * bf16hi(sw)};
  const f32x2 dg = {(d[0] * u[0]) * (sig[0] + silu[0] * (1.0f - sig[0])), (d[1] * u[1]) * (sig[1] + silu[1] * (1.0f - sig[1]))};
  duw = __builtin_bit_cast(uint32_t, __builtin_convertvector(du, bf16x2));
  dgw = __builtin_bit_cast(uint32_t, __builtin_convertvector(dg, bf16x2));
}

// h[rows, 2 * inter] (row stride ld_h), dact[rows, inter] -> dh[rows, 2 * inter] (row stride ld_dh) = d gate | d up.
// One 16-byte vector of 8 activations per thread and step; three streams in, two out.
__global__ __launch_bounds__(256) void swiglu_backward_kernel(const uint16_t* __restrict__ h, int64_t ld_h,
                                                              const uint16_t* __restrict__ dact,
                                                              uint16_t* __restrict__ dh, int64_t ld_dh, int64_t nvec,
                                                              int inter) {
  const int vec_per_row = inter >> 3;
  constexpr int UNROLL = 2;
  const int64_t base = (int64_t)blockIdx.x * (256 * UNROLL) + threadIdx.x;
  uint4 vg[UNROLL], vu[UNROLL], vd[UNROLL];
  int64_t row[UNROLL];
  int col[UNROLL];
#pragma unroll
  for (int k = 0; k < UNROLL; ++k) {
    const int64_t i = base + k * 256;
    const bool ok = i < nvec;
    row[k] = ok ? i / vec_per_row : 0;
    col[k] = ok ? (int)(i - row[k] * vec_per_row) * 8 : 0;
    const uint16_t* src = h + row[k] * ld_h + col[k];
    vg[k] = ok ? nt_load16(src) : make_uint4(0, 0, 0, 0);
    vu[k] = ok ? nt_load16(src + inter) : make_uint4(0, 0, 0, 0);
    vd[k] = ok ? nt_load16(dact + row[k] * (int64_t)inter + col[k]) : make_uint4(0, 0, 0, 0);
  }
#pragma unroll
  for (int k = 0; k < UNROLL; ++k) {
    uint4 dg, du;
    swiglu_bwd2(vg[k].x, vu[k].x, vd[k].x, dg.x, du.x);
    swiglu_bwd2(vg[k].y, vu[k].y, vd[k].y, dg.y, du.y);
    swiglu_bwd2(vg[k].z, vu[k].z, vd[k].z, dg.z, du.z);
    swiglu_bwd2(vg[k].w, vu[k].w, vd[k].w, dg.w, du.w);
    if (base + k * 256 < nvec) {
      uint16_t* dst = dh + row[k] * ld_dh + col[k];
      nt_store16(dst, dg);
      nt_store16(dst + inter, du);
    }
  }
}

// ---------------------------------------------------------------------------------------------
// shared by the two tile kernels below: 128x128 tile, 256 threads
// ---------------------------------------------------------------------------------------------
// Thread t owns column group cg = t%16 (8 columns) and row quad rq = t/16: tile rows
// {4rq..4rq+3} and {64+4rq..64+4rq+3}, i.e. load slot p -> row (p/4)*64 + 4rq + p%4.  Four
// vertically adjacent codes then pack into one 32-bit word of the transposed tile.
__device__ __forceinline__ int tile_row(int rq, int p) { return (p >> 2) * 64 + 4 * rq + (p & 3); }

// 4x4 byte transpose: out[j] byte r = in[r] byte j.
__device__ __forceinline__ void byte_transpose4(const uint32_t in[4], uint32_t out[4]) {
#pragma unroll
  for (int j = 0; j < 4; ++j)
    out[j] = ((in[0] >> (8 * j)) & 0xFFu) | (((in[1] >> (8 * j)) & 0xFFu) << 8) |
             (((in[2] >> (8 * j)) & 0xFFu) << 16) | (((in[3] >> (8 * j)) & 0xFFu) << 24);
}

// Writes the thread's codes c[p] (8 codes of tile row tile_row(rq,p)) into the transposed LDS
// tile (row = tile column, 128 B; 16-byte chunks XOR-swizzled by the column group), then the
// workgroup streams the tile out as 128 rows of dst (row stride ld bytes) with 128-bit stores.
__device__ __forceinline__ void store_tile_transposed(uint8_t* tile, const uint2 c[8], int cg, int rq,
                                                      uint8_t* __restrict__ dst, int64_t ld) {
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const uint32_t lo[4] = {c[4 * h].x, c[4 * h + 1].x, c[4 * h + 2].x, c[4 * h + 3].x};
    const uint32_t hi[4] = {c[4 * h].y, c[4 * h + 1].y, c[4 * h + 2].y, c[4 * h + 3].y};
    uint32_t wcol[8];
    byte_transpose4(lo, wcol);
    byte_transpose4(hi, wcol + 4);
    const int rword = h * 16 + rq;  // 32-bit word inside the 128-byte transposed row
    const int pc = (rword >> 2) ^ (cg & 7);
#pragma unroll
    for (int j = 0; j < 8; ++j)
      *reinterpret_cast<uint32_t*>(&tile[(cg * 8 + j) * 128 + pc * 16 + (rword & 3) * 4]) = wcol[j];
  }
  __syncthreads();
#pragma unroll
  for (int pass = 0; pass < 4; ++pass) {
    const int col = pass * 32 + (threadIdx.x >> 3);
    const int pc = threadIdx.x & 7;
    const int chunk = pc ^ ((col >> 3) & 7);
    uint4 o = *reinterpret_cast<const uint4*>(&tile[col * 128 + pc * 16]);
    nt_store16(reinterpret_cast<char*>(dst) + ((uint32_t)col * (uint32_t)ld + (uint32_t)chunk * 16u), o);
  }
}

// ---------------------------------------------------------------------------------------------
// 128x128 blocks (weights), optional transposed copy of the codes for dgrad
// ---------------------------------------------------------------------------------------------
// One 128x128 tile per workgroup (several tiles per workgroup with the next tile's loads issued ahead were measured
// and were slower: more resident workgroups hide latency better).  The grid is two-dimensional with x the fast index:
// along_k = 1 walks along a tile row of the source, 0 down a tile column (see transpose_grid).
template <bool WITH_T>
__global__ __launch_bounds__(256) void quant_128x128_kernel(const uint16_t* __restrict__ w, int rows,
                                                            int cols, uint8_t* __restrict__ q,
                                                            uint8_t* __restrict__ qt, int64_t ld_t,
                                                            float* __restrict__ scale,
                                                            float* __restrict__ scale_inv, int pow2, int along_k) {
  const int cb = cols >> 7;
  const int cg = threadIdx.x & 15, rq = threadIdx.x >> 4;
  __shared__ uint32_t part[16];
  __shared__ float s_scale;
  __shared__ __attribute__((aligned(16))) uint8_t tile[WITH_T ? 128 * 128 : 16];
  const int br = along_k ? blockIdx.y : blockIdx.x, bc = along_k ? blockIdx.x : blockIdx.y;
  // a tile's first element is a uniform 64-bit address, positions inside the tile are 32-bit byte offsets
  const char* wbase = reinterpret_cast<const char*>(w + (int64_t)br * 128 * cols + bc * 128);
  char* qbase = reinterpret_cast<char*>(q + (int64_t)br * 128 * cols + bc * 128);
  const uint32_t ucols = (uint32_t)cols;
  uint4 v[8];
#pragma unroll
  for (int p = 0; p < 8; ++p) v[p] = nt_load16(wbase + ((uint32_t)tile_row(rq, p) * ucols + (uint32_t)cg * 8u) * 2u);
  const int sidx = br * cb + bc;
  uint32_t m = 0;
#pragma unroll
  for (int p = 0; p < 8; ++p) m = umax(m, mag8(v[p]));
  m = row16_max_u32(m);
  if (cg == 0) part[rq] = m;
  __syncthreads();
  if (threadIdx.x < 16) {
    m = row16_max_u32(part[threadIdx.x]);
    if (threadIdx.x == 0) {
      float s, si;
      scales_from_amax(__uint_as_float(m << 16), s, si, pow2);
      s_scale = s;
      if (scale) scale[sidx] = s;
      scale_inv[sidx] = si;
    }
  }
  __syncthreads();
  const float s = s_scale;
  uint2 c[8];
#pragma unroll
  for (int p = 0; p < 8; ++p) {
    c[p] = cvt8<false>(v[p], s);
    nt_store8(qbase + ((uint32_t)tile_row(rq, p) * ucols + (uint32_t)cg * 8u), c[p]);
  }
  if (WITH_T) store_tile_transposed(tile, c, cg, rq, qt + (int64_t)bc * 128 * ld_t + br * 128, ld_t);
}

// Without the transposed copy and for a large matrix with an even number of tile columns: two neighbouring 128x128
// blocks per workgroup, so that a row of the workgroup's piece is 512 contiguous bytes of the source and 256 of the
// codes instead of 256 and 128 (a copy kernel with this access pattern reaches 78 % of the HBM peak on a
// [36864, 7168] matrix where the one-block pattern reaches 73 %; on a matrix with fewer than a few thousand tiles the
// smaller workgroups of the one-block kernel win).  32 lanes cover a row, a pass 8 rows, 16 passes the tile; lanes
// 0-15 of a row belong to the left block, 16-31 to the right one.  blockIdx.x walks along a tile row.
__global__ __launch_bounds__(256) void quant_128x128_pair_kernel(const uint16_t* __restrict__ w, int cols,
                                                                 uint8_t* __restrict__ q, float* __restrict__ scale,
                                                                 float* __restrict__ scale_inv, int pow2) {
  const int cb = cols >> 7;
  const int lc = threadIdx.x & 31, lr = threadIdx.x >> 5, half = lc >> 4;
  __shared__ uint32_t part[16];
  __shared__ float s_scale[2];
  const int br = blockIdx.y, bc = blockIdx.x * 2;
  const char* wbase = reinterpret_cast<const char*>(w + (int64_t)br * 128 * cols + bc * 128);
  char* qbase = reinterpret_cast<char*>(q + (int64_t)br * 128 * cols + bc * 128);
  const uint32_t ucols = (uint32_t)cols;
  uint4 v[16];
#pragma unroll
  for (int p = 0; p < 16; ++p) v[p] = nt_load16(wbase + ((uint32_t)(p * 8 + lr) * ucols + (uint32_t)lc * 8u) * 2u);
  uint32_t m = 0;
#pragma unroll
  for (int p = 0; p < 16; ++p) m = umax(m, mag8(v[p]));
  m = row16_max_u32(m);
  // part[2 * j + half]: 16-lane group j = threadIdx.x >> 5 (8 of them per block half)
  if ((threadIdx.x & 15) == 0) part[lr * 2 + half] = m;
  __syncthreads();
  if (threadIdx.x < 2) {
    uint32_t mm = 0;
#pragma unroll
    for (int j = 0; j < 8; ++j) mm = umax(mm, part[j * 2 + threadIdx.x]);
    float s, si;
    scales_from_amax(__uint_as_float(mm << 16), s, si, pow2);
    s_scale[threadIdx.x] = s;
    const int sidx = br * cb + bc + threadIdx.x;
    if (scale) scale[sidx] = s;
    scale_inv[sidx] = si;
  }
  __syncthreads();
  const float s = s_scale[half];
#pragma unroll
  for (int p = 0; p < 16; ++p)
    nt_store8(qbase + ((uint32_t)(p * 8 + lr) * ucols + (uint32_t)lc * 8u), cvt8<false>(v[p], s));
}

// ---------------------------------------------------------------------------------------------
// 128x1 groups, transposed output (wgrad operands): x[M,K] -> qt[K,M], scales [K, M/128]
// ---------------------------------------------------------------------------------------------
// With DUAL the same pass also writes the 1x128 quantization of x itself (codes q[M,K], one scale per
// row and 128 columns: [M, K/128], or [K/128, M] with KMAJOR): forward / dgrad operand and wgrad
// operand from one read of the bf16 source.
// With SW (1: exactly specified silu, 2: hardware exponential and reciprocal) the source is h[M, 2K] = gate | up
// and what is quantized is act = silu(gate) * up, computed as the tile is loaded: both operand forms of the
// down projection's input from one read of the gate/up output, the bf16 activation never written.
// With SW = 3 the source is again h[M, K] = gate | up (K = 2 * inter) together with dact[M, K / 2], and what is
// quantized is the gradient of SwiGLU, d gate | d up [M, K], computed as the tile is loaded exactly as
// swiglu_backward_kernel computes it: both operand forms of the gate/up projection's output gradient (dgrad and
// wgrad) without the bf16 gradient ever being written.
// ld_src: row stride of the source in elements (K, or at least 2K with SW = 1, 2).
// With GROUPED (MoE: rows of x sorted by expert) the 128-row groups restart at every expert's first row and the
// transposed output lives on the padded token axis of `layout` (grouped.hip): output block tr belongs to expert
// layout[5E + 1 + tr], holds that expert's rows [128 j, 128 j + 128) (j = tr - the expert's first block) and is
// filled up with zero codes past the expert's last row; m is then the number of source rows (any count), mb the
// number of padded blocks the grid covers, and blocks beyond those in use are left untouched.  The 1x128 form
// (DUAL) is written for the rows that exist, at their own positions.
// Tile order.  The grid is two-dimensional, x the fast index: with `along_k` = 0 consecutive workgroups walk down a
// tile column of the source (tile row fastest: neighbours in x write neighbouring 128-byte pieces of the same
// transposed rows), with 1 along a tile row (tile column fastest: neighbours read neighbouring 256-byte pieces of the
// same source rows).  Which of the two is faster depends on the source's row stride: with a stride that is a multiple
// of 16 KB the 128 rows of a tile column fall on few memory channels, and only the second order keeps all of them busy.
// All address arithmetic per thread is 32-bit: a tile's first element is a uniform 64-bit pointer, a thread's position
// inside the tile an unsigned byte offset (a tile spans less than 4 GB: row strides below 2^24 elements).
// Column sums of a 128x128 bf16 tile in fp32, in a fixed order (so that a CPU restatement gives the same bits): a
// thread adds its 8 rows onto +0 in load-slot order (tile rows 4rq, 4rq+1, 4rq+2, 4rq+3, then the same + 64), cs[i]
// for its column cg * 8 + i; wave_column_sums() combines the four row quads of a wave as (q0 + q1) + (q2 + q3) and
// puts the wave's sums into s_cs[wave][column]; after a workgroup barrier column_sum_of_tile() adds the four waves
// in order.
__device__ __forceinline__ void wave_column_sums(float cs[8], int cg, int wave, float (*s_cs)[128]) {
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    cs[i] += __shfl_xor(cs[i], 16);
    cs[i] += __shfl_xor(cs[i], 32);
  }
  if ((threadIdx.x & 63) < 16) {
    *reinterpret_cast<float4*>(&s_cs[wave][cg * 8]) = make_float4(cs[0], cs[1], cs[2], cs[3]);
    *reinterpret_cast<float4*>(&s_cs[wave][cg * 8 + 4]) = make_float4(cs[4], cs[5], cs[6], cs[7]);
  }
}
__device__ __forceinline__ void tile_column_sums(const uint4 v[8], int cg, int wave, float (*s_cs)[128]) {
  float cs[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
#pragma unroll
  for (int p = 0; p < 8; ++p) {
    const uint32_t ws[4] = {v[p].x, v[p].y, v[p].z, v[p].w};
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      cs[2 * i] += bf16lo(ws[i]);
      cs[2 * i + 1] += bf16hi(ws[i]);
    }
  }
  wave_column_sums(cs, cg, wave, s_cs);
}
__device__ __forceinline__ float column_sum_of_tile(const float (*s_cs)[128], int col) {
  return ((s_cs[0][col] + s_cs[1][col]) + s_cs[2][col]) + s_cs[3][col];
}

// With COLSUM the kernel also writes colsum_part[tr * k + column] = the fp32 sum of the tile's 128 rows per column
// (tile_column_sums): the per-block partial sums of a bias gradient, from the same read of grad_out.
template <bool KMAJOR, bool DUAL, int SW = 0, bool GROUPED = false, bool COLSUM = false>
__global__ __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(5))) void quant_128x1_t_kernel(const uint16_t* __restrict__ x, int64_t ld_src, int m, int k,
                                                            uint8_t* __restrict__ qt, int64_t ld_t,
                                                            float* __restrict__ scale_t,
                                                            float* __restrict__ scale_inv_t,
                                                            uint8_t* __restrict__ q, float* __restrict__ scale_r,
                                                            float* __restrict__ scale_inv_r, int pow2, int along_k = 0,
                                                            const int32_t* __restrict__ layout = nullptr, int experts = 0,
                                                            int padded_blocks = 0, const uint16_t* __restrict__ dact = nullptr,
                                                            float* __restrict__ colsum_part = nullptr) {
  static_assert(!COLSUM || (SW == 0 && !GROUPED), "column sums: plain dense source only");
  const int kb = k >> 7, mb = GROUPED ? padded_blocks : m >> 7;
  const int cg = threadIdx.x & 15, rq = threadIdx.x >> 4;
  const int wave = threadIdx.x >> 6;
  __shared__ uint32_t part[4][64];  // [wave][cg*4 + word]
  __shared__ float s_scale[128];
  __shared__ float s_row[DUAL ? 256 : 2];   // scale, scale_inv of the tile's 128 rows
  __shared__ __attribute__((aligned(16))) float s_cs[COLSUM ? 4 : 1][128];
  __shared__ __attribute__((aligned(16))) uint8_t tile[128 * 128];
  const int tr = along_k ? blockIdx.y : blockIdx.x, tc = along_k ? blockIdx.x : blockIdx.y;
  // first source row of the tile and how many of its 128 rows exist (dense: tr * 128 and all of them)
  int g_row0 = tr * 128, g_valid = 128;
  if (GROUPED) {
    const int e = layout[5 * experts + 1 + tr];
    if (e < 0) return;                                   // (uniform over the workgroup) a block no expert owns
    const int j = tr - layout[4 * e + 2];
    g_row0 = layout[4 * e + 0] + j * 128;
    g_valid = layout[4 * e + 1] - j * 128;
    g_valid = g_valid < 0 ? 0 : (g_valid > 128 ? 128 : g_valid);
  }
  // byte offset of this thread's first element inside the source tile, and the row stride in bytes
  const uint32_t ld_b = (uint32_t)ld_src * 2u;
  const uint32_t t_off = (uint32_t)(4 * rq) * ld_b + (uint32_t)cg * 16u;
  auto row_off = [&](int p) -> uint32_t { return t_off + (uint32_t)((p >> 2) * 64 + (p & 3)) * ld_b; };
  uint4 v[8];
  if (SW == 3) {
    // tile columns [0, inter) are d gate (from gate, up and d act), [inter, 2 inter) are d up (from gate and d act)
    const int inter = k >> 1;
    const bool is_gate = tc * 128 < inter;
    const int c0 = tc * 128 - (is_gate ? 0 : inter);                    // first column inside the gate / up half and inside d act
    const char* gbase = reinterpret_cast<const char*>(x + (int64_t)g_row0 * ld_src + c0);
    const char* dbase = reinterpret_cast<const char*>(dact + (int64_t)g_row0 * inter + c0);
    const uint32_t ldd_b = (uint32_t)inter * 2u;
    const uint32_t d_off = (uint32_t)(4 * rq) * ldd_b + (uint32_t)cg * 16u;
#pragma unroll
    for (int p = 0; p < 8; ++p) {
      const uint4 gv = nt_load16(gbase + row_off(p));
      const uint4 dv = nt_load16(dbase + d_off + (uint32_t)((p >> 2) * 64 + (p & 3)) * ldd_b);
      uint32_t unused;
      if (is_gate) {
        const uint4 uv = nt_load16(gbase + (uint32_t)inter * 2u + row_off(p));
        swiglu_bwd2(gv.x, uv.x, dv.x, v[p].x, unused);
        swiglu_bwd2(gv.y, uv.y, dv.y, v[p].y, unused);
        swiglu_bwd2(gv.z, uv.z, dv.z, v[p].z, unused);
        swiglu_bwd2(gv.w, uv.w, dv.w, v[p].w, unused);
      } else {
        swiglu_bwd2(gv.x, 0u, dv.x, unused, v[p].x);
        swiglu_bwd2(gv.y, 0u, dv.y, unused, v[p].y);
        swiglu_bwd2(gv.z, 0u, dv.z, unused, v[p].z);
        swiglu_bwd2(gv.w, 0u, dv.w, unused, v[p].w);
      }
    }
  } else {
    const char* sbase = reinterpret_cast<const char*>(x + (int64_t)g_row0 * ld_src + tc * 128);
#pragma unroll
    for (int p = 0; p < 8; ++p)
      v[p] = (!GROUPED || tile_row(rq, p) < g_valid) ? nt_load16(sbase + row_off(p)) : make_uint4(0, 0, 0, 0);
    if (SW) {
#pragma unroll
      for (int p = 0; p < 8; ++p) {
        const uint4 u = nt_load16(sbase + (uint32_t)k * 2u + row_off(p));
        v[p].x = swiglu2<SW == 2>(v[p].x, u.x);
        v[p].y = swiglu2<SW == 2>(v[p].y, u.y);
        v[p].z = swiglu2<SW == 2>(v[p].z, u.z);
        v[p].w = swiglu2<SW == 2>(v[p].w, u.w);
      }
    }
  }
  // per-column magnitudes over this thread's 8 rows, two columns per word
  uint32_t cm[4] = {0, 0, 0, 0};
#pragma unroll
  for (int p = 0; p < 8; ++p) {
    cm[0] = pk_max_u16(cm[0], v[p].x & 0x7FFF7FFFu);
    cm[1] = pk_max_u16(cm[1], v[p].y & 0x7FFF7FFFu);
    cm[2] = pk_max_u16(cm[2], v[p].z & 0x7FFF7FFFu);
    cm[3] = pk_max_u16(cm[3], v[p].w & 0x7FFF7FFFu);
  }
  // across the 4 row quads inside the wave (lanes differing in bits 4 and 5)
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    cm[i] = pk_max_u16(cm[i], (uint32_t)__shfl_xor((int)cm[i], 16));
    cm[i] = pk_max_u16(cm[i], (uint32_t)__shfl_xor((int)cm[i], 32));
  }
  if ((threadIdx.x & 63) < 16)
    *reinterpret_cast<uint4*>(&part[wave][cg * 4]) = make_uint4(cm[0], cm[1], cm[2], cm[3]);
  if (DUAL) {
    // the 16 threads of a row quad hold a whole 128-column group of each of their 8 rows
    char* qbase = reinterpret_cast<char*>(q + (int64_t)g_row0 * k + tc * 128);
    const uint32_t q_off = (uint32_t)(4 * rq) * (uint32_t)k + (uint32_t)cg * 8u;
#pragma unroll
    for (int half = 0; half < 2; ++half) {
      uint32_t mr[4];
#pragma unroll
      for (int p = 0; p < 4; ++p) mr[p] = row16_max_u32(mag8(v[4 * half + p]));
      float s[4], mine, mine_inv;
      scales4_from_amax(mr, cg, pow2, s, mine, mine_inv);
#pragma unroll
      for (int p = 0; p < 4; ++p) {
        const int row = tile_row(rq, 4 * half + p);
        if (!GROUPED || row < g_valid)
          nt_store8(qbase + q_off + (uint32_t)(half * 64 + p) * (uint32_t)k, cvt8<false>(v[4 * half + p], s[p]));
      }
      if (cg < 4) {
        const int row = tile_row(rq, 4 * half + cg);
        s_row[row] = mine;
        s_row[128 + row] = mine_inv;
      }
    }
  }
  __syncthreads();
  if (DUAL && threadIdx.x >= 128) {
    const int row = threadIdx.x - 128;
    const int64_t r_abs = (int64_t)g_row0 + row;
    const int64_t o = KMAJOR ? (int64_t)tc * m + r_abs : r_abs * kb + tc;
    if (!GROUPED || row < g_valid) {
      if (scale_r) scale_r[o] = s_row[row];
      scale_inv_r[o] = s_row[128 + row];
    }
  }
  if (threadIdx.x < 128) {
    const int col = threadIdx.x, word = col >> 1;
    uint32_t mw = pk_max_u16(pk_max_u16(part[0][word], part[1][word]), pk_max_u16(part[2][word], part[3][word]));
    uint32_t mag = (col & 1) ? (mw >> 16) : (mw & 0xFFFFu);
    float s, si;
    scales_from_amax(__uint_as_float(mag << 16), s, si, pow2);
    s_scale[col] = s;
    // row-major [k, m/128], or block-major [m/128, k] (unit stride over the output rows)
    int64_t o = KMAJOR ? (int64_t)tr * k + tc * 128 + col : ((int64_t)tc * 128 + col) * mb + tr;
    if (scale_t) scale_t[o] = s;
    scale_inv_t[o] = si;
  }
  __syncthreads();
  const float4 sa = *reinterpret_cast<const float4*>(&s_scale[cg * 8]), sb = *reinterpret_cast<const float4*>(&s_scale[cg * 8 + 4]);
  const float sc[8] = {sa.x, sa.y, sa.z, sa.w, sb.x, sb.y, sb.z, sb.w};
  uint2 c[8];
  float cs[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};     // (COLSUM) this thread's column sums, rows in load-slot order
#pragma unroll
  for (int p = 0; p < 8; ++p) {
    // scale from this very column's amax: the clamp to +-448 would be a no-op (see cvt2)
    const uint32_t ws[4] = {v[p].x, v[p].y, v[p].z, v[p].w};
    float f[8];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      f[2 * i] = bf16lo(ws[i]);
      f[2 * i + 1] = bf16hi(ws[i]);
    }
    if (COLSUM) {
#pragma unroll
      for (int i = 0; i < 8; ++i) cs[i] += f[i];
    }
    uint32_t lo = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(f[0] * sc[0], f[1] * sc[1], 0, false);
    lo = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(f[2] * sc[2], f[3] * sc[3], (int)lo, true);
    uint32_t hi = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(f[4] * sc[4], f[5] * sc[5], 0, false);
    hi = (uint32_t)__builtin_amdgcn_cvt_pk_fp8_f32(f[6] * sc[6], f[7] * sc[7], (int)hi, true);
    c[p].x = lo;
    c[p].y = hi;
  }
  if (COLSUM) wave_column_sums(cs, cg, wave, s_cs);
  store_tile_transposed(tile, c, cg, rq, qt + (int64_t)tc * 128 * ld_t + tr * 128, ld_t);
  // (the barrier inside store_tile_transposed has also made every wave's column sums visible)
  if (COLSUM && threadIdx.x < 128)
    colsum_part[(int64_t)tr * k + tc * 128 + threadIdx.x] = column_sum_of_tile(s_cs, threadIdx.x);
}

// ---------------------------------------------------------------------------------------------
// traffic model of the transposing quantizers (measurement aid)
// ---------------------------------------------------------------------------------------------
// The memory accesses of quant_128x1_t_kernel and nothing else: a workgroup loads its 128x128 bf16 tile with the
// same instructions, folds the loaded words together so that the stores depend on them, and writes 128 rows of 128
// bytes where the transposed codes would go (and, with q, the 128 rows of 128 bytes of the row-major codes): no
// amax, no scales, no conversion, no LDS, no barrier.  What it reaches is what the access pattern allows on the
// machine; the distance of the real kernel to it is what the arithmetic and the LDS transposition cost.
__global__ __launch_bounds__(256) void transpose_traffic_model_kernel(const uint16_t* __restrict__ x, int64_t ld_src, int k,
                                                                      uint8_t* __restrict__ qt, int64_t ld_t,
                                                                      uint8_t* __restrict__ q, int along_k) {
  const int cg = threadIdx.x & 15, rq = threadIdx.x >> 4;
  const int tr = along_k ? blockIdx.y : blockIdx.x, tc = along_k ? blockIdx.x : blockIdx.y;
  const char* sbase = reinterpret_cast<const char*>(x + (int64_t)tr * 128 * ld_src + tc * 128);
  const uint32_t ld_b = (uint32_t)ld_src * 2u;
  uint4 v[8];
#pragma unroll
  for (int p = 0; p < 8; ++p) v[p] = nt_load16(sbase + ((uint32_t)tile_row(rq, p) * ld_b + (uint32_t)cg * 16u));
  uint4 acc = v[0];
#pragma unroll
  for (int p = 1; p < 8; ++p) {
    acc.x ^= v[p].x; acc.y ^= v[p].y; acc.z ^= v[p].z; acc.w ^= v[p].w;
  }
  char* dst = reinterpret_cast<char*>(qt + (int64_t)tc * 128 * ld_t + tr * 128);
#pragma unroll
  for (int pass = 0; pass < 4; ++pass)
    nt_store16(dst + ((uint32_t)(pass * 32 + (threadIdx.x >> 3)) * (uint32_t)ld_t + (uint32_t)(threadIdx.x & 7) * 16u), acc);
  if (q) {
    char* qbase = reinterpret_cast<char*>(q + (int64_t)tr * 128 * k + tc * 128);
#pragma unroll
    for (int p = 0; p < 8; ++p)
      nt_store8(qbase + ((uint32_t)tile_row(rq, p) * (uint32_t)k + (uint32_t)cg * 8u), make_uint2(acc.x ^ v[p].x, acc.y ^ v[p].y));
  }
}

// ---------------------------------------------------------------------------------------------
// column sums (bias gradient): x[m, k] bf16 -> per 128-row block partial sums fp32 [ceil(m/128), k] -> bf16 / fp32 [k]
// ---------------------------------------------------------------------------------------------
// The same tiles, the same order of additions as the COLSUM form of quant_128x1_t_kernel (rows past m count as +0),
// for the callers that do not run that kernel on grad_out.  k a multiple of 128, any m.
__global__ __launch_bounds__(256) void column_sum_partial_kernel(const uint16_t* __restrict__ x, int64_t ld_src, int m, int k,
                                                                 float* __restrict__ colsum_part) {
  const int cg = threadIdx.x & 15, rq = threadIdx.x >> 4, wave = threadIdx.x >> 6;
  const int tr = blockIdx.x, tc = blockIdx.y;
  __shared__ __attribute__((aligned(16))) float s_cs[4][128];
  const int valid = m - tr * 128;                       // rows of this block that exist (>= 1)
  const char* sbase = reinterpret_cast<const char*>(x + (int64_t)tr * 128 * ld_src + tc * 128);
  const uint32_t ld_b = (uint32_t)ld_src * 2u;
  uint4 v[8];
#pragma unroll
  for (int p = 0; p < 8; ++p)
    v[p] = tile_row(rq, p) < valid ? nt_load16(sbase + ((uint32_t)tile_row(rq, p) * ld_b + (uint32_t)cg * 16u)) : make_uint4(0, 0, 0, 0);
  tile_column_sums(v, cg, wave, s_cs);
  __syncthreads();
  if (threadIdx.x < 128) colsum_part[(int64_t)tr * k + tc * 128 + threadIdx.x] = column_sum_of_tile(s_cs, threadIdx.x);
}

// out[col] = ((0 + part[0][col]) + part[1][col]) + ... in block order, as fp32 and / or rounded once to bf16
__global__ __launch_bounds__(64) void column_sum_finish_kernel(const float* __restrict__ part, int blocks, int k,
                                                               uint16_t* __restrict__ out_bf16, float* __restrict__ out_f32) {
  const int col = blockIdx.x * 64 + threadIdx.x;
  if (col >= k) return;
  float s = 0.f;
  int b = 0;
  for (; b + 16 <= blocks; b += 16) {      // sixteen loads in flight, added in block order (the order is the contract)
    float v[16];
#pragma unroll
    for (int u = 0; u < 16; ++u) v[u] = part[(int64_t)(b + u) * k + col];
#pragma unroll
    for (int u = 0; u < 16; ++u) s += v[u];
  }
  for (; b < blocks; ++b) s += part[(int64_t)b * k + col];
  if (out_f32) out_f32[col] = s;
  if (out_bf16) out_bf16[col] = __builtin_bit_cast(uint16_t, (__bf16)s);
}

// ---------------------------------------------------------------------------------------------
// byte transpose of a code matrix: q[rows, cols] -> qt[cols, rows]
// ---------------------------------------------------------------------------------------------
// 128x128 blocks are symmetric, so the transposed codes of a weight (dgrad operand) can be made
// from its codes alone, e.g. after the codes of all shards were gathered; no requantization.
__global__ __launch_bounds__(256) void transpose_codes_kernel(const uint8_t* __restrict__ q, int rows, int cols,
                                                              int64_t ld, uint8_t* __restrict__ qt, int64_t ld_t, int along_k) {
  const int cg = threadIdx.x & 15, rq = threadIdx.x >> 4;
  __shared__ __attribute__((aligned(16))) uint8_t tile[128 * 128];
  const int br = along_k ? blockIdx.y : blockIdx.x, bc = along_k ? blockIdx.x : blockIdx.y;
  const char* src = reinterpret_cast<const char*>(q + (int64_t)br * 128 * ld + bc * 128);
  uint2 c[8];
#pragma unroll
  for (int p = 0; p < 8; ++p) {
    const u32x2 t = __builtin_nontemporal_load(
        reinterpret_cast<const u32x2*>(src + ((uint32_t)tile_row(rq, p) * (uint32_t)ld + (uint32_t)cg * 8u)));
    c[p] = make_uint2(t.x, t.y);
  }
  store_tile_transposed(tile, c, cg, rq, qt + (int64_t)bc * 128 * ld_t + br * 128, ld_t);
}

// ---------------------------------------------------------------------------------------------
// dequantize 1x128 groups back to bf16 (gradient bucket round trip)
// ---------------------------------------------------------------------------------------------
// out = bf16(decode(q) * scale_inv); if grad_scale != 1 the bf16 value is multiplied by it and
// rounded again, the order of the reference's cast-back site
// (hyper_parallel/core/hsdp/hsdp_grad_buffer.py:121-125).
template <int UNROLL>
__global__ __launch_bounds__(256) void dequant_1x128_kernel(const uint2* __restrict__ q,
                                                            const float* __restrict__ scale_inv,
                                                            uint4* __restrict__ out, int64_t nvec,
                                                            float grad_scale, int apply_grad_scale) {
  // nvec counts 8-code vectors (16 per group).  One thread: 8 codes -> one uint4 of bf16, so both the
  // 64-bit loads and the 128-bit stores of a wave are contiguous.
  const int64_t base = (int64_t)blockIdx.x * (256 * UNROLL) + threadIdx.x;
  uint2 c[UNROLL];
  float si[UNROLL];
#pragma unroll
  for (int u = 0; u < UNROLL; ++u) {
    const int64_t i = base + u * 256;
    const bool ok = i < nvec;
    u32x2 t = ok ? __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(&q[i])) : u32x2{0u, 0u};
    c[u] = make_uint2(t.x, t.y);
    si[u] = ok ? scale_inv[i >> 4] : 0.f;
  }
#pragma unroll
  for (int u = 0; u < UNROLL; ++u) {
    const int64_t i = base + u * 256;
    const uint32_t words[2] = {c[u].x, c[u].y};
    uint32_t o[4];
#pragma unroll
    for (int wd = 0; wd < 2; ++wd) {
      v2f lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)words[wd], false);
      v2f hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)words[wd], true);
      float f[4] = {lo.x * si[u], lo.y * si[u], hi.x * si[u], hi.y * si[u]};
      __bf16 b[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) {
        b[e] = (__bf16)f[e];
        if (apply_grad_scale) b[e] = (__bf16)((float)b[e] * grad_scale);
      }
      o[2 * wd] = (uint32_t)__builtin_bit_cast(uint16_t, b[0]) | ((uint32_t)__builtin_bit_cast(uint16_t, b[1]) << 16);
      o[2 * wd + 1] = (uint32_t)__builtin_bit_cast(uint16_t, b[2]) | ((uint32_t)__builtin_bit_cast(uint16_t, b[3]) << 16);
    }
    if (i < nvec) nt_store16(&out[i], make_uint4(o[0], o[1], o[2], o[3]));
  }
}

// main[i] += (decode(q[i]) * scale_inv) * grad_scale in fp32: a reduced FP8 gradient added onto an
// fp32 main gradient in one pass (the `main_grad += reduced_grad` of
// hyper_parallel/platform/torch/fully_shard/param.py:160-167 for an FP8 reduce dtype).
__global__ __launch_bounds__(256) void dequant_1x128_accumulate_kernel(const uint2* __restrict__ q,
                                                                       const float* __restrict__ scale_inv,
                                                                       float4* __restrict__ main_grad, int64_t nvec,
                                                                       float grad_scale) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i >= nvec) return;
  const u32x2 c = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(&q[i]));
  const float si = scale_inv[i >> 4];
  float4 m0 = main_grad[2 * i], m1 = main_grad[2 * i + 1];
  const v2f a = __builtin_amdgcn_cvt_pk_f32_fp8((int)c.x, false), b = __builtin_amdgcn_cvt_pk_f32_fp8((int)c.x, true);
  const v2f d = __builtin_amdgcn_cvt_pk_f32_fp8((int)c.y, false), e = __builtin_amdgcn_cvt_pk_f32_fp8((int)c.y, true);
  m0.x += (a.x * si) * grad_scale; m0.y += (a.y * si) * grad_scale;
  m0.z += (b.x * si) * grad_scale; m0.w += (b.y * si) * grad_scale;
  m1.x += (d.x * si) * grad_scale; m1.y += (d.y * si) * grad_scale;
  m1.z += (e.x * si) * grad_scale; m1.w += (e.y * si) * grad_scale;
  main_grad[2 * i] = m0;
  main_grad[2 * i + 1] = m1;
}

// codes with one scale per 128x128 block (weights) -> bf16
__global__ __launch_bounds__(256) void dequant_128x128_kernel(const uint8_t* __restrict__ q,
                                                              const float* __restrict__ scale_inv,
                                                              uint16_t* __restrict__ out, int rows, int cols) {
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;   // one 16-code vector
  const int64_t nvec = (int64_t)rows * cols / 16;
  if (i >= nvec) return;
  const int64_t e0 = i * 16;
  const int r = (int)(e0 / cols), c = (int)(e0 % cols);
  const float si = scale_inv[(int64_t)(r >> 7) * (cols >> 7) + (c >> 7)];
  uint4 cd = *reinterpret_cast<const uint4*>(q + e0);
  const uint32_t words[4] = {cd.x, cd.y, cd.z, cd.w};
  uint32_t o[8];
#pragma unroll
  for (int wd = 0; wd < 4; ++wd) {
    v2f lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)words[wd], false);
    v2f hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)words[wd], true);
    __bf16 b0 = (__bf16)(lo.x * si), b1 = (__bf16)(lo.y * si), b2 = (__bf16)(hi.x * si), b3 = (__bf16)(hi.y * si);
    o[2 * wd] = (uint32_t)__builtin_bit_cast(uint16_t, b0) | ((uint32_t)__builtin_bit_cast(uint16_t, b1) << 16);
    o[2 * wd + 1] = (uint32_t)__builtin_bit_cast(uint16_t, b2) | ((uint32_t)__builtin_bit_cast(uint16_t, b3) << 16);
  }
  uint4* ov = reinterpret_cast<uint4*>(out + e0);
  ov[0] = make_uint4(o[0], o[1], o[2], o[3]);
  ov[1] = make_uint4(o[4], o[5], o[6], o[7]);
}

// codes with one scale for the whole tensor -> bf16 or fp32: out[i] = decode(q[i]) * scale_inv[0], one
// multiplication and (bf16) one rounding.  16 codes per thread: one 128-bit load, 2 or 4 128-bit stores.
template <bool OUT_F32>
__global__ __launch_bounds__(256) void dequant_per_tensor_kernel(const uint8_t* __restrict__ q,
                                                                 const float* __restrict__ scale_inv,
                                                                 void* __restrict__ out, int64_t n) {
  const float si = *scale_inv;
  const int64_t nvec = n >> 4;
  const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
  if (i < nvec) {
    const uint4 cd = nt_load16(q + i * 16);
    const uint32_t words[4] = {cd.x, cd.y, cd.z, cd.w};
    float f[16];
#pragma unroll
    for (int wd = 0; wd < 4; ++wd) {
      const v2f lo = __builtin_amdgcn_cvt_pk_f32_fp8((int)words[wd], false);
      const v2f hi = __builtin_amdgcn_cvt_pk_f32_fp8((int)words[wd], true);
      f[4 * wd] = lo.x * si; f[4 * wd + 1] = lo.y * si; f[4 * wd + 2] = hi.x * si; f[4 * wd + 3] = hi.y * si;
    }
    if (OUT_F32) {
      float* o = reinterpret_cast<float*>(out) + i * 16;
#pragma unroll
      for (int k = 0; k < 4; ++k)
        nt_store16(o + 4 * k, make_uint4(__float_as_uint(f[4 * k]), __float_as_uint(f[4 * k + 1]),
                                         __float_as_uint(f[4 * k + 2]), __float_as_uint(f[4 * k + 3])));
    } else {
      uint32_t w[8];
#pragma unroll
      for (int k = 0; k < 8; ++k) {
        const __bf16 b0 = (__bf16)f[2 * k], b1 = (__bf16)f[2 * k + 1];
        w[k] = (uint32_t)__builtin_bit_cast(uint16_t, b0) | ((uint32_t)__builtin_bit_cast(uint16_t, b1) << 16);
      }
      uint16_t* o = reinterpret_cast<uint16_t*>(out) + i * 16;
      nt_store16(o, make_uint4(w[0], w[1], w[2], w[3]));
      nt_store16(o + 8, make_uint4(w[4], w[5], w[6], w[7]));
    }
  }
  if (blockIdx.x == 0 && threadIdx.x < (n & 15)) {       // the last n % 16 codes, one per thread
    const int64_t j = (nvec << 4) + threadIdx.x;
    const uint32_t c = q[j];
    const v2f pair = __builtin_amdgcn_cvt_pk_f32_fp8((int)c, false);
    const float v = pair.x * si;
    if (OUT_F32) reinterpret_cast<float*>(out)[j] = v;
    else reinterpret_cast<uint16_t*>(out)[j] = __builtin_bit_cast(uint16_t, (__bf16)v);
  }
}

}  // namespace hpfp8

using namespace hpfp8;

// ---------------------------------------------------------------------------------------------
// C-ABI
// ---------------------------------------------------------------------------------------------
extern "C" {

int hpfp8_amax_bf16(const void* x, int64_t n, float* amax_out, hpfp8_stream_t stream) {
  HPFP8_REQUIRE(n >= 0, HPFP8_ERR_SHAPE, "amax: negative element count");
  HPFP8_REQUIRE(amax_out != nullptr, HPFP8_ERR_ARG, "amax: null output");
  HPFP8_REQUIRE(n == 0 || (x && aligned16(x)), HPFP8_ERR_ALIGN, "amax: input must be 16-byte aligned");
  hipStream_t s = (hipStream_t)stream;
  fill_u32_kernel<<<1, 64, 0, s>>>(reinterpret_cast<uint32_t*>(amax_out), 0u, 1);
  if (n > 0) {
    int64_t nvec = n >> 3;
    int64_t blocks = (nvec + 256 * 8 - 1) / (256 * 8);
    if (blocks < 1) blocks = 1;
    if (blocks > 2048) blocks = 2048;    // 8 resident workgroups per CU on 256 CUs; the rest is the grid-stride loop
    amax_bf16_kernel<<<(unsigned)blocks, 256, 0, s>>>((const uint16_t*)x, n, reinterpret_cast<uint32_t*>(amax_out));
  }
  return check_launch("amax");
}

int hpfp8_cast_per_tensor_bf16(const void* x, int64_t n, const float* amax, void* q, float* scale,
                               float* scale_inv, hpfp8_stream_t stream) {
  HPFP8_REQUIRE(n >= 0, HPFP8_ERR_SHAPE, "cast_per_tensor: negative element count");
  HPFP8_REQUIRE(amax != nullptr, HPFP8_ERR_ARG, "cast_per_tensor: null amax");
  HPFP8_REQUIRE(n == 0 || (x && q && aligned16(x) && aligned16(q)), HPFP8_ERR_ALIGN,
                "cast_per_tensor: buffers must be non-null and 16-byte aligned");
  int64_t nvec = n >> 3;
  int blocks = (int)((nvec + 256 * 4 - 1) / (256 * 4));
  if (blocks < 1) blocks = 1;
  if (blocks > 16384) blocks = 16384;
  cast_per_tensor_kernel<<<blocks, 256, 0, (hipStream_t)stream>>>((const uint16_t*)x, n, amax, (uint8_t*)q,
                                                                  scale, scale_inv);
  return check_launch("cast_per_tensor");
}

int hpfp8_quantize_per_tensor_bf16(const void* x, int64_t n, void* q, float* amax, float* scale,
                                   float* scale_inv, hpfp8_stream_t stream) {
  if (n > 0 && n <= kFusedMaxElems && amax && scale_inv && x && q && aligned16(x) && aligned16(q))
    return launch_per_tensor_fused(x, n, q, reinterpret_cast<uint32_t*>(amax), scale, scale_inv, (hipStream_t)stream);
  int rc = hpfp8_amax_bf16(x, n, amax, stream);      // (also reports the argument errors)
  if (rc != HPFP8_OK) return rc;
  return hpfp8_cast_per_tensor_bf16(x, n, amax, q, scale, scale_inv, stream);
}

void hpfp8_debug_set_spin_limit(uint32_t polls) { g_spin_limit.store(polls, std::memory_order_relaxed); }

int hpfp8_quantize_per_tensor_sync_bf16(const void* x, int64_t n, void* q, float* amax, float* scale, float* scale_inv,
                                        uint32_t* sync, hpfp8_stream_t stream) {
  const char* what = "quantize_per_tensor_sync";
  HPFP8_REQUIRE(n >= 0, HPFP8_ERR_SHAPE, "%s: negative size", what);
  HPFP8_REQUIRE(n <= kFusedMaxElems, HPFP8_ERR_SHAPE, "%s: at most %lld elements (the one-pass form); larger tensors take "
                "hpfp8_quantize_per_tensor_bf16", what, (long long)kFusedMaxElems);
  if (n == 0) return hpfp8_quantize_per_tensor_bf16(x, n, q, amax, scale, scale_inv, stream);
  HPFP8_REQUIRE(x && q && sync, HPFP8_ERR_ARG, "%s: null buffer", what);
  HPFP8_REQUIRE(aligned16(x) && aligned16(q), HPFP8_ERR_ALIGN, "%s: buffers must be 16-byte aligned", what);
  HPFP8_REQUIRE((reinterpret_cast<uintptr_t>(sync) & 255u) == 0, HPFP8_ERR_ALIGN, "%s: sync must be 256-byte aligned", what);
  const int64_t nvec = (n >> 3) > 0 ? (n >> 3) : 1;
  const int64_t per_thread = (nvec + (int64_t)kFusedMaxBlocks * kFusedThreads - 1) / ((int64_t)kFusedMaxBlocks * kFusedThreads);
  const int vec = per_thread <= 1 ? 1 : (per_thread <= 2 ? 2 : (per_thread <= 4 ? 4 : 8));
  const unsigned grid = (unsigned)((nvec + kFusedThreads * vec - 1) / (kFusedThreads * vec));
  const uint16_t* xs = (const uint16_t*)x;
  uint8_t* q8 = (uint8_t*)q;
  hipStream_t s = (hipStream_t)stream;
  switch (vec) {
    case 1: quant_per_tensor_fused_kernel<1, true><<<grid, kFusedThreads, 0, s>>>(xs, n, sync, sync + 64, q8, scale, g_spin_limit.load(std::memory_order_relaxed), amax, scale_inv); break;
    case 2: quant_per_tensor_fused_kernel<2, true><<<grid, kFusedThreads, 0, s>>>(xs, n, sync, sync + 64, q8, scale, g_spin_limit.load(std::memory_order_relaxed), amax, scale_inv); break;
    case 4: quant_per_tensor_fused_kernel<4, true><<<grid, kFusedThreads, 0, s>>>(xs, n, sync, sync + 64, q8, scale, g_spin_limit.load(std::memory_order_relaxed), amax, scale_inv); break;
    default: quant_per_tensor_fused_kernel<8, true><<<grid, kFusedThreads, 0, s>>>(xs, n, sync, sync + 64, q8, scale, g_spin_limit.load(std::memory_order_relaxed), amax, scale_inv); break;
  }
  return check_launch(what);
}

int hpfp8_quantize_per_tensor_noalloc_bf16(const void* x, int64_t n, void* q, float* scale, float* scale_inv,
                                           hpfp8_stream_t stream) {
  HPFP8_REQUIRE(n >= 0, HPFP8_ERR_SHAPE, "quantize_per_tensor_noalloc: negative element count");
  HPFP8_REQUIRE(n <= kFusedMaxElems, HPFP8_ERR_SHAPE,
                "quantize_per_tensor_noalloc: %lld elements exceed the maximum of %lld this entry point serves; use "
                "hpfp8_quantize_per_tensor_bf16 with an amax word of your own",
                (long long)n, (long long)kFusedMaxElems);
  if (n == 0) return HPFP8_OK;
  HPFP8_REQUIRE(x && q && aligned16(x) && aligned16(q), HPFP8_ERR_ALIGN,
                "quantize_per_tensor_noalloc: buffers must be non-null and 16-byte aligned");
  uint32_t* word = scratch_for_current_device();     // (a pointer asked for once per device; never the array's name)
  if (!word) return HPFP8_ERR_DEVICE;
  // word[0]: the amax word; word[1]: stands in for scale_inv (which doubles as the grid's arrival count) when the
  // caller does not want that output
  return launch_per_tensor_fused(x, n, q, word, scale, scale_inv ? scale_inv : reinterpret_cast<float*>(word + 1),
                                 (hipStream_t)stream);
}

int hpfp8_quantize_1x128_bf16(const void* x, int64_t rows, int64_t cols, void* q, float* scale,
                              float* scale_inv, hpfp8_stream_t stream) {
  HPFP8_REQUIRE(rows >= 0 && cols >= 0, HPFP8_ERR_SHAPE, "quantize_1x128: negative shape");
  HPFP8_REQUIRE(cols % kBlock == 0, HPFP8_ERR_SHAPE, "quantize_1x128: last dim %lld is not a multiple of 128",
                (long long)cols);
  const int64_t nvec = rows * cols / 8;
  if (nvec == 0) return HPFP8_OK;
  HPFP8_REQUIRE(x && q && scale_inv, HPFP8_ERR_ARG, "quantize_1x128: null buffer");
  HPFP8_REQUIRE(aligned16(x) && aligned16(q), HPFP8_ERR_ALIGN, "quantize_1x128: buffers must be 16-byte aligned");
  constexpr int UNROLL = 4;
  const int64_t blocks = (nvec + 256 * UNROLL - 1) / (256 * UNROLL);
  HPFP8_REQUIRE(blocks <= 0x7FFFFFFF, HPFP8_ERR_SHAPE, "quantize_1x128: tensor too large");
  quant_1x128_kernel<UNROLL><<<(unsigned)blocks, 256, 0, (hipStream_t)stream>>>(
      (const uint4*)x, (uint2*)q, scale, scale_inv, nvec);
  return check_launch("quantize_1x128");
}

static int quantize_1x128_kmajor_impl(const void* x, int64_t rows, int64_t cols, void* q, float* scale,
                                      float* scale_inv, int pow2, hpfp8_stream_t stream) {
  HPFP8_REQUIRE(rows >= 0 && cols >= 0, HPFP8_ERR_SHAPE, "quantize_1x128_kmajor: negative shape");
  HPFP8_REQUIRE(cols % kBlock == 0, HPFP8_ERR_SHAPE,
                "quantize_1x128_kmajor: last dim %lld is not a multiple of 128", (long long)cols);
  HPFP8_REQUIRE(rows < (1 << 30) && cols < (1 << 30), HPFP8_ERR_SHAPE, "quantize_1x128_kmajor: dimension too large");
  if (rows == 0 || cols == 0) return HPFP8_OK;
  HPFP8_REQUIRE(x && q && scale_inv, HPFP8_ERR_ARG, "quantize_1x128_kmajor: null buffer");
  HPFP8_REQUIRE(aligned16(x) && aligned16(q), HPFP8_ERR_ALIGN,
                "quantize_1x128_kmajor: buffers must be 16-byte aligned");
  const int64_t groups = cols / kBlock;
  const int64_t blocks = ((groups + 3) / 4) * ((rows + 15) / 16);
  HPFP8_REQUIRE(blocks <= 0x7FFFFFFF, HPFP8_ERR_SHAPE, "quantize_1x128_kmajor: tensor too large");
  quant_1x128_kmajor_kernel<<<(unsigned)blocks, 256, 0, (hipStream_t)stream>>>(
      (const uint16_t*)x, (uint8_t*)q, scale, scale_inv, (int)rows, (int)cols, pow2);
  return check_launch("quantize_1x128_kmajor");
}

int hpfp8_quantize_1x128_kmajor_bf16(const void* x, int64_t rows, int64_t cols, void* q, float* scale,
                                     float* scale_inv, hpfp8_stream_t stream) {
  return quantize_1x128_kmajor_impl(x, rows, cols, q, scale, scale_inv, 0, stream);
}

int hpfp8_quantize_1x128_kmajor_pow2_bf16(const void* x, int64_t rows, int64_t cols, void* q, float* scale,
                                          float* scale_inv, hpfp8_stream_t stream) {
  return quantize_1x128_kmajor_impl(x, rows, cols, q, scale, scale_inv, 1, stream);
}

// Grid of the transposing tile kernels: x is the fast index.  along_k = 1 makes consecutive workgroups walk along a
// tile row of the source, 0 down a tile column (which keeps the 128-byte pieces of one transposed row together).
// Measured on MI355X with buffers rotating beyond the Infinity Cache: down a tile column is the faster order unless
// the source's row stride puts a tile column's 128 rows on few memory channels -- a stride that is a multiple of
// 16 KB for a kernel with one output stream, of 4 KB for one that also writes the row-major codes (`streams` = 2:
// x[4096, 16384] both forms 56.6 -> 62.1 % of 8 TB/s, x[4096, 8192] transposed form 53.3 -> 60.3 %, while
// x[16384, 7168], stride 14 KB, loses 7 points the other way round).  streams = 0 never walks along k (the byte
// transpose, measured faster down the column at every stride).  A grid's y extent is limited to 65535, so a matrix
// with more tiles than that in one direction keeps that direction in x.
static dim3 transpose_grid(int64_t mb, int64_t kb, int64_t ld_src_bytes, int streams, int& along_k) {
  along_k = streams == 0 ? 0 : (ld_src_bytes % (streams >= 2 ? 4096 : 16384) == 0 ? 1 : 0);
  if (along_k && mb > 65535) along_k = 0;
  if (!along_k && kb > 65535) along_k = 1;
  return along_k ? dim3((unsigned)kb, (unsigned)mb) : dim3((unsigned)mb, (unsigned)kb);
}

static int quantize_128x128_impl(const void* w, int64_t rows, int64_t cols, void* q, void* q_t, int64_t ld_t,
                                 float* scale, float* scale_inv, int pow2, hpfp8_stream_t stream) {
  HPFP8_REQUIRE(rows >= 0 && cols >= 0, HPFP8_ERR_SHAPE, "quantize_128x128: negative shape");
  HPFP8_REQUIRE(rows % kBlock == 0 && cols % kBlock == 0, HPFP8_ERR_SHAPE,
                "quantize_128x128: shape [%lld, %lld] is not a multiple of 128", (long long)rows, (long long)cols);
  HPFP8_REQUIRE(rows < (1 << 30) && cols < (1 << 30), HPFP8_ERR_SHAPE, "quantize_128x128: dimension too large");
  const int64_t blocks = (rows / kBlock) * (cols / kBlock);
  if (blocks == 0) return HPFP8_OK;
  HPFP8_REQUIRE(blocks <= 0x7FFFFFFF, HPFP8_ERR_SHAPE, "quantize_128x128: tensor too large");
  HPFP8_REQUIRE(w && q && scale_inv, HPFP8_ERR_ARG, "quantize_128x128: null buffer");
  HPFP8_REQUIRE(aligned16(w) && aligned16(q) && (!q_t || aligned16(q_t)), HPFP8_ERR_ALIGN,
                "quantize_128x128: buffers must be 16-byte aligned");
  HPFP8_REQUIRE(cols < (1 << 24) && (!q_t || ld_t < (1 << 24)), HPFP8_ERR_SHAPE,
                "quantize_128x128: cols and ld_t must be below 2^24");
  HPFP8_REQUIRE(!q_t || (ld_t >= rows && ld_t % 16 == 0), HPFP8_ERR_SHAPE,
                "quantize_128x128: ld_t=%lld must be a multiple of 16 and at least rows", (long long)ld_t);
  hipStream_t s = (hipStream_t)stream;
  int ak = 1;
  if (q_t) {
    const dim3 grid = transpose_grid(rows / kBlock, cols / kBlock, cols * 2, 2, ak);
    quant_128x128_kernel<true><<<grid, 256, 0, s>>>((const uint16_t*)w, (int)rows, (int)cols, (uint8_t*)q, (uint8_t*)q_t, ld_t,
                                                    scale, scale_inv, pow2, ak);
  } else if ((cols / kBlock) % 2 == 0 && rows / kBlock <= 65535 && blocks >= 4096) {
    quant_128x128_pair_kernel<<<dim3((unsigned)(cols / kBlock / 2), (unsigned)(rows / kBlock)), 256, 0, s>>>(
        (const uint16_t*)w, (int)cols, (uint8_t*)q, scale, scale_inv, pow2);
  } else {
    // no transposed copy: always along the source rows (a plain streaming order)
    const bool x_is_cols = cols / kBlock <= 65535 || rows / kBlock > 65535;
    ak = x_is_cols ? 1 : 0;
    const dim3 grid = ak ? dim3((unsigned)(cols / kBlock), (unsigned)(rows / kBlock)) : dim3((unsigned)(rows / kBlock), (unsigned)(cols / kBlock));
    quant_128x128_kernel<false><<<grid, 256, 0, s>>>((const uint16_t*)w, (int)rows, (int)cols, (uint8_t*)q, nullptr, 0, scale,
                                                     scale_inv, pow2, ak);
  }
  return check_launch("quantize_128x128");
}

int hpfp8_quantize_128x128_bf16(const void* w, int64_t rows, int64_t cols, void* q, void* q_t, int64_t ld_t,
                                float* scale, float* scale_inv, hpfp8_stream_t stream) {
  return quantize_128x128_impl(w, rows, cols, q, q_t, ld_t, scale, scale_inv, 0, stream);
}

int hpfp8_quantize_128x128_pow2_bf16(const void* w, int64_t rows, int64_t cols, void* q, void* q_t, int64_t ld_t,
                                     float* scale, float* scale_inv, hpfp8_stream_t stream) {
  return quantize_128x128_impl(w, rows, cols, q, q_t, ld_t, scale, scale_inv, 1, stream);
}

// q != nullptr: also the 1x128 quantization of x itself (codes q, scales scale / scale_inv).
static int quantize_128x1_t_impl(const char* what, bool kmajor, const void* x, int64_t m, int64_t k, void* q_t,
                                 int64_t ld_t, float* scale_t, float* scale_inv_t, hpfp8_stream_t stream,
                                 void* q = nullptr, float* scale = nullptr, float* scale_inv = nullptr, int pow2 = 0,
                                 float* colsum_part = nullptr) {
  HPFP8_REQUIRE(m >= 0 && k >= 0, HPFP8_ERR_SHAPE, "%s: negative shape", what);
  HPFP8_REQUIRE(m % kBlock == 0 && k % kBlock == 0, HPFP8_ERR_SHAPE,
                "%s: shape [%lld, %lld] is not a multiple of 128", what, (long long)m, (long long)k);
  HPFP8_REQUIRE(m < (1 << 30) && k < (1 << 24) && ld_t < (1 << 24), HPFP8_ERR_SHAPE,
                "%s: dimension too large (at most 2^30 rows, and columns and ld_t below 2^24)", what);
  const int64_t blocks = (m / kBlock) * (k / kBlock);
  if (blocks == 0) return HPFP8_OK;
  HPFP8_REQUIRE(blocks <= 0x7FFFFFFF, HPFP8_ERR_SHAPE, "%s: tensor too large", what);
  HPFP8_REQUIRE(x && q_t && scale_inv_t, HPFP8_ERR_ARG, "%s: null buffer", what);
  HPFP8_REQUIRE(aligned16(x) && aligned16(q_t), HPFP8_ERR_ALIGN, "%s: buffers must be 16-byte aligned", what);
  HPFP8_REQUIRE(ld_t >= m && ld_t % 16 == 0, HPFP8_ERR_SHAPE, "%s: ld_t=%lld must be a multiple of 16 and at least m",
                what, (long long)ld_t);
  HPFP8_REQUIRE(!q || (scale_inv && aligned16(q)), HPFP8_ERR_ARG, "%s: q needs scale_inv and 16-byte alignment", what);
  hipStream_t s = (hipStream_t)stream;
  int ak = 0;
  const dim3 grid = transpose_grid(m / kBlock, k / kBlock, k * 2, q ? 2 : 1, ak);
  const uint16_t* xs = (const uint16_t*)x;
  uint8_t* qt8 = (uint8_t*)q_t;
  uint8_t* q8 = (uint8_t*)q;
  if (colsum_part) {
    HPFP8_REQUIRE(kmajor, HPFP8_ERR_ARG, "%s: the column sums come with the k-block-major scale layout only", what);
    if (q)
      quant_128x1_t_kernel<true, true, 0, false, true><<<grid, 256, 0, s>>>(xs, k, (int)m, (int)k, qt8, ld_t, scale_t, scale_inv_t, q8,
                                                                            scale, scale_inv, pow2, ak, nullptr, 0, 0, nullptr, colsum_part);
    else
      quant_128x1_t_kernel<true, false, 0, false, true><<<grid, 256, 0, s>>>(xs, k, (int)m, (int)k, qt8, ld_t, scale_t, scale_inv_t, nullptr,
                                                                             nullptr, nullptr, pow2, ak, nullptr, 0, 0, nullptr, colsum_part);
  } else if (q) {
    if (kmajor)
      quant_128x1_t_kernel<true, true><<<grid, 256, 0, s>>>(xs, k, (int)m, (int)k, qt8, ld_t, scale_t, scale_inv_t, q8, scale, scale_inv, pow2, ak);
    else
      quant_128x1_t_kernel<false, true><<<grid, 256, 0, s>>>(xs, k, (int)m, (int)k, qt8, ld_t, scale_t, scale_inv_t, q8, scale, scale_inv, pow2, ak);
  } else {
    if (kmajor)
      quant_128x1_t_kernel<true, false><<<grid, 256, 0, s>>>(xs, k, (int)m, (int)k, qt8, ld_t, scale_t, scale_inv_t, nullptr, nullptr, nullptr, pow2, ak);
    else
      quant_128x1_t_kernel<false, false><<<grid, 256, 0, s>>>(xs, k, (int)m, (int)k, qt8, ld_t, scale_t, scale_inv_t, nullptr, nullptr, nullptr, pow2, ak);
  }
  return check_launch(what);
}

int hpfp8_swiglu_quantize_1x128_and_128x1_t_bf16(const void* h, int64_t rows, int64_t inter, int64_t ld_h, int fast,
                                                 void* q, float* scale, float* scale_inv, void* q_t, int64_t ld_t,
                                                 float* scale_t, float* scale_inv_t, hpfp8_stream_t stream) {
  const char* what = "swiglu_quantize_1x128_and_128x1_t";
  HPFP8_REQUIRE(rows >= 0 && inter >= 0, HPFP8_ERR_SHAPE, "%s: negative shape", what);
  HPFP8_REQUIRE(rows % kBlock == 0 && inter % kBlock == 0, HPFP8_ERR_SHAPE,
                "%s: shape [%lld, %lld] is not a multiple of 128", what, (long long)rows, (long long)inter);
  HPFP8_REQUIRE(rows < (1 << 30) && inter < (1 << 24) && ld_h < (1 << 24) && ld_t < (1 << 24), HPFP8_ERR_SHAPE,
                "%s: dimension too large (at most 2^30 rows; width and row strides below 2^24)", what);
  const int64_t blocks = (rows / kBlock) * (inter / kBlock);
  if (blocks == 0) return HPFP8_OK;
  HPFP8_REQUIRE(blocks <= 0x7FFFFFFF, HPFP8_ERR_SHAPE, "%s: tensor too large", what);
  HPFP8_REQUIRE(h && q && scale_inv && q_t && scale_inv_t, HPFP8_ERR_ARG, "%s: null buffer", what);
  HPFP8_REQUIRE(aligned16(h) && aligned16(q) && aligned16(q_t), HPFP8_ERR_ALIGN, "%s: buffers must be 16-byte aligned", what);
  HPFP8_REQUIRE(ld_h >= 2 * inter && ld_h % 8 == 0, HPFP8_ERR_SHAPE,
                "%s: ld_h=%lld must be a multiple of 8 and at least twice the width", what, (long long)ld_h);
  HPFP8_REQUIRE(ld_t >= rows && ld_t % 16 == 0, HPFP8_ERR_SHAPE, "%s: ld_t=%lld must be a multiple of 16 and at least rows",
                what, (long long)ld_t);
  hipStream_t s = (hipStream_t)stream;
  int ak = 0;
  const dim3 grid = transpose_grid(rows / kBlock, inter / kBlock, ld_h * 2, 2, ak);
  if (fast)
    quant_128x1_t_kernel<true, true, 2><<<grid, 256, 0, s>>>((const uint16_t*)h, ld_h, (int)rows, (int)inter, (uint8_t*)q_t, ld_t,
                                                            scale_t, scale_inv_t, (uint8_t*)q, scale, scale_inv, 0, ak);
  else
    quant_128x1_t_kernel<true, true, 1><<<grid, 256, 0, s>>>((const uint16_t*)h, ld_h, (int)rows, (int)inter, (uint8_t*)q_t, ld_t,
                                                            scale_t, scale_inv_t, (uint8_t*)q, scale, scale_inv, 0, ak);
  return check_launch(what);
}

int hpfp8_swiglu_backward_quantize_1x128_and_128x1_t_bf16(const void* h, int64_t rows, int64_t inter, int64_t ld_h,
                                                          const void* dact, void* q, float* scale, float* scale_inv,
                                                          void* q_t, int64_t ld_t, float* scale_t, float* scale_inv_t,
                                                          hpfp8_stream_t stream) {
  const char* what = "swiglu_backward_quantize_1x128_and_128x1_t";
  HPFP8_REQUIRE(rows >= 0 && inter >= 0, HPFP8_ERR_SHAPE, "%s: negative shape", what);
  HPFP8_REQUIRE(rows % kBlock == 0 && inter % kBlock == 0, HPFP8_ERR_SHAPE,
                "%s: shape [%lld, %lld] is not a multiple of 128", what, (long long)rows, (long long)inter);
  HPFP8_REQUIRE(rows < (1 << 30) && inter < (1 << 23) && ld_h < (1 << 24) && ld_t < (1 << 24), HPFP8_ERR_SHAPE,
                "%s: dimension too large (at most 2^30 rows; width and row strides below 2^24)", what);
  const int64_t blocks = (rows / kBlock) * (2 * inter / kBlock);
  if (blocks == 0) return HPFP8_OK;
  HPFP8_REQUIRE(blocks <= 0x7FFFFFFF, HPFP8_ERR_SHAPE, "%s: tensor too large", what);
  HPFP8_REQUIRE(h && dact && q && scale_inv && q_t && scale_inv_t, HPFP8_ERR_ARG, "%s: null buffer", what);
  HPFP8_REQUIRE(aligned16(h) && aligned16(dact) && aligned16(q) && aligned16(q_t), HPFP8_ERR_ALIGN,
                "%s: buffers must be 16-byte aligned", what);
  HPFP8_REQUIRE(ld_h >= 2 * inter && ld_h % 8 == 0, HPFP8_ERR_SHAPE,
                "%s: ld_h=%lld must be a multiple of 8 and at least twice the width", what, (long long)ld_h);
  HPFP8_REQUIRE(ld_t >= rows && ld_t % 16 == 0, HPFP8_ERR_SHAPE, "%s: ld_t=%lld must be a multiple of 16 and at least rows",
                what, (long long)ld_t);
  int ak = 0;
  const dim3 grid = transpose_grid(rows / kBlock, 2 * inter / kBlock, ld_h * 2, 2, ak);
  quant_128x1_t_kernel<true, true, 3><<<grid, 256, 0, (hipStream_t)stream>>>(
      (const uint16_t*)h, ld_h, (int)rows, (int)(2 * inter), (uint8_t*)q_t, ld_t, scale_t, scale_inv_t, (uint8_t*)q, scale,
      scale_inv, 0, ak, nullptr, 0, 0, (const uint16_t*)dact);
  return check_launch(what);
}

int hpfp8_quantize_128x1_t_grouped_bf16(const void* x, int64_t total_m, int64_t k, const int32_t* layout, int experts,
                                        void* q_t, int64_t ld_t, float* scale_inv_t, void* q, float* scale_inv,
                                        hpfp8_stream_t stream) {
  const char* what = "quantize_128x1_t_grouped";
  HPFP8_REQUIRE(total_m >= 0 && k >= 0, HPFP8_ERR_SHAPE, "%s: negative shape", what);
  HPFP8_REQUIRE(k % kBlock == 0, HPFP8_ERR_SHAPE, "%s: width %lld is not a multiple of 128", what, (long long)k);
  HPFP8_REQUIRE(experts >= 0 && experts <= 4096, HPFP8_ERR_SHAPE, "%s: bad expert count %d", what, experts);
  HPFP8_REQUIRE(total_m < (1 << 30) && k < (1 << 24) && ld_t < (1 << 24), HPFP8_ERR_SHAPE,
                "%s: dimension too large (at most 2^30 rows; width and ld_t below 2^24)", what);
  const int64_t padded_blocks = total_m / kBlock + experts;
  const int64_t blocks = padded_blocks * (k / kBlock);
  if (blocks == 0) return HPFP8_OK;
  HPFP8_REQUIRE(blocks <= 0x7FFFFFFF, HPFP8_ERR_SHAPE, "%s: tensor too large", what);
  HPFP8_REQUIRE((x || total_m == 0) && layout && q_t && scale_inv_t, HPFP8_ERR_ARG, "%s: null buffer", what);
  HPFP8_REQUIRE(aligned16(x) && aligned16(q_t), HPFP8_ERR_ALIGN, "%s: buffers must be 16-byte aligned", what);
  HPFP8_REQUIRE(ld_t >= padded_blocks * kBlock && ld_t % 16 == 0, HPFP8_ERR_SHAPE,
                "%s: ld_t=%lld must be a multiple of 16 and at least the padded row count %lld", what, (long long)ld_t,
                (long long)(padded_blocks * kBlock));
  HPFP8_REQUIRE(!q || (scale_inv && aligned16(q)), HPFP8_ERR_ARG, "%s: q needs scale_inv and 16-byte alignment", what);
  hipStream_t s = (hipStream_t)stream;
  int ak = 0;
  const dim3 grid = transpose_grid(padded_blocks, k / kBlock, k * 2, q ? 2 : 1, ak);
  if (q)
    quant_128x1_t_kernel<true, true, 0, true><<<grid, 256, 0, s>>>(
        (const uint16_t*)x, k, (int)total_m, (int)k, (uint8_t*)q_t, ld_t, nullptr, scale_inv_t, (uint8_t*)q, nullptr, scale_inv, 0,
        ak, layout, experts, (int)padded_blocks);
  else
    quant_128x1_t_kernel<true, false, 0, true><<<grid, 256, 0, s>>>(
        (const uint16_t*)x, k, (int)total_m, (int)k, (uint8_t*)q_t, ld_t, nullptr, scale_inv_t, nullptr, nullptr, nullptr, 0,
        ak, layout, experts, (int)padded_blocks);
  return check_launch(what);
}

int hpfp8_quantize_128x1_t_bf16(const void* x, int64_t m, int64_t k, void* q_t, int64_t ld_t, float* scale_t,
                                float* scale_inv_t, hpfp8_stream_t stream) {
  return quantize_128x1_t_impl("quantize_128x1_t", false, x, m, k, q_t, ld_t, scale_t, scale_inv_t, stream);
}

int hpfp8_quantize_128x1_t_kmajor_bf16(const void* x, int64_t m, int64_t k, void* q_t, int64_t ld_t,
                                       float* scale_t, float* scale_inv_t, hpfp8_stream_t stream) {
  return quantize_128x1_t_impl("quantize_128x1_t_kmajor", true, x, m, k, q_t, ld_t, scale_t, scale_inv_t, stream);
}

int hpfp8_quantize_1x128_and_128x1_t_bf16(const void* x, int64_t m, int64_t k, int kmajor, void* q, float* scale,
                                          float* scale_inv, void* q_t, int64_t ld_t, float* scale_t,
                                          float* scale_inv_t, hpfp8_stream_t stream) {
  HPFP8_REQUIRE(m == 0 || k == 0 || q != nullptr, HPFP8_ERR_ARG, "quantize_1x128_and_128x1_t: null buffer");
  return quantize_128x1_t_impl("quantize_1x128_and_128x1_t", kmajor != 0, x, m, k, q_t, ld_t, scale_t, scale_inv_t,
                               stream, q, scale, scale_inv);
}

int hpfp8_debug_transpose_traffic_model(const void* x, int64_t m, int64_t k, void* q_t, int64_t ld_t, void* q,
                                        hpfp8_stream_t stream) {
  const char* what = "debug_transpose_traffic_model";
  HPFP8_REQUIRE(m > 0 && k > 0 && m % kBlock == 0 && k % kBlock == 0, HPFP8_ERR_SHAPE, "%s: shape must be positive multiples of 128", what);
  HPFP8_REQUIRE(m < (1 << 30) && k < (1 << 24) && ld_t < (1 << 24) && ld_t >= m && ld_t % 16 == 0, HPFP8_ERR_SHAPE, "%s: bad shape", what);
  HPFP8_REQUIRE(x && q_t && aligned16(x) && aligned16(q_t) && (!q || aligned16(q)), HPFP8_ERR_ARG, "%s: bad buffer", what);
  int ak = 0;
  const dim3 grid = transpose_grid(m / kBlock, k / kBlock, k * 2, q ? 2 : 1, ak);
  transpose_traffic_model_kernel<<<grid, 256, 0, (hipStream_t)stream>>>((const uint16_t*)x, k, (int)k, (uint8_t*)q_t, ld_t,
                                                                       (uint8_t*)q, ak);
  return check_launch(what);
}

int hpfp8_quantize_128x1_t_colsum_bf16(const void* x, int64_t m, int64_t k, void* q, float* scale, float* scale_inv, void* q_t,
                                       int64_t ld_t, float* scale_t, float* scale_inv_t, int pow2, float* colsum_partial,
                                       hpfp8_stream_t stream) {
  HPFP8_REQUIRE(m == 0 || k == 0 || colsum_partial != nullptr, HPFP8_ERR_ARG, "quantize_128x1_t_colsum: null buffer");
  return quantize_128x1_t_impl("quantize_128x1_t_colsum", true, x, m, k, q_t, ld_t, scale_t, scale_inv_t, stream, q, scale,
                               scale_inv, pow2 ? 1 : 0, colsum_partial);
}

int hpfp8_column_sum_finish(const float* partial, int64_t blocks, int64_t cols, void* out_bf16, float* out_f32,
                            hpfp8_stream_t stream) {
  HPFP8_REQUIRE(blocks >= 0 && cols >= 0 && blocks < (1 << 30) && cols < (1 << 30), HPFP8_ERR_SHAPE, "column_sum_finish: bad shape");
  if (cols == 0) return HPFP8_OK;
  HPFP8_REQUIRE((partial || blocks == 0) && (out_bf16 || out_f32), HPFP8_ERR_ARG, "column_sum_finish: null buffer");
  column_sum_finish_kernel<<<(unsigned)((cols + 63) / 64), 64, 0, (hipStream_t)stream>>>(partial, (int)blocks, (int)cols,
                                                                                          (uint16_t*)out_bf16, out_f32);
  return check_launch("column_sum_finish");
}

int hpfp8_column_sum_bf16(const void* x, int64_t m, int64_t k, int64_t ld, float* partial, void* out_bf16, float* out_f32,
                          hpfp8_stream_t stream) {
  HPFP8_REQUIRE(m >= 0 && k >= 0, HPFP8_ERR_SHAPE, "column_sum: negative shape");
  HPFP8_REQUIRE(k % kBlock == 0, HPFP8_ERR_SHAPE, "column_sum: width %lld is not a multiple of 128", (long long)k);
  HPFP8_REQUIRE(m < (1 << 30) && k < (1 << 23) && ld < (1 << 24), HPFP8_ERR_SHAPE, "column_sum: dimension too large");
  if (k == 0) return HPFP8_OK;
  const int64_t blocks = (m + kBlock - 1) / kBlock;
  HPFP8_REQUIRE(out_bf16 || out_f32, HPFP8_ERR_ARG, "column_sum: null output");
  if (blocks > 0) {
    HPFP8_REQUIRE(x && partial, HPFP8_ERR_ARG, "column_sum: null buffer");
    HPFP8_REQUIRE(aligned16(x) && ld >= k && ld % 8 == 0, HPFP8_ERR_ALIGN,
                  "column_sum: x must be 16-byte aligned with a row stride that is a multiple of 8 and at least k");
    HPFP8_REQUIRE(k / kBlock <= 65535, HPFP8_ERR_SHAPE, "column_sum: width too large");
    column_sum_partial_kernel<<<dim3((unsigned)blocks, (unsigned)(k / kBlock)), 256, 0, (hipStream_t)stream>>>(
        (const uint16_t*)x, ld, (int)m, (int)k, partial);
    const int rc = check_launch("column_sum");
    if (rc != HPFP8_OK) return rc;
  }
  return hpfp8_column_sum_finish(partial, blocks, k, out_bf16, out_f32, stream);
}

int hpfp8_quantize_128x1_t_kmajor_pow2_bf16(const void* x, int64_t m, int64_t k, void* q_t, int64_t ld_t,
                                            float* scale_t, float* scale_inv_t, hpfp8_stream_t stream) {
  return quantize_128x1_t_impl("quantize_128x1_t_kmajor_pow2", true, x, m, k, q_t, ld_t, scale_t, scale_inv_t, stream,
                               nullptr, nullptr, nullptr, 1);
}

int hpfp8_quantize_1x128_and_128x1_t_pow2_bf16(const void* x, int64_t m, int64_t k, int kmajor, void* q, float* scale,
                                               float* scale_inv, void* q_t, int64_t ld_t, float* scale_t,
                                               float* scale_inv_t, hpfp8_stream_t stream) {
  HPFP8_REQUIRE(m == 0 || k == 0 || q != nullptr, HPFP8_ERR_ARG, "quantize_1x128_and_128x1_t_pow2: null buffer");
  return quantize_128x1_t_impl("quantize_1x128_and_128x1_t_pow2", kmajor != 0, x, m, k, q_t, ld_t, scale_t, scale_inv_t,
                               stream, q, scale, scale_inv, 1);
}

static int swiglu_quantize_impl(const void* h, int64_t rows, int64_t inter, int64_t ld_h, int kmajor, void* q,
                                float* scale, float* scale_inv, void* act, int pow2, int fast, hpfp8_stream_t stream) {
  HPFP8_REQUIRE(rows >= 0 && inter >= 0, HPFP8_ERR_SHAPE, "swiglu_quantize_1x128: negative shape");
  HPFP8_REQUIRE(inter % kBlock == 0, HPFP8_ERR_SHAPE, "swiglu_quantize_1x128: width %lld is not a multiple of 128",
                (long long)inter);
  HPFP8_REQUIRE(rows < (1 << 30) && inter < (1 << 30), HPFP8_ERR_SHAPE, "swiglu_quantize_1x128: dimension too large");
  if (rows == 0 || inter == 0) return HPFP8_OK;
  HPFP8_REQUIRE(ld_h >= 2 * inter && ld_h % 8 == 0, HPFP8_ERR_SHAPE,
                "swiglu_quantize_1x128: ld_h=%lld must be a multiple of 8 and at least twice the width", (long long)ld_h);
  HPFP8_REQUIRE(h && q && scale_inv, HPFP8_ERR_ARG, "swiglu_quantize_1x128: null buffer");
  HPFP8_REQUIRE(aligned16(h) && aligned16(q) && (!act || aligned16(act)), HPFP8_ERR_ALIGN,
                "swiglu_quantize_1x128: buffers must be 16-byte aligned");
  const int64_t groups = inter / kBlock;
  const int64_t blocks = ((groups + 3) / 4) * ((rows + 15) / 16);
  HPFP8_REQUIRE(blocks <= 0x7FFFFFFF, HPFP8_ERR_SHAPE, "swiglu_quantize_1x128: tensor too large");
  hipStream_t s = (hipStream_t)stream;
  auto launch = [&](auto kernel) {
    kernel<<<(unsigned)blocks, 256, 0, s>>>((const uint16_t*)h, ld_h, (uint8_t*)q, scale, scale_inv, (uint16_t*)act,
                                            (int)rows, (int)inter, pow2);
  };
  if (kmajor && fast) launch(swiglu_quant_1x128_kernel<true, true>);
  else if (kmajor) launch(swiglu_quant_1x128_kernel<true, false>);
  else if (fast) launch(swiglu_quant_1x128_kernel<false, true>);
  else launch(swiglu_quant_1x128_kernel<false, false>);
  return check_launch("swiglu_quantize_1x128");
}

int hpfp8_swiglu_quantize_1x128_bf16(const void* h, int64_t rows, int64_t inter, int64_t ld_h, int kmajor, void* q,
                                     float* scale, float* scale_inv, void* act, hpfp8_stream_t stream) {
  return swiglu_quantize_impl(h, rows, inter, ld_h, kmajor, q, scale, scale_inv, act, 0, 0, stream);
}

int hpfp8_swiglu_quantize_1x128_pow2_bf16(const void* h, int64_t rows, int64_t inter, int64_t ld_h, int kmajor, void* q,
                                          float* scale, float* scale_inv, void* act, hpfp8_stream_t stream) {
  return swiglu_quantize_impl(h, rows, inter, ld_h, kmajor, q, scale, scale_inv, act, 1, 0, stream);
}

int hpfp8_swiglu_quantize_1x128_fast_bf16(const void* h, int64_t rows, int64_t inter, int64_t ld_h, int kmajor, int pow2,
                                          void* q, float* scale, float* scale_inv, void* act, hpfp8_stream_t stream) {
  HPFP8_REQUIRE(pow2 == 0 || pow2 == 1, HPFP8_ERR_ARG, "swiglu_quantize_1x128_fast: pow2 must be 0 or 1");
  return swiglu_quantize_impl(h, rows, inter, ld_h, kmajor, q, scale, scale_inv, act, pow2, 1, stream);
}

int hpfp8_swiglu_backward_bf16(const void* h, int64_t rows, int64_t inter, int64_t ld_h, const void* dact, void* dh,
                               int64_t ld_dh, hpfp8_stream_t stream) {
  HPFP8_REQUIRE(rows >= 0 && inter >= 0, HPFP8_ERR_SHAPE, "swiglu_backward: negative shape");
  HPFP8_REQUIRE(inter % 8 == 0, HPFP8_ERR_SHAPE, "swiglu_backward: width %lld is not a multiple of 8", (long long)inter);
  HPFP8_REQUIRE(rows < (1 << 30) && inter < (1 << 30), HPFP8_ERR_SHAPE, "swiglu_backward: dimension too large");
  if (rows == 0 || inter == 0) return HPFP8_OK;
  HPFP8_REQUIRE(ld_h >= 2 * inter && ld_h % 8 == 0 && ld_dh >= 2 * inter && ld_dh % 8 == 0, HPFP8_ERR_SHAPE,
                "swiglu_backward: ld_h=%lld and ld_dh=%lld must be multiples of 8 and at least twice the width",
                (long long)ld_h, (long long)ld_dh);
  HPFP8_REQUIRE(h && dact && dh, HPFP8_ERR_ARG, "swiglu_backward: null buffer");
  HPFP8_REQUIRE(aligned16(h) && aligned16(dact) && aligned16(dh), HPFP8_ERR_ALIGN,
                "swiglu_backward: buffers must be 16-byte aligned");
  const int64_t nvec = rows * (inter / 8);
  const int64_t blocks = (nvec + 511) / 512;
  HPFP8_REQUIRE(blocks <= 0x7FFFFFFF, HPFP8_ERR_SHAPE, "swiglu_backward: tensor too large");
  swiglu_backward_kernel<<<(unsigned)blocks, 256, 0, (hipStream_t)stream>>>((const uint16_t*)h, ld_h, (const uint16_t*)dact,
                                                                           (uint16_t*)dh, ld_dh, nvec, (int)inter);
  return check_launch("swiglu_backward");
}

int hpfp8_transpose_codes(const void* q, int64_t rows, int64_t cols, int64_t ld, void* q_t, int64_t ld_t,
                          hpfp8_stream_t stream) {
  HPFP8_REQUIRE(rows >= 0 && cols >= 0, HPFP8_ERR_SHAPE, "transpose_codes: negative shape");
  HPFP8_REQUIRE(rows % kBlock == 0 && cols % kBlock == 0, HPFP8_ERR_SHAPE,
                "transpose_codes: shape [%lld, %lld] is not a multiple of 128", (long long)rows, (long long)cols);
  HPFP8_REQUIRE(rows < (1 << 30) && cols < (1 << 30), HPFP8_ERR_SHAPE, "transpose_codes: dimension too large");
  const int64_t blocks = (rows / kBlock) * (cols / kBlock);
  if (blocks == 0) return HPFP8_OK;
  HPFP8_REQUIRE(blocks <= 0x7FFFFFFF, HPFP8_ERR_SHAPE, "transpose_codes: tensor too large");
  HPFP8_REQUIRE(q && q_t, HPFP8_ERR_ARG, "transpose_codes: null buffer");
  HPFP8_REQUIRE(aligned16(q) && aligned16(q_t), HPFP8_ERR_ALIGN, "transpose_codes: buffers must be 16-byte aligned");
  HPFP8_REQUIRE(ld_t < (1 << 24) && ld < (1 << 24), HPFP8_ERR_SHAPE, "transpose_codes: ld and ld_t must be below 2^24");
  HPFP8_REQUIRE(ld >= cols && ld % 16 == 0 && ld_t >= rows && ld_t % 16 == 0, HPFP8_ERR_SHAPE,
                "transpose_codes: ld=%lld / ld_t=%lld must be multiples of 16 and at least cols / rows", (long long)ld,
                (long long)ld_t);
  int ak = 0;
  const dim3 grid = transpose_grid(rows / kBlock, cols / kBlock, ld, 0, ak);
  transpose_codes_kernel<<<grid, 256, 0, (hipStream_t)stream>>>((const uint8_t*)q, (int)rows, (int)cols, ld, (uint8_t*)q_t,
                                                                 ld_t, ak);
  return check_launch("transpose_codes");
}

int hpfp8_dequantize_per_tensor(const void* q, int64_t n, const float* scale_inv, void* out, int out_type,
                                hpfp8_stream_t stream) {
  HPFP8_REQUIRE(n >= 0, HPFP8_ERR_SHAPE, "dequantize_per_tensor: negative element count");
  HPFP8_REQUIRE(out_type == HPFP8_OUT_BF16 || out_type == HPFP8_OUT_F32, HPFP8_ERR_ARG, "dequantize_per_tensor: bad out_type");
  if (n == 0) return HPFP8_OK;
  HPFP8_REQUIRE(q && scale_inv && out, HPFP8_ERR_ARG, "dequantize_per_tensor: null buffer");
  HPFP8_REQUIRE(aligned16(q) && aligned16(out), HPFP8_ERR_ALIGN, "dequantize_per_tensor: buffers must be 16-byte aligned");
  int64_t blocks = ((n >> 4) + 255) / 256;
  if (blocks < 1) blocks = 1;
  HPFP8_REQUIRE(blocks <= 0x7FFFFFFF, HPFP8_ERR_SHAPE, "dequantize_per_tensor: tensor too large");
  if (out_type == HPFP8_OUT_F32)
    dequant_per_tensor_kernel<true><<<(unsigned)blocks, 256, 0, (hipStream_t)stream>>>((const uint8_t*)q, scale_inv, out, n);
  else
    dequant_per_tensor_kernel<false><<<(unsigned)blocks, 256, 0, (hipStream_t)stream>>>((const uint8_t*)q, scale_inv, out, n);
  return check_launch("dequantize_per_tensor");
}

int hpfp8_dequantize_1x128_bf16(const void* q, const float* scale_inv, int64_t rows, int64_t cols, void* out,
                                float grad_scale, hpfp8_stream_t stream) {
  HPFP8_REQUIRE(rows >= 0 && cols >= 0, HPFP8_ERR_SHAPE, "dequantize_1x128: negative shape");
  HPFP8_REQUIRE(cols % kBlock == 0, HPFP8_ERR_SHAPE, "dequantize_1x128: last dim %lld is not a multiple of 128",
                (long long)cols);
  const int64_t nvec = rows * cols / 8;
  if (nvec == 0) return HPFP8_OK;
  HPFP8_REQUIRE(q && scale_inv && out, HPFP8_ERR_ARG, "dequantize_1x128: null buffer");
  HPFP8_REQUIRE(aligned16(q) && aligned16(out), HPFP8_ERR_ALIGN, "dequantize_1x128: buffers must be 16-byte aligned");
  constexpr int UNROLL = 4;
  const int64_t blocks = (nvec + 256 * UNROLL - 1) / (256 * UNROLL);
  HPFP8_REQUIRE(blocks <= 0x7FFFFFFF, HPFP8_ERR_SHAPE, "dequantize_1x128: tensor too large");
  dequant_1x128_kernel<UNROLL><<<(unsigned)blocks, 256, 0, (hipStream_t)stream>>>(
      (const uint2*)q, scale_inv, (uint4*)out, nvec, grad_scale, grad_scale != 1.0f ? 1 : 0);
  return check_launch("dequantize_1x128");
}

int hpfp8_dequantize_1x128_accumulate_f32(const void* q, const float* scale_inv, int64_t rows, int64_t cols,
                                          float* main_grad, float grad_scale, hpfp8_stream_t stream) {
  HPFP8_REQUIRE(rows >= 0 && cols >= 0, HPFP8_ERR_SHAPE, "dequantize_1x128_accumulate: negative shape");
  HPFP8_REQUIRE(cols % kBlock == 0, HPFP8_ERR_SHAPE,
                "dequantize_1x128_accumulate: last dim %lld is not a multiple of 128", (long long)cols);
  const int64_t nvec = rows * cols / 8;
  if (nvec == 0) return HPFP8_OK;
  HPFP8_REQUIRE(q && scale_inv && main_grad, HPFP8_ERR_ARG, "dequantize_1x128_accumulate: null buffer");
  HPFP8_REQUIRE(aligned16(q) && aligned16(main_grad), HPFP8_ERR_ALIGN,
                "dequantize_1x128_accumulate: buffers must be 16-byte aligned");
  const int64_t blocks = (nvec + 255) / 256;
  HPFP8_REQUIRE(blocks <= 0x7FFFFFFF, HPFP8_ERR_SHAPE, "dequantize_1x128_accumulate: tensor too large");
  dequant_1x128_accumulate_kernel<<<(unsigned)blocks, 256, 0, (hipStream_t)stream>>>(
      (const uint2*)q, scale_inv, (float4*)main_grad, nvec, grad_scale);
  return check_launch("dequantize_1x128_accumulate");
}

int hpfp8_dequantize_128x128_bf16(const void* q, const float* scale_inv, int64_t rows, int64_t cols, void* out,
                                  hpfp8_stream_t stream) {
  HPFP8_REQUIRE(rows >= 0 && cols >= 0, HPFP8_ERR_SHAPE, "dequantize_128x128: negative shape");
  HPFP8_REQUIRE(rows % kBlock == 0 && cols % kBlock == 0, HPFP8_ERR_SHAPE,
                "dequantize_128x128: shape [%lld, %lld] is not a multiple of 128", (long long)rows, (long long)cols);
  HPFP8_REQUIRE(rows < (1 << 30) && cols < (1 << 30), HPFP8_ERR_SHAPE, "dequantize_128x128: dimension too large");
  const int64_t nvec = rows * cols / 16;
  if (nvec == 0) return HPFP8_OK;
  HPFP8_REQUIRE(q && scale_inv && out, HPFP8_ERR_ARG, "dequantize_128x128: null buffer");
  HPFP8_REQUIRE(aligned16(q) && aligned16(out), HPFP8_ERR_ALIGN, "dequantize_128x128: buffers must be 16-byte aligned");
  const int64_t blocks = (nvec + 255) / 256;
  HPFP8_REQUIRE(blocks <= 0x7FFFFFFF, HPFP8_ERR_SHAPE, "dequantize_128x128: tensor too large");
  dequant_128x128_kernel<<<(unsigned)blocks, 256, 0, (hipStream_t)stream>>>((const uint8_t*)q, scale_inv,
                                                                           (uint16_t*)out, (int)rows, (int)cols);
  return check_launch("dequantize_128x128");
}

}  // extern "C"
