// Shared host/device helpers for the dpk kernels (gfx950, wave64).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stddef.h>

#include "../../include/dpk.h"

#define DPK_ABI_VERSION 3
#define DPK_WAVE 64

// ---- host side -------------------------------------------------------------

// Stores a printf-style message for dpk_last_error() and returns `code`.
int dpk_fail(int code, const char* fmt, ...);

#define DPK_REQUIRE(cond, code, ...)            \
  do {                                          \
    if (!(cond)) return dpk_fail((code), __VA_ARGS__); \
  } while (0)

#define DPK_LAUNCH_CHECK(name)                                                   \
  do {                                                                           \
    hipError_t e_ = hipGetLastError();                                           \
    if (e_ != hipSuccess)                                                        \
      return dpk_fail(DPK_E_LAUNCH, "%s: launch failed: %s", (name), hipGetErrorString(e_)); \
  } while (0)

static inline bool dpk_aligned(const void* p, size_t a) {
  return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0;
}
static inline bool dpk_dtype_ok(int d) { return d == DPK_F32 || d == DPK_BF16; }
static inline size_t dpk_elsize(int d) { return d == DPK_BF16 ? 2 : 4; }
static inline int64_t dpk_cdiv(int64_t a, int64_t b) { return (a + b - 1) / b; }
static inline size_t dpk_align_up(size_t x, size_t a) { return (x + a - 1) / a * a; }

// Grid dimension limits of HIP: x up to 2^31-1, y and z up to 65535.
#define DPK_MAX_GRID_X 2147483647LL
#define DPK_MAX_GRID_YZ 65535LL

// ---- device side -----------------------------------------------------------
#if defined(__HIPCC__)

typedef uint16_t bf16_t;  // raw bfloat16 bits

__device__ __forceinline__ float bf16_to_f32(bf16_t v) {
  return __uint_as_float(static_cast<uint32_t>(v) << 16);
}
// Round to nearest even, NaN kept quiet: what torch's float -> bfloat16 cast does. gfx950
// converts in hardware (v_cvt_pk_bf16_f32, two values per instruction).
__device__ __forceinline__ bf16_t f32_to_bf16(float f) {
  return __builtin_bit_cast(bf16_t, static_cast<__bf16>(f));
}
// lo in bits 0..15, hi in bits 16..31
__device__ __forceinline__ uint32_t f32x2_to_bf16x2(float lo, float hi) {
  typedef float dpk_f2 __attribute__((ext_vector_type(2)));
  typedef __bf16 dpk_bf2 __attribute__((ext_vector_type(2)));
  dpk_f2 v;
  v.x = lo;
  v.y = hi;
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, dpk_bf2));
}

typedef float dpk_vf4 __attribute__((ext_vector_type(4)));
typedef uint32_t dpk_vu2 __attribute__((ext_vector_type(2)));

template <typename T> struct dpk_io;
template <> struct dpk_io<float> {
  // load4 with a non-temporal hint: for data that is streamed through exactly once
  static __device__ __forceinline__ float4 load4_nt(const float* p) {
    const dpk_vf4 v = __builtin_nontemporal_load(reinterpret_cast<const dpk_vf4*>(p));
    return make_float4(v.x, v.y, v.z, v.w);
  }
  // The same four elements as loaded, to be unpacked later: a kernel that wants many loads
  // in flight issues them all as raw4 and unpacks once they are all on their way.
  typedef dpk_vf4 raw4;
  static __device__ __forceinline__ raw4 load4_raw(const float* p) { return *reinterpret_cast<const dpk_vf4*>(p); }
  static __device__ __forceinline__ float4 unpack4(raw4 v) { return make_float4(v.x, v.y, v.z, v.w); }
  static __device__ __forceinline__ float load(const float* p) { return *p; }
  static __device__ __forceinline__ void store(float* p, float v) { *p = v; }
  // 4 consecutive elements, p 16-byte aligned
  static __device__ __forceinline__ float4 load4(const float* p) {
    return *reinterpret_cast<const float4*>(p);
  }
  static __device__ __forceinline__ void store4(float* p, float4 v) {
    *reinterpret_cast<float4*>(p) = v;
  }
  // store4 with a non-temporal hint: for output that nobody re-reads before it has
  // left the caches anyway
  static __device__ __forceinline__ void store4_nt(float* p, float4 v) {
    dpk_vf4 w;
    w.x = v.x;
    w.y = v.y;
    w.z = v.z;
    w.w = v.w;
    __builtin_nontemporal_store(w, reinterpret_cast<dpk_vf4*>(p));
  }
};
template <> struct dpk_io<bf16_t> {
  static __device__ __forceinline__ float4 load4_nt(const bf16_t* p) {
    const dpk_vu2 r = __builtin_nontemporal_load(reinterpret_cast<const dpk_vu2*>(p));
    float4 v;
    v.x = __uint_as_float(r.x << 16);
    v.y = __uint_as_float(r.x & 0xffff0000u);
    v.z = __uint_as_float(r.y << 16);
    v.w = __uint_as_float(r.y & 0xffff0000u);
    return v;
  }
  typedef dpk_vu2 raw4;
  static __device__ __forceinline__ raw4 load4_raw(const bf16_t* p) { return *reinterpret_cast<const dpk_vu2*>(p); }
  static __device__ __forceinline__ float4 unpack4(raw4 r) {
    float4 v;
    v.x = __uint_as_float(r.x << 16);
    v.y = __uint_as_float(r.x & 0xffff0000u);
    v.z = __uint_as_float(r.y << 16);
    v.w = __uint_as_float(r.y & 0xffff0000u);
    return v;
  }
  static __device__ __forceinline__ float load(const bf16_t* p) { return bf16_to_f32(*p); }
  static __device__ __forceinline__ void store(bf16_t* p, float v) { *p = f32_to_bf16(v); }
  // 4 consecutive elements, p 8-byte aligned
  static __device__ __forceinline__ float4 load4(const bf16_t* p) {
    uint2 r = *reinterpret_cast<const uint2*>(p);
    float4 v;
    v.x = __uint_as_float(r.x << 16);
    v.y = __uint_as_float(r.x & 0xffff0000u);
    v.z = __uint_as_float(r.y << 16);
    v.w = __uint_as_float(r.y & 0xffff0000u);
    return v;
  }
  static __device__ __forceinline__ void store4(bf16_t* p, float4 v) {
    uint2 r;
    r.x = f32x2_to_bf16x2(v.x, v.y);
    r.y = f32x2_to_bf16x2(v.z, v.w);
    *reinterpret_cast<uint2*>(p) = r;
  }
  static __device__ __forceinline__ void store4_nt(bf16_t* p, float4 v) {
    dpk_vu2 r;
    r.x = f32x2_to_bf16x2(v.x, v.y);
    r.y = f32x2_to_bf16x2(v.z, v.w);
    __builtin_nontemporal_store(r, reinterpret_cast<dpk_vu2*>(p));
  }
};

// Workgroups are handed to the 8 XCDs round-robin by hardware id. Renumbering
// them so that each XCD works through one contiguous range of work units
// keeps what neighbouring units share (the rows of a sample) in that XCD's L2.
__device__ __forceinline__ uint32_t xcd_contiguous_id(uint32_t bid, uint32_t nb) {
  const uint32_t x = bid & 7u, idx = bid >> 3;
  const uint32_t base = nb >> 3, rem = nb & 7u;
  return x * base + (x < rem ? x : rem) + idx;
}

__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) v += __shfl_xor(v, o, DPK_WAVE);
  return v;
}

// Sum over a block of NWAVES*64 threads; the result is valid in thread 0 only.
// `red` is LDS scratch of at least NWAVES floats. Fixed order.
template <int NWAVES>
__device__ __forceinline__ float block_sum(float v, float* red) {
  v = wave_sum(v);
  const int lane = threadIdx.x & (DPK_WAVE - 1);
  const int wave = threadIdx.x / DPK_WAVE;
  __syncthreads();  // protect `red` against a previous use
  if (lane == 0) red[wave] = v;
  __syncthreads();
  float s = 0.f;
  if (threadIdx.x == 0) {
#pragma unroll
    for (int w = 0; w < NWAVES; ++w) s += red[w];
  }
  return s;
}

// out[r] = post(sum_c part[r*cols + c]) for r < rows: one wave per row, fixed
// order. mode 0: plain sum; mode 1: sqrt(max(0, sum)) * factor.
static __global__ __launch_bounds__(256) void dpk_reduce_rows_kernel(const float* __restrict__ part,
                                                                       int64_t rows, int64_t cols,
                                                                       float* __restrict__ out,
                                                                       int mode, float factor) {
  const int64_t w = (static_cast<int64_t>(blockIdx.x) * 256 + threadIdx.x) / DPK_WAVE;
  const int lane = threadIdx.x & (DPK_WAVE - 1);
  if (w >= rows) return;
  const float* p = part + w * cols;
  float s = 0.f;
  for (int64_t i = lane; i < cols; i += DPK_WAVE) s += p[i];
  s = wave_sum(s);
  if (lane == 0) out[w] = mode == 1 ? sqrtf(fmaxf(s, 0.f)) * factor : s;
}

static inline void dpk_launch_reduce_rows(const float* part, int64_t rows, int64_t cols, float* out,
                                          int mode, float factor, hipStream_t s) {
  hipLaunchKernelGGL(dpk_reduce_rows_kernel, dim3(static_cast<unsigned>(dpk_cdiv(rows, 4))),
                     dim3(256), 0, s, part, rows, cols, out, mode, factor);
}

#endif  // __HIPCC__
