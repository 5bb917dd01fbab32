// Streaming kernels behind DPOptimizer.clip_and_accumulate
// (opacus/optimizers/optimizer.py:432-475): per-sample squared norms, the clip
// factor, and the clip-weighted sum over the batch. All HBM-bound; each reads
// the n x P per-sample gradient tensor exactly once, with 16-byte accesses that
// are contiguous across a wavefront, and reduces in a fixed order.
#include <cstring>

#include "dpk_common.h"
#include "philox_normal.h"

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / DPK_WAVE;
// Elements of one row handled by one block of the sum-of-squares kernel.
constexpr int64_t kSumsqChunk = 8192;

struct MultiArgs {
  const void* gs[DPK_MULTI_MAX];
  void* out[DPK_MULTI_MAX];
  int64_t P[DPK_MULTI_MAX];
  int64_t prefix[DPK_MULTI_MAX + 1];  // blocks (per row for sumsq) before tensor k
  int K;
};

__device__ __forceinline__ int find_tensor(const MultiArgs& a, int64_t c) {
  int k = 0;
  while (k + 1 < a.K && c >= a.prefix[k + 1]) ++k;
  return k;
}

// What one launch of the clip-weighted sum works on: up to DPK_MULTI_MAX column ranges
// ("segments"), each a range of one tensor's columns. A tensor may be split between two
// launches, so a segment carries the tensor's row stride beside its own width, and the
// row of the factor table its tensor uses under per-layer clipping.
struct ClipArgs {
  const void* gs[DPK_MULTI_MAX];      // first column of the segment in row 0
  void* out[DPK_MULTI_MAX];           // the same column of the sum
  int64_t cols[DPK_MULTI_MAX];        // width of the segment
  int64_t stride[DPK_MULTI_MAX];      // elements between rows of the tensor
  int64_t prefix[DPK_MULTI_MAX + 1];  // blocks before segment k
  int tensor[DPK_MULTI_MAX];          // index of the tensor (row of a per-layer factor table)
  int K;
};

__device__ __forceinline__ int find_segment(const ClipArgs& a, int64_t c) {
  int k = 0;
  while (k + 1 < a.K && c >= a.prefix[k + 1]) ++k;
  return k;
}

// ---- sum of squares per row --------------------------------------------------
// grid.x = n * CT where CT = prefix[K] = chunks per row summed over the tensors.
// Block (row, c) reduces chunk c of that row to one float:
//   ws[n * prefix[k] + row * nchunk_k + (c - prefix[k])].
template <typename T, bool VEC>
__global__ __launch_bounds__(kThreads) void sumsq_partial_kernel(MultiArgs a, int64_t n, float* ws) {
  __shared__ float red[kWaves];
  const uint32_t CT = static_cast<uint32_t>(a.prefix[a.K]);  // grid.x = n * CT fits 31 bits
  const int64_t row = blockIdx.x / CT;
  const int64_t c = blockIdx.x - static_cast<uint32_t>(row) * CT;
  const int k = find_tensor(a, c);
  const int64_t P = a.P[k];
  const int64_t nchunk = a.prefix[k + 1] - a.prefix[k];
  const int64_t chunk = c - a.prefix[k];
  const T* rowp = static_cast<const T*>(a.gs[k]) + row * P;
  const int64_t lo = chunk * kSumsqChunk;
  const int64_t hi = (lo + kSumsqChunk < P) ? lo + kSumsqChunk : P;
  float acc0 = 0.f, acc1 = 0.f, acc2 = 0.f, acc3 = 0.f;
  if (VEC && hi - lo == kSumsqChunk) {
    // a whole chunk: all of the thread's loads in flight at once, read-once data
    constexpr int kPer = kSumsqChunk / (kThreads * 4);
    float4 v[kPer];
#pragma unroll
    for (int u = 0; u < kPer; ++u) v[u] = dpk_io<T>::load4_nt(rowp + lo + (u * kThreads + threadIdx.x) * 4);
#pragma unroll
    for (int u = 0; u < kPer; ++u) {
      acc0 += v[u].x * v[u].x;
      acc1 += v[u].y * v[u].y;
      acc2 += v[u].z * v[u].z;
      acc3 += v[u].w * v[u].w;
    }
  } else if (VEC) {
    for (int64_t i = lo + threadIdx.x * 4; i < hi; i += kThreads * 4) {
      float4 v = dpk_io<T>::load4(rowp + i);
      acc0 += v.x * v.x;
      acc1 += v.y * v.y;
      acc2 += v.z * v.z;
      acc3 += v.w * v.w;
    }
  } else {
    for (int64_t i = lo + threadIdx.x; i < hi; i += kThreads) {
      float v = dpk_io<T>::load(rowp + i);
      acc0 += v * v;
    }
  }
  float s = block_sum<kWaves>((acc0 + acc1) + (acc2 + acc3), red);
  if (threadIdx.x == 0) ws[n * a.prefix[k] + row * nchunk + chunk] = s;
}

// One wave per (tensor, row): sumsq[k*n + row] = sum of that row's partials.
__global__ __launch_bounds__(kThreads) void sumsq_final_kernel(MultiArgs a, int64_t n,
                                                                 const float* ws, float* sumsq) {
  const int64_t w = (static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x) / DPK_WAVE;
  const int lane = threadIdx.x & (DPK_WAVE - 1);
  if (w >= static_cast<int64_t>(a.K) * n) return;
  const int k = static_cast<int>(w / n);
  const int64_t row = w % n;
  const int64_t nchunk = a.prefix[k + 1] - a.prefix[k];
  const float* p = ws + n * a.prefix[k] + row * nchunk;
  float s = 0.f;
  for (int64_t i = lane; i < nchunk; i += DPK_WAVE) s += p[i];
  s = wave_sum(s);
  if (lane == 0) sumsq[w] = s;
}

// ---- clip factor -----------------------------------------------------------
__global__ void clip_factor_kernel(const float* __restrict__ v, int64_t K, int64_t n, int is_norm,
                                   float C, float* __restrict__ norm, float* __restrict__ clip) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= n) return;
  float s = 0.f;
  for (int64_t k = 0; k < K; ++k) {
    float x = v[k * n + i];
    s += is_norm ? x * x : x;
  }
  const float nr = sqrtf(s);
  if (norm) norm[i] = nr;
  if (clip) clip[i] = fminf(C / (nr + 1e-6f), 1.0f);
}

// ---- clip-weighted sum over the batch ----------------------------------------
// A block of NT threads owns (NT / RS) * W consecutive columns of one tensor
// (W = 4 with VEC, else 1). Thread (cx, ry) walks rows ry, ry+RS, ... of its
// columns; the RS partial sums meet in LDS in a fixed order. RS = 1 with one
// wave per block is the streaming shape for large P: every lane keeps U
// independent 16-byte non-temporal loads in flight (the tensor is read once and
// never again), and many one-wave blocks measured closest to the HBM read
// ceiling. RS > 1 keeps the chip busy when P is small and n large.
template <typename TG, typename TO, bool VEC, int RS, int NT, int U>
__global__ __launch_bounds__(NT) void clip_accumulate_kernel(ClipArgs a, int64_t n,
                                                               const float* __restrict__ clip_base,
                                                               int64_t clip_stride, int accumulate) {
  constexpr int W = VEC ? 4 : 1;
  constexpr int CX = NT / RS;
  __shared__ float4 part[RS > 1 ? NT : 1];
  const int k = find_segment(a, blockIdx.x);
  // one factor vector for all tensors (stride 0) or one per tensor (per-layer clipping)
  const float* __restrict__ clip = clip_base + a.tensor[k] * clip_stride;
  const int64_t P = a.stride[k];
  const int64_t blk = blockIdx.x - a.prefix[k];
  const int cx = threadIdx.x % CX;
  const int ry = threadIdx.x / CX;
  const int64_t col = (blk * CX + cx) * W;
  const bool live = col < a.cols[k];
  const TG* base = static_cast<const TG*>(a.gs[k]) + col;
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  if (live) {
    int64_t r = ry;
    for (; r + (U - 1) * RS < n; r += U * RS) {
      float4 v[U];
      float c[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const TG* p = base + (r + u * RS) * P;
        if (VEC) {
          v[u] = dpk_io<TG>::load4_nt(p);
        } else {
          v[u] = make_float4(dpk_io<TG>::load(p), 0.f, 0.f, 0.f);
        }
        c[u] = clip[r + u * RS];
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        acc.x = fmaf(c[u], v[u].x, acc.x);
        if (VEC) {
          acc.y = fmaf(c[u], v[u].y, acc.y);
          acc.z = fmaf(c[u], v[u].z, acc.z);
          acc.w = fmaf(c[u], v[u].w, acc.w);
        }
      }
    }
    for (; r < n; r += RS) {
      const TG* p = base + r * P;
      const float c = clip[r];
      if (VEC) {
        float4 v = dpk_io<TG>::load4(p);
        acc.x = fmaf(c, v.x, acc.x);
        acc.y = fmaf(c, v.y, acc.y);
        acc.z = fmaf(c, v.z, acc.z);
        acc.w = fmaf(c, v.w, acc.w);
      } else {
        acc.x = fmaf(c, dpk_io<TG>::load(p), acc.x);
      }
    }
  }
  if (RS > 1) {
    part[threadIdx.x] = acc;
    __syncthreads();
    if (ry != 0) return;
#pragma unroll
    for (int j = 1; j < RS; ++j) {
      float4 o = part[j * CX + cx];
      acc.x += o.x;
      acc.y += o.y;
      acc.z += o.z;
      acc.w += o.w;
    }
  }
  if (!live) return;
  TO* out = static_cast<TO*>(a.out[k]) + col;
  if (VEC) {
    if (accumulate) {
      float4 o = dpk_io<TO>::load4(out);
      acc.x += o.x;
      acc.y += o.y;
      acc.z += o.z;
      acc.w += o.w;
    }
    dpk_io<TO>::store4(out, acc);
  } else {
    if (accumulate) acc.x += dpk_io<TO>::load(out);
    dpk_io<TO>::store(out, acc.x);
  }
}

// ---- a whole DPOptimizer step for a small model in one launch -------------------------------
// clip factors from the per-parameter squared norms, the clip-weighted sum over the batch, the
// noise and the division by the batch size (optimizer.py:444-504), for up to DPK_MULTI_MAX
// tensors of at most kStepMaxN samples: every block recomputes the n factors into LDS (K * n
// floats out of the cache), sums its columns exactly as clip_accumulate_kernel does with RS = 16
// (same loop, same order of additions: the same bits), and carries them on through the noise add
// of add_noise_kernel (noise.hip: the same Philox group per four elements, the same arithmetic)
// into grad. The clipped sum itself is also stored when the caller wants it (summed[k] != NULL).
// For a model of a few ten thousand parameters the step is bound by launches and host work:
// this is one launch where there were four (stacked norms, factors, sum, noise).
constexpr int kStepMaxN = 1024;
constexpr int kStepRS = 16, kStepU = 8;

struct StepArgs {
  const void* gs[DPK_MULTI_MAX];
  const float* sumsq[DPK_MULTI_MAX];  // float[n] per tensor
  void* grad[DPK_MULTI_MAX];
  void* summed[DPK_MULTI_MAX];        // nullable
  int64_t P[DPK_MULTI_MAX];
  int64_t gprefix[DPK_MULTI_MAX + 1];  // Philox groups before tensor k
  uint32_t bprefix[DPK_MULTI_MAX + 1];  // blocks before tensor k
  uint8_t vec[DPK_MULTI_MAX];           // tensor k in 4-element chunks
  int K;
};

template <typename TG, typename TO, bool VEC>
__device__ __forceinline__ void step_columns(const StepArgs& a, int k, int64_t n, const float* clip, float4* part,
                                             float std, float denom, uint64_t seed, uint64_t offset, int draws) {
  constexpr int W = VEC ? 4 : 1, RS = kStepRS, U = kStepU, CX = kThreads / RS;
  const int64_t P = a.P[k];
  const int64_t blk = blockIdx.x - a.bprefix[k];
  const int cx = threadIdx.x % CX;
  const int ry = threadIdx.x / CX;
  const int64_t col = (blk * CX + cx) * W;
  const bool live = col < P;
  const TG* base = static_cast<const TG*>(a.gs[k]) + col;
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  if (live) {
    int64_t r = ry;
    for (; r + (U - 1) * RS < n; r += U * RS) {
      float4 v[U];
      float c[U];
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const TG* p = base + (r + u * RS) * P;
        if (VEC) {
          v[u] = dpk_io<TG>::load4_nt(p);
        } else {
          v[u] = make_float4(dpk_io<TG>::load(p), 0.f, 0.f, 0.f);
        }
        c[u] = clip[r + u * RS];
      }
#pragma unroll
      for (int u = 0; u < U; ++u) {
        acc.x = fmaf(c[u], v[u].x, acc.x);
        if (VEC) {
          acc.y = fmaf(c[u], v[u].y, acc.y);
          acc.z = fmaf(c[u], v[u].z, acc.z);
          acc.w = fmaf(c[u], v[u].w, acc.w);
        }
      }
    }
    for (; r < n; r += RS) {
      const TG* p = base + r * P;
      const float c = clip[r];
      if (VEC) {
        float4 v = dpk_io<TG>::load4(p);
        acc.x = fmaf(c, v.x, acc.x);
        acc.y = fmaf(c, v.y, acc.y);
        acc.z = fmaf(c, v.z, acc.z);
        acc.w = fmaf(c, v.w, acc.w);
      } else {
        acc.x = fmaf(c, dpk_io<TG>::load(p), acc.x);
      }
    }
  }
  part[threadIdx.x] = acc;
  __syncthreads();
  if (ry != 0 || !live) return;
#pragma unroll
  for (int j = 1; j < RS; ++j) {
    float4 o = part[j * CX + cx];
    acc.x += o.x;
    acc.y += o.y;
    acc.z += o.z;
    acc.w += o.w;
  }
  // what summed_grad would hold: the sum rounded to the parameter's type
  TO* summed = static_cast<TO*>(a.summed[k]);
  TO* grad = static_cast<TO*>(a.grad[k]) + col;
  const float inv = 1.0f / denom;
  const bool exact_div = std == 0.f;
  const uint64_t group = static_cast<uint64_t>(a.gprefix[k]) + static_cast<uint64_t>(col >> 2);
  float4 z = make_float4(0.f, 0.f, 0.f, 0.f);
  if (std != 0.f) {
    z = dpk_noise::noise4(group, seed, offset, draws);
    z.x *= std;
    z.y *= std;
    z.z *= std;
    z.w *= std;
  }
  if (VEC) {
    if (sizeof(TO) == 2) {  // one rounding, as the stored sum has
      acc.x = bf16_to_f32(f32_to_bf16(acc.x));
      acc.y = bf16_to_f32(f32_to_bf16(acc.y));
      acc.z = bf16_to_f32(f32_to_bf16(acc.z));
      acc.w = bf16_to_f32(f32_to_bf16(acc.w));
    }
    if (summed) dpk_io<TO>::store4(summed + col, acc);
    float4 v;
    if (exact_div) v = make_float4(acc.x / denom, acc.y / denom, acc.z / denom, acc.w / denom);
    else v = make_float4((acc.x + z.x) * inv, (acc.y + z.y) * inv, (acc.z + z.z) * inv, (acc.w + z.w) * inv);
    dpk_io<TO>::store4(grad, v);
  } else {
    if (sizeof(TO) == 2) acc.x = bf16_to_f32(f32_to_bf16(acc.x));
    if (summed) dpk_io<TO>::store(summed + col, acc.x);
    const int e = static_cast<int>(col & 3);
    const float ze = e == 0 ? z.x : e == 1 ? z.y : e == 2 ? z.z : z.w;
    dpk_io<TO>::store(grad, exact_div ? acc.x / denom : (acc.x + ze) * inv);
  }
}

template <typename TG, typename TO>
__global__ __launch_bounds__(kThreads) void clip_noise_step_kernel(StepArgs a, int64_t n, float C, float std, float denom,
                                                                    uint64_t seed, uint64_t offset, int draws) {
  __shared__ float clip[kStepMaxN];
  __shared__ float4 part[kThreads];
  for (int64_t r = threadIdx.x; r < n; r += kThreads) {
    float s = 0.f;
    for (int k = 0; k < a.K; ++k) s += a.sumsq[k][r];  // (as clip_factor_kernel adds the rows of the stacked table)
    clip[r] = fminf(C / (sqrtf(s) + 1e-6f), 1.0f);
  }
  __syncthreads();
  int k = 0;
  while (k + 1 < a.K && blockIdx.x >= a.bprefix[k + 1]) ++k;
  if (a.vec[k]) step_columns<TG, TO, true>(a, k, n, clip, part, std, denom, seed, offset, draws);
  else step_columns<TG, TO, false>(a, k, n, clip, part, std, denom, seed, offset, draws);
}

// The shape for very large tensors: a block owns kWideChunks * 256 consecutive 16-byte
// (fp32) chunks - 128 KB of every row - and walks the rows one at a time with all of a
// row's loads in flight and the whole sum in registers (kWideChunks float4 per thread,
// one wave per SIMD, one block per CU). Per row the blocks then read few, long
// contiguous stretches, which the memory system serves faster than many short ones:
// 6.7 TB/s against 6.2 TB/s for the one-wave shape above on a 128 x 16.8 M fp32 tensor.
// Every block of this kernel has a whole span: the host gives it whole spans only, in
// multiples of the CU count, and the rest of the columns to the kernel above.
constexpr int kWideChunks = 32;
constexpr int64_t kWideSpan = static_cast<int64_t>(kThreads) * kWideChunks * 4;  // elements per block

// 4 consecutive elements of a row through a buffer descriptor: the row's base and the
// chunk's offset stay in scalar registers and each lane adds one 32-bit byte offset, so
// no vector register holds an address. aux 2 is the non-temporal hint.
typedef int span_vi4 __attribute__((ext_vector_type(4)));
typedef int span_vi2 __attribute__((ext_vector_type(2)));
template <typename T> struct span_io;
// raw_t: the four elements as loaded.
template <> struct span_io<float> {
  typedef span_vi4 raw_t;
  static __device__ __forceinline__ raw_t load_raw_nt(__amdgpu_buffer_rsrc_t row, uint32_t lane_bytes, int chunk_bytes) {
    return __builtin_amdgcn_raw_buffer_load_b128(row, lane_bytes, chunk_bytes, 2);
  }
  static __device__ __forceinline__ float4 unpack(raw_t r) {
    return make_float4(__int_as_float(r.x), __int_as_float(r.y), __int_as_float(r.z), __int_as_float(r.w));
  }
  static __device__ __forceinline__ float4 load4_nt(__amdgpu_buffer_rsrc_t row, uint32_t lane_bytes, int chunk_bytes) {
    return unpack(load_raw_nt(row, lane_bytes, chunk_bytes));
  }
};
template <> struct span_io<bf16_t> {
  typedef span_vi2 raw_t;
  static __device__ __forceinline__ raw_t load_raw_nt(__amdgpu_buffer_rsrc_t row, uint32_t lane_bytes, int chunk_bytes) {
    return __builtin_amdgcn_raw_buffer_load_b64(row, lane_bytes, chunk_bytes, 2);
  }
  static __device__ __forceinline__ float4 unpack(raw_t r) {
    float4 v;
    v.x = __uint_as_float(static_cast<uint32_t>(r.x) << 16);
    v.y = __uint_as_float(static_cast<uint32_t>(r.x) & 0xffff0000u);
    v.z = __uint_as_float(static_cast<uint32_t>(r.y) << 16);
    v.w = __uint_as_float(static_cast<uint32_t>(r.y) & 0xffff0000u);
    return v;
  }
  static __device__ __forceinline__ float4 load4_nt(__amdgpu_buffer_rsrc_t row, uint32_t lane_bytes, int chunk_bytes) {
    return unpack(load_raw_nt(row, lane_bytes, chunk_bytes));
  }
};

template <typename TG, typename TO>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(1, 1))) void clip_accumulate_wide_kernel(
    ClipArgs a, int64_t n, const float* __restrict__ clip_base, int64_t clip_stride, int accumulate) {
  const int k = find_segment(a, blockIdx.x);
  const float* __restrict__ clip = clip_base + a.tensor[k] * clip_stride;
  const int64_t stride = a.stride[k];
  const int64_t span0 = (blockIdx.x - a.prefix[k]) * kWideSpan;
  // the vector registers hold the sum and one row of loads and nothing else
  const TG* row = static_cast<const TG*>(a.gs[k]) + span0;
  const uint32_t lane = threadIdx.x * 4;
  constexpr int kChunkBytes = kThreads * 4 * sizeof(TG);
  float4 acc[kWideChunks];
#pragma unroll
  for (int v = 0; v < kWideChunks; ++v) acc[v] = make_float4(0.f, 0.f, 0.f, 0.f);
  typedef typename span_io<TG>::raw_t raw_t;
  // One row at a time; its loads stay as loaded until every one of them is issued (an
  // unpacking of bf16 pairs placed next to each load would have the wave wait for that
  // load before it asks for the next).
  for (int64_t r = 0; r < n; ++r, row += stride) {
    const float c = clip[r];
    raw_t x[kWideChunks];
    const __amdgpu_buffer_rsrc_t rsrc = __builtin_amdgcn_make_buffer_rsrc(
        const_cast<TG*>(row), 0, kWideChunks * kChunkBytes, 0x00020000);
#pragma unroll
    for (int v = 0; v < kWideChunks; ++v)
      x[v] = span_io<TG>::load_raw_nt(rsrc, lane * static_cast<uint32_t>(sizeof(TG)), v * kChunkBytes);
#pragma unroll
    for (int v = 0; v < kWideChunks; ++v) {
      const float4 f = span_io<TG>::unpack(x[v]);
      acc[v].x = fmaf(c, f.x, acc[v].x);
      acc[v].y = fmaf(c, f.y, acc[v].y);
      acc[v].z = fmaf(c, f.z, acc[v].z);
      acc[v].w = fmaf(c, f.w, acc[v].w);
    }
  }
  TO* out = static_cast<TO*>(a.out[k]) + span0;
  if (accumulate) {
    float4 old[kWideChunks];
#pragma unroll
    for (int v = 0; v < kWideChunks; ++v) old[v] = dpk_io<TO>::load4(out + v * (kThreads * 4) + lane);
#pragma unroll
    for (int v = 0; v < kWideChunks; ++v) {
      acc[v].x += old[v].x;
      acc[v].y += old[v].y;
      acc[v].z += old[v].z;
      acc[v].w += old[v].w;
    }
  }
#pragma unroll
  for (int v = 0; v < kWideChunks; ++v) dpk_io<TO>::store4(out + v * (kThreads * 4) + lane, acc[v]);
}

constexpr int kStreamThreads = 64;  // block size of the RS = 1 streaming shape
constexpr int kStreamUnroll = 16;

template <typename TG, typename TO, bool VEC, int RS>
void launch_clip_accumulate(const ClipArgs& a, int64_t n, const float* clip, int64_t clip_stride,
                            int accumulate, hipStream_t s) {
  constexpr int NT = RS == 1 ? kStreamThreads : kThreads;
  constexpr int U = RS == 1 ? kStreamUnroll : 8;
  hipLaunchKernelGGL((clip_accumulate_kernel<TG, TO, VEC, RS, NT, U>),
                     dim3(static_cast<unsigned>(a.prefix[a.K])), dim3(NT), 0, s, a, n, clip, clip_stride,
                     accumulate);
}

// Columns [lo, lo + cols) of tensor k become the next segment of a launch whose blocks
// cover cols_per_block columns each.
template <typename TG, typename TO>
void add_segment(ClipArgs& a, const void* const* gs, void* const* summed, const int64_t* P, int k, int64_t lo,
                 int64_t cols, int64_t cols_per_block) {
  const int j = a.K++;
  a.gs[j] = static_cast<const TG*>(gs[k]) + lo;
  a.out[j] = static_cast<TO*>(summed[k]) + lo;
  a.cols[j] = cols;
  a.stride[j] = P[k];
  a.tensor[j] = k;
  a.prefix[j + 1] = a.prefix[j] + dpk_cdiv(cols, cols_per_block);
}

// Returns the larger grid of the (up to two) launches; nothing is launched when one
// would exceed the grid limit, which the caller reports.
template <typename TG, typename TO>
int64_t dispatch_clip_accumulate(const void* const* gs, void* const* summed, const int64_t* P, int K, int64_t n,
                                 const float* clip, int64_t clip_stride, int accumulate, bool vec, int rs,
                                 int cus, hipStream_t s) {
  // Whole 128 KB spans, in whole rounds of one block per CU, go to the wide kernel.
  int64_t wide_spans = 0;
  if (vec && rs == 1 && n > 0 && cus > 0) {
    for (int k = 0; k < K; ++k) wide_spans += P[k] / kWideSpan;
    wide_spans -= wide_spans % cus;
  }
  ClipArgs wide, rest;
  wide.K = rest.K = 0;
  wide.prefix[0] = rest.prefix[0] = 0;
  const int64_t cols_per_block =
      static_cast<int64_t>((rs == 1 ? kStreamThreads : kThreads) / rs) * (vec ? 4 : 1);
  for (int k = 0; k < K; ++k) {
    int64_t take = P[k] / kWideSpan;
    if (take > wide_spans) take = wide_spans;
    wide_spans -= take;
    if (take > 0) add_segment<TG, TO>(wide, gs, summed, P, k, 0, take * kWideSpan, kWideSpan);
    if (take * kWideSpan < P[k])
      add_segment<TG, TO>(rest, gs, summed, P, k, take * kWideSpan, P[k] - take * kWideSpan, cols_per_block);
  }
  const int64_t wb = wide.prefix[wide.K], rb = rest.prefix[rest.K];
  const int64_t most = wb > rb ? wb : rb;
  if (most > DPK_MAX_GRID_X) return most;
  if (rest.K > 0) {
    if (vec) {
      if (rs == 1) launch_clip_accumulate<TG, TO, true, 1>(rest, n, clip, clip_stride, accumulate, s);
      else launch_clip_accumulate<TG, TO, true, 16>(rest, n, clip, clip_stride, accumulate, s);
    } else {
      if (rs == 1) launch_clip_accumulate<TG, TO, false, 1>(rest, n, clip, clip_stride, accumulate, s);
      else launch_clip_accumulate<TG, TO, false, 16>(rest, n, clip, clip_stride, accumulate, s);
    }
  }
  if (wide.K > 0)
    hipLaunchKernelGGL((clip_accumulate_wide_kernel<TG, TO>), dim3(static_cast<unsigned>(wb)), dim3(kThreads), 0, s,
                       wide, n, clip, clip_stride, accumulate);
  return most;
}

int fill_sumsq_args(MultiArgs& a, const void* const* gs, const int64_t* P, int64_t K, int dtype,
                    bool* vec, const char* who) {
  DPK_REQUIRE(gs && P, DPK_E_ARG, "%s: NULL pointer table", who);
  DPK_REQUIRE(K >= 1 && K <= DPK_MULTI_MAX, DPK_E_SHAPE, "%s: K=%lld not in [1,%d]", who,
              (long long)K, DPK_MULTI_MAX);
  DPK_REQUIRE(dpk_dtype_ok(dtype), DPK_E_DTYPE, "%s: dtype %d", who, dtype);
  const size_t need = dtype == DPK_BF16 ? 8 : 16;
  *vec = true;
  a.K = static_cast<int>(K);
  a.prefix[0] = 0;
  for (int k = 0; k < K; ++k) {
    DPK_REQUIRE(P[k] >= 1, DPK_E_SHAPE, "%s: P[%d]=%lld", who, k, (long long)P[k]);
    DPK_REQUIRE(gs[k], DPK_E_ARG, "%s: gs[%d] is NULL", who, k);
    DPK_REQUIRE(dpk_aligned(gs[k], dpk_elsize(dtype)), DPK_E_ALIGN, "%s: gs[%d] misaligned", who, k);
    if (P[k] % 4 != 0 || !dpk_aligned(gs[k], need)) *vec = false;
    a.gs[k] = gs[k];
    a.out[k] = nullptr;
    a.P[k] = P[k];
    a.prefix[k + 1] = a.prefix[k] + dpk_cdiv(P[k], kSumsqChunk);
  }
  return DPK_OK;
}

}  // namespace

extern "C" size_t dpk_sumsq_rows_multi_workspace_bytes(int64_t n, const int64_t* P, int64_t K) {
  if (n <= 0 || !P || K <= 0) return 0;
  int64_t ct = 0;
  for (int64_t k = 0; k < K; ++k) ct += dpk_cdiv(P[k] > 0 ? P[k] : 0, kSumsqChunk);
  return dpk_align_up(static_cast<size_t>(n) * ct * sizeof(float), 256);
}

extern "C" size_t dpk_sumsq_rows_workspace_bytes(int64_t n, int64_t P) {
  return dpk_sumsq_rows_multi_workspace_bytes(n, &P, 1);
}

extern "C" int dpk_sumsq_rows_multi(const void* const* gs, const int64_t* P, int64_t K, int dtype,
                                    int64_t n, float* sumsq, void* ws, size_t ws_bytes,
                                    dpk_stream_t stream) {
  const char* who = "dpk_sumsq_rows_multi";
  DPK_REQUIRE(n >= 0, DPK_E_SHAPE, "%s: n=%lld", who, (long long)n);
  if (n == 0) return DPK_OK;
  MultiArgs a;
  bool vec;
  int rc = fill_sumsq_args(a, gs, P, K, dtype, &vec, who);
  if (rc != DPK_OK) return rc;
  DPK_REQUIRE(sumsq, DPK_E_ARG, "%s: sumsq is NULL", who);
  const size_t need = dpk_sumsq_rows_multi_workspace_bytes(n, P, K);
  DPK_REQUIRE(ws && ws_bytes >= need, DPK_E_WORKSPACE, "%s: workspace %zu < %zu bytes", who,
              ws_bytes, need);
  DPK_REQUIRE(dpk_aligned(ws, 4), DPK_E_ALIGN, "%s: workspace misaligned", who);
  const int64_t blocks = n * a.prefix[K];
  DPK_REQUIRE(blocks <= DPK_MAX_GRID_X, DPK_E_SHAPE, "%s: %lld blocks exceed the grid limit", who,
              (long long)blocks);
  hipStream_t s = static_cast<hipStream_t>(stream);
  // Rows of one chunk each (small parameters: norm layers, biases): the block's sum is the row's
  // sum of squares and lands in sumsq directly, ws[n k + row] being sumsq[k n + row]; no second kernel.
  const bool one_chunk = a.prefix[K] == K;
  float* wsf = one_chunk ? sumsq : static_cast<float*>(ws);
  dim3 grid(static_cast<unsigned>(blocks)), block(kThreads);
  if (dtype == DPK_F32) {
    if (vec) hipLaunchKernelGGL((sumsq_partial_kernel<float, true>), grid, block, 0, s, a, n, wsf);
    else hipLaunchKernelGGL((sumsq_partial_kernel<float, false>), grid, block, 0, s, a, n, wsf);
  } else {
    if (vec) hipLaunchKernelGGL((sumsq_partial_kernel<bf16_t, true>), grid, block, 0, s, a, n, wsf);
    else hipLaunchKernelGGL((sumsq_partial_kernel<bf16_t, false>), grid, block, 0, s, a, n, wsf);
  }
  DPK_LAUNCH_CHECK(who);
  if (one_chunk) return DPK_OK;
  const int64_t waves = K * n;
  hipLaunchKernelGGL(sumsq_final_kernel, dim3(static_cast<unsigned>(dpk_cdiv(waves, kWaves))), block,
                     0, s, a, n, wsf, sumsq);
  DPK_LAUNCH_CHECK(who);
  return DPK_OK;
}

extern "C" int dpk_sumsq_rows(const void* gs, int dtype, int64_t n, int64_t P, float* sumsq,
                              void* ws, size_t ws_bytes, dpk_stream_t stream) {
  return dpk_sumsq_rows_multi(&gs, &P, 1, dtype, n, sumsq, ws, ws_bytes, stream);
}

extern "C" int dpk_clip_factor(const float* sumsq, int64_t K, int64_t n, int is_norm,
                               float max_grad_norm, float* norm, float* clip, dpk_stream_t stream) {
  const char* who = "dpk_clip_factor";
  DPK_REQUIRE(n >= 0 && K >= 1, DPK_E_SHAPE, "%s: K=%lld n=%lld", who, (long long)K, (long long)n);
  if (n == 0) return DPK_OK;
  DPK_REQUIRE(sumsq, DPK_E_ARG, "%s: input is NULL", who);
  DPK_REQUIRE(norm || clip, DPK_E_ARG, "%s: both outputs are NULL", who);
  hipLaunchKernelGGL(clip_factor_kernel, dim3(static_cast<unsigned>(dpk_cdiv(n, 256))), dim3(256), 0,
                     static_cast<hipStream_t>(stream), sumsq, K, n, is_norm, max_grad_norm, norm, clip);
  DPK_LAUNCH_CHECK(who);
  return DPK_OK;
}

namespace {
int clip_accumulate_impl(const char* who, const void* const* gs, void* const* summed, const int64_t* P,
                         int64_t K, int gs_dtype, int out_dtype, const float* clip, int64_t clip_stride,
                         int64_t n, int accumulate, dpk_stream_t stream) {
  DPK_REQUIRE(n >= 0, DPK_E_SHAPE, "%s: n=%lld", who, (long long)n);
  DPK_REQUIRE(gs && summed && P, DPK_E_ARG, "%s: NULL pointer table", who);
  DPK_REQUIRE(K >= 1 && K <= DPK_MULTI_MAX, DPK_E_SHAPE, "%s: K=%lld not in [1,%d]", who,
              (long long)K, DPK_MULTI_MAX);
  DPK_REQUIRE(dpk_dtype_ok(gs_dtype) && dpk_dtype_ok(out_dtype), DPK_E_DTYPE, "%s: dtypes %d,%d",
              who, gs_dtype, out_dtype);
  DPK_REQUIRE(n == 0 || clip, DPK_E_ARG, "%s: clip is NULL", who);
  bool vec = true;
  int64_t ptotal = 0;
  const size_t gneed = gs_dtype == DPK_BF16 ? 8 : 16, oneed = out_dtype == DPK_BF16 ? 8 : 16;
  for (int k = 0; k < K; ++k) {
    DPK_REQUIRE(P[k] >= 1, DPK_E_SHAPE, "%s: P[%d]=%lld", who, k, (long long)P[k]);
    DPK_REQUIRE(summed[k] && (n == 0 || gs[k]), DPK_E_ARG, "%s: tensor %d is NULL", who, k);
    DPK_REQUIRE(dpk_aligned(gs[k], dpk_elsize(gs_dtype)) && dpk_aligned(summed[k], dpk_elsize(out_dtype)),
                DPK_E_ALIGN, "%s: tensor %d misaligned", who, k);
    if (P[k] % 4 != 0 || !dpk_aligned(gs[k], gneed) || !dpk_aligned(summed[k], oneed)) vec = false;
    ptotal += P[k];
  }
  // An empty batch contributes a zero sum: with accumulate nothing changes,
  // without it the kernel's row loop runs zero times and writes zeros.
  if (n == 0 && accumulate) return DPK_OK;
  // Split the rows inside a block when the columns alone cannot fill the chip.
  const int rs = (ptotal / (vec ? 4 : 1) < 256LL * 1024 && n >= 64) ? 16 : 1;
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int cus = dpk_device_cus();
  if (cus < 0) return cus;
  const int Ki = static_cast<int>(K);
  int64_t blocks = 0;
  if (gs_dtype == DPK_F32 && out_dtype == DPK_F32)
    blocks = dispatch_clip_accumulate<float, float>(gs, summed, P, Ki, n, clip, clip_stride, accumulate, vec, rs, cus, s);
  else if (gs_dtype == DPK_BF16 && out_dtype == DPK_F32)
    blocks = dispatch_clip_accumulate<bf16_t, float>(gs, summed, P, Ki, n, clip, clip_stride, accumulate, vec, rs, cus, s);
  else if (gs_dtype == DPK_F32 && out_dtype == DPK_BF16)
    blocks = dispatch_clip_accumulate<float, bf16_t>(gs, summed, P, Ki, n, clip, clip_stride, accumulate, vec, rs, cus, s);
  else
    blocks = dispatch_clip_accumulate<bf16_t, bf16_t>(gs, summed, P, Ki, n, clip, clip_stride, accumulate, vec, rs, cus, s);
  DPK_REQUIRE(blocks <= DPK_MAX_GRID_X, DPK_E_SHAPE, "%s: %lld blocks exceed the grid limit", who,
              (long long)blocks);
  DPK_LAUNCH_CHECK(who);
  return DPK_OK;
}
}  // namespace

extern "C" int dpk_clip_accumulate_multi(const void* const* gs, void* const* summed,
                                         const int64_t* P, int64_t K, int gs_dtype, int out_dtype,
                                         const float* clip, int64_t n, int accumulate,
                                         dpk_stream_t stream) {
  return clip_accumulate_impl("dpk_clip_accumulate_multi", gs, summed, P, K, gs_dtype, out_dtype, clip, 0,
                              n, accumulate, stream);
}

extern "C" int dpk_clip_accumulate_per_layer(const void* const* gs, void* const* summed,
                                             const int64_t* P, int64_t K, int gs_dtype, int out_dtype,
                                             const float* clip, int64_t n, int accumulate,
                                             dpk_stream_t stream) {
  return clip_accumulate_impl("dpk_clip_accumulate_per_layer", gs, summed, P, K, gs_dtype, out_dtype, clip,
                              n, n, accumulate, stream);
}

namespace {
struct LayerBounds {
  float C[DPK_MULTI_MAX];
};

__global__ void clip_factor_per_layer_kernel(const float* __restrict__ v, int64_t n, int is_norm,
                                             LayerBounds bounds, float* __restrict__ clip) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * blockDim.x + threadIdx.x;
  if (i >= n) return;
  const int k = blockIdx.y;
  const float x = v[k * n + i];
  const float nr = is_norm ? fabsf(x) : sqrtf(x);
  clip[k * n + i] = fminf(bounds.C[k] / (nr + 1e-6f), 1.0f);
}
}  // namespace

extern "C" int dpk_clip_factor_per_layer(const float* sumsq, int64_t K, int64_t n, int is_norm,
                                         const float* max_grad_norms, float* clip,
                                         dpk_stream_t stream) {
  const char* who = "dpk_clip_factor_per_layer";
  DPK_REQUIRE(K >= 1 && K <= DPK_MULTI_MAX && n >= 0, DPK_E_SHAPE, "%s: K=%lld (1..%d) n=%lld", who,
              (long long)K, DPK_MULTI_MAX, (long long)n);
  if (n == 0) return DPK_OK;
  DPK_REQUIRE(sumsq && clip && max_grad_norms, DPK_E_ARG, "%s: NULL argument", who);
  DPK_REQUIRE(dpk_cdiv(n, 256) <= DPK_MAX_GRID_X, DPK_E_SHAPE, "%s: n too large", who);
  LayerBounds bounds;
  for (int k = 0; k < K; ++k) {
    DPK_REQUIRE(max_grad_norms[k] >= 0.f, DPK_E_ARG, "%s: max_grad_norms[%d]=%g", who, k,
                (double)max_grad_norms[k]);
    bounds.C[k] = max_grad_norms[k];
  }
  hipLaunchKernelGGL(clip_factor_per_layer_kernel,
                     dim3(static_cast<unsigned>(dpk_cdiv(n, 256)), static_cast<unsigned>(K)), dim3(256), 0,
                     static_cast<hipStream_t>(stream), sumsq, n, is_norm, bounds, clip);
  DPK_LAUNCH_CHECK(who);
  return DPK_OK;
}

extern "C" int dpk_clip_accumulate(const void* gs, int gs_dtype, const float* clip, void* summed,
                                   int out_dtype, int64_t n, int64_t P, int accumulate,
                                   dpk_stream_t stream) {
  return dpk_clip_accumulate_multi(&gs, &summed, &P, 1, gs_dtype, out_dtype, clip, n, accumulate,
                                   stream);
}

// The whole step of a small model in one launch (see clip_noise_step_kernel): K <= DPK_MULTI_MAX
// tensors, 64 <= n <= 1024 samples. Results are bit-identical to dpk_clip_factor on the stacked
// sumsq rows + dpk_clip_accumulate_multi (in its small-tensor shape) + dpk_add_noise_multi.
extern "C" int dpk_clip_noise_step(const void* const* gs, const float* const* sumsq, void* const* grad,
                                   void* const* summed, const int64_t* P, int64_t K, int gs_dtype, int out_dtype,
                                   int64_t n, float max_grad_norm, float std, float denom, uint64_t seed,
                                   uint64_t offset, int draws, dpk_stream_t stream) {
  const char* who = "dpk_clip_noise_step";
  DPK_REQUIRE(gs && sumsq && grad && P, DPK_E_ARG, "%s: NULL pointer table", who);
  DPK_REQUIRE(K >= 1 && K <= DPK_MULTI_MAX, DPK_E_SHAPE, "%s: K=%lld not in [1,%d]", who, (long long)K, DPK_MULTI_MAX);
  DPK_REQUIRE(n >= 64 && n <= kStepMaxN, DPK_E_SHAPE, "%s: n=%lld not in [64,%d]", who, (long long)n, kStepMaxN);
  DPK_REQUIRE(dpk_dtype_ok(gs_dtype) && dpk_dtype_ok(out_dtype), DPK_E_DTYPE, "%s: dtypes %d,%d", who, gs_dtype, out_dtype);
  DPK_REQUIRE(draws == 1 || draws == 4, DPK_E_ARG, "%s: draws=%d (1 or 4)", who, draws);
  DPK_REQUIRE(std >= 0.f && denom != 0.f, DPK_E_ARG, "%s: std=%g denom=%g", who, (double)std, (double)denom);
  StepArgs a;
  memset(&a, 0, sizeof(a));
  a.K = static_cast<int>(K);
  const size_t gneed = gs_dtype == DPK_BF16 ? 8 : 16, oneed = out_dtype == DPK_BF16 ? 8 : 16;
  int64_t blocks = 0;
  for (int k = 0; k < K; ++k) {
    DPK_REQUIRE(P[k] >= 1, DPK_E_SHAPE, "%s: P[%d]=%lld", who, k, (long long)P[k]);
    DPK_REQUIRE(gs[k] && sumsq[k] && grad[k], DPK_E_ARG, "%s: tensor %d is NULL", who, k);
    DPK_REQUIRE(dpk_aligned(gs[k], dpk_elsize(gs_dtype)) && dpk_aligned(grad[k], dpk_elsize(out_dtype)) &&
                    dpk_aligned(summed ? summed[k] : nullptr, dpk_elsize(out_dtype)) && dpk_aligned(sumsq[k], 4),
                DPK_E_ALIGN, "%s: tensor %d misaligned", who, k);
    a.gs[k] = gs[k];
    a.sumsq[k] = sumsq[k];
    a.grad[k] = grad[k];
    a.summed[k] = summed ? summed[k] : nullptr;
    a.P[k] = P[k];
    const bool vec = P[k] % 4 == 0 && dpk_aligned(gs[k], gneed) && dpk_aligned(grad[k], oneed) &&
                     dpk_aligned(a.summed[k], oneed);
    a.vec[k] = vec ? 1 : 0;
    a.gprefix[k + 1] = a.gprefix[k] + dpk_cdiv(P[k], 4);
    blocks += dpk_cdiv(P[k], (kThreads / kStepRS) * (vec ? 4 : 1));
    DPK_REQUIRE(blocks <= DPK_MAX_GRID_X, DPK_E_SHAPE, "%s: too many blocks", who);
    a.bprefix[k + 1] = static_cast<uint32_t>(blocks);
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid(static_cast<unsigned>(blocks)), block(kThreads);
#define DPK_STEP(TG, TO) \
  hipLaunchKernelGGL((clip_noise_step_kernel<TG, TO>), grid, block, 0, s, a, n, max_grad_norm, std, denom, seed, offset, draws)
  if (gs_dtype == DPK_F32 && out_dtype == DPK_F32) DPK_STEP(float, float);
  else if (gs_dtype == DPK_BF16 && out_dtype == DPK_F32) DPK_STEP(bf16_t, float);
  else if (gs_dtype == DPK_F32 && out_dtype == DPK_BF16) DPK_STEP(float, bf16_t);
  else DPK_STEP(bf16_t, bf16_t);
#undef DPK_STEP
  DPK_LAUNCH_CHECK(who);
  return DPK_OK;
}
