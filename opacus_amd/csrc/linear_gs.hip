// Per-sample gradients of nn.Linear (opacus/grad_sample/linear.py:29-51).
//   weight: gs[n,i,j] = scale * sum_t b[n,t,i] * a[n,t,j]     (linear.py:47)
//   bias:   gs[n,k]   = scale * sum_t b[n,t,k]                (linear.py:50)
// T == 1 is a rank-1 outer product per sample: no contraction, the kernel is
// bound by the n*out*in store stream. T > 1 is a batched GEMM with K = T on the
// fp32 MFMA path (bf16 inputs are widened on the way into LDS, which is exact).
// Both paths also deliver the per-sample sum of squares of what they wrote (the
// MFMA kernel as one partial per block reduced in a fixed order, the rank-one
// case from its closed form), so the optimizer's norm pass over the n*out*in
// tensor disappears.
#include "dpk_common.h"
#include "mfma_bf16.h"
#include "mfma_bf16_tr.h"
#include "mfma_f32_dlds.h"
#include "mfma_f32.h"

#include <cstring>
#include <type_traits>

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / DPK_WAVE;
constexpr int kOuterRowsPerThread = 8;  // rows of gs each thread writes (T == 1)

// ---- T == 1 ------------------------------------------------------------------
// Block = CX column threads x RY = 256 / CX row groups; a thread keeps its 4 (or
// 1) activations in registers and writes kOuterRowsPerThread rows, so a block
// covers 8 * RY rows of CX * W contiguous elements each. With CX = 256 that is 8
// rows of 4 KB: few rows per block (many small blocks in flight) is what keeps
// the store stream closest to the HBM write ceiling.
template <typename TIN, typename TOUT, bool VEC, int CXLOG2>
__global__ __launch_bounds__(kThreads) void linear_outer_kernel(
    const TIN* __restrict__ b, const TIN* __restrict__ a, TOUT* __restrict__ gs, int64_t M, int64_t N,
    float scale, uint32_t tiles_m, uint32_t tiles_n) {
  constexpr int W = VEC ? 4 : 1;
  constexpr int CX = 1 << CXLOG2, RY = kThreads >> CXLOG2;
  constexpr int ROWS = kOuterRowsPerThread * RY;
  const int cx = threadIdx.x & (CX - 1), ry = threadIdx.x >> CXLOG2;
  // 32-bit index arithmetic: a block only issues a handful of stores, so 64-bit
  // divisions here would cost more instructions than the work itself
  const uint32_t per_sample = tiles_m * tiles_n;
  const uint32_t sample32 = blockIdx.x / per_sample;
  const uint32_t rem = blockIdx.x - sample32 * per_sample;
  const uint32_t tm = rem / tiles_n, tn = rem - tm * tiles_n;
  const int64_t sample = sample32;
  const int64_t i0 = static_cast<int64_t>(tm) * ROWS + ry;
  const int64_t j = (static_cast<int64_t>(tn) * CX + cx) * W;
  if (j >= N) return;
  const TIN* bs = b + sample * M;
  TOUT* out = gs + sample * M * N + j;
  float4 av = make_float4(0.f, 0.f, 0.f, 0.f);
  if (VEC) av = dpk_io<TIN>::load4(a + sample * N + j);
  else av.x = dpk_io<TIN>::load(a + sample * N + j);
  float bv[kOuterRowsPerThread];
#pragma unroll
  for (int r = 0; r < kOuterRowsPerThread; ++r) {
    const int64_t i = i0 + r * RY;
    bv[r] = i < M ? scale * dpk_io<TIN>::load(bs + i) : 0.f;
  }
#pragma unroll
  for (int r = 0; r < kOuterRowsPerThread; ++r) {
    const int64_t i = i0 + r * RY;
    if (i < M) {
      if (VEC) dpk_io<TOUT>::store4_nt(out + i * N, make_float4(bv[r] * av.x, bv[r] * av.y, bv[r] * av.z, bv[r] * av.w));
      else dpk_io<TOUT>::store(out + i * N, bv[r] * av.x);
    }
  }
}

// The same product written as one sequential stream: thread <-> one 4-element chunk of
// the sample's out x in matrix taken in memory order, so that the blocks resident at
// any moment write one contiguous stretch of memory. The gradients are written once
// and next touched by a kernel that streams all of them, long after they have left the
// caches: non-temporal stores keep them from sitting there as dirty lines, whose
// write-back would otherwise fall into that kernel's time (its reads measured 7 %
// slower after plain stores). Non-temporal stores in memory order measured 7.0 TB/s;
// the tiled kernel above, whose blocks each touch eight rows 4 * in bytes apart,
// 5.7 TB/s. More chunks per thread or other block sizes measured slower.
constexpr int kSeqThreads = 256;

// E: elements of a chunk, 4, or 8 for bf16 results (16 bytes a store either way: with
// 8-byte stores the bf16 stream stopped at 5.3 TB/s).
template <typename TIN, typename TOUT, int E>
__global__ __launch_bounds__(kSeqThreads) void linear_outer_seq_kernel(
    const TIN* __restrict__ b, const TIN* __restrict__ a, TOUT* __restrict__ gs, uint32_t M,
    uint32_t cols, float scale, uint32_t blocks_per_sample) {
  static_assert(E == 4 || (E == 8 && sizeof(TOUT) == 2), "one or two 4-element pieces; 16-byte stores at most");
  const uint32_t sample = blockIdx.x / blocks_per_sample;
  const uint32_t blk = blockIdx.x - sample * blocks_per_sample;
  const uint32_t total = M * cols;  // chunks per sample (< 2^32, checked by the host)
  const TIN* bs = b + static_cast<int64_t>(sample) * M;
  const TIN* as = a + static_cast<int64_t>(sample) * cols * E;
  TOUT* out = gs + static_cast<int64_t>(sample) * total * E;
  const uint32_t p = blk * kSeqThreads + threadIdx.x;
  if (p >= total) return;
  const uint32_t i = p / cols, jc = p - i * cols;
  const float bv = scale * dpk_io<TIN>::load(bs + i);
  const float4 av = dpk_io<TIN>::load4(as + jc * E);
  if constexpr (E == 4) {
    dpk_io<TOUT>::store4_nt(out + static_cast<int64_t>(p) * 4, make_float4(bv * av.x, bv * av.y, bv * av.z, bv * av.w));
  } else {
    const float4 aw = dpk_io<TIN>::load4(as + jc * E + 4);
    typedef uint32_t vu4 __attribute__((ext_vector_type(4)));
    vu4 w;
    w.x = f32x2_to_bf16x2(bv * av.x, bv * av.y);
    w.y = f32x2_to_bf16x2(bv * av.z, bv * av.w);
    w.z = f32x2_to_bf16x2(bv * aw.x, bv * aw.y);
    w.w = f32x2_to_bf16x2(bv * aw.z, bv * aw.w);
    __builtin_nontemporal_store(w, reinterpret_cast<vu4*>(out + static_cast<int64_t>(p) * 8));
  }
}

// Sum of squares of a rank-one matrix: sum_ij (s b_i a_j)^2 = (sum_i (s b_i)^2)(sum_j a_j^2).
// One block per sample; keeps the reduction out of the store-bound kernel above.
template <typename TIN>
__global__ __launch_bounds__(kThreads) void rank1_sumsq_kernel(const TIN* __restrict__ b,
                                                                 const TIN* __restrict__ a,
                                                                 float* __restrict__ sumsq, int64_t M,
                                                                 int64_t N, float scale) {
  __shared__ float red[kWaves];
  const int64_t sample = blockIdx.x;
  float sb = 0.f, sa = 0.f;
  for (int64_t i = threadIdx.x; i < M; i += kThreads) {
    const float v = scale * dpk_io<TIN>::load(b + sample * M + i);
    sb = fmaf(v, v, sb);
  }
  for (int64_t i = threadIdx.x; i < N; i += kThreads) {
    const float v = dpk_io<TIN>::load(a + sample * N + i);
    sa = fmaf(v, v, sa);
  }
  const float tb = block_sum<kWaves>(sb, red);
  const float ta = block_sum<kWaves>(sa, red);
  if (threadIdx.x == 0) sumsq[sample] = tb * ta;
}

// ---- T > 1 -------------------------------------------------------------------
template <int BM, int BN, typename TIN, typename TOUT, bool VEC>
__global__ __launch_bounds__(kThreads) void linear_mfma_kernel(
    const TIN* __restrict__ b, const TIN* __restrict__ a, TOUT* __restrict__ gs,
    float* __restrict__ partials, int64_t T, int64_t M, int64_t N, float scale, int64_t tiles_m,
    int64_t tiles_n) {
  __shared__ mf32::Smem<BM, BN> sm;
  __shared__ float red[kWaves];
  const int64_t per_sample = tiles_m * tiles_n;
  const int64_t sample = blockIdx.x / per_sample;
  const int64_t rem = blockIdx.x % per_sample;
  const int64_t m0 = (rem / tiles_n) * BM, n0 = (rem % tiles_n) * BN;
  mf32::LoaderMContig<BM, TIN, VEC> la(b + sample * T * M, M, m0, M, T);
  mf32::LoaderMContig<BN, TIN, VEC> lb(a + sample * T * N, N, n0, N, T);
  mf32::Tile<BM, BN> tile;
  tile.clear();
  mf32::mainloop<BM, BN>(tile, sm, la, lb, T);
  TOUT* out = gs + sample * M * N;
  float ss = 0.f;
  tile.for_each([&](int r, int c, float v) {
    const int64_t i = m0 + r, j = n0 + c;
    if (i < M && j < N) {
      const float x = v * scale;
      if (gs) dpk_io<TOUT>::store(out + i * N + j, x);
      ss = fmaf(x, x, ss);
    }
  });
  if (partials) {
    const float s = block_sum<kWaves>(ss, red);
    if (threadIdx.x == 0) partials[blockIdx.x] = s;
  }
}

// The same contraction for bf16 inputs on the bf16 matrix instruction (8 x the rate of
// the fp32 one): v_mfma_f32_32x32x16_bf16 with fp32 accumulators, operand tiles
// transposed into k-contiguous LDS rows by the loader.
template <int BM, int BN, typename TOUT, bool VEC>
__global__ __launch_bounds__(kThreads) __attribute__((amdgpu_waves_per_eu(2, 2))) void linear_mfma_bf16_kernel(
    const bf16_t* __restrict__ b, const bf16_t* __restrict__ a, TOUT* __restrict__ gs,
    float* __restrict__ partials, int64_t T, int64_t M, int64_t N, float scale, int64_t tiles_m,
    int64_t tiles_n) {
  __shared__ mb16::Smem<BM, BN> sm;
  __shared__ float red[kWaves];
  const int64_t per_sample = tiles_m * tiles_n;
  const int64_t sample = blockIdx.x / per_sample;
  const int64_t rem = blockIdx.x % per_sample;
  const int64_t m0 = (rem / tiles_n) * BM, n0 = (rem % tiles_n) * BN;
  mb16::LoaderMContig<BM, VEC> la(b + sample * T * M, M, m0, M, T);
  mb16::LoaderMContig<BN, VEC> lb(a + sample * T * N, N, n0, N, T);
  mb16::Tile<BM, BN> tile;
  tile.clear();
  mb16::mainloop_pairs<BM, BN>(tile, sm, la, lb, T);
  TOUT* out = gs + sample * M * N;
  float ss = 0.f;
  tile.for_each([&](int r, int c, float v) {
    const int64_t i = m0 + r, j = n0 + c;
    if (i < M && j < N) {
      const float x = v * scale;
      if (gs) dpk_io<TOUT>::store(out + i * N + j, x);
      ss = fmaf(x, x, ss);
    }
  });
  if (partials) {
    const float s = block_sum<kWaves>(ss, red);
    if (threadIdx.x == 0) partials[blockIdx.x] = s;
  }
}

// The same contraction with the transposition left to the LDS read (mfma_bf16_tr.h): tiles
// travel global -> LDS as they lie in memory, four k tiles deep. The product is formed
// transposed, rows = input features, columns = output features, because a lane of the
// accumulator layout owns four consecutive ROWS: that way they are four consecutive elements
// of a row of gs. Results are gathered into whole rows of the output tile in
// the (by then idle) stage memory and leave as 16-byte non-temporal stores.
// M % 8 == 0, N % 8 == 0, T >= 32, 16-byte aligned b, a and gs.
// The output tile passes through the stage memory kRows rows at a time; a row is padded so
// that the 32 rows a half-wave writes into (8 bytes each for bf16: pitch = 2 mod 64 dwords;
// 16 bytes in two passes for fp32: pitch = 4 mod 64 dwords) cover the banks once.
template <typename TOUT> struct TrOut;
template <> struct TrOut<bf16_t> { static constexpr int kPad = 8, kRows = 128; };
template <> struct TrOut<float> { static constexpr int kPad = 16, kRows = 64; };

// The two engines behind the kernel: input element type, stage memory, accumulator tile and
// main loop of mfma_bf16_tr.h (bf16, transposing LDS reads) or mfma_f32_dlds.h (fp32).
struct TrBf16 {
  typedef bf16_t elem;
  static constexpr int kBK = mb16t::BK;
  template <class C> using Smem = mb16t::Smem<C>;
  template <class C> using Tile = mb16t::Tile<C>;
  template <class C, class... A> static __device__ __forceinline__ void mainloop(A&&... args) {
    mb16t::mainloop<C>(static_cast<A&&>(args)...);
  }
  template <class C, class... A> static __device__ __forceinline__ void mainloop_weighted(A&&... args) {
    mb16t::mainloop<C, true>(static_cast<A&&>(args)...);
  }
};
struct DldsF32 {
  typedef float elem;
  static constexpr int kBK = mf32d::BK;
  template <class C> using Smem = mf32d::Smem<C>;
  template <class C> using Tile = mf32d::Tile<C>;
  template <class C, class... A> static __device__ __forceinline__ void mainloop(A&&... args) {
    mf32d::mainloop<C>(static_cast<A&&>(args)...);
  }
  template <class C, class... A> static __device__ __forceinline__ void mainloop_weighted(A&&... args) {
    mf32d::mainloop<C, true>(static_cast<A&&>(args)...);
  }
};

//
// W: a "sample" of the launch is a run of T / unit_rows units of unit_rows
// rows each (unit_rows a multiple of the k tile), and unit u of sample s counts
// coef[s * (T / unit_rows) + u] times: gs[s] = scale * sum_u coef[..] * b_u^T a_u.
// (Two waves per SIMD asked for, which these kernels reach anyway, caps W at 256 registers: the
// accumulators then live in ordinary registers, where they can be multiplied in place.)
// One block tile of the product of one "sample": the tile at (m0, n0) of out = scale * b^T a
// over T rows (b, a and out already at the sample), its sum of squares into partials[slot].
template <class E, class C, typename TOUT, bool W>
__device__ __forceinline__ void linear_dlds_tile(
    typename E::template Smem<C>& sm, float* red, const typename E::elem* __restrict__ b,
    const typename E::elem* __restrict__ a, TOUT* __restrict__ out, float* __restrict__ partials, uint32_t slot,
    int64_t T, int64_t M, int64_t N, float scale, int64_t m0, int64_t n0, const float* __restrict__ coef,
    int64_t unit_rows) {
  typedef typename E::template Smem<C> SmemT;
  // rows of the product = input features (P = a), columns = output features (Q = b)
  constexpr int BJ = C::BP, BI = C::BQ;
  constexpr int kPitch = BJ * sizeof(TOUT) + TrOut<TOUT>::kPad, kRows = TrOut<TOUT>::kRows;
  static_assert(kRows * kPitch <= sizeof(SmemT), "output rows must fit the stage memory");
  static_assert(BI % kRows == 0 && kRows % 32 == 0, "passes of whole MFMA tiles");
  TOUT* const gs = out;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int wj0 = (wave / C::WQ) * (32 * C::TP), wi0 = (wave % C::WQ) * (32 * C::TQ);  // this wave's corner
  typename E::template Tile<C> tile;
  tile.clear();
  if constexpr (W)
    E::template mainloop_weighted<C>(tile, sm, a, N, n0, b, M, m0, T, wj0, wi0, coef, unit_rows / E::kBK);
  else
    E::template mainloop<C>(tile, sm, a, N, n0, b, M, m0, T, wj0, wi0);
  const int kk = lane >> 5, l32 = lane & 31;
  float ss = 0.f;
  unsigned char* stage_out = &sm.stage[0][0];
  if (gs == nullptr) {  // only the squared norm is wanted
#pragma unroll
    for (int it = 0; it < C::TQ; ++it)
#pragma unroll
      for (int jt = 0; jt < C::TP; ++jt)
#pragma unroll
        for (int vg = 0; vg < 4; ++vg) {
          const int il = wi0 + it * 32 + l32, jl = wj0 + jt * 32 + vg * 8 + kk * 4;
          if (m0 + il < M && n0 + jl < N) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
              const float x = tile.acc[jt][it][vg * 4 + e] * scale;
              ss = fmaf(x, x, ss);
            }
          }
        }
  }
  // In a pass the waves that own rows [pass * kRows, + kRows) of the tile put them into the
  // stage memory, then all threads send whole rows on their way.
#pragma unroll
  for (int pass = 0; gs != nullptr && pass < BI / kRows; ++pass) {
    if (pass > 0) __syncthreads();
#pragma unroll
    for (int it = 0; it < C::TQ; ++it) {
      if ((wi0 + it * 32) / kRows != pass) continue;  // wave-uniform
#pragma unroll
      for (int jt = 0; jt < C::TP; ++jt)
#pragma unroll
        for (int vg = 0; vg < 4; ++vg) {
          const int il = wi0 + it * 32 + l32, jl = wj0 + jt * 32 + vg * 8 + kk * 4;
          float4 x;
          x.x = tile.acc[jt][it][vg * 4 + 0] * scale;
          x.y = tile.acc[jt][it][vg * 4 + 1] * scale;
          x.z = tile.acc[jt][it][vg * 4 + 2] * scale;
          x.w = tile.acc[jt][it][vg * 4 + 3] * scale;
          // N % 4 == 0: the four columns are inside or outside together
          if (m0 + il < M && n0 + jl < N) ss = fmaf(x.x, x.x, fmaf(x.y, x.y, fmaf(x.z, x.z, fmaf(x.w, x.w, ss))));
          dpk_io<TOUT>::store4(reinterpret_cast<TOUT*>(stage_out + (il - pass * kRows) * kPitch) + jl, x);
        }
    }
    __syncthreads();
    constexpr int kChunksPerRow = BJ * sizeof(TOUT) / 16, kPerChunk = 16 / sizeof(TOUT);
    static_assert(kRows * kChunksPerRow % C::kThreads == 0, "whole trips of the block over the rows");
#pragma unroll
    for (int r = 0; r < kRows * kChunksPerRow / C::kThreads; ++r) {
      const int idx = threadIdx.x + r * C::kThreads;
      const int il = idx / kChunksPerRow, c = idx % kChunksPerRow;
      const int64_t i = m0 + pass * kRows + il, j = n0 + c * kPerChunk;
      if (i < M && j < N) {  // N is a multiple of the chunk: whole chunks
        const uint2* src = reinterpret_cast<const uint2*>(stage_out + il * kPitch + c * 16);
        const uint2 lo = src[0], hi = src[1];
        typedef uint32_t vu4 __attribute__((ext_vector_type(4)));
        vu4 w;
        w.x = lo.x;
        w.y = lo.y;
        w.z = hi.x;
        w.w = hi.y;
        __builtin_nontemporal_store(w, reinterpret_cast<vu4*>(out + i * N + j));
      }
    }
  }
  if (partials) {
    const float s = block_sum<C::kWaves>(ss, red);
    if (threadIdx.x == 0) partials[slot] = s;
  }
}

template <class E, class C, typename TOUT, bool W = false>
__global__ __launch_bounds__(C::kThreads, W ? 2 : 1) void linear_dlds_kernel(
    const typename E::elem* __restrict__ b, const typename E::elem* __restrict__ a, TOUT* __restrict__ gs,
    float* __restrict__ partials, int64_t T, int64_t M, int64_t N, float scale, int64_t tiles_m,
    int64_t tiles_n, const float* __restrict__ coef = nullptr, int64_t unit_rows = 0) {
  __shared__ typename E::template Smem<C> sm;
  __shared__ float red[C::kWaves];
  // neighbouring tiles of a sample share operand panels: keep them on one XCD
  const uint32_t bid = xcd_contiguous_id(blockIdx.x, gridDim.x);
  const int64_t per_sample = tiles_m * tiles_n;
  const int64_t sample = bid / per_sample;
  const int64_t rem = bid % per_sample;
  const float* c = coef;
  if constexpr (W) c = coef + sample * (T / unit_rows);  // this run of samples' coefficients
  linear_dlds_tile<E, C, TOUT, W>(sm, red, b + sample * T * M, a + sample * T * N, gs ? gs + sample * M * N : gs, partials,
                                  bid, T, M, N, scale, (rem / tiles_n) * C::BQ, (rem % tiles_n) * C::BP, c, unit_rows);
}

// The clip-weighted sums of up to kWsumMax Linear layers in one launch: block -> (layer, tile)
// through the prefix sums of the layers' tile counts. A layer on its own fills the GPU in
// whole rounds of blocks only by luck (22 x 8 tiles of 256 x 256 on 256 CUs leave 80 idle for
// the whole contraction); pooled, the layers' tiles follow one another without a gap.
constexpr int kWsumMax = 32;
struct WsumMultiArgs {
  const bf16_t* b[kWsumMax];
  const bf16_t* a[kWsumMax];
  const float* coef[kWsumMax];
  void* out[kWsumMax];
  int64_t rows[kWsumMax];       // n * T
  int32_t unit_rows[kWsumMax];  // T
  int32_t M[kWsumMax], N[kWsumMax];
  int32_t tiles_n[kWsumMax];  // tiles along N, columns of tiles varying fastest; or minus the tiles along M, rows fastest
  uint32_t tile_prefix[kWsumMax + 1];  // blocks of the layers before: tiles x pieces
  float scale[kWsumMax];
  int32_t nlayers;
  // pieces > 1: a layer's samples are cut into that many runs, each with blocks of its own; piece p of
  // layer l leaves its fp32 sum at part[l] + p * M * N and add_pieces_multi_kernel adds the pieces
  int32_t pieces;
  float* part[kWsumMax];
};

template <class C, typename TOUT>
__global__ __launch_bounds__(C::kThreads, 2) void linear_wsum_multi_kernel(const WsumMultiArgs A) {
  __shared__ typename TrBf16::template Smem<C> sm;
  __shared__ float red[C::kWaves];
  // consecutive tiles (one layer, neighbouring operand panels) on one XCD
  const uint32_t bid = xcd_contiguous_id(blockIdx.x, gridDim.x);
  int l = 0;
  while (l + 1 < A.nlayers && bid >= A.tile_prefix[l + 1]) ++l;
  // Tiles that run at the same time on an XCD should need few operand panels between them: with
  // the shorter tile dimension varying fastest, a CU-count's worth of consecutive tiles is a
  // block of a few rows by a few columns rather than a strip across the wide dimension.
  uint32_t rem = bid - A.tile_prefix[l];
  const uint32_t per_piece = (A.tile_prefix[l + 1] - A.tile_prefix[l]) / static_cast<uint32_t>(A.pieces);
  const uint32_t piece = rem / per_piece;  // a piece's tiles are consecutive: its operand rows stay in one L2
  rem -= piece * per_piece;
  const int32_t tn = A.tiles_n[l];  // negative: rows of tiles vary fastest, -tn rows
  const uint32_t tm_i = tn > 0 ? rem / static_cast<uint32_t>(tn) : rem % static_cast<uint32_t>(-tn);
  const uint32_t tn_i = tn > 0 ? rem % static_cast<uint32_t>(tn) : rem / static_cast<uint32_t>(-tn);
  const int64_t rows = A.rows[l] / A.pieces, row0 = rows * piece;
  const int64_t M = A.M[l], N = A.N[l];
  TOUT* out = static_cast<TOUT*>(A.out[l]);
  if constexpr (std::is_same<TOUT, float>::value) {
    if (A.pieces > 1) out = A.part[l] + static_cast<int64_t>(piece) * M * N;
  }
  linear_dlds_tile<TrBf16, C, TOUT, true>(sm, red, A.b[l] + row0 * M, A.a[l] + row0 * N, out, nullptr, 0u, rows, M, N,
                                          A.scale[l], static_cast<int64_t>(tm_i) * C::BQ,
                                          static_cast<int64_t>(tn_i) * C::BP,
                                          A.coef[l] + row0 / A.unit_rows[l], A.unit_rows[l]);
}

// out[l][e] = sum_p part[l][p * count + e] for the layers of a pooled launch, four elements per thread.
struct AddPiecesMultiArgs {
  const float* part[kWsumMax];
  void* out[kWsumMax];
  int64_t count4[kWsumMax];
  uint32_t block_prefix[kWsumMax + 1];
  int32_t nlayers, pieces;
};

template <typename TOUT>
__global__ __launch_bounds__(kThreads) void add_pieces_multi_kernel(const AddPiecesMultiArgs A) {
  int l = 0;
  while (l + 1 < A.nlayers && blockIdx.x >= A.block_prefix[l + 1]) ++l;
  const int64_t e = static_cast<int64_t>(blockIdx.x - A.block_prefix[l]) * kThreads + threadIdx.x;
  const int64_t count4 = A.count4[l];
  if (e >= count4) return;
  typedef float vf4 __attribute__((ext_vector_type(4)));
  const vf4* src = reinterpret_cast<const vf4*>(A.part[l]) + e;
  vf4 sum = __builtin_nontemporal_load(src);
  for (int p = 1; p < A.pieces; ++p) sum += __builtin_nontemporal_load(src + p * count4);
  dpk_io<TOUT>::store4(static_cast<TOUT*>(A.out[l]) + 4 * e, make_float4(sum.x, sum.y, sum.z, sum.w));
}

using DldsF32Cfg = mf32d::Config<2, 2, 2, 2, 4>;  // 128 x 128, 4 waves, 64 KB: two blocks per CU
using TrSmall = mb16t::Config<2, 2, 2, 2, 4>;  // 128 x 128, 4 waves, 64 KB: two blocks per CU
using TrLarge = mb16t::Config<4, 2, 2, 4, 4>;  // 256 x 256, 8 waves, 128 KB: one block per CU
// time of a 256 x 256 block relative to four 128 x 128 blocks run two at a time
constexpr double kTrLargeGain = 0.9;

// ---- bias / row sums -----------------------------------------------------------
// out[n,k] = scale * sum_t b[n,t,k]; threads along k, RS row groups along t.
template <typename TIN, typename TOUT, int RS>
__global__ __launch_bounds__(kThreads) void colsum_kernel(const TIN* __restrict__ b,
                                                            TOUT* __restrict__ out, int64_t T,
                                                            int64_t Kdim, float scale,
                                                            int64_t blocks_per_sample) {
  constexpr int CX = kThreads / RS;
  __shared__ float part[kThreads];
  const int64_t sample = blockIdx.x / blocks_per_sample;
  const int64_t k = (blockIdx.x % blocks_per_sample) * CX + threadIdx.x % CX;
  const int ry = threadIdx.x / CX;
  float acc = 0.f;
  if (k < Kdim) {
    const TIN* p = b + sample * T * Kdim + k;
    for (int64_t t = ry; t < T; t += RS) acc += dpk_io<TIN>::load(p + t * Kdim);
  }
  if (RS > 1) {
    part[threadIdx.x] = acc;
    __syncthreads();
    if (ry != 0) return;
#pragma unroll
    for (int j = 1; j < RS; ++j) acc += part[j * CX + threadIdx.x];
  }
  if (k < Kdim) dpk_io<TOUT>::store(out + sample * Kdim + k, acc * scale);
}

// The same with four consecutive columns per thread (16-byte loads for fp32, 8-byte for bf16)
// and eight rows of loads in flight, kept as loaded until all eight are issued. K % 4 == 0,
// b and out aligned to four elements.
template <typename TIN, typename TOUT, int RS>
__global__ __launch_bounds__(kThreads) void colsum4_kernel(const TIN* __restrict__ b, TOUT* __restrict__ out,
                                                             int64_t T, int64_t Kdim, float scale,
                                                             int64_t blocks_per_sample) {
  constexpr int CXT = kThreads / RS, U = 8;
  __shared__ float4 part[kThreads];
  const int64_t sample = blockIdx.x / blocks_per_sample;
  const int64_t k = ((blockIdx.x % blocks_per_sample) * CXT + threadIdx.x % CXT) * 4;
  const int ry = threadIdx.x / CXT;
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  auto add = [&](float4 v) {
    acc.x += v.x;
    acc.y += v.y;
    acc.z += v.z;
    acc.w += v.w;
  };
  if (k < Kdim) {
    const TIN* p = b + sample * T * Kdim + k;
    int64_t t = ry;
    for (; t + (U - 1) * RS < T; t += U * RS) {
      typename dpk_io<TIN>::raw4 x[U];
#pragma unroll
      for (int u = 0; u < U; ++u) x[u] = dpk_io<TIN>::load4_raw(p + (t + u * RS) * Kdim);
#pragma unroll
      for (int u = 0; u < U; ++u) add(dpk_io<TIN>::unpack4(x[u]));
    }
    for (; t < T; t += RS) add(dpk_io<TIN>::unpack4(dpk_io<TIN>::load4_raw(p + t * Kdim)));
  }
  if (RS > 1) {
    part[threadIdx.x] = acc;
    __syncthreads();
    if (ry != 0) return;
#pragma unroll
    for (int j = 1; j < RS; ++j) add(part[j * CXT + threadIdx.x]);
  }
  if (k < Kdim) {
    acc.x *= scale;
    acc.y *= scale;
    acc.z *= scale;
    acc.w *= scale;
    dpk_io<TOUT>::store4(out + sample * Kdim + k, acc);
  }
}

// out[r] = scale * sum_q b[r,q]: one wave per row (conv bias, conv.py:117). VEC: rows of whole,
// aligned 4-element chunks, read four chunks a lane at a time with all of them in flight.
template <typename TIN, typename TOUT, bool VEC>
__global__ __launch_bounds__(kThreads) void rowsum_kernel(const TIN* __restrict__ b,
                                                            TOUT* __restrict__ out, int64_t rows,
                                                            int64_t q, float scale) {
  const int64_t w = (static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x) / DPK_WAVE;
  const int lane = threadIdx.x & (DPK_WAVE - 1);
  if (w >= rows) return;
  const TIN* p = b + w * q;
  float s = 0.f;
  if (VEC) {
    constexpr int U = 4, kStep = DPK_WAVE * 4;
    int64_t i = lane * 4;
    for (; i + (U - 1) * kStep < q; i += U * kStep) {
      typename dpk_io<TIN>::raw4 x[U];
#pragma unroll
      for (int u = 0; u < U; ++u) x[u] = dpk_io<TIN>::load4_raw(p + i + u * kStep);
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const float4 v = dpk_io<TIN>::unpack4(x[u]);
        s += (v.x + v.y) + (v.z + v.w);
      }
    }
    for (; i < q; i += kStep) {
      const float4 v = dpk_io<TIN>::unpack4(dpk_io<TIN>::load4_raw(p + i));
      s += (v.x + v.y) + (v.z + v.w);
    }
  } else {
    for (int64_t i = lane; i < q; i += DPK_WAVE) s += dpk_io<TIN>::load(p + i);
  }
  s = wave_sum(s);
  if (lane == 0) dpk_io<TOUT>::store(out + w, s * scale);
}

struct Plan {
  bool outer;
  int cx_log2;
  int rows_pb;
  int bm;
  int tr;  // 0, or the tile edge of the transposing-read bf16 kernel (it replaces bm)
  int64_t tiles_m, tiles_n;
};

Plan make_plan(int64_t T, int64_t M, int64_t N, bool vec) {
  Plan p;
  p.tr = 0;
  p.outer = (T == 1);
  if (p.outer) {
    const int64_t cols = dpk_cdiv(N, vec ? 4 : 1);
    // column threads per block: 8, 32, 128 or 256 (the instantiated shapes)
    const int lg = cols > 128 ? 8 : cols > 32 ? 7 : cols > 8 ? 5 : 3;
    p.cx_log2 = lg;
    p.bm = 0;
    p.rows_pb = kOuterRowsPerThread * (kThreads >> lg);
    p.tiles_m = dpk_cdiv(M, p.rows_pb);
    p.tiles_n = dpk_cdiv(cols, 1LL << lg);
  } else {
    p.cx_log2 = 0;
    p.rows_pb = 0;
    p.bm = (M > 64 && N > 64) ? 128 : 64;
    p.tiles_m = dpk_cdiv(M, p.bm);
    p.tiles_n = dpk_cdiv(N, p.bm);
  }
  return p;
}

// Whether the transposing-read bf16 kernel takes the shape, and with which tile: whole
// 16-byte chunks, at least one whole k tile, per-lane byte offsets inside a k tile that fit
// 32 bits. The 256-tile blocks move half the operand bytes per product and run one to a
// CU; the 128-tile blocks two to a CU. The cheaper of the two by rounds of resident blocks
// times work per block wins. `tile` (DPK_TILE_128 or DPK_TILE_256) overrides the choice
// (for tests that want both kernels on small shapes).
void plan_tr(Plan& p, const void* b, const void* a, const void* gs, int64_t n, int64_t T, int64_t M, int64_t N,
             int cus, int tile) {
  if (cus <= 0) cus = 256;
  if (p.outer || p.bm != 128 || T < mb16t::BK || M % 8 != 0 || N % 8 != 0 || M >= (1LL << 24) || N >= (1LL << 24) ||
      !dpk_aligned(b, 16) || !dpk_aligned(a, 16) || !dpk_aligned(gs, 16))
    return;
  const int64_t small = n * dpk_cdiv(M, 128) * dpk_cdiv(N, 128), large = n * dpk_cdiv(M, 256) * dpk_cdiv(N, 256);
  const double cost_small = static_cast<double>(dpk_cdiv(small, 2 * cus)) * 2.0;
  const double cost_large = static_cast<double>(dpk_cdiv(large, cus)) * 4.0 * kTrLargeGain;
  p.tr = (M >= 256 && N >= 256 && cost_large < cost_small) ? 256 : 128;
  if (tile != DPK_TILE_AUTO) p.tr = tile == DPK_TILE_256 ? 256 : 128;
  p.bm = p.tr;
  p.tiles_m = dpk_cdiv(M, p.tr);
  p.tiles_n = dpk_cdiv(N, p.tr);
}

// Whether the direct-load fp32 kernel takes the shape: whole 16-byte chunks, at least one whole
// k tile, a bf16 result only in whole 16-byte chunks too. Same 128 x 128 tiling as the plan.
void plan_dlds_f32(Plan& p, const void* b, const void* a, const void* gs, int gs_dtype, int64_t T, int64_t M,
                   int64_t N) {
  const int64_t out_chunk = gs_dtype == DPK_BF16 ? 8 : 4;
  if (p.outer || p.bm != 128 || T < mf32d::BK || M % 4 != 0 || N % out_chunk != 0 || M >= (1LL << 24) || N >= (1LL << 24) ||
      !dpk_aligned(b, 16) || !dpk_aligned(a, 16) || !dpk_aligned(gs, 16))
    return;
  p.tr = 128;
}

template <typename TIN, typename TOUT>
void launch_linear(const Plan& p, bool vec, const void* b, const void* a, void* gs, float* partials,
                   int64_t n, int64_t T, int64_t M, int64_t N, float scale, hipStream_t s) {
  const dim3 grid(static_cast<unsigned>(n * p.tiles_m * p.tiles_n)), block(kThreads);
  const TIN* bp = static_cast<const TIN*>(b);
  const TIN* ap = static_cast<const TIN*>(a);
  TOUT* gp = static_cast<TOUT*>(gs);
  if (p.outer) {
#define DPK_OUTER(V, LG)                                                                          \
  hipLaunchKernelGGL((linear_outer_kernel<TIN, TOUT, V, LG>), grid, block, 0, s, bp, ap, gp, M, N, \
                     scale, static_cast<uint32_t>(p.tiles_m), static_cast<uint32_t>(p.tiles_n))
    const int64_t cols4 = N / 4, chunks = M * cols4;
    const int64_t bps = dpk_cdiv(chunks, kSeqThreads);
    const bool wide16 = sizeof(TOUT) == 2 && N % 8 == 0 && dpk_aligned(gs, 16);
    if (vec && wide16 && n * dpk_cdiv(chunks / 2, kSeqThreads) <= DPK_MAX_GRID_X && chunks / 2 < (1LL << 32)) {
      if constexpr (sizeof(TOUT) == 2) {
        const int64_t bps8 = dpk_cdiv(chunks / 2, kSeqThreads);
        hipLaunchKernelGGL((linear_outer_seq_kernel<TIN, TOUT, 8>), dim3(static_cast<unsigned>(n * bps8)),
                           dim3(kSeqThreads), 0, s, bp, ap, gp, static_cast<uint32_t>(M), static_cast<uint32_t>(N / 8),
                           scale, static_cast<uint32_t>(bps8));
      }
    } else if (vec && chunks < (1LL << 32) && n * bps <= DPK_MAX_GRID_X) {
      hipLaunchKernelGGL((linear_outer_seq_kernel<TIN, TOUT, 4>), dim3(static_cast<unsigned>(n * bps)),
                         dim3(kSeqThreads), 0, s, bp, ap, gp, static_cast<uint32_t>(M), static_cast<uint32_t>(cols4), scale,
                         static_cast<uint32_t>(bps));
    } else if (vec) {
      if (p.cx_log2 == 8) DPK_OUTER(true, 8);
      else if (p.cx_log2 == 7) DPK_OUTER(true, 7);
      else if (p.cx_log2 == 5) DPK_OUTER(true, 5);
      else DPK_OUTER(true, 3);
    } else {
      if (p.cx_log2 == 8) DPK_OUTER(false, 8);
      else if (p.cx_log2 == 7) DPK_OUTER(false, 7);
      else if (p.cx_log2 == 5) DPK_OUTER(false, 5);
      else DPK_OUTER(false, 3);
    }
#undef DPK_OUTER
  } else if constexpr (std::is_same<TIN, bf16_t>::value) {
    // 16-byte rows of 8 elements for the transposing loader
    const bool vec8 = M % 8 == 0 && N % 8 == 0 && dpk_aligned(b, 16) && dpk_aligned(a, 16) &&
                      T * (M > N ? M : N) * 2 < (1LL << 30);
#define DPK_BF16(BMN, V)                                                                              \
  hipLaunchKernelGGL((linear_mfma_bf16_kernel<BMN, BMN, TOUT, V>), grid, block, 0, s, bp, ap, gp, partials, \
                     T, M, N, scale, p.tiles_m, p.tiles_n)
    if (p.tr == 256) {
      hipLaunchKernelGGL((linear_dlds_kernel<TrBf16, TrLarge, TOUT>), grid, dim3(TrLarge::kThreads), 0, s, bp, ap, gp,
                         partials, T, M, N, scale, p.tiles_m, p.tiles_n);
    } else if (p.tr == 128) {
      hipLaunchKernelGGL((linear_dlds_kernel<TrBf16, TrSmall, TOUT>), grid, dim3(TrSmall::kThreads), 0, s, bp, ap, gp,
                         partials, T, M, N, scale, p.tiles_m, p.tiles_n);
    } else if (p.bm == 128) {
      if (vec8) DPK_BF16(128, true);
      else DPK_BF16(128, false);
    } else {
      if (vec8) DPK_BF16(64, true);
      else DPK_BF16(64, false);
    }
#undef DPK_BF16
  } else if (p.tr == 128) {
    hipLaunchKernelGGL((linear_dlds_kernel<DldsF32, DldsF32Cfg, TOUT>), grid, dim3(DldsF32Cfg::kThreads), 0, s, bp, ap,
                       gp, partials, T, M, N, scale, p.tiles_m, p.tiles_n);
  } else if (p.bm == 128) {
    if (vec)
      hipLaunchKernelGGL((linear_mfma_kernel<128, 128, TIN, TOUT, true>), grid, block, 0, s, bp, ap,
                         gp, partials, T, M, N, scale, p.tiles_m, p.tiles_n);
    else
      hipLaunchKernelGGL((linear_mfma_kernel<128, 128, TIN, TOUT, false>), grid, block, 0, s, bp, ap,
                         gp, partials, T, M, N, scale, p.tiles_m, p.tiles_n);
  } else {
    if (vec)
      hipLaunchKernelGGL((linear_mfma_kernel<64, 64, TIN, TOUT, true>), grid, block, 0, s, bp, ap,
                         gp, partials, T, M, N, scale, p.tiles_m, p.tiles_n);
    else
      hipLaunchKernelGGL((linear_mfma_kernel<64, 64, TIN, TOUT, false>), grid, block, 0, s, bp, ap,
                         gp, partials, T, M, N, scale, p.tiles_m, p.tiles_n);
  }
}

// out[e] = sum_p part[p * count + e], four elements per thread (count % 4 == 0).
template <typename TOUT>
__global__ __launch_bounds__(kThreads) void add_pieces_kernel(const float* __restrict__ part, TOUT* __restrict__ out,
                                                            int64_t count4, int pieces) {
  const int64_t e = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (e >= count4) return;
  typedef float vf4 __attribute__((ext_vector_type(4)));
  const vf4* src = reinterpret_cast<const vf4*>(part) + e;
  vf4 sum = __builtin_nontemporal_load(src);
  for (int p = 1; p < pieces; ++p) sum += __builtin_nontemporal_load(src + p * count4);
  const float4 acc = make_float4(sum.x, sum.y, sum.z, sum.w);
  dpk_io<TOUT>::store4(out + 4 * e, acc);
}

// ---- clip-weighted sums for the shapes and dtypes the transposing-read kernel does not take ----
// w[r] = coef[r / T] for the n * T rows of a layer's operands: the weight of a row.
__global__ __launch_bounds__(kThreads) void row_weights_kernel(const float* __restrict__ coef, float* __restrict__ w,
                                                                 int64_t rows, int64_t T) {
  const int64_t r = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (r < rows) w[r] = coef[r / T];
}

// LoaderMContig whose rows are multiplied by their weights on the way into LDS (in fp32, as the
// reference multiplies the backprops by the coefficients before its second pass,
// fast_gradient_clipping_utils.py:193-196; bf16 rows are widened first, which is exact).
template <int BMN, typename T, bool VEC>
struct LoaderMContigWeighted : mf32::LoaderMContig<BMN, T, VEC> {
  typedef mf32::LoaderMContig<BMN, T, VEC> Base;
  const float* w;
  __device__ __forceinline__ LoaderMContigWeighted(const T* base_, int64_t ld_, int64_t m0_, int64_t M_, int64_t K_,
                                                   const float* w_)
      : Base(base_, ld_, m0_, M_, K_), w(w_) {}
  __device__ __forceinline__ void fetch(int64_t k0) {
    Base::fetch(k0);
#pragma unroll
    for (int r = 0; r < Base::R; ++r) {
      const int idx = threadIdx.x + r * mf32::NTHREADS;
      const int64_t k = k0 + idx / (BMN / 4);
      const float c = k < this->K ? w[k] : 0.f;
      this->st[r].x *= c;
      this->st[r].y *= c;
      this->st[r].z *= c;
      this->st[r].w *= c;
    }
  }
};

// out (or piece p's fp32 partial) = scale * sum_r w[r] * b[r, :]^T a[r, :] over the rows of piece p,
// on the fp32 MFMA whatever the input type: any T, any feature sizes, any alignment.
template <int BM, int BN, typename TIN, typename TOUT, bool VEC>
__global__ __launch_bounds__(kThreads) void linear_wsum_generic_kernel(
    const TIN* __restrict__ b, const TIN* __restrict__ a, const float* __restrict__ w, TOUT* __restrict__ out,
    int64_t rows, int64_t rows_per_piece, int64_t M, int64_t N, float scale, int64_t tiles_m, int64_t tiles_n) {
  __shared__ mf32::Smem<BM, BN> sm;
  const int64_t per_piece = tiles_m * tiles_n;
  const int64_t piece = blockIdx.x / per_piece;
  const int64_t rem = blockIdx.x % per_piece;
  const int64_t m0 = (rem / tiles_n) * BM, n0 = (rem % tiles_n) * BN;
  const int64_t k0 = piece * rows_per_piece;
  const int64_t k1 = k0 + rows_per_piece < rows ? k0 + rows_per_piece : rows;
  LoaderMContigWeighted<BM, TIN, VEC> la(b, M, m0, M, k1, w);
  mf32::LoaderMContig<BN, TIN, VEC> lb(a, N, n0, N, k1);
  mf32::Tile<BM, BN> tile;
  tile.clear();
  if (k0 < k1) mf32::mainloop<BM, BN>(tile, sm, la, lb, k0, k1);
  TOUT* dst = out + piece * M * N;
  tile.for_each([&](int r, int c, float v) {
    const int64_t i = m0 + r, j = n0 + c;
    if (i < M && j < N) dpk_io<TOUT>::store(dst + i * N + j, v * scale);
  });
}

// part[chunk, k] = sum over the chunk's rows of w[r] * b[r, k]: thread <-> 4 columns (VEC) or one,
// eight rows of loads in flight.
template <typename TIN, bool VEC>
__global__ __launch_bounds__(kThreads) void wcolsum_partial_kernel(const TIN* __restrict__ b, const float* __restrict__ w,
                                                                     float* __restrict__ part, int64_t rows,
                                                                     int64_t rows_per_chunk, int64_t Kdim,
                                                                     int64_t col_blocks) {
  constexpr int W = VEC ? 4 : 1, U = 8;
  const int64_t chunk = blockIdx.x / col_blocks;
  const int64_t k = ((blockIdx.x % col_blocks) * kThreads + threadIdx.x) * W;
  if (k >= Kdim) return;
  const int64_t r0 = chunk * rows_per_chunk;
  const int64_t r1 = r0 + rows_per_chunk < rows ? r0 + rows_per_chunk : rows;
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  const TIN* p = b + k;
  int64_t r = r0;
  if (VEC) {
    for (; r + U <= r1; r += U) {
      typename dpk_io<TIN>::raw4 x[U];
#pragma unroll
      for (int u = 0; u < U; ++u) x[u] = dpk_io<TIN>::load4_raw(p + (r + u) * Kdim);
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const float4 v = dpk_io<TIN>::unpack4(x[u]);
        const float c = w[r + u];
        acc.x = fmaf(c, v.x, acc.x);
        acc.y = fmaf(c, v.y, acc.y);
        acc.z = fmaf(c, v.z, acc.z);
        acc.w = fmaf(c, v.w, acc.w);
      }
    }
  }
  for (; r < r1; ++r) {
    const float c = w[r];
    if (VEC) {
      const float4 v = dpk_io<TIN>::load4(p + r * Kdim);
      acc.x = fmaf(c, v.x, acc.x);
      acc.y = fmaf(c, v.y, acc.y);
      acc.z = fmaf(c, v.z, acc.z);
      acc.w = fmaf(c, v.w, acc.w);
    } else {
      acc.x = fmaf(c, dpk_io<TIN>::load(p + r * Kdim), acc.x);
    }
  }
  float* o = part + chunk * Kdim + k;
  if (VEC) {
    *reinterpret_cast<float4*>(o) = acc;
  } else {
    *o = acc.x;
  }
}

// out[k] = scale * sum_chunk part[chunk, k]: a block owns 64 columns, its four waves take every fourth
// chunk each (eight loads in flight) and their sums meet in LDS; the order of addition is fixed.
template <typename TOUT>
__global__ __launch_bounds__(kThreads) void wcolsum_final_kernel(const float* __restrict__ part, TOUT* __restrict__ out,
                                                                   int64_t chunks, int64_t Kdim, float scale) {
  __shared__ float red[kWaves][DPK_WAVE];
  const int lane = threadIdx.x & (DPK_WAVE - 1), wave = threadIdx.x / DPK_WAVE;
  const int64_t k = static_cast<int64_t>(blockIdx.x) * DPK_WAVE + lane;
  float s = 0.f;
  if (k < Kdim) {
    constexpr int U = 8;
    int64_t c = wave;
    for (; c + (U - 1) * kWaves < chunks; c += U * kWaves) {
      float x[U];
#pragma unroll
      for (int u = 0; u < U; ++u) x[u] = part[(c + u * kWaves) * Kdim + k];
#pragma unroll
      for (int u = 0; u < U; ++u) s += x[u];
    }
    for (; c < chunks; c += kWaves) s += part[c * Kdim + k];
  }
  red[wave][lane] = s;
  __syncthreads();
  if (wave == 0 && k < Kdim) {
    float t = red[0][lane];
#pragma unroll
    for (int w = 1; w < kWaves; ++w) t += red[w][lane];
    dpk_io<TOUT>::store(out + k, t * scale);
  }
}

bool linear_vec(const void* b, const void* a, const void* gs, int in_dtype, int gs_dtype, int64_t M,
                int64_t N) {
  const size_t ia = in_dtype == DPK_BF16 ? 8 : 16, oa = gs_dtype == DPK_BF16 ? 8 : 16;
  return M % 4 == 0 && N % 4 == 0 && dpk_aligned(b, ia) && dpk_aligned(a, ia) && dpk_aligned(gs, oa);
}

}  // namespace

extern "C" size_t dpk_linear_gs_workspace_bytes(int64_t n, int64_t T, int64_t out, int64_t in) {
  if (n <= 0 || T <= 1 || out <= 0 || in <= 0) return 0;  // the rank-one path needs none
  // The scalar plan never has fewer blocks than the vector plan.
  const Plan p = make_plan(T, out, in, false);
  return dpk_align_up(static_cast<size_t>(n * p.tiles_m * p.tiles_n) * sizeof(float), 256);
}

extern "C" int dpk_linear_gs(const void* b, const void* a, int in_dtype, void* gs, int gs_dtype,
                             float* sumsq, int64_t n, int64_t T, int64_t out, int64_t in,
                             float scale, int tile, void* ws, size_t ws_bytes, dpk_stream_t stream) {
  const char* who = "dpk_linear_gs";
  DPK_REQUIRE(tile == DPK_TILE_AUTO || tile == DPK_TILE_128 || tile == DPK_TILE_256, DPK_E_ARG, "%s: tile %d", who,
              tile);
  DPK_REQUIRE(n >= 0 && T >= 1 && out >= 1 && in >= 1, DPK_E_SHAPE,
              "%s: n=%lld T=%lld out=%lld in=%lld", who, (long long)n, (long long)T, (long long)out,
              (long long)in);
  if (n == 0) return DPK_OK;
  DPK_REQUIRE(b && a && (gs || sumsq), DPK_E_ARG, "%s: NULL tensor", who);
  DPK_REQUIRE(dpk_dtype_ok(in_dtype) && dpk_dtype_ok(gs_dtype), DPK_E_DTYPE, "%s: dtypes %d,%d", who,
              in_dtype, gs_dtype);
  DPK_REQUIRE(dpk_aligned(b, dpk_elsize(in_dtype)) && dpk_aligned(a, dpk_elsize(in_dtype)) &&
                  dpk_aligned(gs, dpk_elsize(gs_dtype)),
              DPK_E_ALIGN, "%s: misaligned tensor", who);
  const bool vec = linear_vec(b, a, gs, in_dtype, gs_dtype, out, in);
  Plan p = make_plan(T, out, in, vec);
  if (in_dtype == DPK_BF16) plan_tr(p, b, a, gs, n, T, out, in, dpk_device_cus(), tile);
  else plan_dlds_f32(p, b, a, gs, gs_dtype, T, out, in);
  const int64_t blocks = n * p.tiles_m * p.tiles_n;
  DPK_REQUIRE(blocks <= DPK_MAX_GRID_X, DPK_E_SHAPE, "%s: %lld blocks exceed the grid limit", who,
              (long long)blocks);
  float* partials = nullptr;
  if (sumsq && !p.outer) {
    const size_t need = static_cast<size_t>(blocks) * sizeof(float);
    DPK_REQUIRE(ws && ws_bytes >= need, DPK_E_WORKSPACE, "%s: workspace %zu < %zu bytes", who,
                ws_bytes, need);
    DPK_REQUIRE(dpk_aligned(ws, 4), DPK_E_ALIGN, "%s: workspace misaligned", who);
    partials = static_cast<float*>(ws);
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (sumsq && p.outer) {
    // Ahead of the store-bound kernel: the operands are still warm from the backward
    // pass, and the pass leaves them in the cache for the kernel that follows.
    if (in_dtype == DPK_F32)
      hipLaunchKernelGGL(rank1_sumsq_kernel<float>, dim3(static_cast<unsigned>(n)), dim3(kThreads), 0, s,
                         static_cast<const float*>(b), static_cast<const float*>(a), sumsq, out, in, scale);
    else
      hipLaunchKernelGGL(rank1_sumsq_kernel<bf16_t>, dim3(static_cast<unsigned>(n)), dim3(kThreads), 0, s,
                         static_cast<const bf16_t*>(b), static_cast<const bf16_t*>(a), sumsq, out, in, scale);
    DPK_LAUNCH_CHECK(who);
  }
  if (p.outer && !gs)
    ;  // norm only, rank one: the closed form above is the whole answer
  else if (in_dtype == DPK_F32 && gs_dtype == DPK_F32)
    launch_linear<float, float>(p, vec, b, a, gs, partials, n, T, out, in, scale, s);
  else if (in_dtype == DPK_BF16 && gs_dtype == DPK_BF16)
    launch_linear<bf16_t, bf16_t>(p, vec, b, a, gs, partials, n, T, out, in, scale, s);
  else if (in_dtype == DPK_BF16 && gs_dtype == DPK_F32)
    launch_linear<bf16_t, float>(p, vec, b, a, gs, partials, n, T, out, in, scale, s);
  else
    launch_linear<float, bf16_t>(p, vec, b, a, gs, partials, n, T, out, in, scale, s);
  DPK_LAUNCH_CHECK(who);
  if (sumsq && !p.outer) {
    dpk_launch_reduce_rows(partials, n, p.tiles_m * p.tiles_n, sumsq, 0, 1.f, s);
    DPK_LAUNCH_CHECK(who);
  }
  return DPK_OK;
}

namespace {
// Whether the transposing-read bf16 kernel takes the layer (the fast path of dpk_linear_weighted_sum
// and the only one of dpk_linear_weighted_sum_multi).
bool wsum_fast_shape(int in_dtype, int64_t T, int64_t out, int64_t in) {
  return in_dtype == DPK_BF16 && T % mb16t::BK == 0 && out % 8 == 0 && in % 8 == 0 && out > 64 && in > 64 &&
         out < (1LL << 24) && in < (1LL << 24);
}
// ... and the direct-load fp32 kernel with the coefficients on its accumulators
bool wsum_fast_shape_f32(int in_dtype, int out_dtype, int64_t T, int64_t out, int64_t in) {
  return in_dtype == DPK_F32 && T % mf32d::BK == 0 && out % 4 == 0 && in % (out_dtype == DPK_BF16 ? 8 : 4) == 0 &&
         out > 64 && in > 64 && out < (1LL << 24) && in < (1LL << 24);
}

struct WsumGenericLayout {
  size_t weights, total;  // [0, weights): float[n * T] row weights; then float[pieces, out, in] when pieces > 1
};
WsumGenericLayout wsum_generic_layout(int64_t n, int64_t T, int64_t out, int64_t in, int pieces) {
  WsumGenericLayout l;
  l.weights = dpk_align_up(static_cast<size_t>(n * T) * sizeof(float), 256);
  l.total = l.weights + (pieces > 1 ? dpk_align_up(static_cast<size_t>(pieces) * out * in * sizeof(float), 256) : 0);
  return l;
}
}  // namespace

extern "C" size_t dpk_linear_weighted_sum_workspace_bytes(int64_t n, int64_t T, int64_t out, int64_t in, int in_dtype,
                                                          int pieces) {
  if (n <= 0 || T <= 0 || out <= 0 || in <= 0 || pieces < 1) return 0;
  (void)in_dtype;
  // room for either path: a shape the fast kernel takes still goes the generic way when a tensor
  // turns out not to be 16-byte aligned
  return wsum_generic_layout(n, T, out, in, pieces).total;
}

// out_sum = scale * sum_s coef[s] * b[s]^T a[s]: the clip-weighted sum of a Linear layer's
// per-sample gradients, contracted over samples and positions at once
// (what the second backward pass leaves in weight.grad, fast_gradient_clipping_utils.py:193-201).
// bf16 operands in whole k tiles per sample go to the transposing-read kernel with the coefficients
// on its accumulators; with pieces > 1 piece p (samples p * n / pieces .. + n / pieces - 1) leaves
// its fp32 sum in the workspace and a second kernel adds the pieces into out_sum. Everything else
// (fp32 operands, any T, any feature sizes and alignment) goes to the fp32 MFMA kernel whose loader
// multiplies the rows of b by their weights; its pieces are runs of rows.
extern "C" int dpk_linear_weighted_sum(const void* b, const void* a, int in_dtype, const float* coef, void* out_sum,
                                       int out_dtype, int64_t n, int64_t T, int64_t out, int64_t in, float scale,
                                       int pieces, void* ws, size_t ws_bytes, dpk_stream_t stream) {
  const char* who = "dpk_linear_weighted_sum";
  DPK_REQUIRE(n >= 1 && T >= 1 && out >= 1 && in >= 1 && pieces >= 1, DPK_E_SHAPE,
              "%s: n=%lld T=%lld out=%lld in=%lld pieces=%d", who, (long long)n, (long long)T, (long long)out,
              (long long)in, pieces);
  DPK_REQUIRE(b && a && coef && out_sum, DPK_E_ARG, "%s: NULL tensor", who);
  DPK_REQUIRE(dpk_dtype_ok(in_dtype) && dpk_dtype_ok(out_dtype), DPK_E_DTYPE, "%s: dtypes %d,%d", who, in_dtype,
              out_dtype);
  DPK_REQUIRE(dpk_aligned(coef, 4) && dpk_aligned(b, dpk_elsize(in_dtype)) && dpk_aligned(a, dpk_elsize(in_dtype)) &&
                  dpk_aligned(out_sum, dpk_elsize(out_dtype)),
              DPK_E_ALIGN, "%s: misaligned tensor", who);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int64_t count = out * in;
  const bool fast = (wsum_fast_shape(in_dtype, T, out, in) || wsum_fast_shape_f32(in_dtype, out_dtype, T, out, in)) &&
                    n % pieces == 0 && dpk_aligned(b, 16) && dpk_aligned(a, 16) && dpk_aligned(out_sum, 16);
  if (!fast) {
    // generic path: row weights, then the fp32 MFMA kernel over all n * T rows (in `pieces` runs of rows)
    const int64_t rows = n * T;
    const WsumGenericLayout l = wsum_generic_layout(n, T, out, in, pieces);
    DPK_REQUIRE(ws && ws_bytes >= l.total, DPK_E_WORKSPACE, "%s: workspace %zu < %zu bytes", who, ws_bytes, l.total);
    DPK_REQUIRE(dpk_aligned(ws, 256), DPK_E_ALIGN, "%s: workspace must be 256-byte aligned", who);
    float* w = static_cast<float*>(ws);
    float* part = reinterpret_cast<float*>(static_cast<char*>(ws) + l.weights);
    const int64_t rows_per_piece = dpk_cdiv(dpk_cdiv(rows, pieces), mf32::BK) * mf32::BK;
    const int bm = (out > 64 && in > 64) ? 128 : 64;
    const int64_t tiles_m = dpk_cdiv(out, bm), tiles_n = dpk_cdiv(in, bm);
    const int64_t blocks = pieces * tiles_m * tiles_n;
    DPK_REQUIRE(blocks <= DPK_MAX_GRID_X && dpk_cdiv(rows, kThreads) <= DPK_MAX_GRID_X && (pieces == 1 || count % 4 == 0),
                DPK_E_SHAPE, "%s: %lld blocks exceed the grid limit, or out * in = %lld is not a multiple of 4 with pieces",
                who, (long long)blocks, (long long)count);
    hipLaunchKernelGGL(row_weights_kernel, dim3(static_cast<unsigned>(dpk_cdiv(rows, kThreads))), dim3(kThreads), 0, s,
                       coef, w, rows, T);
    DPK_LAUNCH_CHECK(who);
    const bool vec = out % 4 == 0 && in % 4 == 0 && dpk_aligned(b, 4 * dpk_elsize(in_dtype)) &&
                     dpk_aligned(a, 4 * dpk_elsize(in_dtype));
    const dim3 grid(static_cast<unsigned>(blocks));
    const bool split = pieces > 1;
#define DPK_WG(BMN, TIN, TOUT, V)                                                                                   \
  hipLaunchKernelGGL((linear_wsum_generic_kernel<BMN, BMN, TIN, TOUT, V>), grid, dim3(kThreads), 0, s,              \
                     static_cast<const TIN*>(b), static_cast<const TIN*>(a), w,                                     \
                     split ? reinterpret_cast<TOUT*>(part) : static_cast<TOUT*>(out_sum), rows, rows_per_piece, out, \
                     in, scale, tiles_m, tiles_n)
#define DPK_WG_V(BMN, TIN, TOUT) \
  do {                           \
    if (vec) DPK_WG(BMN, TIN, TOUT, true); \
    else DPK_WG(BMN, TIN, TOUT, false);    \
  } while (0)
#define DPK_WG_B(TIN, TOUT)                  \
  do {                                       \
    if (bm == 128) DPK_WG_V(128, TIN, TOUT); \
    else DPK_WG_V(64, TIN, TOUT);            \
  } while (0)
    const bool f32_dst = split || out_dtype == DPK_F32;
    if (in_dtype == DPK_F32 && f32_dst) DPK_WG_B(float, float);
    else if (in_dtype == DPK_F32) DPK_WG_B(float, bf16_t);
    else if (f32_dst) DPK_WG_B(bf16_t, float);
    else DPK_WG_B(bf16_t, bf16_t);
#undef DPK_WG_B
#undef DPK_WG_V
#undef DPK_WG
    DPK_LAUNCH_CHECK(who);
    if (split) {
      const dim3 g2(static_cast<unsigned>(dpk_cdiv(count / 4, kThreads)));
      if (out_dtype == DPK_BF16)
        hipLaunchKernelGGL(add_pieces_kernel<bf16_t>, g2, dim3(kThreads), 0, s, part, static_cast<bf16_t*>(out_sum),
                           count / 4, pieces);
      else
        hipLaunchKernelGGL(add_pieces_kernel<float>, g2, dim3(kThreads), 0, s, part, static_cast<float*>(out_sum),
                           count / 4, pieces);
      DPK_LAUNCH_CHECK(who);
    }
    return DPK_OK;
  }
  const bool split = pieces > 1;
  if (split) {
    const size_t need = static_cast<size_t>(pieces) * out * in * sizeof(float);
    DPK_REQUIRE(ws && ws_bytes >= need, DPK_E_WORKSPACE, "%s: workspace %zu < %zu bytes", who, ws_bytes, need);
    DPK_REQUIRE(dpk_aligned(ws, 16), DPK_E_ALIGN, "%s: workspace misaligned", who);
  }
  void* dst = split ? ws : out_sum;
  const int dst_dtype = split ? DPK_F32 : out_dtype;
  const int64_t rows = (n / pieces) * T;
  Plan p = make_plan(rows, out, in, true);
  if (in_dtype == DPK_BF16) plan_tr(p, b, a, out_sum, pieces, rows, out, in, dpk_device_cus(), DPK_TILE_AUTO);
  else plan_dlds_f32(p, b, a, out_sum, dst_dtype, rows, out, in);
  DPK_REQUIRE(p.tr != 0, DPK_E_SHAPE, "%s: out=%lld in=%lld: no tile plan", who, (long long)out, (long long)in);
  const int64_t blocks = pieces * p.tiles_m * p.tiles_n;
  const int64_t count4 = out * in / 4;  // out, in multiples of 4
  DPK_REQUIRE(blocks <= DPK_MAX_GRID_X && dpk_cdiv(count4, kThreads) <= DPK_MAX_GRID_X, DPK_E_SHAPE,
              "%s: %lld blocks exceed the grid limit", who, (long long)blocks);
  const dim3 grid(static_cast<unsigned>(blocks));
  float* none = nullptr;
  if (in_dtype == DPK_F32) {
    const float* bf = static_cast<const float*>(b);
    const float* af = static_cast<const float*>(a);
    if (dst_dtype == DPK_BF16)
      hipLaunchKernelGGL((linear_dlds_kernel<DldsF32, DldsF32Cfg, bf16_t, true>), grid, dim3(DldsF32Cfg::kThreads), 0, s,
                         bf, af, static_cast<bf16_t*>(dst), none, rows, out, in, scale, p.tiles_m, p.tiles_n, coef, T);
    else
      hipLaunchKernelGGL((linear_dlds_kernel<DldsF32, DldsF32Cfg, float, true>), grid, dim3(DldsF32Cfg::kThreads), 0, s,
                         bf, af, static_cast<float*>(dst), none, rows, out, in, scale, p.tiles_m, p.tiles_n, coef, T);
  } else {
  const bf16_t* bp = static_cast<const bf16_t*>(b);
  const bf16_t* ap = static_cast<const bf16_t*>(a);
#define DPK_WSUM(CFG, TOUT)                                                                                    \
  hipLaunchKernelGGL((linear_dlds_kernel<TrBf16, CFG, TOUT, true>), grid, dim3(CFG::kThreads), 0, s, bp, ap, \
                     static_cast<TOUT*>(dst), none, rows, out, in, scale, p.tiles_m, p.tiles_n, coef, T)
  if (p.tr == 256 && dst_dtype == DPK_BF16) DPK_WSUM(TrLarge, bf16_t);
  else if (p.tr == 256) DPK_WSUM(TrLarge, float);
  else if (dst_dtype == DPK_BF16) DPK_WSUM(TrSmall, bf16_t);
  else DPK_WSUM(TrSmall, float);
#undef DPK_WSUM
  }
  DPK_LAUNCH_CHECK(who);
  if (split) {
    const dim3 g2(static_cast<unsigned>(dpk_cdiv(count4, kThreads)));
    if (out_dtype == DPK_BF16)
      hipLaunchKernelGGL(add_pieces_kernel<bf16_t>, g2, dim3(kThreads), 0, s, static_cast<const float*>(ws),
                         static_cast<bf16_t*>(out_sum), count4, pieces);
    else
      hipLaunchKernelGGL(add_pieces_kernel<float>, g2, dim3(kThreads), 0, s, static_cast<const float*>(ws),
                         static_cast<float*>(out_sum), count4, pieces);
    DPK_LAUNCH_CHECK(who);
  }
  return DPK_OK;
}

// out_sum[k] = scale * sum_s coef[s] * sum_t b[s, t, k]: the clip-weighted sum of a Linear layer's
// per-sample bias gradients (linear.py:50 weighted as fast_gradient_clipping_utils.py:193-201
// weights the loss), one pass over b in chunks of rows and a fixed-order sum of the chunks.
namespace {
constexpr int64_t kWcolChunks = 256;
struct WcolLayout {
  size_t weights, total;
  int64_t chunks, rows_per_chunk;
};
WcolLayout wcol_layout(int64_t n, int64_t T, int64_t out) {
  WcolLayout l;
  const int64_t rows = n * T;
  l.chunks = rows < kWcolChunks ? rows : kWcolChunks;
  l.rows_per_chunk = dpk_cdiv(rows, l.chunks);
  l.chunks = dpk_cdiv(rows, l.rows_per_chunk);
  l.weights = dpk_align_up(static_cast<size_t>(rows) * sizeof(float), 256);
  l.total = l.weights + dpk_align_up(static_cast<size_t>(l.chunks) * out * sizeof(float), 256);
  return l;
}
}  // namespace

extern "C" size_t dpk_linear_bias_weighted_sum_workspace_bytes(int64_t n, int64_t T, int64_t out) {
  if (n <= 0 || T <= 0 || out <= 0) return 0;
  return wcol_layout(n, T, out).total;
}

extern "C" int dpk_linear_bias_weighted_sum(const void* b, int in_dtype, const float* coef, void* out_sum, int out_dtype,
                                            int64_t n, int64_t T, int64_t out, float scale, void* ws, size_t ws_bytes,
                                            dpk_stream_t stream) {
  const char* who = "dpk_linear_bias_weighted_sum";
  DPK_REQUIRE(n >= 1 && T >= 1 && out >= 1, DPK_E_SHAPE, "%s: n=%lld T=%lld out=%lld", who, (long long)n, (long long)T,
              (long long)out);
  DPK_REQUIRE(b && coef && out_sum, DPK_E_ARG, "%s: NULL tensor", who);
  DPK_REQUIRE(dpk_dtype_ok(in_dtype) && dpk_dtype_ok(out_dtype), DPK_E_DTYPE, "%s: dtypes %d,%d", who, in_dtype, out_dtype);
  DPK_REQUIRE(dpk_aligned(coef, 4) && dpk_aligned(b, dpk_elsize(in_dtype)) && dpk_aligned(out_sum, dpk_elsize(out_dtype)),
              DPK_E_ALIGN, "%s: misaligned tensor", who);
  const WcolLayout l = wcol_layout(n, T, out);
  DPK_REQUIRE(ws && ws_bytes >= l.total, DPK_E_WORKSPACE, "%s: workspace %zu < %zu bytes", who, ws_bytes, l.total);
  DPK_REQUIRE(dpk_aligned(ws, 256), DPK_E_ALIGN, "%s: workspace must be 256-byte aligned", who);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int64_t rows = n * T;
  float* w = static_cast<float*>(ws);
  float* part = reinterpret_cast<float*>(static_cast<char*>(ws) + l.weights);
  const bool vec = out % 4 == 0 && dpk_aligned(b, 4 * dpk_elsize(in_dtype));
  const int64_t col_blocks = dpk_cdiv(out, kThreads * (vec ? 4 : 1));
  DPK_REQUIRE(l.chunks * col_blocks <= DPK_MAX_GRID_X && dpk_cdiv(rows, kThreads) <= DPK_MAX_GRID_X, DPK_E_SHAPE,
              "%s: too many blocks", who);
  hipLaunchKernelGGL(row_weights_kernel, dim3(static_cast<unsigned>(dpk_cdiv(rows, kThreads))), dim3(kThreads), 0, s, coef,
                     w, rows, T);
  DPK_LAUNCH_CHECK(who);
  const dim3 grid(static_cast<unsigned>(l.chunks * col_blocks));
#define DPK_WCOL(TIN, V)                                                                                        \
  hipLaunchKernelGGL((wcolsum_partial_kernel<TIN, V>), grid, dim3(kThreads), 0, s, static_cast<const TIN*>(b), w, \
                     part, rows, l.rows_per_chunk, out, col_blocks)
  if (in_dtype == DPK_F32 && vec) DPK_WCOL(float, true);
  else if (in_dtype == DPK_F32) DPK_WCOL(float, false);
  else if (vec) DPK_WCOL(bf16_t, true);
  else DPK_WCOL(bf16_t, false);
#undef DPK_WCOL
  DPK_LAUNCH_CHECK(who);
  const dim3 g2(static_cast<unsigned>(dpk_cdiv(out, DPK_WAVE)));
  if (out_dtype == DPK_BF16)
    hipLaunchKernelGGL(wcolsum_final_kernel<bf16_t>, g2, dim3(kThreads), 0, s, part, static_cast<bf16_t*>(out_sum),
                       l.chunks, out, scale);
  else
    hipLaunchKernelGGL(wcolsum_final_kernel<float>, g2, dim3(kThreads), 0, s, part, static_cast<float*>(out_sum), l.chunks,
                       out, scale);
  DPK_LAUNCH_CHECK(who);
  return DPK_OK;
}

// The same sums for several layers at once (dpk_wsum_layer records, host array): one launch per
// group of up to 32 layers whose results share a dtype. A pool with too few tiles to fill the GPU
// in whole rounds of blocks has every layer's samples cut into `pieces` runs (each piece's fp32
// sum to the workspace, one more launch adds them), so that blocks = tiles x pieces does.
namespace {
struct WsumPoolPlan {
  int tile;    // 128 or 256
  int pieces;  // 1, 2, 4 or 8, dividing every layer's n
};

// The pooled launch runs at a rate that hardly depends on how its work is spread once most CUs
// have a block (measured on two layers of 1024 x 4096, 16384 rows: 64 + 64 tiles of 256 x 256 in one
// piece 306 us, in two pieces, 256 blocks, 290 us with the pass that adds them, in four 314 us;
// 512 tiles of 128 x 128 335 us), so pieces are only used to give every CU a block: the smallest
// count that does. 256 x 256 tiles wherever every layer is at least that wide.
WsumPoolPlan wsum_pool_plan(const dpk_wsum_layer* layers, int count, int cus) {
  int64_t tiles256 = 0, tiles128 = 0;
  bool all_wide = true;
  int64_t g = 0;  // pieces must divide every n
  for (int i = 0; i < count; ++i) {
    const dpk_wsum_layer& L = layers[i];
    tiles256 += dpk_cdiv(L.out, 256) * dpk_cdiv(L.in, 256);
    tiles128 += dpk_cdiv(L.out, 128) * dpk_cdiv(L.in, 128);
    all_wide = all_wide && L.out >= 256 && L.in >= 256;
    int64_t a = L.n, b = g;
    while (b) {
      const int64_t t = a % b;
      a = b;
      b = t;
    }
    g = a;
  }
  WsumPoolPlan best{all_wide ? 256 : 128, 1};
  const int64_t tiles = all_wide ? tiles256 : tiles128;
  const int64_t resident = all_wide ? cus : 2 * cus;
  while (best.pieces < 8 && tiles * best.pieces < resident && g % (2 * best.pieces) == 0) best.pieces *= 2;
  return best;
}
}  // namespace

extern "C" size_t dpk_linear_weighted_sum_multi_workspace_bytes(const dpk_wsum_layer* layers, int count) {
  if (!layers || count <= 0) return 0;
  int cus = dpk_device_cus();
  if (cus <= 0) cus = 256;
  const WsumPoolPlan plan = wsum_pool_plan(layers, count, cus);
  if (plan.pieces == 1) return 0;
  size_t total = 0;
  for (int i = 0; i < count; ++i)
    total += dpk_align_up(static_cast<size_t>(plan.pieces) * layers[i].out * layers[i].in * sizeof(float), 256);
  return total;
}

extern "C" int dpk_linear_weighted_sum_multi(const dpk_wsum_layer* layers, int count, int in_dtype, int out_dtype,
                                             void* ws, size_t ws_bytes, dpk_stream_t stream) {
  const char* who = "dpk_linear_weighted_sum_multi";
  DPK_REQUIRE(count >= 0 && (layers || count == 0), DPK_E_ARG, "%s: count=%d, layers=%p", who, count, (const void*)layers);
  DPK_REQUIRE(in_dtype == DPK_BF16 && dpk_dtype_ok(out_dtype), DPK_E_DTYPE, "%s: dtypes %d,%d (bf16 input only)", who,
              in_dtype, out_dtype);
  for (int i = 0; i < count; ++i) {
    const dpk_wsum_layer& L = layers[i];
    DPK_REQUIRE(L.n >= 1 && L.T >= 1 && L.out >= 1 && L.in >= 1, DPK_E_SHAPE, "%s: layer %d: n=%lld T=%lld out=%lld in=%lld",
                who, i, (long long)L.n, (long long)L.T, (long long)L.out, (long long)L.in);
    DPK_REQUIRE(L.b && L.a && L.coef && L.out_sum, DPK_E_ARG, "%s: layer %d: NULL tensor", who, i);
    DPK_REQUIRE(L.T % mb16t::BK == 0 && L.T < (int64_t{1} << 31), DPK_E_SHAPE, "%s: layer %d: T=%lld must be a multiple of %d",
                who, i, (long long)L.T, mb16t::BK);
    DPK_REQUIRE(L.out % 8 == 0 && L.in % 8 == 0 && L.out > 64 && L.in > 64 && L.out < (1LL << 24) && L.in < (1LL << 24) &&
                    dpk_aligned(L.b, 16) && dpk_aligned(L.a, 16) && dpk_aligned(L.out_sum, 16) && dpk_aligned(L.coef, 4),
                DPK_E_SHAPE, "%s: layer %d: out=%lld and in=%lld must be multiples of 8 above 64 and the tensors 16-byte aligned",
                who, i, (long long)L.out, (long long)L.in);
  }
  if (count == 0) return DPK_OK;
  int cus = dpk_device_cus();
  if (cus <= 0) cus = 256;
  const WsumPoolPlan plan = wsum_pool_plan(layers, count, cus);
  const int tile = plan.tile, pieces = plan.pieces;
  if (pieces > 1) {
    const size_t need = dpk_linear_weighted_sum_multi_workspace_bytes(layers, count);
    DPK_REQUIRE(ws && ws_bytes >= need, DPK_E_WORKSPACE, "%s: workspace %zu < %zu bytes", who, ws_bytes, need);
    DPK_REQUIRE(dpk_aligned(ws, 256), DPK_E_ALIGN, "%s: workspace must be 256-byte aligned", who);
  }
  hipStream_t s = static_cast<hipStream_t>(stream);
  char* part = static_cast<char*>(ws);
  for (int lo = 0; lo < count; lo += kWsumMax) {
    const int nl = count - lo < kWsumMax ? count - lo : kWsumMax;
    WsumMultiArgs A;
    AddPiecesMultiArgs R;
    memset(&A, 0, sizeof(A));
    memset(&R, 0, sizeof(R));
    A.nlayers = nl;
    A.pieces = pieces;
    R.nlayers = nl;
    R.pieces = pieces;
    int64_t total = 0, add_blocks = 0;
    for (int i = 0; i < nl; ++i) {
      const dpk_wsum_layer& L = layers[lo + i];
      A.b[i] = static_cast<const bf16_t*>(L.b);
      A.a[i] = static_cast<const bf16_t*>(L.a);
      A.coef[i] = L.coef;
      A.out[i] = L.out_sum;
      A.rows[i] = L.n * L.T;
      A.unit_rows[i] = static_cast<int32_t>(L.T);
      A.M[i] = static_cast<int32_t>(L.out);
      A.N[i] = static_cast<int32_t>(L.in);
      const int32_t tm = static_cast<int32_t>(dpk_cdiv(L.out, tile)), tn = static_cast<int32_t>(dpk_cdiv(L.in, tile));
      A.tiles_n[i] = tm < tn ? -tm : tn;  // the shorter dimension varies fastest
      A.scale[i] = L.scale;
      total += dpk_cdiv(L.out, tile) * dpk_cdiv(L.in, tile) * pieces;
      DPK_REQUIRE(total <= DPK_MAX_GRID_X, DPK_E_SHAPE, "%s: %lld blocks exceed the grid limit", who, (long long)total);
      A.tile_prefix[i + 1] = static_cast<uint32_t>(total);
      if (pieces > 1) {
        A.part[i] = reinterpret_cast<float*>(part);
        R.part[i] = A.part[i];
        R.out[i] = L.out_sum;
        R.count4[i] = L.out * L.in / 4;
        add_blocks += dpk_cdiv(R.count4[i], kThreads);
        DPK_REQUIRE(add_blocks <= DPK_MAX_GRID_X, DPK_E_SHAPE, "%s: %lld blocks exceed the grid limit", who, (long long)add_blocks);
        R.block_prefix[i + 1] = static_cast<uint32_t>(add_blocks);
        part += dpk_align_up(static_cast<size_t>(pieces) * L.out * L.in * sizeof(float), 256);
      }
    }
    const dim3 grid(static_cast<unsigned>(total));
    const bool f32 = out_dtype == DPK_F32 || pieces > 1;  // pieces are summed in fp32
    if (tile == 256 && !f32)
      hipLaunchKernelGGL((linear_wsum_multi_kernel<TrLarge, bf16_t>), grid, dim3(TrLarge::kThreads), 0, s, A);
    else if (tile == 256)
      hipLaunchKernelGGL((linear_wsum_multi_kernel<TrLarge, float>), grid, dim3(TrLarge::kThreads), 0, s, A);
    else if (!f32)
      hipLaunchKernelGGL((linear_wsum_multi_kernel<TrSmall, bf16_t>), grid, dim3(TrSmall::kThreads), 0, s, A);
    else
      hipLaunchKernelGGL((linear_wsum_multi_kernel<TrSmall, float>), grid, dim3(TrSmall::kThreads), 0, s, A);
    DPK_LAUNCH_CHECK(who);
    if (pieces > 1) {
      const dim3 g2(static_cast<unsigned>(add_blocks));
      if (out_dtype == DPK_BF16) hipLaunchKernelGGL(add_pieces_multi_kernel<bf16_t>, g2, dim3(kThreads), 0, s, R);
      else hipLaunchKernelGGL(add_pieces_multi_kernel<float>, g2, dim3(kThreads), 0, s, R);
      DPK_LAUNCH_CHECK(who);
    }
  }
  return DPK_OK;
}

namespace {
template <typename TIN, typename TOUT>
void launch_colsum(const void* b, void* out, int64_t n, int64_t T, int64_t K, float scale,
                   hipStream_t s) {
  const size_t ia = 4 * sizeof(TIN), oa = 4 * sizeof(TOUT);
  if (K % 4 == 0 && dpk_aligned(b, ia) && dpk_aligned(out, oa)) {
    // four row groups of 64 column threads (1 KB of a row per wave) when that already makes
    // enough blocks; sixteen groups of 16 otherwise
    if (n * dpk_cdiv(K, 256) >= 1024 || T < 64) {
      const int64_t bps = dpk_cdiv(K, 4 * (kThreads / 4));
      hipLaunchKernelGGL((colsum4_kernel<TIN, TOUT, 4>), dim3(static_cast<unsigned>(n * bps)), dim3(kThreads), 0, s,
                         static_cast<const TIN*>(b), static_cast<TOUT*>(out), T, K, scale, bps);
    } else {
      const int64_t bps = dpk_cdiv(K, 4 * (kThreads / 16));
      hipLaunchKernelGGL((colsum4_kernel<TIN, TOUT, 16>), dim3(static_cast<unsigned>(n * bps)), dim3(kThreads), 0, s,
                         static_cast<const TIN*>(b), static_cast<TOUT*>(out), T, K, scale, bps);
    }
    return;
  }
  // Split the t loop inside the block when there are few columns to go round.
  if (n * K < 64 * 1024 && T >= 32) {
    const int64_t bps = dpk_cdiv(K, kThreads / 16);
    hipLaunchKernelGGL((colsum_kernel<TIN, TOUT, 16>), dim3(static_cast<unsigned>(n * bps)),
                       dim3(kThreads), 0, s, static_cast<const TIN*>(b), static_cast<TOUT*>(out), T,
                       K, scale, bps);
  } else {
    const int64_t bps = dpk_cdiv(K, kThreads);
    hipLaunchKernelGGL((colsum_kernel<TIN, TOUT, 1>), dim3(static_cast<unsigned>(n * bps)),
                       dim3(kThreads), 0, s, static_cast<const TIN*>(b), static_cast<TOUT*>(out), T,
                       K, scale, bps);
  }
}
// sumsq[r] = sum_k v[r,k]^2 of the values as stored: one wave per row.
template <typename T>
__global__ __launch_bounds__(kThreads) void rowsq_kernel(const T* __restrict__ v, float* __restrict__ sumsq,
                                                          int64_t rows, int64_t K) {
  const int64_t w = (static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x) / DPK_WAVE;
  const int lane = threadIdx.x & (DPK_WAVE - 1);
  if (w >= rows) return;
  const T* p = v + w * K;
  float s = 0.f;
  for (int64_t i = lane; i < K; i += DPK_WAVE) {
    const float x = dpk_io<T>::load(p + i);
    s = fmaf(x, x, s);
  }
  s = wave_sum(s);
  if (lane == 0) sumsq[w] = s;
}
// The same with a block per row and 4-element loads, for rows long enough to keep a block busy:
// a lone wave walks a row of 4096 values in 64 dependent steps.
template <typename T>
__global__ __launch_bounds__(kThreads) void rowsq_block_kernel(const T* __restrict__ v, float* __restrict__ sumsq,
                                                                int64_t K) {
  __shared__ float red[kWaves];
  const T* p = v + static_cast<int64_t>(blockIdx.x) * K;
  float s = 0.f;
  for (int64_t i = threadIdx.x * 4; i < K; i += kThreads * 4) {
    const float4 x = dpk_io<T>::load4(p + i);
    s += (x.x * x.x + x.y * x.y) + (x.z * x.z + x.w * x.w);
  }
  const float t = block_sum<kWaves>(s, red);
  if (threadIdx.x == 0) sumsq[blockIdx.x] = t;
}
void launch_rowsq(const void* v, int dtype, float* sumsq, int64_t rows, int64_t K, hipStream_t s) {
  if (K >= 1024 && K % 4 == 0 && dpk_aligned(v, dtype == DPK_BF16 ? 8 : 16) && rows <= DPK_MAX_GRID_X) {
    const dim3 grid(static_cast<unsigned>(rows)), block(kThreads);
    if (dtype == DPK_F32)
      hipLaunchKernelGGL(rowsq_block_kernel<float>, grid, block, 0, s, static_cast<const float*>(v), sumsq, K);
    else
      hipLaunchKernelGGL(rowsq_block_kernel<bf16_t>, grid, block, 0, s, static_cast<const bf16_t*>(v), sumsq, K);
    return;
  }
  const dim3 grid(static_cast<unsigned>(dpk_cdiv(rows, kWaves))), block(kThreads);
  if (dtype == DPK_F32)
    hipLaunchKernelGGL(rowsq_kernel<float>, grid, block, 0, s, static_cast<const float*>(v), sumsq, rows, K);
  else
    hipLaunchKernelGGL(rowsq_kernel<bf16_t>, grid, block, 0, s, static_cast<const bf16_t*>(v), sumsq, rows, K);
}

template <typename TIN, typename TOUT>
void launch_rowsum(const void* b, void* out, int64_t rows, int64_t q, float scale, hipStream_t s) {
  const dim3 grid(static_cast<unsigned>(dpk_cdiv(rows, kWaves))), block(kThreads);
  if (q % 4 == 0 && dpk_aligned(b, 4 * sizeof(TIN)))
    hipLaunchKernelGGL((rowsum_kernel<TIN, TOUT, true>), grid, block, 0, s, static_cast<const TIN*>(b),
                       static_cast<TOUT*>(out), rows, q, scale);
  else
    hipLaunchKernelGGL((rowsum_kernel<TIN, TOUT, false>), grid, block, 0, s, static_cast<const TIN*>(b),
                       static_cast<TOUT*>(out), rows, q, scale);
}
}  // namespace

extern "C" int dpk_linear_bias_gs(const void* b, int in_dtype, void* gs_bias, int gs_dtype, float* sumsq,
                                  int64_t n, int64_t T, int64_t out, float scale,
                                  dpk_stream_t stream) {
  const char* who = "dpk_linear_bias_gs";
  DPK_REQUIRE(n >= 0 && T >= 1 && out >= 1, DPK_E_SHAPE, "%s: n=%lld T=%lld out=%lld", who,
              (long long)n, (long long)T, (long long)out);
  if (n == 0) return DPK_OK;
  DPK_REQUIRE(b && gs_bias, DPK_E_ARG, "%s: NULL tensor", who);
  DPK_REQUIRE(dpk_dtype_ok(in_dtype) && dpk_dtype_ok(gs_dtype), DPK_E_DTYPE, "%s: dtypes %d,%d", who,
              in_dtype, gs_dtype);
  DPK_REQUIRE(dpk_aligned(b, dpk_elsize(in_dtype)) && dpk_aligned(gs_bias, dpk_elsize(gs_dtype)),
              DPK_E_ALIGN, "%s: misaligned tensor", who);
  DPK_REQUIRE(n * dpk_cdiv(out, 16) <= DPK_MAX_GRID_X, DPK_E_SHAPE, "%s: too many blocks", who);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (in_dtype == DPK_F32 && gs_dtype == DPK_F32) launch_colsum<float, float>(b, gs_bias, n, T, out, scale, s);
  else if (in_dtype == DPK_BF16 && gs_dtype == DPK_BF16) launch_colsum<bf16_t, bf16_t>(b, gs_bias, n, T, out, scale, s);
  else if (in_dtype == DPK_BF16 && gs_dtype == DPK_F32) launch_colsum<bf16_t, float>(b, gs_bias, n, T, out, scale, s);
  else launch_colsum<float, bf16_t>(b, gs_bias, n, T, out, scale, s);
  if (sumsq) launch_rowsq(gs_bias, gs_dtype, sumsq, n, out, s);
  DPK_LAUNCH_CHECK(who);
  return DPK_OK;
}

extern "C" int dpk_conv_bias_gs(const void* b, int in_dtype, void* gs_bias, int gs_dtype, float* sumsq,
                                int64_t n, int64_t O, int64_t q, float scale, dpk_stream_t stream) {
  const char* who = "dpk_conv_bias_gs";
  DPK_REQUIRE(n >= 0 && O >= 1 && q >= 1, DPK_E_SHAPE, "%s: n=%lld O=%lld q=%lld", who,
              (long long)n, (long long)O, (long long)q);
  if (n == 0) return DPK_OK;
  DPK_REQUIRE(b && gs_bias, DPK_E_ARG, "%s: NULL tensor", who);
  DPK_REQUIRE(dpk_dtype_ok(in_dtype) && dpk_dtype_ok(gs_dtype), DPK_E_DTYPE, "%s: dtypes %d,%d", who,
              in_dtype, gs_dtype);
  DPK_REQUIRE(dpk_aligned(b, dpk_elsize(in_dtype)) && dpk_aligned(gs_bias, dpk_elsize(gs_dtype)),
              DPK_E_ALIGN, "%s: misaligned tensor", who);
  DPK_REQUIRE(dpk_cdiv(n * O, kWaves) <= DPK_MAX_GRID_X, DPK_E_SHAPE, "%s: too many rows", who);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (in_dtype == DPK_F32 && gs_dtype == DPK_F32) launch_rowsum<float, float>(b, gs_bias, n * O, q, scale, s);
  else if (in_dtype == DPK_BF16 && gs_dtype == DPK_BF16) launch_rowsum<bf16_t, bf16_t>(b, gs_bias, n * O, q, scale, s);
  else if (in_dtype == DPK_BF16 && gs_dtype == DPK_F32) launch_rowsum<bf16_t, float>(b, gs_bias, n * O, q, scale, s);
  else launch_rowsum<float, bf16_t>(b, gs_bias, n * O, q, scale, s);
  if (sumsq) launch_rowsq(gs_bias, gs_dtype, sumsq, n, O, s);
  DPK_LAUNCH_CHECK(who);
  return DPK_OK;
}
