// fp32 MFMA block-tile machinery for gfx950 (wave64), shared by the per-sample
// contraction kernels. A block of 256 threads (4 waves, 2 x 2) owns a BM x BN
// tile of C[m][n] = sum_k A(k,m) * B(k,n). Operand tiles are staged in LDS as
// [k][m] so that the 64 lanes of v_mfma_f32_32x32x2f32 read 32 consecutive
// floats for each of the instruction's two k values: conflict-free ds_read_b32.
// How a tile gets from global memory into that layout is the loader's business
// (rows contiguous along m, rows contiguous along k, or an implicit im2col).
//
// v_mfma_f32_32x32x2f32 operand layout (lane l of 64):
//   a = A[m = l % 32][k = l / 32], b = B[k = l / 32][n = l % 32]
//   c[v], v = 0..15: row = (v / 4) * 8 + (l / 32) * 4 + (v % 4), col = l % 32
#pragma once

#include "dpk_common.h"

namespace mf32 {

typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int BK = 16;         // k extent of one staged tile
constexpr int PAD = 4;         // keeps LDS rows 16-byte aligned and skews banks
constexpr int NTHREADS = 256;  // 4 waves

template <int BM, int BN>
struct Smem {
  float a[2][BK][BM + PAD];
  float b[2][BK][BN + PAD];
};

template <int BM, int BN>
struct Tile {
  static constexpr int WM = BM / 2, WN = BN / 2;    // wave tile
  static constexpr int TM = WM / 32, TN = WN / 32;  // 32x32 MFMA tiles per wave
  static_assert(TM >= 1 && TN >= 1, "block tile must be at least 64 x 64");
  floatx16 acc[TM][TN];

  __device__ __forceinline__ void clear() {
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
  }

  __device__ __forceinline__ void mma(const float (*As)[BM + PAD], const float (*Bs)[BN + PAD]) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wm0 = (wave >> 1) * WM, wn0 = (wave & 1) * WN;
    const int kk = lane >> 5, l32 = lane & 31;
    // all operand reads of the k-tile first, then its MFMAs: LDS latency is paid
    // once per tile instead of once per k step
    float av[BK / 2][TM], bv[BK / 2][TN];
#pragma unroll
    for (int k2 = 0; k2 < BK / 2; ++k2) {
#pragma unroll
      for (int i = 0; i < TM; ++i) av[k2][i] = As[2 * k2 + kk][wm0 + i * 32 + l32];
#pragma unroll
      for (int j = 0; j < TN; ++j) bv[k2][j] = Bs[2 * k2 + kk][wn0 + j * 32 + l32];
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int k2 = 0; k2 < BK / 2; ++k2)
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[k2][i], bv[k2][j], acc[i][j], 0, 0, 0);
  }

  // f(row, col, value) for every accumulator element this thread owns; row and
  // col are relative to the block tile.
  template <typename F>
  __device__ __forceinline__ void for_each(F f) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wm0 = (wave >> 1) * WM, wn0 = (wave & 1) * WN;
    const int kk = lane >> 5, l32 = lane & 31;
#pragma unroll
    for (int i = 0; i < TM; ++i)
#pragma unroll
      for (int j = 0; j < TN; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v)
          f(wm0 + i * 32 + (v >> 2) * 8 + kk * 4 + (v & 3), wn0 + j * 32 + l32, acc[i][j][v]);
  }
};

// Source rows run along m: element (k, m) at base[k * ld + m]. (Linear layers:
// backprops [T, out] and activations [T, in] of one sample.)
template <int BMN, typename T, bool VEC>
struct LoaderMContig {
  static constexpr int R = BK * BMN / 4 / NTHREADS;
  static_assert(R >= 1, "tile too small for this loader");
  const T* base;
  int64_t ld, m0, M, K;
  float4 st[R];
  __device__ __forceinline__ LoaderMContig(const T* base_, int64_t ld_, int64_t m0_, int64_t M_,
                                           int64_t K_)
      : base(base_), ld(ld_), m0(m0_), M(M_), K(K_) {}
  __device__ __forceinline__ void fetch(int64_t k0) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int idx = threadIdx.x + r * NTHREADS;
      const int64_t k = k0 + idx / (BMN / 4);
      const int64_t m = m0 + (idx % (BMN / 4)) * 4;
      float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
      if (k < K && m < M) {
        const T* p = base + k * ld + m;
        if (VEC) {
          v = dpk_io<T>::load4(p);
        } else {
          v.x = dpk_io<T>::load(p);
          if (m + 1 < M) v.y = dpk_io<T>::load(p + 1);
          if (m + 2 < M) v.z = dpk_io<T>::load(p + 2);
          if (m + 3 < M) v.w = dpk_io<T>::load(p + 3);
        }
      }
      st[r] = v;
    }
  }
  __device__ __forceinline__ void commit(float (*S)[BMN + PAD]) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int idx = threadIdx.x + r * NTHREADS;
      *reinterpret_cast<float4*>(&S[idx / (BMN / 4)][(idx % (BMN / 4)) * 4]) = st[r];
    }
  }
};

// Source rows run along k: element (k, m) at base[m * ld + k]. (Conv backprops
// [O, q]; Gram operands [T, d].) The transpose happens on the way into LDS.
template <int BMN, typename T, bool VEC>
struct LoaderKContig {
  static constexpr int R = BK * BMN / 4 / NTHREADS;
  static_assert(R >= 1, "tile too small for this loader");
  const T* base;
  int64_t ld, m0, M, K;
  float4 st[R];
  __device__ __forceinline__ LoaderKContig(const T* base_, int64_t ld_, int64_t m0_, int64_t M_,
                                           int64_t K_)
      : base(base_), ld(ld_), m0(m0_), M(M_), K(K_) {}
  __device__ __forceinline__ void fetch(int64_t k0) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int idx = threadIdx.x + r * NTHREADS;
      const int64_t m = m0 + idx / (BK / 4);
      const int64_t k = k0 + (idx % (BK / 4)) * 4;
      float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
      if (m < M && k < K) {
        const T* p = base + m * ld + k;
        if (VEC) {
          v = dpk_io<T>::load4(p);
        } else {
          v.x = dpk_io<T>::load(p);
          if (k + 1 < K) v.y = dpk_io<T>::load(p + 1);
          if (k + 2 < K) v.z = dpk_io<T>::load(p + 2);
          if (k + 3 < K) v.w = dpk_io<T>::load(p + 3);
        }
      }
      st[r] = v;
    }
  }
  __device__ __forceinline__ void commit(float (*S)[BMN + PAD]) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int idx = threadIdx.x + r * NTHREADS;
      const int m = idx / (BK / 4), k = (idx % (BK / 4)) * 4;
      S[k + 0][m] = st[r].x;
      S[k + 1][m] = st[r].y;
      S[k + 2][m] = st[r].z;
      S[k + 3][m] = st[r].w;
    }
  }
};

// Software-pipelined k loop: while the MFMAs consume LDS buffer `cur`, the next
// tile is already in flight from global memory into registers; it is committed
// to the other buffer afterwards. One barrier per k tile.
// The k range is [k_begin, k_end), k_begin a multiple of BK; the loaders bound k themselves.
template <int BM, int BN, class LA, class LB>
__device__ __forceinline__ void mainloop(Tile<BM, BN>& t, Smem<BM, BN>& sm, LA& la, LB& lb,
                                         int64_t k_begin, int64_t k_end) {
  const int64_t nk = (k_end - k_begin + BK - 1) / BK;
  la.fetch(k_begin);
  lb.fetch(k_begin);
  la.commit(sm.a[0]);
  lb.commit(sm.b[0]);
  __syncthreads();
  for (int64_t kt = 0; kt < nk; ++kt) {
    const int cur = static_cast<int>(kt & 1);
    const bool more = kt + 1 < nk;
    if (more) {
      la.fetch(k_begin + (kt + 1) * BK);
      lb.fetch(k_begin + (kt + 1) * BK);
    }
    t.mma(sm.a[cur], sm.b[cur]);
    if (more) {
      la.commit(sm.a[cur ^ 1]);
      lb.commit(sm.b[cur ^ 1]);
    }
    __syncthreads();
  }
}

template <int BM, int BN, class LA, class LB>
__device__ __forceinline__ void mainloop(Tile<BM, BN>& t, Smem<BM, BN>& sm, LA& la, LB& lb, int64_t K) {
  mainloop<BM, BN>(t, sm, la, lb, 0, K);
}

}  // namespace mf32
