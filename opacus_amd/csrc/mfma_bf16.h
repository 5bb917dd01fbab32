// bf16 MFMA block-tile machinery for gfx950 (wave64): C[m][n] = sum_k A[m][k] * B[n][k]
// with both operands stored with k contiguous (rows of a [T, d] matrix), fp32
// accumulation. A block of 256 threads (4 waves, 2 x 2) owns a BM x BN tile.
//
// v_mfma_f32_32x32x16_bf16 operand layout (lane l of 64):
//   a = A[m = l % 32][k = (l / 32) * 8 .. + 7]   (8 bf16 = 16 bytes, k contiguous)
//   b = B[n = l % 32][k = (l / 32) * 8 .. + 7]
//   c[v], v = 0..15: row = (v / 4) * 8 + (l / 32) * 4 + (v % 4), col = l % 32
// so a k-contiguous row-major tile in LDS feeds the instruction with one 16-byte
// read per operand and no transposition. LDS rows are padded by 16 bytes to
// spread the 32 rows a half-wave reads over the banks.
#pragma once

#include "dpk_common.h"

namespace mb16 {

typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));

constexpr int BK = 64;        // k extent of a staged tile (bf16 elements)
constexpr int LDK = BK + 8;   // padded LDS row, in bf16 elements (144 bytes)
constexpr int NTHREADS = 256;

template <int BM, int BN>
struct Smem {
  bf16_t a[2][BM][LDK];
  bf16_t b[2][BN][LDK];
};

template <int BM, int BN>
struct Tile {
  static constexpr int WM = BM / 2, WN = BN / 2;
  static constexpr int TM = WM / 32, TN = WN / 32;
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

  __device__ __forceinline__ void mma(const bf16_t (*As)[LDK], const bf16_t (*Bs)[LDK]) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int wm0 = (wave >> 1) * WM, wn0 = (wave & 1) * WN;
    const int kg = (lane >> 5) * 8, l32 = lane & 31;
#pragma unroll
    for (int k0 = 0; k0 < BK; k0 += 16) {
      bf16x8 av[TM], bv[TN];
#pragma unroll
      for (int i = 0; i < TM; ++i)
        av[i] = *reinterpret_cast<const bf16x8*>(&As[wm0 + i * 32 + l32][k0 + kg]);
#pragma unroll
      for (int j = 0; j < TN; ++j)
        bv[j] = *reinterpret_cast<const bf16x8*>(&Bs[wn0 + j * 32 + l32][k0 + kg]);
#pragma unroll
      for (int i = 0; i < TM; ++i)
#pragma unroll
        for (int j = 0; j < TN; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av[i], bv[j], acc[i][j], 0, 0, 0);
    }
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

// Rows of the source run along k: element (m, k) at base[m * ld + k].
// VEC: ld % 8 == 0 and base 16-byte aligned, so every 8-element group is one
// 16-byte load; otherwise elements are fetched one by one with bounds checks.
// Two register slots, so that the tile after next is already in flight while
// the next one waits in registers for its LDS buffer to become free.
template <int BMN, bool VEC>
struct Loader {
  static constexpr int R = BMN * BK / 8 / NTHREADS;
  static_assert(R >= 1, "tile too small for this loader");
  const bf16_t* base;
  int64_t ld, m0, M, K;
  uint4 st[2][R];
  __device__ __forceinline__ Loader(const bf16_t* base_, int64_t ld_, int64_t m0_, int64_t M_,
                                    int64_t K_)
      : base(base_), ld(ld_), m0(m0_), M(M_), K(K_) {}
  template <int SLOT>
  __device__ __forceinline__ void fetch(int64_t k0) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int idx = threadIdx.x + r * NTHREADS;
      const int64_t m = m0 + idx / (BK / 8);
      const int64_t k = k0 + (idx % (BK / 8)) * 8;
      uint4 v = make_uint4(0u, 0u, 0u, 0u);
      if (m < M && k < K) {
        const bf16_t* p = base + m * ld + k;
        if (VEC) {
          v = *reinterpret_cast<const uint4*>(p);
        } else {
          uint32_t w[4] = {0u, 0u, 0u, 0u};
#pragma unroll
          for (int e = 0; e < 8; ++e)
            if (k + e < K) w[e >> 1] |= static_cast<uint32_t>(p[e]) << ((e & 1) * 16);
          v = make_uint4(w[0], w[1], w[2], w[3]);
        }
      }
      st[SLOT][r] = v;
    }
  }
  template <int SLOT>
  __device__ __forceinline__ void commit(bf16_t (*S)[LDK]) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int idx = threadIdx.x + r * NTHREADS;
      *reinterpret_cast<uint4*>(&S[idx / (BK / 8)][(idx % (BK / 8)) * 8]) = st[SLOT][r];
    }
  }
};

// Rows of the source run along m: element (m, k) at base[k * ld + m] (a [T, features]
// matrix contracted over T). The instruction wants k contiguous, so the tile is transposed
// on its way into LDS: a thread loads an 8 (m) x 4 (k) patch as four 16-byte rows, regroups
// it in registers (one v_perm_b32 per output dword) and writes eight 8-byte pieces, one per
// m. Lanes 0..15 of a wave take consecutive k quads of the same 8 m, so their LDS writes
// fall into 32 consecutive dwords of a row, and four such groups share a 64-byte stretch
// of every source row they read.
// VEC: ld % 8 == 0, m0 % 8 == 0, base 16-byte aligned and the matrix below 1 GiB. Its loads
// go through a buffer descriptor over the K x ld matrix: the row offset of the k tile sits
// in a scalar register, each lane adds one constant byte offset, and rows past K read as
// zero without a test.
__device__ __forceinline__ uint32_t dword(const uint4& v, int i) {
  return i == 0 ? v.x : i == 1 ? v.y : i == 2 ? v.z : v.w;
}

template <int BMN, bool VEC>
struct LoaderMContig {
  static constexpr int PATCHES = (BMN / 8) * (BK / 4);
  static constexpr int R = (PATCHES + NTHREADS - 1) / NTHREADS;
  // per patch: pointer to its element (k = kq * 4, m) of the k tile at k0 = 0, advanced
  // by whole k tiles; the bounds are 32-bit and the column test is made once
  const bf16_t* ptr[R];
  int64_t ld;
  int kfirst[R], K, mleft[R];
  uint32_t voff[R];
  __amdgpu_buffer_rsrc_t rsrc;
  uint4 st[2][R][4];
  __device__ __forceinline__ LoaderMContig(const bf16_t* base, int64_t ld_, int64_t m0, int64_t M,
                                           int64_t K_)
      : ld(ld_), K(static_cast<int>(K_)) {
    if (VEC)
      rsrc = __builtin_amdgcn_make_buffer_rsrc(const_cast<bf16_t*>(base), 0, static_cast<int>(K_ * ld_ * 2), 0x00020000);
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int idx = threadIdx.x + r * NTHREADS;
      const int kq = idx % (BK / 4), mg = idx / (BK / 4);
      const int64_t m = m0 + mg * 8;
      kfirst[r] = kq * 4;
      // elements of the patch's 8 columns that exist (0: the patch is outside the matrix)
      mleft[r] = (idx < PATCHES && m < M) ? static_cast<int>(M - m < 8 ? M - m : 8) : 0;
      ptr[r] = base + kfirst[r] * ld + m;
      // a patch outside the matrix points past the descriptor's end and reads zeros
      voff[r] = mleft[r] > 0 ? static_cast<uint32_t>((kfirst[r] * ld + m) * 2) : 0x7fffffffu;
    }
  }
  // k0 must advance by BK from call to call of the same slot sequence: the loader keeps no
  // pointer per slot, it recomputes from k0
  template <int SLOT>
  __device__ __forceinline__ void fetch(int64_t k0) {
    const int k0i = static_cast<int>(k0);
    if (VEC) {
      typedef int vi4 __attribute__((ext_vector_type(4)));
      const int row_bytes = static_cast<int>(ld) * 2;
      const int tile_off = k0i * row_bytes;
#pragma unroll
      for (int r = 0; r < R; ++r) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const vi4 v = __builtin_amdgcn_raw_buffer_load_b128(rsrc, voff[r], tile_off + j * row_bytes, 0);
          st[SLOT][r][j] = make_uint4(v.x, v.y, v.z, v.w);
        }
      }
      return;
    }
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const bf16_t* p = ptr[r] + k0 * ld;
#pragma unroll
      for (int j = 0; j < 4; ++j) {
        uint4 v = make_uint4(0u, 0u, 0u, 0u);
        if (mleft[r] > 0 && k0i + kfirst[r] + j < K) {
          if (VEC) {
            v = *reinterpret_cast<const uint4*>(p + j * ld);
          } else {
            uint32_t w[4] = {0u, 0u, 0u, 0u};
#pragma unroll
            for (int e = 0; e < 8; ++e)
              if (e < mleft[r]) w[e >> 1] |= static_cast<uint32_t>(p[j * ld + e]) << ((e & 1) * 16);
            v = make_uint4(w[0], w[1], w[2], w[3]);
          }
        }
        st[SLOT][r][j] = v;
      }
    }
  }
  template <int SLOT>
  __device__ __forceinline__ void commit(bf16_t (*S)[LDK]) {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int idx = threadIdx.x + r * NTHREADS;
      if (idx >= PATCHES) continue;
      const int kq = idx % (BK / 4), mg = idx / (BK / 4);
      bf16_t* dst = &S[mg * 8][kq * 4];
#pragma unroll
      for (int c = 0; c < 8; ++c) {
        // element c of rows k, k+1 | rows k+2, k+3: low halves of the dwords for even c,
        // high halves for odd c
        const uint32_t sel = (c & 1) ? 0x07060302u : 0x05040100u;
        uint2 o;
        o.x = __builtin_amdgcn_perm(dword(st[SLOT][r][1], c >> 1), dword(st[SLOT][r][0], c >> 1), sel);
        o.y = __builtin_amdgcn_perm(dword(st[SLOT][r][3], c >> 1), dword(st[SLOT][r][2], c >> 1), sel);
        *reinterpret_cast<uint2*>(dst + c * LDK) = o;
      }
    }
  }
};

// Software pipeline over k, two tiles per trip so that every register slot and
// LDS buffer index is a compile-time constant:
//   LDS buffer (kt & 1) holds tile kt, register slot ((kt + 1) & 1) holds tile
//   kt + 1 (loaded during the previous step), and the loads of tile kt + 2 are
//   issued before the MFMAs of tile kt start. Global-memory latency is thus
//   covered by a whole step of MFMAs rather than by a fraction of one.
template <int BM, int BN, class LA, class LB>
__device__ __forceinline__ void mainloop(Tile<BM, BN>& t, Smem<BM, BN>& sm, LA& la, LB& lb,
                                         int64_t K) {
  const int64_t nk = (K + BK - 1) / BK;
  la.template fetch<0>(0);
  lb.template fetch<0>(0);
  if (nk > 1) {
    la.template fetch<1>(BK);
    lb.template fetch<1>(BK);
  }
  la.template commit<0>(sm.a[0]);
  lb.template commit<0>(sm.b[0]);
  __syncthreads();
  for (int64_t kt = 0; kt < nk; kt += 2) {
    if (kt + 2 < nk) {
      la.template fetch<0>((kt + 2) * BK);
      lb.template fetch<0>((kt + 2) * BK);
    }
    t.mma(sm.a[0], sm.b[0]);
    if (kt + 1 < nk) {
      la.template commit<1>(sm.a[1]);
      lb.template commit<1>(sm.b[1]);
    }
    __syncthreads();
    if (kt + 1 >= nk) break;
    if (kt + 3 < nk) {
      la.template fetch<1>((kt + 3) * BK);
      lb.template fetch<1>((kt + 3) * BK);
    }
    t.mma(sm.a[1], sm.b[1]);
    if (kt + 2 < nk) {
      la.template commit<0>(sm.a[0]);
      lb.template commit<0>(sm.b[0]);
    }
    __syncthreads();
  }
}

}  // namespace mb16

namespace mb16 {

// The same pipeline without a way out in the middle of a trip, for loaders that deliver
// zeros for k tiles past K (both of the above do): tiles are taken in pairs, and for an odd
// count the last pair's second tile is all zeros. One basic block per trip keeps the
// accumulators in place.
template <int BM, int BN, class LA, class LB>
__device__ __forceinline__ void mainloop_pairs(Tile<BM, BN>& t, Smem<BM, BN>& sm, LA& la, LB& lb,
                                               int64_t K) {
  const int64_t nk = (K + BK - 1) / BK;
  la.template fetch<0>(0);
  lb.template fetch<0>(0);
  la.template fetch<1>(BK);
  lb.template fetch<1>(BK);
  la.template commit<0>(sm.a[0]);
  lb.template commit<0>(sm.b[0]);
  __syncthreads();
  for (int64_t kt = 0; kt < nk; kt += 2) {
    la.template fetch<0>((kt + 2) * BK);
    lb.template fetch<0>((kt + 2) * BK);
    t.mma(sm.a[0], sm.b[0]);
    la.template commit<1>(sm.a[1]);
    lb.template commit<1>(sm.b[1]);
    __syncthreads();
    la.template fetch<1>((kt + 3) * BK);
    lb.template fetch<1>((kt + 3) * BK);
    t.mma(sm.a[1], sm.b[1]);
    la.template commit<0>(sm.a[0]);
    lb.template commit<0>(sm.b[0]);
    __syncthreads();
  }
}

}  // namespace mb16
