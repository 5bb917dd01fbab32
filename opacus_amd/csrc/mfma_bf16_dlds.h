// bf16 MFMA Gram tiles fed by direct global->LDS loads (gfx950).
//
// Same contraction as mfma_bf16.h (C[m][n] = sum_k A[m][k] B[n][k], operands with
// k contiguous), but the operand tiles never pass through VGPRs: each lane issues
// global_load_lds_dwordx4, which drops its 16 bytes at LDS[base + lane * 16], and
// an NS-deep ring of LDS stages keeps NS - 1 k-tiles in flight behind the MFMAs.
// A block is NWR x NWC waves, each owning a 64 x 64 piece (2 x 2 MFMA tiles of
// 32 x 32) of the (64 NWR) x (64 NWC) block tile.
// Requirements of this path (the caller falls back to mfma_bf16.h otherwise):
// K % 64 == 0, row stride % 8 == 0, 16-byte aligned base.
//
// fp32 operands take the same road (element type float: a stage row of 128 bytes is then 32
// k values, K % 32 == 0). v_mfma_f32_32x32x2f32 wants lane l to hold k = l / 32 of row
// l % 32; which two k values meet in one instruction does not matter to a contraction as
// long as both operands agree, so lanes 0..31 read the 16-byte chunk 2 c of their row and
// lanes 32..63 chunk 2 c + 1, exactly as for bf16, and the e-th float of the two chunks
// (k = 8 c + e and 8 c + 4 + e) feeds the e-th of four instructions.
//
// LDS stage layout: row-major [rows][64 bf16] = 128 bytes per row, no padding
// (a wave's 64 lanes must land contiguously), 16-byte chunks XOR-swizzled:
//   physical chunk = logical chunk ^ ((row >> 1) & 7).
// For the MFMA operand read (16 consecutive rows, one logical chunk, 16 bytes
// per lane) the 16 lanes then hit 16 distinct 16-byte slots of the 256-byte bank
// space: conflict-free. Rows beyond the matrix are fetched from the last valid
// row instead (no fault, finite values); the caller masks them out of its
// reduction.
#pragma once

#include <type_traits>

#include "dpk_common.h"
#include "mfma_bf16.h"

namespace mb16d {

typedef float floatx4 __attribute__((ext_vector_type(4)));

using mb16::bf16x8;
using mb16::floatx16;


typedef __attribute__((address_space(3))) void* lptr_t;

template <int NWR, int NWC, int NS, int BK_ = 64>
struct Config {
  static_assert(BK_ == 64 || BK_ == 32, "k extent of a stage: 64 or 32 bf16");
  static constexpr int BK = BK_;
  static constexpr int ROW_BYTES = BK * 2;          // 128 or 64
  static constexpr int kChunks = ROW_BYTES / 16;    // 16-byte chunks per row: 8 or 4
  static constexpr int kRowsPerKB = 1024 / ROW_BYTES;  // rows covered by one wave instruction
  static constexpr int kWaveRows = NWR, kWaveCols = NWC;
  static constexpr int kWaves = NWR * NWC;
  static constexpr int kThreads = 64 * kWaves;
  static constexpr int BM = 64 * NWR, BN = 64 * NWC;
  static constexpr int kStages = NS;
  static constexpr int kStageBytes = (BM + BN) * ROW_BYTES;
  // global->LDS instructions per thread and k-tile: one per 1 KB of tile per wave
  static constexpr int kLoadsA = BM * ROW_BYTES / 1024 / kWaves;
  static constexpr int kLoadsB = BN * ROW_BYTES / 1024 / kWaves;
  static constexpr int kLoadsPerTile = kLoadsA + kLoadsB;
  static_assert(BM * ROW_BYTES % (1024 * kWaves) == 0 && BN * ROW_BYTES % (1024 * kWaves) == 0,
                "tile rows must split evenly over the waves");
};

template <class C>
struct Smem {
  alignas(1024) unsigned char stage[C::kStages][C::kStageBytes];  // per stage: A tile, then B tile
};

// 8 chunks per row: chunk ^ ((row >> 1) & 7); 4 chunks per row: chunk ^ ((row >> 2) & 3).
// Either way 16 consecutive rows at one logical chunk cover the 256-byte bank space once.
template <class C>
__device__ __forceinline__ int swz(int row, int chunk) {
  return C::kChunks == 8 ? chunk ^ ((row >> 1) & 7) : chunk ^ ((row >> 2) & 3);
}

// One direct global->LDS load of 16 bytes per lane: lane l's bytes land at
// LDS[lds_base + l * 16]. Written as inline assembly so that waiting for it stays
// in this file's hands: the ring below wants loads of later tiles to remain in
// flight across the barrier and across the LDS reads of the current tile.
__device__ __forceinline__ void load16_to_lds(const void* gptr, uint32_t lds_base) {
  asm volatile(
      "s_mov_b32 m0, %0\n\t"
      "s_nop 0\n\t"
      "global_load_lds_dwordx4 %1, off\n\t"
      :
      : "s"(lds_base), "v"(gptr)
      : "memory", "m0");
}

__device__ __forceinline__ uint32_t lds_offset(const void* p) {
  return static_cast<uint32_t>(reinterpret_cast<uintptr_t>((lptr_t)p));
}

// The same with the address split into a wave-uniform base (scalar registers) and a
// 32-bit per-lane byte offset: the per-lane part of a tile's addresses never changes
// along k, so the main loop computes it once and only moves the scalar base.
__device__ __forceinline__ void load16_to_lds(const void* sbase, uint32_t voff, uint32_t lds_base) {
  asm volatile(
      "s_mov_b32 m0, %0\n\t"
      "s_nop 0\n\t"
      "global_load_lds_dwordx4 %1, %2\n\t"
      :
      : "s"(lds_base), "v"(voff), "s"(sbase)
      : "memory", "m0");
}

// The r-th global->LDS load of a tile covers 1 KB of consecutive tile rows per wave:
// group r * kWaves + wave. lane_offset: this lane's byte offset from the matrix base
// for that load (rows >= M read row M - 1 instead); group_lds: where the group lands
// in the tile's LDS image.
template <class C, int ES = 2>
__device__ __forceinline__ uint32_t lane_offset(int64_t ld, int64_t m0, int64_t M, int r) {
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int grp = r * C::kWaves + wave;
  const int row = grp * C::kRowsPerKB + lane / C::kChunks;
  const int lc = swz<C>(row, lane % C::kChunks);  // which logical chunk lives at this physical slot
  int64_t m = m0 + row;
  m = m < M ? m : M - 1;
  return static_cast<uint32_t>(m * ld * ES + lc * 16);  // ld in elements of ES bytes
}

template <class C>
__device__ __forceinline__ uint32_t group_lds(int r) {
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  return static_cast<uint32_t>((r * C::kWaves + wave) * 1024);
}

// Waits until at most N of this wave's loads are outstanding, then meets the
// other waves. No fence beyond that: the LDS reads of the previous tile were
// consumed by MFMAs already, and nothing else is shared.
template <int N>
__device__ __forceinline__ void wait_and_barrier() {
  static_assert(N == 0 || N == 4 || N == 6 || N == 8 || N == 12 || N == 16 || N == 18 || N == 24,
                "add the vmcnt value to the switch below");
  switch (N) {
    case 0: asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory"); break;
    case 4: asm volatile("s_waitcnt vmcnt(4)\n\ts_barrier" ::: "memory"); break;
    case 6: asm volatile("s_waitcnt vmcnt(6)\n\ts_barrier" ::: "memory"); break;
    case 8: asm volatile("s_waitcnt vmcnt(8)\n\ts_barrier" ::: "memory"); break;
    case 12: asm volatile("s_waitcnt vmcnt(12)\n\ts_barrier" ::: "memory"); break;
    case 16: asm volatile("s_waitcnt vmcnt(16)\n\ts_barrier" ::: "memory"); break;
    case 18: asm volatile("s_waitcnt vmcnt(18)\n\ts_barrier" ::: "memory"); break;
    default: asm volatile("s_waitcnt vmcnt(24)\n\ts_barrier" ::: "memory"); break;
  }
}

// The 64 x 64 accumulator piece of one wave.
struct Tile {
  floatx16 acc[2][2];

  __device__ __forceinline__ void clear() {
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
  }

  // As / Bs: the stage's operand tiles; (wm0, wn0): this wave's corner in the block tile;
  // issue(q), q < NLOADS: issues the q-th load of the tile being prefetched.
  template <class C, int NLOADS, typename T = bf16_t, class IssueFn>
  __device__ __forceinline__ void mma(const unsigned char* As, const unsigned char* Bs, int wm0, int wn0,
                                      IssueFn issue) {
    const int lane = threadIdx.x & 63;
    const int kh = lane >> 5, l32 = lane & 31;
    // All operand fragments of the k-tile are requested up front (16 reads of 16
    // bytes per lane); the MFMAs of step ks then only wait for their own four,
    // so LDS latency is paid once per tile instead of once per step.
    constexpr int KS = C::BK / 16, ROW_BYTES = C::ROW_BYTES;
    constexpr bool kF32 = std::is_same<T, float>::value;
    typedef typename std::conditional<kF32, floatx4, bf16x8>::type frag_t;  // 16 bytes either way
    frag_t av[KS][2], bv[KS][2];
    // bf16: the next tile's loads go out before anything else of this tile. A tile's MFMAs are
    // 512 cycles of the pipe; loads issued in their shadow, a few per k step, left the last of
    // them a stage's wait at the next barrier (waves stalled half their cycles; 2048 -> 32000:
    // 835 -> 728 us with the loads first). fp32 tiles take four times as long to multiply and
    // run 6 % faster with the loads dealt out between the steps.
    constexpr bool kLoadsFirst = !kF32;
    if constexpr (kLoadsFirst) {
#pragma unroll
      for (int q = 0; q < NLOADS; ++q) issue(q);
    }
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
#pragma unroll
      for (int i = 0; i < 2; ++i) {
        const int row = wm0 + i * 32 + l32;
        av[ks][i] = *reinterpret_cast<const frag_t*>(As + row * ROW_BYTES + swz<C>(row, ks * 2 + kh) * 16);
      }
#pragma unroll
      for (int j = 0; j < 2; ++j) {
        const int row = wn0 + j * 32 + l32;
        bv[ks][j] = *reinterpret_cast<const frag_t*>(Bs + row * ROW_BYTES + swz<C>(row, ks * 2 + kh) * 16);
      }
    }
    __builtin_amdgcn_sched_barrier(0);  // keep the reads ahead of the MFMAs
    // MFMAs execute asynchronously: the global->LDS loads of the tile after next
    // (and their address arithmetic) are issued in their shadow, a few per step.
    constexpr int PER_STEP = (NLOADS + KS - 1) / KS;
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) {
      if constexpr (kF32) {
#pragma unroll
        for (int e = 0; e < 4; ++e)
#pragma unroll
          for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
              acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(av[ks][i][e], bv[ks][j][e], acc[i][j], 0, 0, 0);
      } else {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int j = 0; j < 2; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(av[ks][i], bv[ks][j], acc[i][j], 0, 0, 0);
      }
      if constexpr (!kLoadsFirst) {
#pragma unroll
        for (int q = ks * PER_STEP; q < (ks + 1) * PER_STEP && q < NLOADS; ++q) issue(q);
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  }
};

// C tile += A[m0a.., :K] . B[m0b.., :K]^T with an NS-stage ring. Every iteration
// issues exactly one tile's worth of loads (past the end the last tile is
// fetched again into a stage nobody reads), so the number of loads that may
// stay outstanding while tile kt is awaited is the constant
// kLoadsPerTile * (NS - 2). abase / bbase must be wave-uniform and every byte
// offset inside the matrices must fit 32 bits (M * ld * 2 < 2^32).
// Ma / Mb: rows of the two operand matrices (the same matrix for a Gram).
// (A diagonal tile of a Gram has the same rows as both operands. Fetching them once and
// pointing both operand reads at the one image measured 5 % faster on a launch of one
// round of blocks and 4.5 % slower on a launch of 24 rounds, and was not kept.)
template <class C, typename T = bf16_t>
__device__ __forceinline__ void mainloop(Tile& t, Smem<C>& sm, const T* abase,
                                         const T* bbase, int64_t ld, int64_t m0a, int64_t m0b,
                                         int64_t Ma, int64_t Mb, int64_t K, int wm0, int wn0) {
  constexpr int NS = C::kStages;
  constexpr int ROW_BYTES = C::ROW_BYTES, ES = sizeof(T);
  constexpr int BK = ROW_BYTES / ES;  // k values of a stage row: 64 bf16 or 32 floats
  const int64_t nk = K / BK;
  const uint32_t lds0 = lds_offset(&sm.stage[0][0]);
  // Per-lane offsets of the tile's loads, fixed for the whole k loop. The empty asm
  // makes them opaque values: recomputing them per load (a 64-bit multiply and a
  // clamp each) would cost more vector instructions than the MFMAs they feed.
  uint32_t off[C::kLoadsPerTile];
#pragma unroll
  for (int q = 0; q < C::kLoadsPerTile; ++q) {
    off[q] = q < C::kLoadsA ? lane_offset<C, ES>(ld, m0a, Ma, q) : lane_offset<C, ES>(ld, m0b, Mb, q - C::kLoadsA);
    asm volatile("" : "+v"(off[q]));
  }
  auto issue_q = [&](int64_t kt, uint32_t st, int q) {
    if (q < C::kLoadsA) load16_to_lds(abase + kt * BK, off[q], st + group_lds<C>(q));
    else load16_to_lds(bbase + kt * BK, off[q], st + C::BM * ROW_BYTES + group_lds<C>(q - C::kLoadsA));
  };
#pragma unroll
  for (int s = 0; s < NS - 1; ++s) {
    const int64_t kc = s < nk ? s : nk - 1;
#pragma unroll
    for (int q = 0; q < C::kLoadsPerTile; ++q) issue_q(kc, lds0 + s * C::kStageBytes, q);
  }
  int stage = 0;  // stage of tile kt
  for (int64_t kt = 0; kt < nk; ++kt) {
    // tile kt has landed for every wave, and the stage of tile kt - 1 is free again
    wait_and_barrier<C::kLoadsPerTile*(NS - 2)>();
    const int64_t kn = kt + NS - 1 < nk ? kt + NS - 1 : nk - 1;
    const uint32_t dst = lds0 + (stage == 0 ? NS - 1 : stage - 1) * C::kStageBytes;
    const unsigned char* st = sm.stage[stage];
    t.template mma<C, C::kLoadsPerTile, T>(st, st + C::BM * ROW_BYTES, wm0, wn0,
                                           [&](int q) { issue_q(kn, dst, q); });
    stage = stage + 1 == NS ? 0 : stage + 1;
  }
  wait_and_barrier<0>();  // the ring may be reused by the caller's next main loop
}

template <class C, typename T = bf16_t>
__device__ __forceinline__ void mainloop(Tile& t, Smem<C>& sm, const T* abase,
                                         const T* bbase, int64_t ld, int64_t m0a, int64_t m0b,
                                         int64_t M, int64_t K, int wm0, int wn0) {
  mainloop<C, T>(t, sm, abase, bbase, ld, m0a, m0b, M, M, K, wm0, wn0);
}

}  // namespace mb16d
