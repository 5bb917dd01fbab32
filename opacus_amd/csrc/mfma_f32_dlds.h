// fp32 MFMA tiles for operands whose contraction index is the slow one in memory, fed by
// direct global -> LDS loads (gfx950): the fp32 sibling of mfma_bf16_tr.h.
//
// C[p][q] = sum_k P[k][p] * Q[k][q], P = [K, ldp] and Q = [K, ldq] row-major.
// v_mfma_f32_32x32x2f32 wants lane l to hold element (k = l / 32, column l % 32) of each
// operand: 32 consecutive floats of one row per half-wave, which is how the matrices lie in
// memory, so no transposition is involved. Tiles go global -> LDS untouched
// (global_load_lds_dwordx4) through a ring of stages, and two sets of operand registers let
// the LDS reads of tile kt + 1 run between the MFMAs of tile kt.
//
// A stage holds BK = 16 rows of every operand tile, in sub-tiles of 128 columns (512 bytes
// a row, 8 KB a sub-tile). The two half-waves of an operand read touch two consecutive rows
// at the same columns; 16-byte chunks of odd rows are moved by 128 bytes (physical chunk =
// logical chunk ^ 8) so that the two rows fall into different halves of the bank space.
// The swizzle is applied on the global side: a direct load lands at LDS[base + lane * 16]
// unconditionally, so each lane fetches the chunk that belongs at its slot.
//
// Edges as in mfma_bf16_tr.h: columns past the matrix are fetched from a clamped in-row
// position (the caller discards their results); a last k tile that is not whole is fetched
// as the last 16 rows of the matrix and the rows it shares with the tile before are zeroed
// in one operand's stage before the read. K >= 16, ld % 4 == 0, 16-byte aligned bases,
// 16 * ld * 4 < 2^32.
#pragma once

#include "dpk_common.h"
#include "mfma_bf16_dlds.h"
#include "mfma_bf16_tr.h"

namespace mf32d {

using mb16::floatx16;
using mb16d::load16_to_lds;
using mb16d::lds_offset;
using mb16d::wait_and_barrier;

// s_waitcnt lgkmcnt(0) with the other counters left alone (gfx9 encoding: vmcnt 63, expcnt 7)
constexpr int kWaitLgkm0 = 0xC07F;
constexpr int BK = 16;                      // rows (k) of a stage
constexpr int SUB = 128;                    // columns of a sub-tile
constexpr int ROW_BYTES = SUB * 4;          // 512
constexpr int SUB_BYTES = BK * ROW_BYTES;   // 8 KB: one sub-tile of one stage

template <int WP_, int WQ_, int TP_, int TQ_, int NS_>
struct Config {
  static constexpr int WP = WP_, WQ = WQ_, TP = TP_, TQ = TQ_, NS = NS_;
  static constexpr int kWaves = WP * WQ, kThreads = 64 * kWaves;
  static constexpr int BP = 32 * WP * TP, BQ = 32 * WQ * TQ;
  static constexpr int SUBP = BP / SUB, SUBQ = BQ / SUB;
  static constexpr int kStageBytes = (SUBP + SUBQ) * SUB_BYTES;  // P sub-tiles, then Q sub-tiles
  static constexpr int kLoads = (SUBP + SUBQ) * (SUB_BYTES / 1024) / kWaves;  // per wave and stage
  static_assert(BP % SUB == 0 && BQ % SUB == 0, "block tile: multiples of 128 columns");
  static_assert(kWaves == 4 || kWaves == 8, "a sub-tile's eight 1 KB groups must split evenly over the waves");
  static_assert((NS & (NS - 1)) == 0 && NS >= 2, "ring depth: a power of two");
};

template <class C>
struct Smem {
  alignas(1024) unsigned char stage[C::NS][C::kStageBytes];
};

// The q-th load of a wave moves 1 KB group G = q * kWaves + wave of the stage image: rows
// 2 (G % 8) and 2 (G % 8) + 1 of sub-tile G / 8. Byte offset, from the first row of a k tile
// and the operand's first column, of the 16 bytes this lane fetches for it.
template <class C>
__device__ __forceinline__ uint32_t load_offset(int64_t ld, int64_t col0, int q) {
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int G = q * C::kWaves + wave;
  const int row = (G & 7) * 2 + (lane >> 5);
  const int chunk = (lane & 31) ^ ((lane >> 5) << 3);  // logical chunk that lives at this slot
  int64_t col = col0 + chunk * 4;
  col = col + 4 <= ld ? col : ld - 4;
  return static_cast<uint32_t>((row * ld + col) * 4);
}

// LDS byte offset, inside an operand's part of a stage, of this lane's element of the
// 32-column piece that starts at column c0 (a multiple of 32) of the operand tile, k2 step 0
// (rows 0 and 1); add 2 s * ROW_BYTES for step s.
__device__ __forceinline__ uint32_t frag_offset(int c0) {
  const int lane = threadIdx.x & 63;
  const int r = lane >> 5;
  const int m = (c0 & (SUB - 1)) + (lane & 31);
  const int chunk = (m >> 2) ^ (r << 3);
  return static_cast<uint32_t>((c0 / SUB) * SUB_BYTES + r * ROW_BYTES + chunk * 16 + (m & 3) * 4);
}

// The operand registers of one k tile for one wave.
template <class C>
struct Frags {
  static constexpr int KS = BK / 2;
  static constexpr int kPerStep = C::TP + C::TQ;
  static constexpr int kReads = KS * kPerStep;
  float p[KS][C::TP], q[KS][C::TQ];

  // the r-th read of the tile, r < kReads: k2 steps in order, P's pieces before Q's
  __device__ __forceinline__ void read(int r, const unsigned char* Ps, const unsigned char* Qs,
                                       const uint32_t (&fp)[C::TP], const uint32_t (&fq)[C::TQ]) {
    const int s = r / kPerStep, x = r % kPerStep;
    if (x < C::TP) p[s][x] = *reinterpret_cast<const float*>(Ps + fp[x] + 2 * s * ROW_BYTES);
    else q[s][x - C::TP] = *reinterpret_cast<const float*>(Qs + fq[x - C::TP] + 2 * s * ROW_BYTES);
  }
};

// The accumulator piece of one wave: acc[i][j] covers rows (columns of P) wp0 + 32 i ..,
// columns (columns of Q) wq0 + 32 j ..; element v of lane l is row
// (v / 4) * 8 + (l / 32) * 4 + (v % 4), column l % 32 of its 32 x 32 tile.
template <class C>
struct Tile {
  floatx16 acc[C::TP][C::TQ];

  __device__ __forceinline__ void clear() {
#pragma unroll
    for (int i = 0; i < C::TP; ++i)
#pragma unroll
      for (int j = 0; j < C::TQ; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][j][v] = 0.f;
  }

  __device__ __forceinline__ void scale(float f) {
#pragma unroll
    for (int i = 0; i < C::TP; ++i)
#pragma unroll
      for (int j = 0; j < C::TQ; ++j)
#pragma unroll
        for (int v = 0; v < 16; ++v) acc[i][j][v] *= f;
  }

  // The MFMAs of the tile in `cur`, with the LDS reads of the next tile (into `nxt`) and the
  // global -> LDS loads of a later one (issue(q), q < kLoads) dealt out evenly between them.
  template <class IssueFn>
  __device__ __forceinline__ void mma(const Frags<C>& cur, Frags<C>& nxt, const unsigned char* Ps,
                                      const unsigned char* Qs, const uint32_t (&fp)[C::TP],
                                      const uint32_t (&fq)[C::TQ], IssueFn issue) {
    constexpr int KS = Frags<C>::KS, M = KS * C::TP * C::TQ, R = Frags<C>::kReads, L = C::kLoads;
#pragma unroll
    for (int m = 0; m < M; ++m) {
      const int s = m / (C::TP * C::TQ), i = (m / C::TQ) % C::TP, j = m % C::TQ;
      acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(cur.p[s][i], cur.q[s][j], acc[i][j], 0, 0, 0);
#pragma unroll
      for (int r = m * R / M; r < (m + 1) * R / M; ++r) nxt.read(r, Ps, Qs, fp, fq);
#pragma unroll
      for (int q = m * L / M; q < (m + 1) * L / M; ++q) issue(q);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
};

// acc += P[:, p0 .. p0 + BP - 1]^T . Q[:, q0 .. q0 + BQ - 1] over all K rows. (wp0, wq0):
// this wave's corner in the block tile. Tile kt lives in stage kt % NS, which is refilled
// (with tile kt + NS) as soon as every wave holds tile kt in registers. Every step issues
// exactly one tile's loads (past the end the last tile again), so kLoads * (NS - 2) loads may
// stay in flight while a tile is awaited.
//
// kWeighted: as in mfma_bf16_tr.h. The K rows are units of tiles_per_unit k tiles each and unit u
// counts coef[u] times; the accumulator is kept in units of the current unit's coefficient,
// rescaled by coef[u - 1] / coef[u] at a unit's first tile (an fp32 tile's 64 MFMAs of 64 cycles
// each dwarf the 64 multiplications) and by the last coefficient at the end, with the same floors.
template <class C, bool kWeighted = false>
__device__ __forceinline__ void mainloop(Tile<C>& t, Smem<C>& sm, const float* P, int64_t ldp, int64_t p0,
                                         const float* Q, int64_t ldq, int64_t q0, int64_t K, int wp0,
                                         int wq0, const float* coef = nullptr, int64_t tiles_per_unit = 0) {
  constexpr int NS = C::NS;
  const int64_t nk = (K + BK - 1) / BK;
  int64_t boundary = 0, unit = 0, units = 0;
  float c_cur = 1.f, c_nxt = 1.f;
  if constexpr (kWeighted) {
    units = nk / tiles_per_unit;
    boundary = tiles_per_unit;
    c_cur = mb16t::floored_coef(coef[0], 0.f);
    c_nxt = coef[units > 1 ? 1 : 0];
  }
  const int dup = static_cast<int>(nk * BK - K);  // rows the last tile repeats
  const uint32_t lds0 = lds_offset(&sm.stage[0][0]);
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  // which sub-tile a load belongs to does not depend on the wave (8 % kWaves == 0)
  auto sub_of = [](int q) { return q * C::kWaves / 8; };
  uint32_t off[C::kLoads];
#pragma unroll
  for (int q = 0; q < C::kLoads; ++q) {
    const int S = sub_of(q);
    off[q] = S < C::SUBP ? load_offset<C>(ldp, p0 + S * SUB, q) : load_offset<C>(ldq, q0 + (S - C::SUBP) * SUB, q);
    asm volatile("" : "+v"(off[q]));
  }
  uint32_t fp[C::TP], fq[C::TQ];
#pragma unroll
  for (int i = 0; i < C::TP; ++i) fp[i] = frag_offset(wp0 + 32 * i);
#pragma unroll
  for (int j = 0; j < C::TQ; ++j) fq[j] = frag_offset(wq0 + 32 * j);
  auto issue_q = [&](int64_t kt, int q) {
    const int64_t kc = kt < nk ? kt : nk - 1;
    const int64_t row = kc + 1 < nk ? kc * BK : K - BK;
    const uint32_t dst = lds0 + static_cast<uint32_t>(kt & (NS - 1)) * C::kStageBytes +
                         static_cast<uint32_t>((q * C::kWaves + wave) * 1024);
    if (sub_of(q) < C::SUBP) load16_to_lds(P + row * ldp, off[q], dst);
    else load16_to_lds(Q + row * ldq, off[q], dst);
  };
  // rows of the last tile that repeat the tile before: zero them in P's part of the stage
  auto zero_repeated_rows = [&](int64_t kt) {
    if (kt + 1 != nk || dup == 0) return;
    unsigned char* st = sm.stage[kt & (NS - 1)];
    for (int idx = threadIdx.x; idx < C::SUBP * dup * (ROW_BYTES / 16); idx += C::kThreads) {
      const int sub = idx / (dup * (ROW_BYTES / 16)), rest = idx % (dup * (ROW_BYTES / 16));
      *reinterpret_cast<uint4*>(st + sub * SUB_BYTES + rest * 16) = make_uint4(0u, 0u, 0u, 0u);
    }
    __syncthreads();
  };
#pragma unroll
  for (int s = 0; s < NS; ++s)
#pragma unroll
    for (int q = 0; q < C::kLoads; ++q) issue_q(s, q);
  Frags<C> f0, f1;
  wait_and_barrier<C::kLoads*(NS - 1)>();  // tile 0 has landed for every wave
  zero_repeated_rows(0);
  {
    const unsigned char* st = sm.stage[0];
#pragma unroll
    for (int r = 0; r < Frags<C>::kReads; ++r) f0.read(r, st, st + C::SUBP * SUB_BYTES, fp, fq);
  }
  // Step kt: MFMAs of tile kt out of `cur` while the reads of tile kt + 1 fill `nxt`.
  // Before the barrier every wave has received its reads of tile kt (so stage kt % NS may be
  // refilled) and its loads of tile kt + 1 have landed. The wait is a builtin, not inline
  // assembly: the compiler's own wait insertion then knows that `cur` is complete and does
  // not wait for the reads of `nxt` before an MFMA.
  auto step = [&](int64_t kt, const Frags<C>& cur, Frags<C>& nxt) {
    __builtin_amdgcn_s_waitcnt(kWaitLgkm0);
    __builtin_amdgcn_sched_barrier(0);
    wait_and_barrier<C::kLoads*(NS - 2)>();
    zero_repeated_rows(kt + 1);
    const unsigned char* st = sm.stage[(kt + 1) & (NS - 1)];
    if constexpr (kWeighted) {
      if (kt == boundary) {  // first tile of the next unit (uniform over the block)
        const float c_new = mb16t::floored_coef(c_nxt, c_cur);
        t.scale(c_cur / c_new);
        c_cur = c_new;
        ++unit;
        boundary += tiles_per_unit;
        c_nxt = coef[unit + 1 < units ? unit + 1 : units - 1];
      }
    }
    t.mma(cur, nxt, st, st + C::SUBP * SUB_BYTES, fp, fq, [&](int q) { issue_q(kt + NS, q); });
  };
  int64_t kt = 0;
  for (; kt + 1 < nk; kt += 2) {
    step(kt, f0, f1);
    step(kt + 1, f1, f0);
  }
  if (kt < nk) step(kt, f0, f1);
  __builtin_amdgcn_s_waitcnt(kWaitLgkm0);
  wait_and_barrier<0>();  // the stage memory is the caller's again
  if constexpr (kWeighted) t.scale(c_cur);
}

}  // namespace mf32d
