// bf16 MFMA tiles for operands whose contraction index is the SLOW one in memory (gfx950).
//
// C[p][q] = sum_k P[k][p] * Q[k][q], with P = [K, ldp] and Q = [K, ldq] row-major: the
// per-sample weight gradient of a Linear layer, contracted over the sequence positions.
// v_mfma_f32_32x32x16_bf16 wants every lane to hold 8 consecutive k of one row, which is a
// column of the matrices as they lie in memory. Instead of transposing in registers, the
// tiles go global -> LDS untouched (global_load_lds_dwordx4, as in mfma_bf16_dlds.h) and
// the transposition is done by the LDS read itself: ds_read_b64_tr_b16 hands lane i of
// each group of 16 lanes the i-th 16-bit column of the 4 x 16 block that the group's
// sixteen 8-byte addresses describe. With source lane 4 e + c of a group pointing at
// (row k + e, columns m + 4 c .. + 3), result lane i holds column m + i of rows k .. k + 3;
// two such reads make one MFMA operand (8 k).
//
// A stage holds BK = 32 rows of every operand tile, in sub-tiles of 128 columns (256 bytes
// a row, 8 KB a sub-tile). 16-byte chunks are
// XOR-swizzled, physical chunk = logical chunk ^ ((row & 3) << 2), so that the four rows a
// half-wave's transposing read touches fall into four different 64-byte bank windows. The
// swizzle is applied on the global side (each lane fetches the chunk that belongs at its
// fixed LDS slot), since a direct load lands at LDS[base + lane * 16] unconditionally.
//
// Edges: columns past the matrix are fetched from a clamped in-row position (their results
// are discarded by the caller); a last k tile that is not whole is fetched as the last 32
// rows of the matrix and the rows it shares with the tile before are zeroed in one operand's
// stage before the read. K >= 32, ld % 8 == 0, 16-byte aligned bases, 32 * ld * 2 < 2^32.
#pragma once

#include "dpk_common.h"
#include "mfma_bf16_dlds.h"

namespace mb16t {

using mb16::bf16x8;
using mb16::floatx16;
using mb16d::load16_to_lds;
using mb16d::lds_offset;
using mb16d::wait_and_barrier;

typedef short shortx4 __attribute__((ext_vector_type(4)));
typedef short shortx8 __attribute__((ext_vector_type(8)));
typedef __attribute__((address_space(3))) shortx4* lds_shortx4_ptr;

// s_waitcnt lgkmcnt(0) with the other counters left alone (gfx9 encoding: vmcnt 63, expcnt 7)
constexpr int kWaitLgkm0 = 0xC07F;
constexpr int BK = 32;                      // rows (k) of a stage
constexpr int SUB = 128;                    // columns of a sub-tile
constexpr int ROW_BYTES = SUB * 2;          // 256
constexpr int SUB_BYTES = BK * ROW_BYTES;   // 8 KB: one sub-tile of one stage

// WP x WQ waves, each owning TP x TQ MFMA tiles of 32 x 32: a block tile of
// (32 WP TP) columns of P by (32 WQ TQ) columns of Q, both multiples of 128. An operand
// tile is kept as sub-tiles of 128 columns, each laid out as described above.
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

// The q-th load of a wave moves 1 KB group G = q * kWaves + wave of the stage image:
// rows 4 (G % 8) .. + 3 of sub-tile G / 8. Byte offset, from the first row of a k tile and
// the operand's first column, of the 16 bytes this lane fetches for it.
template <class C>
__device__ __forceinline__ uint32_t load_offset(int64_t ld, int64_t col0, int q) {
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int G = q * C::kWaves + wave;
  const int row = (G & 7) * 4 + (lane >> 4);
  const int chunk = (lane & 15) ^ ((lane >> 4) << 2);  // logical chunk that lives at this slot
  int64_t col = col0 + chunk * 8;
  col = col + 8 <= ld ? col : ld - 8;
  return static_cast<uint32_t>((row * ld + col) * 2);
}

// LDS byte offset, inside an operand's part of a stage, of this lane's address for the
// transposing read of the 32-column piece that starts at column c0 (a multiple of 32) of
// the operand tile, rows 0 .. 3 of k half (lane / 32); add (16 s + 4 r) * ROW_BYTES for
// k16 step s and read r.
__device__ __forceinline__ uint32_t frag_offset(int c0) {
  const int lane = threadIdx.x & 63;
  const int e = (lane & 15) >> 2;                       // row inside the 4-row block
  const int m = (c0 & (SUB - 1)) + ((lane >> 4) & 1) * 16 + (lane & 3) * 4;
  const int chunk = (m >> 3) ^ (e << 2);
  return static_cast<uint32_t>((c0 / SUB) * SUB_BYTES + ((lane >> 5) * 8 + e) * ROW_BYTES + chunk * 16 +
                               ((m >> 2) & 1) * 8);
}

__device__ __forceinline__ shortx4 read_tr(const unsigned char* p) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_shortx4_ptr)(p));
}

// The operand registers of one k tile for one wave, as the halves that one transposing read
// delivers: half h of operand (s, i) is k = 16 s + (lane / 32) * 8 + 4 h .. + 3 of column
// (lane % 32) of the i-th 32-column piece.
template <class C>
struct Frags {
  static constexpr int KS = BK / 16;
  static constexpr int kPerStep = 2 * (C::TP + C::TQ);  // reads of one k16 step
  static constexpr int kReads = KS * kPerStep;
  shortx4 p[KS][C::TP][2], q[KS][C::TQ][2];

  // the r-th read of the tile, r < kReads: k16 steps in order, P's pieces before Q's
  __device__ __forceinline__ void read(int r, const unsigned char* Ps, const unsigned char* Qs,
                                       const uint32_t (&fp)[C::TP], const uint32_t (&fq)[C::TQ]) {
    const int s = r / kPerStep, x = (r % kPerStep) / 2, h = r % 2;
    const int row_bytes = (16 * s + 4 * h) * ROW_BYTES;
    if (x < C::TP) p[s][x][h] = read_tr(Ps + fp[x] + row_bytes);
    else q[s][x - C::TP][h] = read_tr(Qs + fq[x - C::TP] + row_bytes);
  }
  __device__ __forceinline__ bf16x8 operand_p(int s, int i) const {
    return __builtin_bit_cast(bf16x8, __builtin_shufflevector(p[s][i][0], p[s][i][1], 0, 1, 2, 3, 4, 5, 6, 7));
  }
  __device__ __forceinline__ bf16x8 operand_q(int s, int j) const {
    return __builtin_bit_cast(bf16x8, __builtin_shufflevector(q[s][j][0], q[s][j][1], 0, 1, 2, 3, 4, 5, 6, 7));
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

  // The MFMAs of the tile in `cur`, with the LDS reads of the next tile (into `nxt`) and
  // the global -> LDS loads of a later one (issue(q), q < kLoads) dealt out evenly between
  // them: a wave issues in order, so reads queued in one burst would hold its MFMAs back for
  // as long as the LDS takes to accept them.
  //
  // kRescale: every 32 x 32 piece of the accumulator is multiplied by f just before the first
  // MFMA that adds to it, so that the multiplications of one piece run under the MFMA of the
  // piece before.
  template <bool kRescale = false, class IssueFn>
  __device__ __forceinline__ void mma(const Frags<C>& cur, Frags<C>& nxt, const unsigned char* Ps,
                                      const unsigned char* Qs, const uint32_t (&fp)[C::TP],
                                      const uint32_t (&fq)[C::TQ], IssueFn issue, float f = 1.f) {
    constexpr int KS = Frags<C>::KS, M = KS * C::TP * C::TQ, R = Frags<C>::kReads, L = C::kLoads;
#pragma unroll
    for (int m = 0; m < M; ++m) {
      const int s = m / (C::TP * C::TQ), i = (m / C::TQ) % C::TP, j = m % C::TQ;
      if constexpr (kRescale) {
        if (s == 0) {
#pragma unroll
          for (int v = 0; v < 16; ++v) acc[i][j][v] *= f;
        }
      }
      acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(cur.operand_p(s, i), cur.operand_q(s, j), acc[i][j], 0, 0, 0);
#pragma unroll
      for (int r = m * R / M; r < (m + 1) * R / M; ++r) nxt.read(r, Ps, Qs, fp, fq);
#pragma unroll
      for (int q = m * L / M; q < (m + 1) * L / M; ++q) issue(q);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
};

// acc += P[:, p0 .. p0 + BP - 1]^T . Q[:, q0 .. q0 + BQ - 1] over all K rows. (wp0, wq0):
// this wave's corner in the block tile.
//
// Software pipeline: while the MFMAs of tile kt run out of one set of operand registers,
// the LDS reads of tile kt + 1 fill the other set and NS - 1 further tiles are on their way
// from memory. Tile kt lives in stage kt % NS, which is refilled as soon as every wave holds
// tile kt in registers. Every step issues exactly one tile's loads (past the end the last
// tile again), so kLoads * (NS - 2) loads may stay in flight while a tile is awaited.
//
// kWeighted: the K rows are units of tiles_per_unit k tiles each (K a whole number of them)
// and unit u counts coef[u] times: acc = sum_u coef[u] * (P_u^T Q_u). The accumulator is kept
// in units of the current unit's coefficient: at a unit's first tile it is rescaled by
// coef[u - 1] / coef[u], and by the last coefficient at the end. What it holds is then at most
// (sum of the weighted terms so far) / coef[u], so it overflows only where the unit's own
// unweighted product nearly does. No rescaling multiplies by more than 2^40: a coefficient smaller
// than 2^-40 of the one before it (an exact zero: a masked sample) counts as that fraction of it,
// and any coefficient below kMinCoef as kMinCoef. Such a unit then enters the sum with a weight
// of at most 2^-40 of its neighbour's, far below fp32 resolution, where an exact zero would turn
// the rescaling into a division by zero and a fixed floor alone would let a partial sum above
// 3e8 overflow. (Leaving the unit's MFMAs out instead, by a second copy of the step or by zeroing
// one operand's registers under a branch, cost the 256 x 256 kernel 12 % of its rate.)
// Coefficients are non-negative; a NaN stays a NaN.
constexpr float kMinCoef = 1e-30f;
constexpr float kMinRatio = 9.094947017729282e-13f;  // 2^-40
__device__ __forceinline__ float floored_coef(float c, float prev) {
  const float floor = prev * kMinRatio > kMinCoef ? prev * kMinRatio : kMinCoef;
  return c < floor ? floor : c;
}

template <class C, bool kWeighted = false>
__device__ __forceinline__ void mainloop(Tile<C>& t, Smem<C>& sm, const bf16_t* P, int64_t ldp, int64_t p0,
                                         const bf16_t* Q, int64_t ldq, int64_t q0, int64_t K, int wp0,
                                         int wq0, const float* coef = nullptr, int64_t tiles_per_unit = 0) {
  constexpr int NS = C::NS;
  const int64_t nk = (K + BK - 1) / BK;
  int64_t boundary = 0, unit = 0, units = 0;
  float c_cur = 1.f, c_nxt = 1.f;
  if constexpr (kWeighted) {
    units = nk / tiles_per_unit;
    boundary = tiles_per_unit;
    // (read one unit ahead and not looked at before its unit begins: nothing waits for the load)
    c_cur = floored_coef(coef[0], 0.f);
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
  // tile kt lives in stage kt % NS; tiles past the end are the last tile again (their
  // stages are read into registers that no MFMA uses, or not at all)
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
  // refilled, with tile kt + NS) and its loads of tile kt + 1 have landed.
  auto step = [&](int64_t kt, const Frags<C>& cur, Frags<C>& nxt) {
    // as a builtin, not inline assembly: the compiler's own wait insertion then knows that
    // `cur` is complete and does not wait for the reads of `nxt` before an MFMA
    __builtin_amdgcn_s_waitcnt(kWaitLgkm0);
    __builtin_amdgcn_sched_barrier(0);
    wait_and_barrier<C::kLoads*(NS - 2)>();
    zero_repeated_rows(kt + 1);
    const unsigned char* st = sm.stage[(kt + 1) & (NS - 1)];
    if constexpr (kWeighted) {
      if (kt == boundary) {  // first tile of the next unit (uniform over the block)
        const float c_new = floored_coef(c_nxt, c_cur);
        const float ratio = c_cur / c_new;
        c_cur = c_new;
        ++unit;
        boundary += tiles_per_unit;
        c_nxt = coef[unit + 1 < units ? unit + 1 : units - 1];
        // a wave with a small accumulator has the registers to spare for a second copy of the
        // step with the multiplications dealt out between its MFMAs; a large one (a long step:
        // the multiplications are a small part of a unit) rescales first
        if constexpr (C::TP * C::TQ <= 4) {
          t.template mma<true>(cur, nxt, st, st + C::SUBP * SUB_BYTES, fp, fq, [&](int q) { issue_q(kt + NS, q); }, ratio);
          return;
        } else {
          t.scale(ratio);
        }
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

}  // namespace mb16t
