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

// Operand of one MFMA: k = 16 s + (lane / 32) * 8 .. + 7 of column (lane % 32) of the piece.
__device__ __forceinline__ bf16x8 read_operand(const unsigned char* opnd, uint32_t frag, int s) {
  const shortx4 lo = read_tr(opnd + frag + (16 * s) * ROW_BYTES);
  const shortx4 hi = read_tr(opnd + frag + (16 * s + 4) * ROW_BYTES);
  return __builtin_bit_cast(bf16x8, __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7));
}

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

  template <class IssueFn>
  __device__ __forceinline__ void mma(const unsigned char* Ps, const unsigned char* Qs, const uint32_t (&fp)[C::TP],
                                      const uint32_t (&fq)[C::TQ], IssueFn issue) {
    constexpr int KS = BK / 16;
    bf16x8 pv[KS][C::TP], qv[KS][C::TQ];
#pragma unroll
    for (int s = 0; s < KS; ++s) {
#pragma unroll
      for (int i = 0; i < C::TP; ++i) pv[s][i] = read_operand(Ps, fp[i], s);
#pragma unroll
      for (int j = 0; j < C::TQ; ++j) qv[s][j] = read_operand(Qs, fq[j], s);
    }
    __builtin_amdgcn_sched_barrier(0);
    constexpr int PER_STEP = (C::kLoads + KS - 1) / KS;
#pragma unroll
    for (int s = 0; s < KS; ++s) {
#pragma unroll
      for (int i = 0; i < C::TP; ++i)
#pragma unroll
        for (int j = 0; j < C::TQ; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(pv[s][i], qv[s][j], acc[i][j], 0, 0, 0);
#pragma unroll
      for (int q = s * PER_STEP; q < (s + 1) * PER_STEP && q < C::kLoads; ++q) issue(q);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
};

// acc += P[:, p0 .. p0 + BP - 1]^T . Q[:, q0 .. q0 + BQ - 1] over all K rows. (wp0, wq0):
// this wave's corner in the block tile. Every trip issues exactly one tile's loads (past
// the end the last tile again, into a stage nobody reads), so kLoads * (NS - 2) loads may
// stay in flight while a tile is awaited.
template <class C>
__device__ __forceinline__ void mainloop(Tile<C>& t, Smem<C>& sm, const bf16_t* P, int64_t ldp, int64_t p0,
                                         const bf16_t* Q, int64_t ldq, int64_t q0, int64_t K, int wp0,
                                         int wq0) {
  constexpr int NS = C::NS;
  const int64_t nk = (K + BK - 1) / BK;
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
  auto first_row = [&](int64_t kt) { return kt + 1 < nk ? kt * BK : K - BK; };
  auto issue_q = [&](int64_t kt, uint32_t st, int q) {
    const int64_t row = first_row(kt);
    const uint32_t dst = st + static_cast<uint32_t>((q * C::kWaves + wave) * 1024);
    if (sub_of(q) < C::SUBP) load16_to_lds(P + row * ldp, off[q], dst);
    else load16_to_lds(Q + row * ldq, off[q], dst);
  };
#pragma unroll
  for (int s = 0; s < NS - 1; ++s) {
    const int64_t kc = s < nk ? s : nk - 1;
#pragma unroll
    for (int q = 0; q < C::kLoads; ++q) issue_q(kc, lds0 + s * C::kStageBytes, q);
  }
  // One trip: wait for tile kt, refill the stage read in the trip before with tile
  // kt + NS - 1, multiply. A last tile that repeats rows of the one before has them zeroed
  // in P's part of its stage first.
  int stage = 0;
  for (int64_t kt = 0; kt < nk; ++kt) {
    wait_and_barrier<C::kLoads*(NS - 2)>();
    if (kt + 1 == nk && dup > 0) {
      for (int idx = threadIdx.x; idx < C::SUBP * dup * (ROW_BYTES / 16); idx += C::kThreads) {
        const int sub = idx / (dup * (ROW_BYTES / 16)), rest = idx % (dup * (ROW_BYTES / 16));
        *reinterpret_cast<uint4*>(&sm.stage[stage][sub * SUB_BYTES + rest * 16]) = make_uint4(0u, 0u, 0u, 0u);
      }
      __syncthreads();
    }
    const int64_t kn = kt + NS - 1 < nk ? kt + NS - 1 : nk - 1;
    const uint32_t dst = lds0 + ((stage + NS - 1) & (NS - 1)) * C::kStageBytes;
    const unsigned char* st = sm.stage[stage];
    t.mma(st, st + C::SUBP * SUB_BYTES, fp, fq, [&](int q) { issue_q(kn, dst, q); });
    stage = (stage + 1) & (NS - 1);
  }
  wait_and_barrier<0>();  // the stage memory is the caller's again
}

}  // namespace mb16t
