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
// A stage is BK = 32 rows of 128 columns (256 bytes a row) per operand. 16-byte chunks are
// XOR-swizzled, physical chunk = logical chunk ^ ((row & 3) << 2), so that the four rows a
// half-wave's transposing read touches fall into four different 64-byte bank windows. The
// swizzle is applied on the global side (each lane fetches the chunk that belongs at its
// fixed LDS slot), since a direct load lands at LDS[base + lane * 16] unconditionally.
//
// Edges: columns past the matrix are fetched from a clamped in-row position (their results
// are discarded by the caller); a last k tile that is not whole is fetched as the last 32
// rows of the matrix and the rows it shares with the tile before are zeroed in one operand
// after the read. K >= 32, ld % 8 == 0, 16-byte aligned bases, 32 * ld * 2 < 2^32.
#pragma once

#include <type_traits>

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

constexpr int BK = 32;              // rows (k) of a stage
constexpr int BT = 128;             // columns of an operand tile
constexpr int ROW_BYTES = BT * 2;   // 256
constexpr int OPND_BYTES = BK * ROW_BYTES;   // 8 KB
constexpr int STAGE_BYTES = 2 * OPND_BYTES;  // P tile, then Q tile
constexpr int NS = 4;               // ring depth
constexpr int NTHREADS = 256, NWAVES = 4;
constexpr int LOADS_PER_OPND = OPND_BYTES / 1024 / NWAVES;  // per wave and stage: 2
constexpr int LOADS = 2 * LOADS_PER_OPND;

struct Smem {
  alignas(1024) unsigned char stage[NS][STAGE_BYTES];
};

// Byte offset, from the first row of a k tile, of the 16 bytes this lane fetches with the
// r-th load of an operand tile: group g = r * NWAVES + wave covers tile rows 4 g .. 4 g + 3.
__device__ __forceinline__ uint32_t load_offset(int64_t ld, int64_t col0, int r) {
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int row = (r * NWAVES + wave) * 4 + (lane >> 4);
  const int chunk = (lane & 15) ^ ((lane >> 4) << 2);  // logical chunk that lives at this slot
  int64_t col = col0 + chunk * 8;
  col = col + 8 <= ld ? col : ld - 8;
  return static_cast<uint32_t>((row * ld + col) * 2);
}

__device__ __forceinline__ uint32_t load_lds(int r) {
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  return static_cast<uint32_t>((r * NWAVES + wave) * 1024);
}

// LDS byte offset, inside an operand tile, of this lane's address for the transposing read
// of the 32-column piece that starts at column c0 (a multiple of 32), rows 0 .. 3 of k half
// (lane / 32); add (16 s + 4 r) * ROW_BYTES for k16 step s and read r.
__device__ __forceinline__ uint32_t frag_offset(int c0) {
  const int lane = threadIdx.x & 63;
  const int e = (lane & 15) >> 2;                       // row inside the 4-row block
  const int m = c0 + ((lane >> 4) & 1) * 16 + (lane & 3) * 4;
  const int chunk = (m >> 3) ^ (e << 2);
  return static_cast<uint32_t>(((lane >> 5) * 8 + e) * ROW_BYTES + chunk * 16 + ((m >> 2) & 1) * 8);
}

__device__ __forceinline__ shortx4 read_tr(const unsigned char* p) {
  return __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_shortx4_ptr)(p));
}

// Operand of one MFMA: k = 16 s + (lane / 32) * 8 .. + 7 of column (lane % 32) of the piece.
// dup > 0: rows below dup of the tile repeat the tile before and are zeroed.
template <bool MASK>
__device__ __forceinline__ bf16x8 read_operand(const unsigned char* opnd, uint32_t frag, int s, int dup) {
  const shortx4 lo = read_tr(opnd + frag + (16 * s) * ROW_BYTES);
  const shortx4 hi = read_tr(opnd + frag + (16 * s + 4) * ROW_BYTES);
  shortx8 v = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  if (MASK) {
    const int k0 = 16 * s + ((threadIdx.x & 63) >> 5) * 8;
#pragma unroll
    for (int j = 0; j < 8; ++j)
      if (k0 + j < dup) v[j] = 0;
  }
  return __builtin_bit_cast(bf16x8, v);
}

// The 64 x 64 accumulator piece of one wave: acc[i][j] covers rows (of P's columns)
// wp0 + 32 i .., columns (of Q's columns) wq0 + 32 j ..; element v of lane l is
// row (v / 4) * 8 + (l / 32) * 4 + (v % 4), column l % 32 of its 32 x 32 tile.
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

  template <bool MASK, class IssueFn>
  __device__ __forceinline__ void mma(const unsigned char* Ps, const unsigned char* Qs, const uint32_t (&fp)[2],
                                      const uint32_t (&fq)[2], int dup, IssueFn issue) {
    constexpr int KS = BK / 16;
    bf16x8 pv[KS][2], qv[KS][2];
#pragma unroll
    for (int s = 0; s < KS; ++s) {
#pragma unroll
      for (int i = 0; i < 2; ++i) pv[s][i] = read_operand<MASK>(Ps, fp[i], s, dup);
#pragma unroll
      for (int j = 0; j < 2; ++j) qv[s][j] = read_operand<false>(Qs, fq[j], s, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int s = 0; s < KS; ++s) {
#pragma unroll
      for (int i = 0; i < 2; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
          acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(pv[s][i], qv[s][j], acc[i][j], 0, 0, 0);
#pragma unroll
      for (int q = s * (LOADS / KS); q < (s + 1) * (LOADS / KS); ++q) issue(q);
      __builtin_amdgcn_sched_barrier(0);
    }
  }
};

// acc += P[:, p0 .. p0 + 127]^T . Q[:, q0 .. q0 + 127] over all K rows. (wp0, wq0): this
// wave's corner in the block tile. Every trip issues exactly one tile's loads (past the end
// the last tile again, into a stage nobody reads), so LOADS * (NS - 2) loads may stay in
// flight while a tile is awaited.
__device__ __forceinline__ void mainloop(Tile& t, Smem& sm, const bf16_t* P, int64_t ldp, int64_t p0,
                                         const bf16_t* Q, int64_t ldq, int64_t q0, int64_t K, int wp0,
                                         int wq0) {
  const int64_t nk = (K + BK - 1) / BK;
  const int dup = static_cast<int>(nk * BK - K);  // rows the last tile repeats
  const uint32_t lds0 = lds_offset(&sm.stage[0][0]);
  uint32_t off[LOADS];
#pragma unroll
  for (int q = 0; q < LOADS; ++q) {
    off[q] = q < LOADS_PER_OPND ? load_offset(ldp, p0, q) : load_offset(ldq, q0, q - LOADS_PER_OPND);
    asm volatile("" : "+v"(off[q]));
  }
  const uint32_t fp[2] = {frag_offset(wp0), frag_offset(wp0 + 32)};
  const uint32_t fq[2] = {frag_offset(wq0), frag_offset(wq0 + 32)};
  auto first_row = [&](int64_t kt) { return kt + 1 < nk ? kt * BK : K - BK; };
  auto issue_q = [&](int64_t kt, uint32_t st, int q) {
    const int64_t row = first_row(kt);
    if (q < LOADS_PER_OPND) load16_to_lds(P + row * ldp, off[q], st + load_lds(q));
    else load16_to_lds(Q + row * ldq, off[q], st + OPND_BYTES + load_lds(q - LOADS_PER_OPND));
  };
#pragma unroll
  for (int s = 0; s < NS - 1; ++s) {
    const int64_t kc = s < nk ? s : nk - 1;
#pragma unroll
    for (int q = 0; q < LOADS; ++q) issue_q(kc, lds0 + s * STAGE_BYTES, q);
  }
  // One trip: wait for tile kt, refill the stage read in the trip before with tile
  // kt + NS - 1, multiply. The last tile is taken outside the loop because it alone may
  // need the mask.
  int stage = 0;
  auto trip = [&](int64_t kt, auto masked) {
    wait_and_barrier<LOADS*(NS - 2)>();
    const int64_t kn = kt + NS - 1 < nk ? kt + NS - 1 : nk - 1;
    const uint32_t dst = lds0 + ((stage + NS - 1) & (NS - 1)) * STAGE_BYTES;
    const unsigned char* st = sm.stage[stage];
    t.mma<decltype(masked)::value>(st, st + OPND_BYTES, fp, fq, dup, [&](int q) { issue_q(kn, dst, q); });
    stage = (stage + 1) & (NS - 1);
  };
  for (int64_t kt = 0; kt + 1 < nk; ++kt) trip(kt, std::false_type{});
  if (dup > 0) trip(nk - 1, std::true_type{});
  else trip(nk - 1, std::false_type{});
  wait_and_barrier<0>();  // the stage memory is the caller's again
}

}  // namespace mb16t
