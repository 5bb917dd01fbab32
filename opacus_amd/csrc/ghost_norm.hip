// Ghost-clipping per-sample gradient norms of nn.Linear
// (opacus/grad_sample/linear.py:54-93) without forming the gradients:
//   |gs_w[n]|_F^2 = sum_{t,t'} (b_t . b_t') (a_t . a_t'),   |gs_b[n]|^2 = sum_{t,t'} b_t . b_t'
// The reference writes both T x T Gram matrices to memory and reads them back for
// the elementwise contraction. Here a block owns one (ti, tj) tile pair of one
// sample: it forms the b b^T tile in MFMA accumulators (k loop over out), then
// the a a^T tile (k loop over in) - same accumulator layout - multiplies them
// element by element and reduces. The Grams are symmetric, so only tiles with
// ti <= tj are visited and off-diagonal ones count twice. One float per block
// goes to the workspace; a fixed-order reduction applies clamp(min=0) and sqrt
// (linear.py:87-89, :92).
#include <cstring>
#include <mutex>

#include "dpk_common.h"
#include "mfma_bf16.h"
#include "mfma_bf16_dlds.h"
#include "mfma_f32.h"

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / DPK_WAVE;

__device__ __forceinline__ void decode_pair(int pair, int nt, int& ti, int& tj) {
  ti = 0;
  while (pair >= nt - ti) {
    pair -= nt - ti;
    ++ti;
  }
  tj = ti + pair;
}

// Sums acc_g (.) acc_a and acc_g over the block; thread 0 writes the partials.
template <class TileT>
__device__ __forceinline__ void contract_and_store(const TileT& tg, const TileT& ta, bool have_a,
                                                   float weight, float* pw, float* pb, float* red) {
  float sw = 0.f, sb = 0.f;
#pragma unroll
  for (int i = 0; i < TileT::TM; ++i)
#pragma unroll
    for (int j = 0; j < TileT::TN; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const float g = tg.acc[i][j][v];
        sb += g;
        if (have_a) sw = fmaf(g, ta.acc[i][j][v], sw);
      }
  if (pw) {
    const float s = block_sum<kWaves>(sw, red);
    if (threadIdx.x == 0) pw[blockIdx.x] = s * weight;
  }
  if (pb) {
    const float s = block_sum<kWaves>(sb, red);
    if (threadIdx.x == 0) pb[blockIdx.x] = s * weight;
  }
}

template <int B, bool VEC>
__global__ __launch_bounds__(kThreads) void ghost_norm_f32_kernel(
    const float* __restrict__ b, const float* __restrict__ a, float* __restrict__ pw,
    float* __restrict__ pb, int64_t T, int64_t Dout, int64_t Din, int nt, int npairs) {
  __shared__ mf32::Smem<B, B> sm;
  __shared__ float red[kWaves];
  const int64_t sample = blockIdx.x / npairs;
  int ti, tj;
  decode_pair(static_cast<int>(blockIdx.x % npairs), nt, ti, tj);
  mf32::Tile<B, B> tg, ta;
  tg.clear();
  ta.clear();
  {
    const float* bs = b + sample * T * Dout;
    mf32::LoaderKContig<B, float, VEC> la(bs, Dout, static_cast<int64_t>(ti) * B, T, Dout);
    mf32::LoaderKContig<B, float, VEC> lb(bs, Dout, static_cast<int64_t>(tj) * B, T, Dout);
    mf32::mainloop<B, B>(tg, sm, la, lb, Dout);
  }
  if (pw) {
    const float* as = a + sample * T * Din;
    mf32::LoaderKContig<B, float, VEC> la(as, Din, static_cast<int64_t>(ti) * B, T, Din);
    mf32::LoaderKContig<B, float, VEC> lb(as, Din, static_cast<int64_t>(tj) * B, T, Din);
    mf32::mainloop<B, B>(ta, sm, la, lb, Din);
  }
  contract_and_store(tg, ta, pw != nullptr, ti == tj ? 1.f : 2.f, pw, pb, red);
}

template <int B, bool VEC>
__global__ __launch_bounds__(kThreads) void ghost_norm_bf16_kernel(
    const bf16_t* __restrict__ b, const bf16_t* __restrict__ a, float* __restrict__ pw,
    float* __restrict__ pb, int64_t T, int64_t Dout, int64_t Din, int nt, int npairs) {
  __shared__ mb16::Smem<B, B> sm;
  __shared__ float red[kWaves];
  const int64_t sample = blockIdx.x / npairs;
  int ti, tj;
  decode_pair(static_cast<int>(blockIdx.x % npairs), nt, ti, tj);
  mb16::Tile<B, B> tg, ta;
  tg.clear();
  ta.clear();
  {
    const bf16_t* bs = b + sample * T * Dout;
    mb16::Loader<B, VEC> la(bs, Dout, static_cast<int64_t>(ti) * B, T, Dout);
    mb16::Loader<B, VEC> lb(bs, Dout, static_cast<int64_t>(tj) * B, T, Dout);
    mb16::mainloop<B, B>(tg, sm, la, lb, Dout);
  }
  if (pw) {
    const bf16_t* as = a + sample * T * Din;
    mb16::Loader<B, VEC> la(as, Din, static_cast<int64_t>(ti) * B, T, Din);
    mb16::Loader<B, VEC> lb(as, Din, static_cast<int64_t>(tj) * B, T, Din);
    mb16::mainloop<B, B>(ta, sm, la, lb, Din);
  }
  contract_and_store(tg, ta, pw != nullptr, ti == tj ? 1.f : 2.f, pw, pb, red);
}

// Fast path: operand tiles go global -> LDS directly through a ring of stages
// (mfma_bf16_dlds.h). Needs Dout % 64 == Din % 64 == 0 and 16-byte aligned rows.
// The block tile is BM x BN with BM = R * BN: row blocks I, column blocks J, and
// the block-triangle J >= R * I is visited. Column blocks inside the row block's
// own diagonal square (J < R * (I + 1)) count once - together they cover that
// square completely - the ones beyond it twice.
//
// Work units are (sample, tile pair), numbered sample-major. The first nbig units
// get a block each; when the launch would otherwise end in a thinly filled round
// of resident blocks, each remaining unit is cut into kGhostPieces pieces that get a
// block each. A unit cannot be cut along both contractions (it is the sum of the
// products of two Gram tiles), but it is linear in either Gram alone: piece p forms the
// longer-contraction Gram over the p-th part of its k range only, the other Gram in
// full, and the pieces' partial sums add up to the unit's. A piece keeps the 128 x 128
// tile (the operand bytes per MFMA of a whole unit) and does (K_long / pieces +
// K_short) / (K_long + K_short) of its work. (Cutting the tile into quadrants of 64 x 64
// whose waves split k measured worse: a quadrant block alone on a CU took 26 us where
// the whole unit takes 37.) Unit u writes its partial sums at u * slots (+ piece).
constexpr int kGhostPieces = 4;

// One work unit: tile pair `pair` of one sample of one layer, whole (big) or as piece
// `piece` of it. The partial sums of unit `unit_index` (sample * npairs + pair) go
// to pw / pb at unit_index * slots (+ piece).
// TE: bf16_t, or float (a stage row of 128 bytes is then 32 k values).
template <class C, typename TE>
__device__ __forceinline__ void ghost_unit(mb16d::Smem<C>& sm, float* red, const TE* __restrict__ bs,
                                           const TE* __restrict__ as, float* __restrict__ pw,
                                           float* __restrict__ pb, int64_t T, int64_t Dout, int64_t Din, int nJ,
                                           int pair, bool big, uint32_t piece, size_t unit_index, int slots) {
  constexpr int R = C::BM / C::BN;
  constexpr int BKE = C::ROW_BYTES / static_cast<int>(sizeof(TE));  // k values of a stage row
  int I = 0;
  while (pair >= nJ - R * I) {
    pair -= nJ - R * I;
    ++I;
  }
  const int J = R * I + pair;
  const float weight = J < R * (I + 1) ? 1.f : 2.f;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int kh = lane >> 5, l32 = lane & 31;
  float sw = 0.f, sb = 0.f;
  const size_t slot = unit_index * slots + (big ? 0u : piece);
  // the k ranges of the two Grams: whole, or the piece's part of the longer one
  int64_t kb0 = 0, kb1 = Dout, ka0 = 0, ka1 = Din;
  bool count_bias = true;
  if (!big) {
    const bool split_b = !pw || Dout >= Din;
    const int64_t nk = (split_b ? Dout : Din) / BKE;
    const int64_t t0 = nk * piece / kGhostPieces * BKE, t1 = nk * (piece + 1) / kGhostPieces * BKE;
    if (split_b) {
      kb0 = t0;
      kb1 = t1;
    } else {
      ka0 = t0;
      ka1 = t1;
      count_bias = piece == 0;  // the whole b Gram is formed by every piece: its sum counts once
    }
  }
  const int64_t m0a = static_cast<int64_t>(I) * C::BM, m0b = static_cast<int64_t>(J) * C::BN;
  const int wm0 = (wave / C::kWaveCols) * 64, wn0 = (wave % C::kWaveCols) * 64;
  mb16d::Tile tg, ta;
  tg.clear();
  ta.clear();
  if (kb1 > kb0) mb16d::mainloop<C, TE>(tg, sm, bs + kb0, bs + kb0, Dout, m0a, m0b, T, kb1 - kb0, wm0, wn0);
  if (pw && ka1 > ka0) mb16d::mainloop<C, TE>(ta, sm, as + ka0, as + ka0, Din, m0a, m0b, T, ka1 - ka0, wm0, wn0);
  // rows past T hold copies of row T - 1: leave them out
  const int rmax = static_cast<int>(T - m0a < C::BM ? T - m0a : C::BM);
  const int cmax = static_cast<int>(T - m0b < C::BN ? T - m0b : C::BN);
#pragma unroll
  for (int i = 0; i < 2; ++i)
#pragma unroll
    for (int j = 0; j < 2; ++j)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int row = wm0 + i * 32 + (v >> 2) * 8 + kh * 4 + (v & 3), col = wn0 + j * 32 + l32;
        if (row < rmax && col < cmax) {
          const float g = tg.acc[i][j][v];
          sb += g;
          sw = fmaf(g, ta.acc[i][j][v], sw);
        }
      }
  if (pw) {
    const float s = block_sum<C::kWaves>(sw, red);
    if (threadIdx.x == 0) pw[slot] = s * weight;
    // a whole unit leaves the other pieces' slots empty
    if (big && slots > 1 && threadIdx.x < slots && threadIdx.x > 0) pw[slot + threadIdx.x] = 0.f;
  }
  if (pb) {
    const float s = block_sum<C::kWaves>(sb, red);
    if (threadIdx.x == 0) pb[slot] = count_bias ? s * weight : 0.f;
    if (big && slots > 1 && threadIdx.x < slots && threadIdx.x > 0) pb[slot + threadIdx.x] = 0.f;
  }
}

template <class C, typename TE = bf16_t>
__global__ __launch_bounds__(C::kThreads) void ghost_norm_bf16_dlds_kernel(
    const TE* __restrict__ b, const TE* __restrict__ a, float* __restrict__ pw,
    float* __restrict__ pb, int64_t T, int64_t Dout, int64_t Din, int nJ, int npairs, uint32_t nbig,
    int slots) {
  __shared__ mb16d::Smem<C> sm;
  __shared__ float red[C::kWaves];
  const bool big = blockIdx.x < nbig;
  uint32_t unit, quad = 0;
  if (big) {
    unit = xcd_contiguous_id(blockIdx.x, nbig);
  } else {
    // nbig is a multiple of 8, so the low bits still name the XCD
    const uint32_t sid = xcd_contiguous_id(blockIdx.x - nbig, gridDim.x - nbig);
    unit = nbig + sid / kGhostPieces;
    quad = sid % kGhostPieces;
  }
  const int64_t sample = unit / static_cast<uint32_t>(npairs);
  const int pair = static_cast<int>(unit % static_cast<uint32_t>(npairs));
  ghost_unit<C, TE>(sm, red, b + sample * T * Dout, a + sample * T * Din, pw, pb, T, Dout, Din, nJ, pair, big, quad,
                    unit, slots);
}

// ---- several layers in one launch ------------------------------------------------------
// The ghost norms of one layer at a benchmark shape are a launch of a few hundred units on
// 512 resident blocks: its last round of blocks is mostly empty, and every layer pays that
// again. Pooled, the units of all layers of a backward pass fill the rounds, and the one
// tail is cut into pieces (see above). Layers are given in descending order of feature count,
// so that every XCD starts with its longest units.
//
// Hardware block id i runs on XCD i % 8, and an XCD takes its blocks in id order. XCD x is
// given the samples [s0[x], s0[x] + cnt[x]) of every layer (units that share a sample's
// rows share that XCD's L2), layer after layer: `len[x]` units, of which the last `tail[x]`
// are run as kGhostPieces blocks each.
constexpr int kGhostMultiMax = 32;               // layers per launch
constexpr int kGhostMultiLayers = DPK_GHOST_MULTI_MAX;  // layers per call (several launches)

struct GhostMultiArgs {
  const void* b[kGhostMultiMax];
  const void* a[kGhostMultiMax];  // NULL: no weight norm for this layer
  float* pw[kGhostMultiMax];
  float* pb[kGhostMultiMax];
  int32_t T[kGhostMultiMax], Dout[kGhostMultiMax], Din[kGhostMultiMax], nJ[kGhostMultiMax], npairs[kGhostMultiMax];
  uint32_t pair_prefix[kGhostMultiMax + 1];  // tile pairs per sample of the layers before this one
  int32_t nlayers, slots;
  uint32_t s0[8], cnt[8], len[8], tail[8];
};

template <class C, typename TE>
__global__ __launch_bounds__(C::kThreads) void ghost_norm_multi_kernel(const GhostMultiArgs A) {
  __shared__ mb16d::Smem<C> sm;
  __shared__ float red[C::kWaves];
  const uint32_t x = blockIdx.x & 7u, idx = blockIdx.x >> 3;
  const uint32_t tail = A.tail[x], nbig = A.len[x] - tail;
  if (idx >= nbig + kGhostPieces * tail) return;
  const bool big = idx < nbig;
  const uint32_t u = big ? idx : nbig + (idx - nbig) / kGhostPieces;
  const uint32_t quad = big ? 0u : (idx - nbig) % kGhostPieces;
  const uint32_t cnt = A.cnt[x];
  int l = 0;
  while (l + 1 < A.nlayers && u >= cnt * A.pair_prefix[l + 1]) ++l;
  const uint32_t local = u - cnt * A.pair_prefix[l];
  const uint32_t npairs = static_cast<uint32_t>(A.npairs[l]);
  const int64_t sample = static_cast<int64_t>(A.s0[x]) + local / npairs;
  const int pair = static_cast<int>(local % npairs);
  const int64_t T = A.T[l], Dout = A.Dout[l], Din = A.Din[l];
  const TE* a = static_cast<const TE*>(A.a[l]);
  ghost_unit<C, TE>(sm, red, static_cast<const TE*>(A.b[l]) + sample * T * Dout, a ? a + sample * T * Din : nullptr,
                    a ? A.pw[l] : nullptr, A.pb[l], T, Dout, Din, A.nJ[l], pair, big, quad,
                    static_cast<size_t>(sample) * npairs + pair, A.slots);
}

// out = sqrt(max(0, sum of a row of partials)) * factor, for every layer's weight and bias
// rows: one wave per (layer, which, sample), fixed order.
struct GhostReduceArgs {
  const float* part[2 * kGhostMultiMax];  // layer l: pw at 2 l, pb at 2 l + 1 (NULL: skip)
  float* out[2 * kGhostMultiMax];
  int32_t cols[kGhostMultiMax];
  float factor[kGhostMultiMax];
  int32_t nlayers, n;
};

__global__ __launch_bounds__(kThreads) void ghost_reduce_multi_kernel(const GhostReduceArgs A) {
  const int64_t w = (static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x) / DPK_WAVE;
  const int lane = threadIdx.x & (DPK_WAVE - 1);
  if (w >= static_cast<int64_t>(A.nlayers) * 2 * A.n) return;
  const int which = static_cast<int>(w / A.n), row = static_cast<int>(w % A.n), l = which >> 1;
  const float* p = A.part[which];
  if (!p) return;
  const int cols = A.cols[l];
  p += static_cast<int64_t>(row) * cols;
  float s = 0.f;
  for (int i = lane; i < cols; i += DPK_WAVE) s += p[i];
  s = wave_sum(s);
  if (lane == 0) A.out[which][row] = sqrtf(fmaxf(s, 0.f)) * A.factor[l];
}

// 128 x 128 tile, 4 waves, two 32 KB stages: two blocks fit a CU, which measured
// better than one block with a deeper ring or a 256 x 128 tile (8 waves, 3 stages).
#ifndef DPK_GHOST_CFG
#define DPK_GHOST_CFG 2, 2, 2, 64
#endif
using GhostCfg = mb16d::Config<DPK_GHOST_CFG>;

// Tile pairs per sample for a BM x BN tiling of the T x T block-triangle.
int64_t ghost_pairs(int64_t T, int bm, int bn) {
  const int64_t nI = dpk_cdiv(T, bm), nJ = dpk_cdiv(T, bn), R = bm / bn;
  int64_t p = 0;
  for (int64_t I = 0; I < nI; ++I) p += nJ - R * I;
  return p;
}

// T == 1: closed forms of linear.py:71-79. One block per sample.
template <typename T_>
__global__ __launch_bounds__(kThreads) void ghost_norm_rank1_kernel(
    const T_* __restrict__ b, const T_* __restrict__ a, float* __restrict__ nw,
    float* __restrict__ nb, int64_t Dout, int64_t Din, float absscale) {
  __shared__ float red[kWaves];
  const int64_t sample = blockIdx.x;
  float sb = 0.f, sa = 0.f;
  for (int64_t i = threadIdx.x; i < Dout; i += kThreads) {
    const float v = dpk_io<T_>::load(b + sample * Dout + i);
    sb = fmaf(v, v, sb);
  }
  if (nw)
    for (int64_t i = threadIdx.x; i < Din; i += kThreads) {
      const float v = dpk_io<T_>::load(a + sample * Din + i);
      sa = fmaf(v, v, sa);
    }
  const float tb = block_sum<kWaves>(sb, red);
  const float ta = block_sum<kWaves>(sa, red);
  if (threadIdx.x == 0) {
    if (nw) nw[sample] = sqrtf(tb * ta) * absscale;
    if (nb) nb[sample] = sqrtf(tb) * absscale;
  }
}

int tile_edge(int64_t T) { return T > 64 ? 128 : 64; }

}  // namespace

// The Gram route costs 2 T'^2 (in + out) multiply-adds per sample over the tile pairs it
// visits, forming the gradient and squaring it 2 T in out: for thin layers (a low-rank
// adapter, a narrow head) the second is far cheaper although the gradient tile exists for a
// moment in registers.
// The caller's `route` argument overrides the choice (tests drive both routes on one shape).
bool direct_is_cheaper(int route, int64_t T, int64_t out, int64_t in) {
  if (route == DPK_ROUTE_GRAM) return false;
  if (route == DPK_ROUTE_DIRECT) return true;
  const int B = T > 64 ? 128 : 64;
  const int64_t nt = dpk_cdiv(T, B);
  const double gram = static_cast<double>(nt * (nt + 1) / 2) * B * B * static_cast<double>(in + out);
  const double direct = static_cast<double>(T) * static_cast<double>(in) * static_cast<double>(out);
  // the two routes run at about the same rate for either element type
  return direct < 0.9 * gram;
}

// Whether the direct-to-LDS tile kernel takes the layer: 128-row tiles, feature sizes that
// fill whole 128-byte stage rows (64 bf16 or 32 fp32 values), 16-byte aligned operands, a
// sample small enough for 32-bit byte offsets inside it.
bool dlds_takes(const void* b, const void* a, int dtype, bool want_w, int64_t T, int64_t out, int64_t in) {
  const int64_t widest = out > in ? out : in;
  const int64_t es = dpk_elsize(dtype), kmul = 128 / es;
  return T > 64 && out % kmul == 0 && (in % kmul == 0 || !want_w) && dpk_aligned(b, 16) && dpk_aligned(a, 16) &&
         T * widest * es < (int64_t{1} << 32);
}

struct DirectLayout {
  size_t bias, total;  // [0, bias): the Linear kernel's partial sums; then float[n, out]
};

DirectLayout direct_layout(int64_t n, int64_t T, int64_t out, int64_t in) {
  DirectLayout l;
  l.bias = dpk_align_up(dpk_linear_gs_workspace_bytes(n, T, out, in), 256);
  l.total = l.bias + dpk_align_up(static_cast<size_t>(n) * out * sizeof(float), 256);
  return l;
}

extern "C" size_t dpk_linear_ghost_norm_workspace_bytes(int64_t n, int64_t T, int64_t out,
                                                        int64_t in) {
  if (n <= 0 || T <= 1) return 0;
  // Room for any tiling: 64-row tile pairs, or 128-row tile pairs with four
  // piece slots each (2 m^2 + 2 m slots per sample covers both).
  const int64_t m = dpk_cdiv(T, 128);
  const size_t gram = dpk_align_up(static_cast<size_t>(2 * n * (2 * m * m + 2 * m)) * sizeof(float), 256);
  // ... and for the direct route, whichever of the two a call ends up taking
  const size_t direct = direct_layout(n, T, out, in).total;
  return gram > direct ? gram : direct;
}

extern "C" int dpk_linear_ghost_norm(const void* b, const void* a, int dtype, float* norm_w,
                                     float* norm_b, int64_t n, int64_t T, int64_t out, int64_t in,
                                     float scale, int route, void* ws, size_t ws_bytes,
                                     dpk_stream_t stream) {
  const char* who = "dpk_linear_ghost_norm";
  DPK_REQUIRE(route == DPK_ROUTE_AUTO || route == DPK_ROUTE_GRAM || route == DPK_ROUTE_DIRECT, DPK_E_ARG,
              "%s: route %d", who, route);
  DPK_REQUIRE(n >= 0 && T >= 1 && out >= 1 && in >= 1, DPK_E_SHAPE,
              "%s: n=%lld T=%lld out=%lld in=%lld", who, (long long)n, (long long)T, (long long)out,
              (long long)in);
  if (n == 0 || (!norm_w && !norm_b)) return DPK_OK;
  DPK_REQUIRE(b && (a || !norm_w), DPK_E_ARG, "%s: NULL tensor", who);
  DPK_REQUIRE(dpk_dtype_ok(dtype), DPK_E_DTYPE, "%s: dtype %d", who, dtype);
  DPK_REQUIRE(dpk_aligned(b, dpk_elsize(dtype)) && dpk_aligned(a, dpk_elsize(dtype)), DPK_E_ALIGN,
              "%s: misaligned tensor", who);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const float absscale = fabsf(scale);
  if (T == 1) {
    DPK_REQUIRE(n <= DPK_MAX_GRID_X, DPK_E_SHAPE, "%s: n too large", who);
    if (dtype == DPK_F32)
      hipLaunchKernelGGL(ghost_norm_rank1_kernel<float>, dim3((unsigned)n), dim3(kThreads), 0, s,
                         static_cast<const float*>(b), static_cast<const float*>(a), norm_w, norm_b,
                         out, in, absscale);
    else
      hipLaunchKernelGGL(ghost_norm_rank1_kernel<bf16_t>, dim3((unsigned)n), dim3(kThreads), 0, s,
                         static_cast<const bf16_t*>(b), static_cast<const bf16_t*>(a), norm_w, norm_b,
                         out, in, absscale);
    DPK_LAUNCH_CHECK(who);
    return DPK_OK;
  }
  if (norm_w && direct_is_cheaper(route, T, out, in)) {
    // |sum_t b_t a_t^T|_F from the per-sample gradient tiles themselves, never stored;
    // the bias norm from the column sums of b
    const DirectLayout l = direct_layout(n, T, out, in);
    DPK_REQUIRE(ws && ws_bytes >= l.total, DPK_E_WORKSPACE, "%s: workspace %zu < %zu bytes", who, ws_bytes, l.total);
    DPK_REQUIRE(dpk_aligned(ws, 256), DPK_E_ALIGN, "%s: workspace must be 256-byte aligned", who);
    char* base = static_cast<char*>(ws);
    int rc = dpk_linear_gs(b, a, dtype, nullptr, dtype, norm_w, n, T, out, in, 1.0f, DPK_TILE_AUTO, base, l.bias,
                           stream);
    if (rc != DPK_OK) return rc;
    dpk_launch_reduce_rows(norm_w, n, 1, norm_w, 1, absscale, s);  // in place: sqrt, times |scale|
    DPK_LAUNCH_CHECK(who);
    if (norm_b) {
      rc = dpk_linear_bias_gs(b, dtype, base + l.bias, DPK_F32, norm_b, n, T, out, 1.0f, stream);
      if (rc != DPK_OK) return rc;
      dpk_launch_reduce_rows(norm_b, n, 1, norm_b, 1, absscale, s);
      DPK_LAUNCH_CHECK(who);
    }
    return DPK_OK;
  }
  const int B = tile_edge(T);
  const int64_t nt = dpk_cdiv(T, B);
  // bf16 with 64-aligned feature sizes takes the direct-to-LDS kernel
  // (and a sample small enough for 32-bit byte offsets inside it)
  // (fp32 too: 32 k values fill the 128-byte stage row that 64 bf16 do)
  const bool dlds = dlds_takes(b, a, dtype, norm_w != nullptr, T, out, in);
  const int64_t npairs = dlds ? ghost_pairs(T, GhostCfg::BM, GhostCfg::BN) : nt * (nt + 1) / 2;
  const int64_t blocks = n * npairs;
  // The units of a last round of resident blocks (two per CU) that is at most a quarter
  // full are cut into pieces, which then fit one round of their own: left whole, they
  // would take a full round's time on a quarter of the CUs.
  int64_t tail = 0;
  if (dlds) {
    const int cus = dpk_device_cus();
    DPK_REQUIRE(cus > 0, DPK_E_LAUNCH, "%s: cannot query the device", who);
    const int64_t resident = 2 * static_cast<int64_t>(cus);
    const int64_t r = blocks % resident;
    if (resident % 8 == 0 && r > 0 && r * kGhostPieces <= resident) tail = r;
  }
  const int slots = tail ? kGhostPieces : 1;
  const int64_t grid_blocks = blocks - tail + kGhostPieces * tail;
  DPK_REQUIRE(nt < 32768 && grid_blocks <= DPK_MAX_GRID_X && blocks * slots <= DPK_MAX_GRID_X, DPK_E_SHAPE,
              "%s: %lld blocks exceed the grid limit", who, (long long)grid_blocks);
  const size_t need = static_cast<size_t>(2 * blocks * slots) * sizeof(float);
  DPK_REQUIRE(ws && ws_bytes >= need, DPK_E_WORKSPACE, "%s: workspace %zu < %zu bytes", who, ws_bytes,
              need);
  DPK_REQUIRE(dpk_aligned(ws, 4), DPK_E_ALIGN, "%s: workspace misaligned", who);
  float* pw = norm_w ? static_cast<float*>(ws) : nullptr;
  float* pb = norm_b ? static_cast<float*>(ws) + blocks * slots : nullptr;
  const dim3 grid(static_cast<unsigned>(blocks)), block(kThreads);
  if (dtype == DPK_F32 && dlds) {
    hipLaunchKernelGGL((ghost_norm_bf16_dlds_kernel<GhostCfg, float>), dim3(static_cast<unsigned>(grid_blocks)),
                       dim3(GhostCfg::kThreads), 0, s, static_cast<const float*>(b), static_cast<const float*>(a),
                       pw, pb, T, out, in, (int)dpk_cdiv(T, GhostCfg::BN), (int)npairs,
                       static_cast<uint32_t>(blocks - tail), slots);
  } else if (dtype == DPK_F32) {
    const bool vec = out % 4 == 0 && in % 4 == 0 && dpk_aligned(b, 16) && dpk_aligned(a, 16);
    const float* bp = static_cast<const float*>(b);
    const float* ap = static_cast<const float*>(a);
#define DPK_GN_LAUNCH(B_, V_)                                                                 \
  hipLaunchKernelGGL((ghost_norm_f32_kernel<B_, V_>), grid, block, 0, s, bp, ap, pw, pb, T, out, \
                     in, (int)nt, (int)npairs)
    if (B == 128) {
      if (vec) DPK_GN_LAUNCH(128, true);
      else DPK_GN_LAUNCH(128, false);
    } else {
      if (vec) DPK_GN_LAUNCH(64, true);
      else DPK_GN_LAUNCH(64, false);
    }
#undef DPK_GN_LAUNCH
  } else {
    const bool vec = out % 8 == 0 && in % 8 == 0 && dpk_aligned(b, 16) && dpk_aligned(a, 16);
    const bf16_t* bp = static_cast<const bf16_t*>(b);
    const bf16_t* ap = static_cast<const bf16_t*>(a);
    if (dlds) {
      hipLaunchKernelGGL((ghost_norm_bf16_dlds_kernel<GhostCfg>), dim3(static_cast<unsigned>(grid_blocks)),
                         dim3(GhostCfg::kThreads), 0, s, bp, ap, pw, pb, T, out, in,
                         (int)dpk_cdiv(T, GhostCfg::BN), (int)npairs, static_cast<uint32_t>(blocks - tail),
                         slots);
      DPK_LAUNCH_CHECK(who);
    } else {
#define DPK_GN_LAUNCH(B_, V_)                                                                  \
  hipLaunchKernelGGL((ghost_norm_bf16_kernel<B_, V_>), grid, block, 0, s, bp, ap, pw, pb, T, out, \
                     in, (int)nt, (int)npairs)
    if (B == 128) {
      if (vec) DPK_GN_LAUNCH(128, true);
      else DPK_GN_LAUNCH(128, false);
    } else {
      if (vec) DPK_GN_LAUNCH(64, true);
      else DPK_GN_LAUNCH(64, false);
    }
#undef DPK_GN_LAUNCH
    }
  }
  DPK_LAUNCH_CHECK(who);
  if (pw) {
    dpk_launch_reduce_rows(pw, n, npairs * slots, norm_w, 1, absscale, s);
    DPK_LAUNCH_CHECK(who);
  }
  if (pb) {
    dpk_launch_reduce_rows(pb, n, npairs * slots, norm_b, 1, absscale, s);
    DPK_LAUNCH_CHECK(who);
  }
  return DPK_OK;
}

// ---- all Linear layers of a backward pass in one call ----------------------------------
namespace {
size_t multi_single_region(const dpk_ghost_layer* layers, int count, int64_t n) {
  size_t m = 0;
  for (int k = 0; k < count; ++k) {
    const size_t need = dpk_linear_ghost_norm_workspace_bytes(n, layers[k].T, layers[k].out, layers[k].in);
    m = need > m ? need : m;
  }
  return dpk_align_up(m, 256);
}
size_t multi_partials_bytes(int64_t n, int64_t T) {  // pw and pb of one pooled layer, four slots a unit
  return dpk_align_up(static_cast<size_t>(2 * n * ghost_pairs(T, GhostCfg::BM, GhostCfg::BN) * 4) * sizeof(float), 256);
}
}  // namespace

extern "C" size_t dpk_linear_ghost_norm_multi_workspace_bytes(const dpk_ghost_layer* layers, int count, int64_t n) {
  if (!layers || count <= 0 || n <= 0) return 0;
  size_t total = multi_single_region(layers, count, n);
  for (int k = 0; k < count; ++k)
    if (layers[k].T > 1) total += multi_partials_bytes(n, layers[k].T);
  return total;
}

extern "C" int dpk_linear_ghost_norm_multi(const dpk_ghost_layer* layers, int count, int dtype, int64_t n,
                                           void* ws, size_t ws_bytes, dpk_stream_t stream) {
  const char* who = "dpk_linear_ghost_norm_multi";
  DPK_REQUIRE(count >= 0 && count <= kGhostMultiLayers && n >= 0, DPK_E_SHAPE, "%s: count=%d (at most %d) n=%lld", who,
              count, kGhostMultiLayers, (long long)n);
  if (count == 0 || n == 0) return DPK_OK;
  DPK_REQUIRE(layers, DPK_E_ARG, "%s: NULL layer table", who);
  DPK_REQUIRE(dpk_dtype_ok(dtype), DPK_E_DTYPE, "%s: dtype %d", who, dtype);
  const size_t need = dpk_linear_ghost_norm_multi_workspace_bytes(layers, count, n);
  DPK_REQUIRE(need == 0 || (ws && ws_bytes >= need), DPK_E_WORKSPACE, "%s: workspace %zu < %zu bytes", who, ws_bytes,
              need);
  DPK_REQUIRE(dpk_aligned(ws, 256), DPK_E_ALIGN, "%s: workspace must be 256-byte aligned", who);
  char* base = static_cast<char*>(ws);
  const size_t single_region = multi_single_region(layers, count, n);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const int cus = dpk_device_cus();
  DPK_REQUIRE(cus > 0, DPK_E_LAUNCH, "%s: cannot query the device", who);

  // Layers the tile kernel takes by the Gram route are pooled; every other layer (T == 1, thin
  // layers on the direct route, feature sizes the tile kernel does not take) goes through the
  // single-layer entry point, one after the other on the same stream and scratch.
  int pooled[kGhostMultiLayers];
  int npooled = 0;
  for (int k = 0; k < count; ++k) {
    const dpk_ghost_layer& L = layers[k];
    DPK_REQUIRE(L.T >= 1 && L.out >= 1 && L.in >= 1, DPK_E_SHAPE, "%s: layer %d: T=%lld out=%lld in=%lld", who, k,
                (long long)L.T, (long long)L.out, (long long)L.in);
    if (!L.norm_w && !L.norm_b) continue;
    DPK_REQUIRE(L.b && (L.a || !L.norm_w), DPK_E_ARG, "%s: layer %d: NULL tensor", who, k);
    const bool pool = L.T > 1 && !(L.norm_w && direct_is_cheaper(DPK_ROUTE_AUTO, L.T, L.out, L.in)) &&
                      dlds_takes(L.b, L.a, dtype, L.norm_w != nullptr, L.T, L.out, L.in) &&
                      dpk_cdiv(L.T, 128) < 32768;
    if (pool) {
      pooled[npooled++] = k;
    } else {
      const int rc = dpk_linear_ghost_norm(L.b, L.a, dtype, L.norm_w, L.norm_b, n, L.T, L.out, L.in, L.scale,
                                           DPK_ROUTE_AUTO, base, single_region, stream);
      if (rc != DPK_OK) return rc;
    }
  }
  if (npooled == 1) {  // nothing to pool with: the single-layer launch has the same kernel and its own tail
    const dpk_ghost_layer& L = layers[pooled[0]];
    return dpk_linear_ghost_norm(L.b, L.a, dtype, L.norm_w, L.norm_b, n, L.T, L.out, L.in, L.scale, DPK_ROUTE_GRAM,
                                 base, single_region, stream);
  }
  // longest units first (insertion sort: a few dozen layers)
  for (int i = 1; i < npooled; ++i) {
    const int k = pooled[i];
    const int64_t cost = layers[k].out + (layers[k].norm_w ? layers[k].in : 0);
    int j = i;
    for (; j > 0; --j) {
      const dpk_ghost_layer& P = layers[pooled[j - 1]];
      if (P.out + (P.norm_w ? P.in : 0) >= cost) break;
      pooled[j] = pooled[j - 1];
    }
    pooled[j] = k;
  }
  // every layer with T > 1 has its partial-sum region at a fixed place in table order (the
  // workspace query sums over exactly these), whichever of them end up pooled
  size_t lay_off[kGhostMultiLayers];
  {
    size_t o = single_region;
    for (int k = 0; k < count; ++k) {
      lay_off[k] = o;
      if (layers[k].T > 1) o += multi_partials_bytes(n, layers[k].T);
    }
  }
  const uint32_t resident = static_cast<uint32_t>(2 * cus / 8);  // blocks an XCD holds at once
  for (int c0 = 0; c0 < npooled; c0 += kGhostMultiMax) {
    const int nl = npooled - c0 < kGhostMultiMax ? npooled - c0 : kGhostMultiMax;
    GhostMultiArgs A;
    GhostReduceArgs R;
    memset(&A, 0, sizeof(A));
    memset(&R, 0, sizeof(R));
    A.nlayers = nl;
    R.nlayers = nl;
    R.n = static_cast<int32_t>(n);
    uint32_t P = 0;
    for (int i = 0; i < nl; ++i) {
      const dpk_ghost_layer& L = layers[pooled[c0 + i]];
      A.b[i] = L.b;
      A.a[i] = L.norm_w ? L.a : nullptr;
      A.T[i] = static_cast<int32_t>(L.T);
      A.Dout[i] = static_cast<int32_t>(L.out);
      A.Din[i] = static_cast<int32_t>(L.in);
      A.nJ[i] = static_cast<int32_t>(dpk_cdiv(L.T, GhostCfg::BN));
      A.npairs[i] = static_cast<int32_t>(ghost_pairs(L.T, GhostCfg::BM, GhostCfg::BN));
      A.pair_prefix[i] = P;
      P += static_cast<uint32_t>(A.npairs[i]);
    }
    A.pair_prefix[nl] = P;
    DPK_REQUIRE(static_cast<uint64_t>(n) * P < (1ull << 28), DPK_E_SHAPE, "%s: too many tile pairs", who);
    uint32_t longest = 0;
    bool any_tail = false;
    for (uint32_t x = 0; x < 8; ++x) {
      A.s0[x] = static_cast<uint32_t>(x * n / 8);
      A.cnt[x] = static_cast<uint32_t>((x + 1) * n / 8) - A.s0[x];
      A.len[x] = A.cnt[x] * P;
      const uint32_t r = resident > 0 ? A.len[x] % resident : 0;
      A.tail[x] = (cus % 8 == 0 && r > 0 && r * kGhostPieces <= resident) ? r : 0;
      any_tail = any_tail || A.tail[x] > 0;
      const uint32_t blocks = A.len[x] - A.tail[x] + kGhostPieces * A.tail[x];
      longest = blocks > longest ? blocks : longest;
    }
    A.slots = any_tail ? kGhostPieces : 1;
    for (int i = 0; i < nl; ++i) {
      const dpk_ghost_layer& L = layers[pooled[c0 + i]];
      float* part = reinterpret_cast<float*>(base + lay_off[pooled[c0 + i]]);
      const int64_t per = n * A.npairs[i] * A.slots;
      A.pw[i] = L.norm_w ? part : nullptr;
      A.pb[i] = L.norm_b ? part + per : nullptr;
      R.part[2 * i] = A.pw[i];
      R.part[2 * i + 1] = A.pb[i];
      R.out[2 * i] = L.norm_w;
      R.out[2 * i + 1] = L.norm_b;
      R.cols[i] = A.npairs[i] * A.slots;
      R.factor[i] = fabsf(L.scale);
    }
    const dim3 grid(8u * longest), block(GhostCfg::kThreads);
    if (dtype == DPK_F32) hipLaunchKernelGGL((ghost_norm_multi_kernel<GhostCfg, float>), grid, block, 0, s, A);
    else hipLaunchKernelGGL((ghost_norm_multi_kernel<GhostCfg, bf16_t>), grid, block, 0, s, A);
    DPK_LAUNCH_CHECK(who);
    const int64_t waves = static_cast<int64_t>(nl) * 2 * n;
    hipLaunchKernelGGL(ghost_reduce_multi_kernel, dim3(static_cast<unsigned>(dpk_cdiv(waves, kWaves))), dim3(kThreads), 0,
                       s, R);
    DPK_LAUNCH_CHECK(who);
  }
  return DPK_OK;
}

// ---- the same entry point for callers that cannot allocate ---------------------------
// Partial sums (and, on the direct route, the column sums of b) live in a file-scope
// device array instead of a caller-provided workspace. Every GPU holds its own copy of the
// array at its own address; the name below is only the host-side handle by which
// hipGetSymbolAddress finds the copy of the current device. Host code passes that address,
// never the name, to the kernels. Each block writes every slot the final reduction reads,
// so nothing has to start at zero and what an earlier call left behind is never read.
static __device__ __align__(256) unsigned char scratch[DPK_STATIC_SCRATCH_BYTES];

namespace {
constexpr int kMaxDevices = 64;
std::mutex g_scratch_mutex;
void* g_scratch_ptr[kMaxDevices] = {};

// Address of the current device's copy of `scratch`, resolved once per device.
int scratch_of_current_device(const char* who, void** out) {
  int dev = -1;
  hipError_t e = hipGetDevice(&dev);
  DPK_REQUIRE(e == hipSuccess, DPK_E_LAUNCH, "%s: hipGetDevice: %s", who, hipGetErrorString(e));
  DPK_REQUIRE(dev >= 0 && dev < kMaxDevices, DPK_E_LAUNCH, "%s: device index %d out of range", who, dev);
  std::lock_guard<std::mutex> lock(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* ptr = nullptr;
    e = hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch));
    DPK_REQUIRE(e == hipSuccess && ptr, DPK_E_LAUNCH, "%s: hipGetSymbolAddress: %s", who, hipGetErrorString(e));
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return DPK_OK;
}
}  // namespace

extern "C" int dpk_linear_ghost_norm_static(const void* b, const void* a, int dtype, float* norm_w,
                                            float* norm_b, int64_t n, int64_t T, int64_t out, int64_t in,
                                            float scale, int route, dpk_stream_t stream) {
  const char* who = "dpk_linear_ghost_norm_static";
  DPK_REQUIRE(n >= 0 && T >= 1 && out >= 1 && in >= 1, DPK_E_SHAPE, "%s: n=%lld T=%lld out=%lld in=%lld", who,
              (long long)n, (long long)T, (long long)out, (long long)in);
  if (n == 0 || (!norm_w && !norm_b)) return DPK_OK;
  const size_t need = dpk_linear_ghost_norm_workspace_bytes(n, T, out, in);
  DPK_REQUIRE(need <= DPK_STATIC_SCRATCH_BYTES, DPK_E_SHAPE,
              "%s: n=%lld T=%lld out=%lld in=%lld needs %zu bytes of scratch, the built-in buffer holds %zu; "
              "use dpk_linear_ghost_norm with a workspace",
              who, (long long)n, (long long)T, (long long)out, (long long)in, need,
              static_cast<size_t>(DPK_STATIC_SCRATCH_BYTES));
  void* ptr = nullptr;
  if (need > 0) {
    const int rc = scratch_of_current_device(who, &ptr);
    if (rc != DPK_OK) return rc;
  }
  return dpk_linear_ghost_norm(b, a, dtype, norm_w, norm_b, n, T, out, in, scale, route, ptr,
                               need > 0 ? static_cast<size_t>(DPK_STATIC_SCRATCH_BYTES) : 0, stream);
}
