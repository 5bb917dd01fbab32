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
// of resident blocks, the remaining units are cut into quadrants of 64 x 64 and
// every quadrant gets a block of its own that splits k over its waves. Unit u
// writes its partial sums at u * slots (a quadrant at u * slots + quadrant).
template <class C>
constexpr bool ghost_cfg_has_quadrants() {
  return C::BM == 128 && C::BN == 128 && C::BK == 64 && C::kWaves == 4 && C::kStages == 2;
}

// TE: bf16_t, or float (a stage row of 128 bytes is then 32 k values).
template <class C, typename TE = bf16_t>
__global__ __launch_bounds__(C::kThreads) void ghost_norm_bf16_dlds_kernel(
    const TE* __restrict__ b, const TE* __restrict__ a, float* __restrict__ pw,
    float* __restrict__ pb, int64_t T, int64_t Dout, int64_t Din, int nJ, int npairs, uint32_t nbig,
    int slots) {
  constexpr int R = C::BM / C::BN;
  constexpr bool kQuadrants = ghost_cfg_has_quadrants<C>();
  __shared__ mb16d::Smem<C> sm;
  __shared__ float red[C::kWaves];
  const bool big = !kQuadrants || blockIdx.x < nbig;
  uint32_t unit, quad = 0;
  if (big) {
    unit = xcd_contiguous_id(blockIdx.x, nbig);
  } else {
    // nbig is a multiple of 8, so the low bits still name the XCD
    const uint32_t sid = xcd_contiguous_id(blockIdx.x - nbig, gridDim.x - nbig);
    unit = nbig + (sid >> 2);
    quad = sid & 3u;
  }
  const int64_t sample = unit / static_cast<uint32_t>(npairs);
  int pair = static_cast<int>(unit % static_cast<uint32_t>(npairs));
  int I = 0;
  while (pair >= nJ - R * I) {
    pair -= nJ - R * I;
    ++I;
  }
  const int J = R * I + pair;
  const float weight = J < R * (I + 1) ? 1.f : 2.f;
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int kh = lane >> 5, l32 = lane & 31;
  const TE* bs = b + sample * T * Dout;
  const TE* as = a + sample * T * Din;
  float sw = 0.f, sb = 0.f;
  size_t slot;
  if (big) {
    const int64_t m0a = static_cast<int64_t>(I) * C::BM, m0b = static_cast<int64_t>(J) * C::BN;
    const int wm0 = (wave / C::kWaveCols) * 64, wn0 = (wave % C::kWaveCols) * 64;
    mb16d::Tile tg, ta;
    tg.clear();
    ta.clear();
    mb16d::mainloop<C, TE>(tg, sm, bs, bs, Dout, m0a, m0b, T, Dout, wm0, wn0);
    if (pw) mb16d::mainloop<C, TE>(ta, sm, as, as, Din, m0a, m0b, T, Din, wm0, wn0);
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
    slot = static_cast<size_t>(unit) * slots;
  } else if constexpr (kQuadrants) {
    // quadrant (quad >> 1, quad & 1) of the unit's tile; R == 1 on this path
    const int64_t m0a = static_cast<int64_t>(I) * C::BM + (quad >> 1) * 64;
    const int64_t m0b = static_cast<int64_t>(J) * C::BN + (quad & 1u) * 64;
    slot = static_cast<size_t>(unit) * slots + quad;
    if (m0a < T && m0b < T) {  // block-uniform
      mb16d::Tile t;
      t.clear();
      mb16d::mainloop_splitk<C, TE>(t, sm, bs, bs, Dout, m0a, m0b, T, Dout);
      const mb16d::floatx16 g = mb16d::splitk_reduce<C>(t, sm);
      mb16d::floatx16 h;
      if (pw) {
        t.clear();
        mb16d::mainloop_splitk<C, TE>(t, sm, as, as, Din, m0a, m0b, T, Din);
        h = mb16d::splitk_reduce<C>(t, sm);
      }
      const int rmax = static_cast<int>(T - m0a < 64 ? T - m0a : 64);
      const int cmax = static_cast<int>(T - m0b < 64 ? T - m0b : 64);
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int row = (wave >> 1) * 32 + (v >> 2) * 8 + kh * 4 + (v & 3), col = (wave & 1) * 32 + l32;
        if (row < rmax && col < cmax) {
          sb += g[v];
          if (pw) sw = fmaf(g[v], h[v], sw);
        }
      }
    }
  }
  if (pw) {
    const float s = block_sum<C::kWaves>(sw, red);
    if (threadIdx.x == 0) pw[slot] = s * weight;
    // a whole unit leaves the other quadrant slots empty
    if (big && slots > 1 && threadIdx.x < slots && threadIdx.x > 0) pw[slot + threadIdx.x] = 0.f;
  }
  if (pb) {
    const float s = block_sum<C::kWaves>(sb, red);
    if (threadIdx.x == 0) pb[slot] = s * weight;
    if (big && slots > 1 && threadIdx.x < slots && threadIdx.x > 0) pb[slot + threadIdx.x] = 0.f;
  }
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
  // quadrant slots each (2 m^2 + 2 m slots per sample covers both).
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
  const int64_t widest = out > in ? out : in;
  // (fp32 too: 32 k values fill the 128-byte stage row that 64 bf16 do)
  const int64_t es = dpk_elsize(dtype), kmul = 128 / es;
  const bool dlds = B == 128 && out % kmul == 0 && (in % kmul == 0 || !norm_w) &&
                    dpk_aligned(b, 16) && dpk_aligned(a, 16) && T * widest * es < (int64_t{1} << 32);
  const int64_t npairs = dlds ? ghost_pairs(T, GhostCfg::BM, GhostCfg::BN) : nt * (nt + 1) / 2;
  const int64_t blocks = n * npairs;
  // A last round of resident blocks (two per CU) that is at most a quarter full is
  // served by quadrant blocks instead, which then fit one round of their own: a lone
  // tile block per CU runs latency-bound and takes most of a full round's time, a
  // round of quadrant blocks about a third of it.
  int64_t tail = 0;
  if (dlds && ghost_cfg_has_quadrants<GhostCfg>()) {
    const int cus = dpk_device_cus();
    DPK_REQUIRE(cus > 0, DPK_E_LAUNCH, "%s: cannot query the device", who);
    const int64_t resident = 2 * static_cast<int64_t>(cus);
    const int64_t r = blocks % resident;
    if (resident % 8 == 0 && r > 0 && r * 4 <= resident) tail = r;
  }
  const int slots = tail ? 4 : 1;
  const int64_t grid_blocks = blocks - tail + 4 * tail;
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
