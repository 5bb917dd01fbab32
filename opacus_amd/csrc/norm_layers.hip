// Per-sample gradients of the affine parameters of normalisation layers:
//   GroupNorm  opacus/grad_sample/group_norm.py:26-47
//   RMSNorm    opacus/grad_sample/rms_norm.py:27-47
// Both re-normalise the layer input without the affine part, multiply by the
// backprops and sum over everything but (sample, channel/feature). The reference
// materialises normalize(x) and the product; here the statistics are computed
// and applied in registers, x is read from HBM once (re-reads hit the cache) and
// b once. HBM-bound.
#include "dpk_common.h"

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / DPK_WAVE;

// ---- GroupNorm ----------------------------------------------------------------
// One block per (sample, group). The group's Cg*S elements are contiguous.
// Mean, then centred second moment (two passes: the same arithmetic as a direct
// evaluation of the definition, no cancellation), then per channel the two sums,
// one wave per channel.
template <typename TIN, typename TOUT>
__global__ __launch_bounds__(kThreads) void group_norm_gs_kernel(
    const TIN* __restrict__ x, const TIN* __restrict__ b, TOUT* __restrict__ gw,
    TOUT* __restrict__ gb, int64_t C, int64_t S, int64_t G, float eps, float scale) {
  __shared__ float red[kWaves];
  __shared__ float stat[2];
  const int64_t sample = blockIdx.x / G, grp = blockIdx.x % G;
  const int64_t Cg = C / G, len = Cg * S;
  const int64_t base = (sample * C + grp * Cg) * S;
  const TIN* xg = x + base;
  const TIN* bg = b + base;
  float s = 0.f;
  for (int64_t i = threadIdx.x; i < len; i += kThreads) s += dpk_io<TIN>::load(xg + i);
  s = block_sum<kWaves>(s, red);
  if (threadIdx.x == 0) stat[0] = s / static_cast<float>(len);
  __syncthreads();
  const float mean = stat[0];
  float v = 0.f;
  for (int64_t i = threadIdx.x; i < len; i += kThreads) {
    const float d = dpk_io<TIN>::load(xg + i) - mean;
    v = fmaf(d, d, v);
  }
  v = block_sum<kWaves>(v, red);
  if (threadIdx.x == 0) stat[1] = 1.0f / sqrtf(v / static_cast<float>(len) + eps);
  __syncthreads();
  const float rstd = stat[1];
  const int lane = threadIdx.x & (DPK_WAVE - 1), wave = threadIdx.x / DPK_WAVE;
  for (int64_t c = wave; c < Cg; c += kWaves) {
    const TIN* xc = xg + c * S;
    const TIN* bc = bg + c * S;
    float sw = 0.f, sb = 0.f;
    for (int64_t i = lane; i < S; i += DPK_WAVE) {
      const float bv = dpk_io<TIN>::load(bc + i);
      sw = fmaf((dpk_io<TIN>::load(xc + i) - mean) * rstd, bv, sw);
      sb += bv;
    }
    sw = wave_sum(sw);
    sb = wave_sum(sb);
    if (lane == 0) {
      const int64_t o = sample * C + grp * Cg + c;
      if (gw) dpk_io<TOUT>::store(gw + o, sw * scale);
      if (gb) dpk_io<TOUT>::store(gb + o, sb * scale);
    }
  }
}

// ---- RMSNorm ------------------------------------------------------------------
// rstd[row] = rsqrt(mean_d x[row,:]^2 + eps), one wave per row.
template <typename TIN>
__global__ __launch_bounds__(kThreads) void rms_rstd_kernel(const TIN* __restrict__ x, int64_t rows,
                                                             int64_t D, float eps,
                                                             float* __restrict__ rstd) {
  const int64_t w = (static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x) / DPK_WAVE;
  const int lane = threadIdx.x & (DPK_WAVE - 1);
  if (w >= rows) return;
  const TIN* p = x + w * D;
  float s = 0.f;
  for (int64_t i = lane; i < D; i += DPK_WAVE) {
    const float v = dpk_io<TIN>::load(p + i);
    s = fmaf(v, v, s);
  }
  s = wave_sum(s);
  if (lane == 0) rstd[w] = 1.0f / sqrtf(s / static_cast<float>(D) + eps);
}

// part[ts][sample][d] = sum over the t range of split ts of x * rstd * b.
// grid = n * dch * TS; thread <-> 4 (VEC) or 1 feature.
template <typename TIN, bool VEC>
__global__ __launch_bounds__(kThreads) void rms_partial_kernel(
    const TIN* __restrict__ x, const TIN* __restrict__ b, const float* __restrict__ rstd, int64_t n,
    int64_t T, int64_t D, int dch, int TS, float* __restrict__ part) {
  constexpr int W = VEC ? 4 : 1;
  int64_t bid = blockIdx.x;
  const int ts = static_cast<int>(bid % TS);
  bid /= TS;
  const int dc = static_cast<int>(bid % dch);
  const int64_t sample = bid / dch;
  const int64_t d = (static_cast<int64_t>(dc) * kThreads + threadIdx.x) * W;
  if (d >= D) return;
  const int64_t per = (T + TS - 1) / TS;
  const int64_t t0 = ts * per, t1 = (t0 + per < T) ? t0 + per : T;
  const TIN* xs = x + sample * T * D + d;
  const TIN* bs = b + sample * T * D + d;
  const float* rs = rstd + sample * T;
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f);
  for (int64_t t = t0; t < t1; ++t) {
    const float r = rs[t];
    if (VEC) {
      const float4 xv = dpk_io<TIN>::load4(xs + t * D), bv = dpk_io<TIN>::load4(bs + t * D);
      acc.x = fmaf(xv.x * r, bv.x, acc.x);
      acc.y = fmaf(xv.y * r, bv.y, acc.y);
      acc.z = fmaf(xv.z * r, bv.z, acc.z);
      acc.w = fmaf(xv.w * r, bv.w, acc.w);
    } else {
      acc.x = fmaf(dpk_io<TIN>::load(xs + t * D) * r, dpk_io<TIN>::load(bs + t * D), acc.x);
    }
  }
  float* o = part + (static_cast<int64_t>(ts) * n + sample) * D + d;
  if (VEC) *reinterpret_cast<float4*>(o) = acc;
  else *o = acc.x;
}

template <typename TOUT>
__global__ __launch_bounds__(kThreads) void rms_final_kernel(const float* __restrict__ part,
                                                              int64_t nD, int TS, float scale,
                                                              TOUT* __restrict__ gw) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i >= nD) return;
  float s = 0.f;
  for (int ts = 0; ts < TS; ++ts) s += part[static_cast<int64_t>(ts) * nD + i];
  dpk_io<TOUT>::store(gw + i, s * scale);
}

int rms_splits(int64_t T) {
  int64_t ts = dpk_cdiv(T, 64);
  return static_cast<int>(ts < 1 ? 1 : (ts > 16 ? 16 : ts));
}

}  // namespace

extern "C" int dpk_group_norm_gs(const void* x, const void* b, int in_dtype, void* gs_w, void* gs_b,
                                 int gs_dtype, int64_t n, int64_t C, int64_t S, int64_t groups,
                                 float eps, float scale, dpk_stream_t stream) {
  const char* who = "dpk_group_norm_gs";
  DPK_REQUIRE(n >= 0 && C >= 1 && S >= 1 && groups >= 1, DPK_E_SHAPE,
              "%s: n=%lld C=%lld S=%lld groups=%lld", who, (long long)n, (long long)C, (long long)S,
              (long long)groups);
  DPK_REQUIRE(C % groups == 0, DPK_E_SHAPE, "%s: groups=%lld does not divide C=%lld", who,
              (long long)groups, (long long)C);
  if (n == 0 || (!gs_w && !gs_b)) return DPK_OK;
  DPK_REQUIRE(x && b, DPK_E_ARG, "%s: NULL tensor", who);
  DPK_REQUIRE(dpk_dtype_ok(in_dtype) && dpk_dtype_ok(gs_dtype), DPK_E_DTYPE, "%s: dtypes %d,%d", who,
              in_dtype, gs_dtype);
  DPK_REQUIRE(dpk_aligned(x, dpk_elsize(in_dtype)) && dpk_aligned(b, dpk_elsize(in_dtype)) &&
                  dpk_aligned(gs_w, dpk_elsize(gs_dtype)) && dpk_aligned(gs_b, dpk_elsize(gs_dtype)),
              DPK_E_ALIGN, "%s: misaligned tensor", who);
  DPK_REQUIRE(n * groups <= DPK_MAX_GRID_X, DPK_E_SHAPE, "%s: too many blocks", who);
  const dim3 grid(static_cast<unsigned>(n * groups)), block(kThreads);
  hipStream_t s = static_cast<hipStream_t>(stream);
#define DPK_GN(TI, TO)                                                                           \
  hipLaunchKernelGGL((group_norm_gs_kernel<TI, TO>), grid, block, 0, s, static_cast<const TI*>(x), \
                     static_cast<const TI*>(b), static_cast<TO*>(gs_w), static_cast<TO*>(gs_b), C, S, \
                     groups, eps, scale)
  if (in_dtype == DPK_F32 && gs_dtype == DPK_F32) DPK_GN(float, float);
  else if (in_dtype == DPK_BF16 && gs_dtype == DPK_BF16) DPK_GN(bf16_t, bf16_t);
  else if (in_dtype == DPK_BF16 && gs_dtype == DPK_F32) DPK_GN(bf16_t, float);
  else DPK_GN(float, bf16_t);
#undef DPK_GN
  DPK_LAUNCH_CHECK(who);
  return DPK_OK;
}

extern "C" size_t dpk_rms_norm_gs_workspace_bytes(int64_t n, int64_t T, int64_t D) {
  if (n <= 0 || T <= 0 || D <= 0) return 0;
  return dpk_align_up(static_cast<size_t>(n * T) * 4, 256) +
         dpk_align_up(static_cast<size_t>(rms_splits(T)) * n * D * 4, 256);
}

extern "C" int dpk_rms_norm_gs(const void* x, const void* b, int in_dtype, void* gs_w, int gs_dtype,
                               int64_t n, int64_t T, int64_t D, float eps, float scale, void* ws,
                               size_t ws_bytes, dpk_stream_t stream) {
  const char* who = "dpk_rms_norm_gs";
  DPK_REQUIRE(n >= 0 && T >= 1 && D >= 1, DPK_E_SHAPE, "%s: n=%lld T=%lld D=%lld", who, (long long)n,
              (long long)T, (long long)D);
  if (n == 0) return DPK_OK;
  DPK_REQUIRE(x && b && gs_w, DPK_E_ARG, "%s: NULL tensor", who);
  DPK_REQUIRE(dpk_dtype_ok(in_dtype) && dpk_dtype_ok(gs_dtype), DPK_E_DTYPE, "%s: dtypes %d,%d", who,
              in_dtype, gs_dtype);
  DPK_REQUIRE(dpk_aligned(x, dpk_elsize(in_dtype)) && dpk_aligned(b, dpk_elsize(in_dtype)) &&
                  dpk_aligned(gs_w, dpk_elsize(gs_dtype)),
              DPK_E_ALIGN, "%s: misaligned tensor", who);
  const size_t need = dpk_rms_norm_gs_workspace_bytes(n, T, D);
  DPK_REQUIRE(ws && ws_bytes >= need, DPK_E_WORKSPACE, "%s: workspace %zu < %zu bytes", who, ws_bytes,
              need);
  DPK_REQUIRE(dpk_aligned(ws, 256), DPK_E_ALIGN, "%s: workspace must be 256-byte aligned", who);
  float* rstd = static_cast<float*>(ws);
  float* part = reinterpret_cast<float*>(static_cast<char*>(ws) +
                                         dpk_align_up(static_cast<size_t>(n * T) * 4, 256));
  const int TS = rms_splits(T);
  const size_t va = in_dtype == DPK_BF16 ? 8 : 16;
  const bool vec = D % 4 == 0 && dpk_aligned(x, va) && dpk_aligned(b, va);
  const int dch = static_cast<int>(dpk_cdiv(D, kThreads * (vec ? 4 : 1)));
  DPK_REQUIRE(n * dch * TS <= DPK_MAX_GRID_X && dpk_cdiv(n * T, kWaves) <= DPK_MAX_GRID_X, DPK_E_SHAPE,
              "%s: too many blocks", who);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 block(kThreads);
  const dim3 g1(static_cast<unsigned>(dpk_cdiv(n * T, kWaves))), g2(static_cast<unsigned>(n * dch * TS));
  if (in_dtype == DPK_F32) {
    const float* xp = static_cast<const float*>(x);
    const float* bp = static_cast<const float*>(b);
    hipLaunchKernelGGL(rms_rstd_kernel<float>, g1, block, 0, s, xp, n * T, D, eps, rstd);
    if (vec) hipLaunchKernelGGL((rms_partial_kernel<float, true>), g2, block, 0, s, xp, bp, rstd, n, T, D, dch, TS, part);
    else hipLaunchKernelGGL((rms_partial_kernel<float, false>), g2, block, 0, s, xp, bp, rstd, n, T, D, dch, TS, part);
  } else {
    const bf16_t* xp = static_cast<const bf16_t*>(x);
    const bf16_t* bp = static_cast<const bf16_t*>(b);
    hipLaunchKernelGGL(rms_rstd_kernel<bf16_t>, g1, block, 0, s, xp, n * T, D, eps, rstd);
    if (vec) hipLaunchKernelGGL((rms_partial_kernel<bf16_t, true>), g2, block, 0, s, xp, bp, rstd, n, T, D, dch, TS, part);
    else hipLaunchKernelGGL((rms_partial_kernel<bf16_t, false>), g2, block, 0, s, xp, bp, rstd, n, T, D, dch, TS, part);
  }
  DPK_LAUNCH_CHECK(who);
  const dim3 g3(static_cast<unsigned>(dpk_cdiv(n * D, kThreads)));
  if (gs_dtype == DPK_F32)
    hipLaunchKernelGGL(rms_final_kernel<float>, g3, block, 0, s, part, n * D, TS, scale, static_cast<float*>(gs_w));
  else
    hipLaunchKernelGGL(rms_final_kernel<bf16_t>, g3, block, 0, s, part, n * D, TS, scale, static_cast<bf16_t*>(gs_w));
  DPK_LAUNCH_CHECK(who);
  return DPK_OK;
}
