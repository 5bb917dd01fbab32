// Per-sample gradients of the affine parameters of normalisation layers:
//   GroupNorm  opacus/grad_sample/group_norm.py:26-47
//   RMSNorm    opacus/grad_sample/rms_norm.py:27-47
//   LayerNorm  opacus/grad_sample/layer_norm.py:27-52
// Both re-normalise the layer input without the affine part, multiply by the
// backprops and sum over everything but (sample, channel/feature). The reference
// materialises normalize(x) and the product; here the statistics are computed
// and applied in registers, x is read from HBM once (re-reads hit the cache) and
// b once. HBM-bound.
#include <algorithm>

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

// Groups of at most 1024 * K elements whose channels are whole multiples of four
// elements: every thread keeps its K four-element chunks of x in registers, so x and
// b are read from memory exactly once. Per-chunk products go to LDS and one wave per
// channel adds them up in a fixed order.
template <typename TIN, typename TOUT, int K>
__global__ __launch_bounds__(kThreads) void group_norm_gs_reg_kernel(
    const TIN* __restrict__ x, const TIN* __restrict__ b, TOUT* __restrict__ gw,
    TOUT* __restrict__ gb, int64_t C, int64_t S, int64_t G, float eps, float scale) {
  __shared__ float red[kWaves];
  __shared__ float stat[2];
  __shared__ float cw[kThreads * K], cb[kThreads * K];
  const int64_t sample = blockIdx.x / G, grp = blockIdx.x % G;
  const int Cg = static_cast<int>(C / G);
  const int len4 = static_cast<int>(Cg * S / 4), S4 = static_cast<int>(S / 4);
  const int64_t base = (sample * C + grp * Cg) * S;
  const TIN* xg = x + base;
  const TIN* bg = b + base;
  float4 xv[K];
  float s = 0.f;
#pragma unroll
  for (int k = 0; k < K; ++k) {
    const int j = k * kThreads + threadIdx.x;
    xv[k] = j < len4 ? dpk_io<TIN>::load4(xg + j * 4) : make_float4(0.f, 0.f, 0.f, 0.f);
    s += (xv[k].x + xv[k].y) + (xv[k].z + xv[k].w);
  }
  s = block_sum<kWaves>(s, red);
  if (threadIdx.x == 0) stat[0] = s / static_cast<float>(len4 * 4);
  __syncthreads();
  const float mean = stat[0];
  float v = 0.f;
#pragma unroll
  for (int k = 0; k < K; ++k) {
    const int j = k * kThreads + threadIdx.x;
    if (j < len4) {
      xv[k].x -= mean;
      xv[k].y -= mean;
      xv[k].z -= mean;
      xv[k].w -= mean;
      v = fmaf(xv[k].x, xv[k].x, v);
      v = fmaf(xv[k].y, xv[k].y, v);
      v = fmaf(xv[k].z, xv[k].z, v);
      v = fmaf(xv[k].w, xv[k].w, v);
    }
  }
  v = block_sum<kWaves>(v, red);
  if (threadIdx.x == 0) stat[1] = 1.0f / sqrtf(v / static_cast<float>(len4 * 4) + eps);
  __syncthreads();
  const float rstd = stat[1];
#pragma unroll
  for (int k = 0; k < K; ++k) {
    const int j = k * kThreads + threadIdx.x;
    if (j < len4) {
      const float4 bv = dpk_io<TIN>::load4(bg + j * 4);
      float pw = xv[k].x * rstd * bv.x;
      pw = fmaf(xv[k].y * rstd, bv.y, pw);
      pw = fmaf(xv[k].z * rstd, bv.z, pw);
      pw = fmaf(xv[k].w * rstd, bv.w, pw);
      cw[j] = pw;
      cb[j] = (bv.x + bv.y) + (bv.z + bv.w);
    }
  }
  __syncthreads();
  const int lane = threadIdx.x & (DPK_WAVE - 1), wave = threadIdx.x / DPK_WAVE;
  for (int c = wave; c < Cg; c += kWaves) {
    float sw = 0.f, sb = 0.f;
    for (int i = lane; i < S4; i += DPK_WAVE) {
      sw += cw[c * S4 + i];
      sb += cb[c * S4 + i];
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

// ---- RMSNorm and LayerNorm --------------------------------------------------------
// Both normalise every row of D features on its own and reduce norm(x) * b over the
// rows t of a sample. LN = false: x * rsqrt(mean x^2 + eps). LN = true: centred, with
// the variance taken around the mean, and the bias gradient sum_t b on the side.

// rstd[row] (and mean[row] for LN), one wave per row.
template <typename TIN, bool LN>
__global__ __launch_bounds__(kThreads) void row_stat_kernel(const TIN* __restrict__ x, int64_t rows,
                                                             int64_t D, float eps,
                                                             float* __restrict__ rstd,
                                                             float* __restrict__ mean) {
  const int64_t w = (static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x) / DPK_WAVE;
  const int lane = threadIdx.x & (DPK_WAVE - 1);
  if (w >= rows) return;
  const TIN* p = x + w * D;
  float m = 0.f;
  if (LN) {
    for (int64_t i = lane; i < D; i += DPK_WAVE) m += dpk_io<TIN>::load(p + i);
    m = wave_sum(m) / static_cast<float>(D);
  }
  float s = 0.f;
  for (int64_t i = lane; i < D; i += DPK_WAVE) {
    const float v = dpk_io<TIN>::load(p + i) - m;
    s = fmaf(v, v, s);
  }
  s = wave_sum(s);
  if (lane == 0) {
    rstd[w] = 1.0f / sqrtf(s / static_cast<float>(D) + eps);
    if (LN) mean[w] = m;
  }
}

// part[ts][sample][d] = sum over the t range of split ts of (x - mean) * rstd * b, and
// partb[ts][sample][d] = sum of b for LN. grid = n * dch * TS; thread <-> 4 (VEC) or 1 feature.
template <typename TIN, bool VEC, bool LN>
__global__ __launch_bounds__(kThreads) void row_partial_kernel(
    const TIN* __restrict__ x, const TIN* __restrict__ b, const float* __restrict__ rstd,
    const float* __restrict__ mean, int64_t n, int64_t T, int64_t D, int dch, int TS,
    float* __restrict__ part, float* __restrict__ partb) {
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
  const float* ms = mean + sample * T;
  float4 acc = make_float4(0.f, 0.f, 0.f, 0.f), accb = make_float4(0.f, 0.f, 0.f, 0.f);
  for (int64_t t = t0; t < t1; ++t) {
    const float r = rs[t], m = LN ? ms[t] : 0.f;
    if (VEC) {
      const float4 xv = dpk_io<TIN>::load4(xs + t * D), bv = dpk_io<TIN>::load4(bs + t * D);
      acc.x = fmaf((xv.x - m) * r, bv.x, acc.x);
      acc.y = fmaf((xv.y - m) * r, bv.y, acc.y);
      acc.z = fmaf((xv.z - m) * r, bv.z, acc.z);
      acc.w = fmaf((xv.w - m) * r, bv.w, acc.w);
      if (LN) {
        accb.x += bv.x;
        accb.y += bv.y;
        accb.z += bv.z;
        accb.w += bv.w;
      }
    } else {
      const float bv = dpk_io<TIN>::load(bs + t * D);
      acc.x = fmaf((dpk_io<TIN>::load(xs + t * D) - m) * r, bv, acc.x);
      if (LN) accb.x += bv;
    }
  }
  const int64_t o = (static_cast<int64_t>(ts) * n + sample) * D + d;
  if (VEC) *reinterpret_cast<float4*>(part + o) = acc;
  else part[o] = acc.x;
  if (LN && partb) {
    if (VEC) *reinterpret_cast<float4*>(partb + o) = accb;
    else partb[o] = accb.x;
  }
}

template <typename TOUT>
__global__ __launch_bounds__(kThreads) void row_final_kernel(const float* __restrict__ part,
                                                              int64_t nD, int TS, float scale,
                                                              TOUT* __restrict__ gw) {
  const int64_t i = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  if (i >= nD) return;
  // four independent chains keep several loads in flight; the order is fixed
  float s0 = 0.f, s1 = 0.f, s2 = 0.f, s3 = 0.f;
  int ts = 0;
  for (; ts + 4 <= TS; ts += 4) {
    s0 += part[static_cast<int64_t>(ts) * nD + i];
    s1 += part[static_cast<int64_t>(ts + 1) * nD + i];
    s2 += part[static_cast<int64_t>(ts + 2) * nD + i];
    s3 += part[static_cast<int64_t>(ts + 3) * nD + i];
  }
  for (; ts < TS; ++ts) s0 += part[static_cast<int64_t>(ts) * nD + i];
  dpk_io<TOUT>::store(gw + i, ((s0 + s1) + (s2 + s3)) * scale);
}

// Per-sample sum of squares of the [n, D] result (as stored), a block per sample: the optimizer's
// norm pass then has nothing to read. The result is a few KB per sample and still in cache; a
// final sum with a block per sample that squared on the way was tried and is slower (16 blocks
// read 8 MB of partial sums).
template <typename TOUT>
__global__ __launch_bounds__(kThreads) void row_sumsq_kernel(const TOUT* __restrict__ gw, int64_t D,
                                                              float* __restrict__ sumsq) {
  __shared__ float red[kWaves];
  const TOUT* row = gw + static_cast<int64_t>(blockIdx.x) * D;
  float ss = 0.f;
  for (int64_t d = threadIdx.x; d < D; d += kThreads) {
    const float v = dpk_io<TOUT>::load(row + d);
    ss = fmaf(v, v, ss);
  }
  const float total = block_sum<kWaves>(ss, red);
  if (threadIdx.x == 0) sumsq[blockIdx.x] = total;
}

// Cross-wave sum of per-lane float4 chunks through LDS, written to o[0..D).
template <int NCH>
__device__ __forceinline__ void rows_meet(const float4 (&acc)[NCH], float (&red)[kWaves][256 * NCH],
                                          float* __restrict__ o) {
  constexpr int D = 256 * NCH;
  const int lane = threadIdx.x & (DPK_WAVE - 1), wave = threadIdx.x / DPK_WAVE;
#pragma unroll
  for (int c = 0; c < NCH; ++c) *reinterpret_cast<float4*>(&red[wave][c * 256 + lane * 4]) = acc[c];
  __syncthreads();
  for (int d = threadIdx.x * 4; d < D; d += kThreads * 4) {
    float4 s = *reinterpret_cast<const float4*>(&red[0][d]);
#pragma unroll
    for (int w = 1; w < kWaves; ++w) {
      const float4 v = *reinterpret_cast<const float4*>(&red[w][d]);
      s.x += v.x;
      s.y += v.y;
      s.z += v.z;
      s.w += v.w;
    }
    *reinterpret_cast<float4*>(o + d) = s;
  }
  __syncthreads();
}

// One pass: a wave keeps a whole row of x in registers (D = 256 * NCH elements, four
// per lane and chunk), reduces its statistics across the wave, then streams the
// matching row of b and accumulates norm(x) * b per feature. Rows t of a block's
// stretch are dealt to its waves round-robin; the waves' partial sums meet in LDS.
// part / partb as above. x and b cross HBM exactly once.
template <typename TIN, int NCH, bool LN>
__global__ __launch_bounds__(kThreads) void row_fused_kernel(const TIN* __restrict__ x,
                                                              const TIN* __restrict__ b, int64_t n,
                                                              int64_t T, float eps, int TS,
                                                              float* __restrict__ part,
                                                              float* __restrict__ partb) {
  constexpr int D = 256 * NCH;
  constexpr int NB = LN ? NCH : 1;
  __shared__ float red[kWaves][D];
  const int ts = static_cast<int>(blockIdx.x % TS);
  const int64_t sample = blockIdx.x / TS;
  const int lane = threadIdx.x & (DPK_WAVE - 1), wave = threadIdx.x / DPK_WAVE;
  const int64_t per = (T + TS - 1) / TS;
  const int64_t t0 = ts * per, t1 = (t0 + per < T) ? t0 + per : T;
  float4 acc[NCH], accb[NB];
#pragma unroll
  for (int c = 0; c < NCH; ++c) acc[c] = make_float4(0.f, 0.f, 0.f, 0.f);
#pragma unroll
  for (int c = 0; c < NB; ++c) accb[c] = make_float4(0.f, 0.f, 0.f, 0.f);
  for (int64_t t = t0 + wave; t < t1; t += kWaves) {
    const TIN* xr = x + (sample * T + t) * D + lane * 4;
    const TIN* br = b + (sample * T + t) * D + lane * 4;
    // both rows are asked for before either is used: the row of b does not wait for the
    // statistics of x
    typename dpk_io<TIN>::raw4 xraw[NCH], braw[NCH];
#pragma unroll
    for (int c = 0; c < NCH; ++c) xraw[c] = dpk_io<TIN>::load4_raw(xr + c * 256);
#pragma unroll
    for (int c = 0; c < NCH; ++c) braw[c] = dpk_io<TIN>::load4_raw(br + c * 256);
    float4 xv[NCH];
    float sum = 0.f;
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
      xv[c] = dpk_io<TIN>::unpack4(xraw[c]);
      if (LN) sum += (xv[c].x + xv[c].y) + (xv[c].z + xv[c].w);
    }
    if (LN) {
      const float m = wave_sum(sum) / static_cast<float>(D);
#pragma unroll
      for (int c = 0; c < NCH; ++c) {
        xv[c].x -= m;
        xv[c].y -= m;
        xv[c].z -= m;
        xv[c].w -= m;
      }
    }
    float ss = 0.f;
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
      ss = fmaf(xv[c].x, xv[c].x, ss);
      ss = fmaf(xv[c].y, xv[c].y, ss);
      ss = fmaf(xv[c].z, xv[c].z, ss);
      ss = fmaf(xv[c].w, xv[c].w, ss);
    }
    ss = wave_sum(ss);
    const float r = 1.0f / sqrtf(ss / static_cast<float>(D) + eps);
#pragma unroll
    for (int c = 0; c < NCH; ++c) {
      const float4 bv = dpk_io<TIN>::unpack4(braw[c]);
      acc[c].x = fmaf(xv[c].x * r, bv.x, acc[c].x);
      acc[c].y = fmaf(xv[c].y * r, bv.y, acc[c].y);
      acc[c].z = fmaf(xv[c].z * r, bv.z, acc[c].z);
      acc[c].w = fmaf(xv[c].w * r, bv.w, acc[c].w);
      if (LN) {
        accb[c].x += bv.x;
        accb[c].y += bv.y;
        accb[c].z += bv.z;
        accb[c].w += bv.w;
      }
    }
  }
  const int64_t obase = (static_cast<int64_t>(ts) * n + sample) * D;
  rows_meet<NCH>(acc, red, part + obase);
  if constexpr (LN) {
    if (partb) rows_meet<NCH>(accb, red, partb + obase);  // uniform
  }
}

// Feature sizes the one-pass kernel is instantiated for (D = 256 * NCH).
bool row_fused_ok(int64_t D) {
  if (D % 256 != 0) return false;
  const int64_t c = D / 256;
  return c == 1 || c == 2 || c == 3 || c == 4 || c == 6 || c == 8 || c == 12 || c == 16;
}

// Stretches of t per sample for the one-pass kernel: enough blocks to fill the
// device, at least one row per wave.
int row_fused_splits(int64_t n, int64_t T) {
  int64_t ts = dpk_cdiv(1024, n);
  const int64_t most = dpk_cdiv(T, kWaves);
  if (ts > most) ts = most;
  if (ts > 256) ts = 256;
  return static_cast<int>(ts < 1 ? 1 : ts);
}

template <typename TIN, bool LN>
void launch_row_fused(const TIN* x, const TIN* b, int64_t n, int64_t T, int64_t D, float eps, int TS,
                      float* part, float* partb, hipStream_t s) {
  const dim3 grid(static_cast<unsigned>(n * TS)), block(kThreads);
#define DPK_RF(N_)                                                                                 \
  case N_:                                                                                         \
    hipLaunchKernelGGL((row_fused_kernel<TIN, N_, LN>), grid, block, 0, s, x, b, n, T, eps, TS, part, \
                       partb);                                                                     \
    break
  switch (D / 256) {
    DPK_RF(1);
    DPK_RF(2);
    DPK_RF(3);
    DPK_RF(4);
    DPK_RF(6);
    DPK_RF(8);
    DPK_RF(12);
    default:
      hipLaunchKernelGGL((row_fused_kernel<TIN, 16, LN>), grid, block, 0, s, x, b, n, T, eps, TS, part,
                         partb);
      break;
  }
#undef DPK_RF
}

int row_splits(int64_t T) {
  int64_t ts = dpk_cdiv(T, 64);
  return static_cast<int>(ts < 1 ? 1 : (ts > 16 ? 16 : ts));
}

// Workspace: rstd[n*T], mean[n*T], then splits * n * D partial sums, twice (weight, bias).
struct RowWs {
  size_t stat_bytes, part_bytes;
  size_t total() const { return 2 * stat_bytes + 2 * part_bytes; }
  float* rstd(void* ws) const { return reinterpret_cast<float*>(static_cast<char*>(ws)); }
  float* mean(void* ws) const { return reinterpret_cast<float*>(static_cast<char*>(ws) + stat_bytes); }
  float* part(void* ws) const { return reinterpret_cast<float*>(static_cast<char*>(ws) + 2 * stat_bytes); }
  float* partb(void* ws) const {
    return reinterpret_cast<float*>(static_cast<char*>(ws) + 2 * stat_bytes + part_bytes);
  }
};

RowWs row_ws(int64_t n, int64_t T, int64_t D) {
  const int64_t splits = std::max<int64_t>(row_splits(T), row_fused_ok(D) ? row_fused_splits(n, T) : 0);
  RowWs w;
  w.stat_bytes = dpk_align_up(static_cast<size_t>(n * T) * 4, 256);
  w.part_bytes = dpk_align_up(static_cast<size_t>(splits) * n * D * 4, 256);
  return w;
}

template <typename TIN, bool LN>
void launch_rows(const TIN* x, const TIN* b, int64_t n, int64_t T, int64_t D, float eps, bool vec,
                 bool fused, int TS, float* rstd, float* mean, float* part, float* partb, hipStream_t s) {
  if (fused) {
    launch_row_fused<TIN, LN>(x, b, n, T, D, eps, TS, part, partb, s);
    return;
  }
  const int dch = static_cast<int>(dpk_cdiv(D, kThreads * (vec ? 4 : 1)));
  const dim3 block(kThreads);
  const dim3 g1(static_cast<unsigned>(dpk_cdiv(n * T, kWaves))), g2(static_cast<unsigned>(n * dch * TS));
  hipLaunchKernelGGL((row_stat_kernel<TIN, LN>), g1, block, 0, s, x, n * T, D, eps, rstd, mean);
  if (vec)
    hipLaunchKernelGGL((row_partial_kernel<TIN, true, LN>), g2, block, 0, s, x, b, rstd, mean, n, T, D, dch,
                       TS, part, partb);
  else
    hipLaunchKernelGGL((row_partial_kernel<TIN, false, LN>), g2, block, 0, s, x, b, rstd, mean, n, T, D, dch,
                       TS, part, partb);
}

// Shared body of the two entry points. gs_b is only meaningful with layer_norm.
int row_norm_gs(const char* who, bool layer_norm, const void* x, const void* b, int in_dtype, void* gs_w,
                void* gs_b, int gs_dtype, float* sumsq_w, float* sumsq_b, int64_t n, int64_t T, int64_t D, float eps,
                float scale, void* ws, size_t ws_bytes, dpk_stream_t stream) {
  DPK_REQUIRE(n >= 0 && T >= 1 && D >= 1, DPK_E_SHAPE, "%s: n=%lld T=%lld D=%lld", who, (long long)n,
              (long long)T, (long long)D);
  if (n == 0 || (!gs_w && !gs_b)) return DPK_OK;
  DPK_REQUIRE(x && b, DPK_E_ARG, "%s: NULL tensor", who);
  DPK_REQUIRE(dpk_dtype_ok(in_dtype) && dpk_dtype_ok(gs_dtype), DPK_E_DTYPE, "%s: dtypes %d,%d", who,
              in_dtype, gs_dtype);
  DPK_REQUIRE(dpk_aligned(x, dpk_elsize(in_dtype)) && dpk_aligned(b, dpk_elsize(in_dtype)) &&
                  dpk_aligned(gs_w, dpk_elsize(gs_dtype)) && dpk_aligned(gs_b, dpk_elsize(gs_dtype)),
              DPK_E_ALIGN, "%s: misaligned tensor", who);
  const RowWs w = row_ws(n, T, D);
  DPK_REQUIRE(ws && ws_bytes >= w.total(), DPK_E_WORKSPACE, "%s: workspace %zu < %zu bytes", who, ws_bytes,
              w.total());
  DPK_REQUIRE(dpk_aligned(ws, 256), DPK_E_ALIGN, "%s: workspace must be 256-byte aligned", who);
  const size_t va = in_dtype == DPK_BF16 ? 8 : 16;
  const bool vec = D % 4 == 0 && dpk_aligned(x, va) && dpk_aligned(b, va);
  const bool fused = vec && row_fused_ok(D) && n * row_fused_splits(n, T) <= DPK_MAX_GRID_X;
  const int TS = fused ? row_fused_splits(n, T) : row_splits(T);
  const int64_t dch = dpk_cdiv(D, kThreads * (vec ? 4 : 1));
  DPK_REQUIRE(n * dch * TS <= DPK_MAX_GRID_X && dpk_cdiv(n * T, kWaves) <= DPK_MAX_GRID_X, DPK_E_SHAPE,
              "%s: too many blocks", who);
  hipStream_t s = static_cast<hipStream_t>(stream);
  float* partb = gs_b ? w.partb(ws) : nullptr;
  if (in_dtype == DPK_F32) {
    const float* xp = static_cast<const float*>(x);
    const float* bp = static_cast<const float*>(b);
    if (layer_norm)
      launch_rows<float, true>(xp, bp, n, T, D, eps, vec, fused, TS, w.rstd(ws), w.mean(ws), w.part(ws), partb, s);
    else
      launch_rows<float, false>(xp, bp, n, T, D, eps, vec, fused, TS, w.rstd(ws), w.mean(ws), w.part(ws), partb, s);
  } else {
    const bf16_t* xp = static_cast<const bf16_t*>(x);
    const bf16_t* bp = static_cast<const bf16_t*>(b);
    if (layer_norm)
      launch_rows<bf16_t, true>(xp, bp, n, T, D, eps, vec, fused, TS, w.rstd(ws), w.mean(ws), w.part(ws), partb, s);
    else
      launch_rows<bf16_t, false>(xp, bp, n, T, D, eps, vec, fused, TS, w.rstd(ws), w.mean(ws), w.part(ws), partb, s);
  }
  DPK_LAUNCH_CHECK(who);
  const dim3 block(kThreads), g3(static_cast<unsigned>(dpk_cdiv(n * D, kThreads)));
  for (int pass = 0; pass < 2; ++pass) {
    void* out = pass == 0 ? gs_w : gs_b;
    float* ssq = pass == 0 ? sumsq_w : sumsq_b;
    const float* src = pass == 0 ? w.part(ws) : w.partb(ws);
    if (!out) continue;
    if (gs_dtype == DPK_F32)
      hipLaunchKernelGGL(row_final_kernel<float>, g3, block, 0, s, src, n * D, TS, scale, static_cast<float*>(out));
    else
      hipLaunchKernelGGL(row_final_kernel<bf16_t>, g3, block, 0, s, src, n * D, TS, scale,
                         static_cast<bf16_t*>(out));
    if (ssq) {
      const dim3 gn(static_cast<unsigned>(n));
      if (gs_dtype == DPK_F32)
        hipLaunchKernelGGL(row_sumsq_kernel<float>, gn, block, 0, s, static_cast<const float*>(out), D, ssq);
      else
        hipLaunchKernelGGL(row_sumsq_kernel<bf16_t>, gn, block, 0, s, static_cast<const bf16_t*>(out), D, ssq);
    }
  }
  DPK_LAUNCH_CHECK(who);
  return DPK_OK;
}

}  // namespace

extern "C" int dpk_group_norm_gs(const void* x, const void* b, int in_dtype, void* gs_w, void* gs_b,
                                 int gs_dtype, float* sumsq_w, float* sumsq_b, int64_t n, int64_t C,
                                 int64_t S, int64_t groups, float eps, float scale, dpk_stream_t stream) {
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
  // register-resident path: whole chunks of four per channel, group of at most 8192
  const int64_t len = (C / groups) * S;
  const size_t va = in_dtype == DPK_BF16 ? 8 : 16;
  const bool reg = S % 4 == 0 && len <= 1024 * 8 && dpk_aligned(x, va) && dpk_aligned(b, va);
  const int K = len <= 1024 ? 1 : len <= 2048 ? 2 : len <= 4096 ? 4 : 8;
#define DPK_GN_ARGS(TI, TO)                                                                    \
  grid, block, 0, s, static_cast<const TI*>(x), static_cast<const TI*>(b), static_cast<TO*>(gs_w), \
      static_cast<TO*>(gs_b), C, S, groups, eps, scale
#define DPK_GN(TI, TO)                                                                           \
  do {                                                                                           \
    if (!reg) hipLaunchKernelGGL((group_norm_gs_kernel<TI, TO>), DPK_GN_ARGS(TI, TO));           \
    else if (K == 1) hipLaunchKernelGGL((group_norm_gs_reg_kernel<TI, TO, 1>), DPK_GN_ARGS(TI, TO)); \
    else if (K == 2) hipLaunchKernelGGL((group_norm_gs_reg_kernel<TI, TO, 2>), DPK_GN_ARGS(TI, TO)); \
    else if (K == 4) hipLaunchKernelGGL((group_norm_gs_reg_kernel<TI, TO, 4>), DPK_GN_ARGS(TI, TO)); \
    else hipLaunchKernelGGL((group_norm_gs_reg_kernel<TI, TO, 8>), DPK_GN_ARGS(TI, TO));         \
  } while (0)
  if (in_dtype == DPK_F32 && gs_dtype == DPK_F32) DPK_GN(float, float);
  else if (in_dtype == DPK_BF16 && gs_dtype == DPK_BF16) DPK_GN(bf16_t, bf16_t);
  else if (in_dtype == DPK_BF16 && gs_dtype == DPK_F32) DPK_GN(bf16_t, float);
  else DPK_GN(float, bf16_t);
#undef DPK_GN
#undef DPK_GN_ARGS
  DPK_LAUNCH_CHECK(who);
  // per-sample sums of squares of the [n, C] results, for the optimizer's norm pass
  for (int pass = 0; pass < 2; ++pass) {
    const void* out = pass == 0 ? gs_w : gs_b;
    float* ssq = pass == 0 ? sumsq_w : sumsq_b;
    if (!out || !ssq) continue;
    const dim3 gn(static_cast<unsigned>(n));
    if (gs_dtype == DPK_F32)
      hipLaunchKernelGGL(row_sumsq_kernel<float>, gn, block, 0, s, static_cast<const float*>(out), C, ssq);
    else
      hipLaunchKernelGGL(row_sumsq_kernel<bf16_t>, gn, block, 0, s, static_cast<const bf16_t*>(out), C, ssq);
    DPK_LAUNCH_CHECK(who);
  }
  return DPK_OK;
}

extern "C" size_t dpk_rms_norm_gs_workspace_bytes(int64_t n, int64_t T, int64_t D) {
  if (n <= 0 || T <= 0 || D <= 0) return 0;
  return row_ws(n, T, D).total();
}

extern "C" int dpk_rms_norm_gs(const void* x, const void* b, int in_dtype, void* gs_w, int gs_dtype,
                               float* sumsq, int64_t n, int64_t T, int64_t D, float eps, float scale,
                               void* ws, size_t ws_bytes, dpk_stream_t stream) {
  DPK_REQUIRE(gs_w || n == 0, DPK_E_ARG, "dpk_rms_norm_gs: NULL tensor");
  return row_norm_gs("dpk_rms_norm_gs", false, x, b, in_dtype, gs_w, nullptr, gs_dtype, sumsq, nullptr, n, T, D,
                     eps, scale, ws, ws_bytes, stream);
}

extern "C" size_t dpk_layer_norm_gs_workspace_bytes(int64_t n, int64_t T, int64_t D) {
  return dpk_rms_norm_gs_workspace_bytes(n, T, D);
}

extern "C" int dpk_layer_norm_gs(const void* x, const void* b, int in_dtype, void* gs_w, void* gs_b,
                                 int gs_dtype, float* sumsq_w, float* sumsq_b, int64_t n, int64_t T, int64_t D,
                                 float eps, float scale, void* ws, size_t ws_bytes, dpk_stream_t stream) {
  return row_norm_gs("dpk_layer_norm_gs", true, x, b, in_dtype, gs_w, gs_b, gs_dtype, sumsq_w, sumsq_b, n, T, D,
                     eps, scale, ws, ws_bytes, stream);
}
