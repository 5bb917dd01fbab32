// Per-sample gradients of nn.Conv2d (opacus/grad_sample/conv.py:28-119, Conv2d
// branch) as an implicit-GEMM on the fp32 MFMA path:
//   gs[n, g*Og + m, p] = scale * sum_q b[n, g*Og + m, q] * U[n, g, p, q]
// with q = (oh, ow) running over output positions and p = (c, kh, kw) over one
// group's kernel elements. U is the unfolded activation of
// opacus/utils/tensor_utils.py:116-172,
//   U[n, g, (c,kh,kw), (oh,ow)] = xpad[n, g*Cg + c, oh*sh + kh*dh, ow*sw + kw*dw],
// which is gathered straight from x into the LDS tile (zero where the padding
// is): the n x C*KH*KW x OH*OW matrix the reference writes and re-reads never
// exists. Only the group-diagonal blocks are computed, where the reference forms
// the full O x p product and discards the rest (conv.py:102-112).
#include "dpk_common.h"
#include "mfma_f32.h"

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / DPK_WAVE;

struct ConvGeom {
  int H, W, OW, Q;      // input rows/cols, output cols, output positions
  int KH, KW, Pg;       // kernel, kernel elements per group (Cg*KH*KW)
  int sh, sw, dh, dw;   // stride, dilation
  int ph, pw;           // top / left padding
  // Conv3d only (all 1 / 0 for two dimensions): input depth, kernel depth, depth
  // stride / dilation / front padding, output positions per depth slice (OH*OW).
  int Dd, KD, sd, dd, pd, OHW;
};

// Element (k = q, col = p) of the unfolded activation, staged as S[k][p].
// D3: the input has a depth dimension as well (nn.Conv3d), p = (c, kd, kh, kw) and
// q = (od, oh, ow).
template <int BN, typename T, bool D3 = false>
struct LoaderIm2col {
  static constexpr int R = mf32::BK * BN / mf32::NTHREADS;
  static constexpr int PSTEP = mf32::NTHREADS / mf32::BK;
  const T* x;  // first channel of this sample's group
  ConvGeom g;
  int kq, pl0;
  int off[R], dy[R], dx[R], dz[D3 ? R : 1];
  float st[R];
  __device__ __forceinline__ LoaderIm2col(const T* x_, const ConvGeom& g_, int p0) : x(x_), g(g_) {
    kq = threadIdx.x % mf32::BK;
    pl0 = threadIdx.x / mf32::BK;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int p = p0 + pl0 + r * PSTEP;
      if (p < g.Pg) {
        const int kvol = g.KD * g.KH * g.KW;
        const int c = p / kvol;
        int rem = p % kvol;
        off[r] = c * g.Dd * g.H * g.W;
        if (D3) {
          dz[r] = (rem / (g.KH * g.KW)) * g.dd - g.pd;
          rem %= g.KH * g.KW;
        }
        dy[r] = (rem / g.KW) * g.dh - g.ph;
        dx[r] = (rem % g.KW) * g.dw - g.pw;
      } else {
        off[r] = -1;
        dy[r] = dx[r] = 0;
        if (D3) dz[r] = 0;
      }
    }
  }
  __device__ __forceinline__ void fetch(int64_t k0) {
    const int q = static_cast<int>(k0) + kq;
    int q2 = q, iz0 = 0;
    if (D3) {
      const int od = q / g.OHW;
      q2 = q - od * g.OHW;
      iz0 = od * g.sd;
    }
    const int oh = q2 / g.OW, ow = q2 - oh * g.OW;
    const int iy0 = oh * g.sh, ix0 = ow * g.sw;
    const bool inq = q < g.Q;
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int iy = iy0 + dy[r], ix = ix0 + dx[r];
      bool ok = inq && off[r] >= 0 && static_cast<unsigned>(iy) < static_cast<unsigned>(g.H) &&
                static_cast<unsigned>(ix) < static_cast<unsigned>(g.W);
      int plane = 0;
      if (D3) {
        const int iz = iz0 + dz[r];
        ok = ok && static_cast<unsigned>(iz) < static_cast<unsigned>(g.Dd);
        plane = iz * g.H;
      }
      st[r] = ok ? dpk_io<T>::load(x + off[r] + (plane + iy) * g.W + ix) : 0.f;
    }
  }
  __device__ __forceinline__ void commit(float (*S)[BN + mf32::PAD]) {
#pragma unroll
    for (int r = 0; r < R; ++r) S[kq][pl0 + r * PSTEP] = st[r];
  }
};

template <int BM, int BN, typename TIN, typename TOUT, bool VEC, bool D3>
__global__ __launch_bounds__(kThreads) void conv2d_gs_kernel(
    const TIN* __restrict__ x, const TIN* __restrict__ b, TOUT* __restrict__ gs,
    float* __restrict__ partials, ConvGeom g, int C, int O, int groups, float scale, int tiles_m,
    int tiles_n) {
  __shared__ mf32::Smem<BM, BN> sm;
  __shared__ float red[kWaves];
  const int Og = O / groups, Cg = C / groups;
  int64_t bid = blockIdx.x;
  const int tn = static_cast<int>(bid % tiles_n);
  bid /= tiles_n;
  const int tm = static_cast<int>(bid % tiles_m);
  bid /= tiles_m;
  const int grp = static_cast<int>(bid % groups);
  const int64_t sample = bid / groups;
  const int m0 = tm * BM, p0 = tn * BN;
  const TIN* bg = b + (sample * O + static_cast<int64_t>(grp) * Og) * g.Q;
  const TIN* xg = x + (sample * C + static_cast<int64_t>(grp) * Cg) * g.Dd * g.H * g.W;
  mf32::LoaderKContig<BM, TIN, VEC> la(bg, g.Q, m0, Og, g.Q);
  LoaderIm2col<BN, TIN, D3> lb(xg, g, p0);
  mf32::Tile<BM, BN> tile;
  tile.clear();
  mf32::mainloop<BM, BN>(tile, sm, la, lb, g.Q);
  TOUT* out = gs + (sample * O + static_cast<int64_t>(grp) * Og) * g.Pg;
  float ss = 0.f;
  tile.for_each([&](int r, int c, float v) {
    const int m = m0 + r, p = p0 + c;
    if (m < Og && p < g.Pg) {
      const float val = v * scale;
      dpk_io<TOUT>::store(out + static_cast<int64_t>(m) * g.Pg + p, val);
      ss = fmaf(val, val, ss);
    }
  });
  if (partials) {
    const float s = block_sum<kWaves>(ss, red);
    if (threadIdx.x == 0) partials[blockIdx.x] = s;
  }
}

// ---- small images: the padded input patch lives in LDS -------------------------
// When the channels a column tile touches fit in LDS with their zero padding
// (nch x Hp x Wp floats), the unfolded matrix needs no index arithmetic at all in
// the k loop: element (q, p) is xs[base(p) + qtab[q]] with
//   base(p) = (c - c_lo) * Hp * Wp + kh * dh * Wp + kw * dw      (fixed per lane)
//   qtab[q] = oh * sh * Wp + ow * sw                              (table in LDS)
// and the MFMA's B operand is read straight from the patch. The gather kernel
// above spends more VALU cycles on (iy, ix) bounds and addresses than the MFMAs
// take; here the k loop is MFMAs, LDS reads and the staging of the backprop tile.
template <int BM, int BN, typename TIN, typename TOUT, bool VEC>
__global__ __launch_bounds__(kThreads) void conv2d_gs_patch_kernel(
    const TIN* __restrict__ x, const TIN* __restrict__ b, TOUT* __restrict__ gs,
    float* __restrict__ partials, ConvGeom g, int C, int O, int groups, float scale, int tiles_m,
    int tiles_n, int Hp, int Wp, int pr, int nch_max) {
  using Tile = mf32::Tile<BM, BN>;
  extern __shared__ __align__(16) unsigned char dyn_lds[];
  // layout: A stages | qtab | patch
  typedef float (*AStage)[BM + mf32::PAD];
  float* a_mem = reinterpret_cast<float*>(dyn_lds);
  constexpr int kAStage = mf32::BK * (BM + mf32::PAD);
  const int Qpad = (g.Q + mf32::BK - 1) / mf32::BK * mf32::BK;
  int* qtab = reinterpret_cast<int*>(a_mem + 2 * kAStage);
  float* xs = reinterpret_cast<float*>(qtab + Qpad);
  __shared__ float red[kWaves];

  const int Og = O / groups, Cg = C / groups;
  int64_t bid = blockIdx.x;
  const int tn = static_cast<int>(bid % tiles_n);
  bid /= tiles_n;
  const int tm = static_cast<int>(bid % tiles_m);
  bid /= tiles_m;
  const int grp = static_cast<int>(bid % groups);
  const int64_t sample = bid / groups;
  const int m0 = tm * BM, p0 = tn * BN;
  const int KK = g.KH * g.KW;
  const int c_lo = p0 / KK;
  int c_hi = (p0 + BN - 1) / KK;
  c_hi = c_hi < Cg ? c_hi : Cg - 1;
  const int nch = c_hi - c_lo + 1;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;

  // stage the patch (zero outside the image): 8 independent loads per thread are
  // issued before any of them is stored, so the block pays global latency once per
  // batch rather than once per element
  const TIN* xg = x + ((sample * C + static_cast<int64_t>(grp) * Cg + c_lo) * g.H) * g.W;
  const int plane = Hp * Wp, total = nch * plane;
  for (int i0 = threadIdx.x; i0 < total; i0 += kThreads * 8) {
    float v[8];
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int i = i0 + u * kThreads;
      const int c = i / plane, r = i - c * plane;
      const int y = r / Wp, xx = r - y * Wp;
      const int iy = y - g.ph, ix = xx - g.pw;
      const bool in = i < total && static_cast<unsigned>(iy) < static_cast<unsigned>(g.H) &&
                      static_cast<unsigned>(ix) < static_cast<unsigned>(g.W);
      v[u] = in ? dpk_io<TIN>::load(xg + (static_cast<int64_t>(c) * g.H + iy) * g.W + ix) : 0.f;
    }
#pragma unroll
    for (int u = 0; u < 8; ++u) {
      const int i = i0 + u * kThreads;
      if (i < total) xs[i] = v[u];
    }
  }
  for (int q = threadIdx.x; q < Qpad; q += kThreads) {
    const int oh = q / g.OW, ow = q - oh * g.OW;
    qtab[q] = q < g.Q ? oh * g.sh * Wp + ow * g.sw : 0;
  }
  // this lane's columns of the tile
  const int wm0 = (wave >> 1) * Tile::WM, wn0 = (wave & 1) * Tile::WN;
  const int kk = lane >> 5, l32 = lane & 31;
  int base_p[Tile::TN];
#pragma unroll
  for (int j = 0; j < Tile::TN; ++j) {
    const int p = p0 + wn0 + j * 32 + l32;
    if (p < g.Pg) {
      const int c = p / KK, rem = p - c * KK;
      const int kh = rem / g.KW, kw = rem - kh * g.KW;
      base_p[j] = (c - c_lo) * Hp * Wp + kh * g.dh * Wp + kw * g.dw;
    } else {
      base_p[j] = 0;  // result discarded below; any address inside the patch will do
    }
  }
  (void)pr;
  (void)nch_max;

  // Backprop tile pipeline: BM x 16 floats per k-tile is one 16-byte load per
  // thread, so D tiles are kept in flight in registers (slot = tile % D) and global
  // latency is covered by D - 1 steps of MFMAs even with few waves per SIMD.
  static_assert(BM == 64, "one 16-byte load per thread and k-tile");
  constexpr int D = 4;
  const TIN* bg = b + (sample * O + static_cast<int64_t>(grp) * Og) * g.Q;
  const int am = threadIdx.x / (mf32::BK / 4), ak = (threadIdx.x % (mf32::BK / 4)) * 4;
  const int64_t arow = m0 + am;
  const TIN* ap = bg + arow * g.Q + ak;
  float4 slot[D];
  auto fetch = [&](int64_t kt, float4& dst) {
    const int64_t k = kt * mf32::BK + ak;
    float4 v = make_float4(0.f, 0.f, 0.f, 0.f);
    if (arow < Og && k < g.Q) {
      const TIN* p = ap + kt * mf32::BK;
      if (VEC) {
        v = dpk_io<TIN>::load4(p);
      } else {
        v.x = dpk_io<TIN>::load(p);
        if (k + 1 < g.Q) v.y = dpk_io<TIN>::load(p + 1);
        if (k + 2 < g.Q) v.z = dpk_io<TIN>::load(p + 2);
        if (k + 3 < g.Q) v.w = dpk_io<TIN>::load(p + 3);
      }
    }
    dst = v;
  };
  auto commit = [&](const float4& v, AStage S) {
    S[ak + 0][am] = v.x;
    S[ak + 1][am] = v.y;
    S[ak + 2][am] = v.z;
    S[ak + 3][am] = v.w;
  };
  Tile tile;
  tile.clear();
  const int64_t nk = (g.Q + mf32::BK - 1) / mf32::BK;
#pragma unroll
  for (int d = 0; d < D - 1; ++d)
    if (d < nk) fetch(d, slot[d]);
  commit(slot[0], reinterpret_cast<AStage>(a_mem));
  __syncthreads();  // also publishes the patch and qtab
  for (int64_t kt0 = 0; kt0 < nk; kt0 += D) {
#pragma unroll
    for (int d = 0; d < D; ++d) {
      const int64_t kt = kt0 + d;
      if (kt < nk) {
        if (kt + D - 1 < nk) fetch(kt + D - 1, slot[(d + D - 1) % D]);
        AStage As = reinterpret_cast<AStage>(a_mem + (d & 1) * kAStage);
        const int* qt = qtab + kt * mf32::BK;
        int qo[mf32::BK / 2];
#pragma unroll
        for (int k2 = 0; k2 < mf32::BK / 2; ++k2) qo[k2] = qt[2 * k2 + kk];
        // all operand reads of the k-tile first, then its MFMAs: LDS latency is paid once
        float av[mf32::BK / 2][Tile::TM], bv[mf32::BK / 2][Tile::TN];
#pragma unroll
        for (int k2 = 0; k2 < mf32::BK / 2; ++k2) {
#pragma unroll
          for (int i = 0; i < Tile::TM; ++i) av[k2][i] = As[2 * k2 + kk][wm0 + i * 32 + l32];
#pragma unroll
          for (int j = 0; j < Tile::TN; ++j) bv[k2][j] = xs[base_p[j] + qo[k2]];
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int k2 = 0; k2 < mf32::BK / 2; ++k2)
#pragma unroll
          for (int i = 0; i < Tile::TM; ++i)
#pragma unroll
            for (int j = 0; j < Tile::TN; ++j)
              tile.acc[i][j] =
                  __builtin_amdgcn_mfma_f32_32x32x2f32(av[k2][i], bv[k2][j], tile.acc[i][j], 0, 0, 0);
        if (kt + 1 < nk) commit(slot[(d + 1) % D], reinterpret_cast<AStage>(a_mem + ((d + 1) & 1) * kAStage));
        __syncthreads();
      }
    }
  }
  TOUT* out = gs + (sample * O + static_cast<int64_t>(grp) * Og) * g.Pg;
  float ss = 0.f;
  tile.for_each([&](int r, int c, float v) {
    const int m = m0 + r, p = p0 + c;
    if (m < Og && p < g.Pg) {
      const float val = v * scale;
      dpk_io<TOUT>::store(out + static_cast<int64_t>(m) * g.Pg + p, val);
      ss = fmaf(val, val, ss);
    }
  });
  if (partials) {
    const float s = block_sum<kWaves>(ss, red);
    if (threadIdx.x == 0) partials[blockIdx.x] = s;
  }
}

// LDS bytes of the patch kernel for a 64 x 64 tile, or 0 if the geometry does not fit.
size_t patch_lds_bytes(const ConvGeom& g, int Cg, int Hp, int Wp) {
  const int KK = g.KH * g.KW;
  int nch = (64 + KK - 2) / KK + 1;  // channels a run of 64 columns can touch
  if (nch > Cg) nch = Cg;
  const size_t a_bytes = 2 * mf32::BK * (64 + mf32::PAD) * sizeof(float);
  const size_t q_bytes = static_cast<size_t>((g.Q + mf32::BK - 1) / mf32::BK * mf32::BK) * sizeof(int);
  const size_t x_bytes = static_cast<size_t>(nch) * Hp * Wp * sizeof(float);
  const size_t total = a_bytes + q_bytes + x_bytes;
  return total <= 64 * 1024 - 64 ? total : 0;
}

struct Plan {
  int bm, bn, tiles_m, tiles_n;
};

// The workspace query does not know the image size, so it sizes for the plan with
// the most blocks (64 x 64 tiles); make_plan(.., small = true) is that plan.
Plan make_plan(int64_t Og, int64_t Pg, bool small = false) {
  Plan p;
  if (small) {
    p.bm = p.bn = 64;
    p.tiles_m = static_cast<int>(dpk_cdiv(Og, 64));
    p.tiles_n = static_cast<int>(dpk_cdiv(Pg, 64));
    return p;
  }
  p.bm = Og > 64 ? 128 : 64;
  p.bn = (Pg > 64 && p.bm == 128) ? 128 : 64;
  if (p.bn == 64) p.bm = 64;
  p.tiles_m = static_cast<int>(dpk_cdiv(Og, p.bm));
  p.tiles_n = static_cast<int>(dpk_cdiv(Pg, p.bn));
  return p;
}

template <typename TIN, typename TOUT>
void launch(const Plan& p, bool vec, const void* x, const void* b, void* gs, float* partials,
            const ConvGeom& g, int64_t n, int C, int O, int groups, float scale, hipStream_t s,
            size_t patch_bytes, int Hp, int Wp) {
  const dim3 grid(static_cast<unsigned>(n * groups * p.tiles_m * p.tiles_n)), block(kThreads);
  const TIN* xp = static_cast<const TIN*>(x);
  const TIN* bp = static_cast<const TIN*>(b);
  TOUT* gp = static_cast<TOUT*>(gs);
  if (patch_bytes > 0) {
    if (vec)
      hipLaunchKernelGGL((conv2d_gs_patch_kernel<64, 64, TIN, TOUT, true>), grid, block, patch_bytes, s, xp,
                         bp, gp, partials, g, C, O, groups, scale, p.tiles_m, p.tiles_n, Hp, Wp, 0, 0);
    else
      hipLaunchKernelGGL((conv2d_gs_patch_kernel<64, 64, TIN, TOUT, false>), grid, block, patch_bytes, s,
                         xp, bp, gp, partials, g, C, O, groups, scale, p.tiles_m, p.tiles_n, Hp, Wp, 0, 0);
    return;
  }
#define DPK_CONV_LAUNCH(BM, BN, V, D3)                                                            \
  hipLaunchKernelGGL((conv2d_gs_kernel<BM, BN, TIN, TOUT, V, D3>), grid, block, 0, s, xp, bp, gp, \
                     partials, g, C, O, groups, scale, p.tiles_m, p.tiles_n)
  const bool d3 = g.Dd > 1 || g.KD > 1 || g.pd > 0;
  if (p.bm == 128) {
    if (vec && d3) DPK_CONV_LAUNCH(128, 128, true, true);
    else if (vec) DPK_CONV_LAUNCH(128, 128, true, false);
    else if (d3) DPK_CONV_LAUNCH(128, 128, false, true);
    else DPK_CONV_LAUNCH(128, 128, false, false);
  } else {
    if (vec && d3) DPK_CONV_LAUNCH(64, 64, true, true);
    else if (vec) DPK_CONV_LAUNCH(64, 64, true, false);
    else if (d3) DPK_CONV_LAUNCH(64, 64, false, true);
    else DPK_CONV_LAUNCH(64, 64, false, false);
  }
#undef DPK_CONV_LAUNCH
}

// Depth extents of a Conv3d call; {1, 1, 1, 0, 0, 1} for two dimensions.
struct Depth {
  int64_t D, KD, sd, pd_lo, pd_hi, dd;
};

int conv_gs(const char* who, const void* x, const void* b, int in_dtype, void* gs, int gs_dtype,
            float* sumsq, int64_t n, int64_t C, const Depth& z, int64_t H, int64_t W, int64_t O,
            int64_t KH, int64_t KW, int64_t sh, int64_t sw, int64_t ph_lo, int64_t ph_hi, int64_t pw_lo,
            int64_t pw_hi, int64_t dh, int64_t dw, int64_t groups, float scale, void* ws, size_t ws_bytes,
            dpk_stream_t stream);

}  // namespace

extern "C" size_t dpk_conv2d_gs_workspace_bytes(int64_t n, int64_t C, int64_t O, int64_t KH,
                                                int64_t KW, int64_t groups) {
  if (n <= 0 || C <= 0 || O <= 0 || KH <= 0 || KW <= 0 || groups <= 0) return 0;
  if (C % groups != 0 || O % groups != 0) return 0;
  const Plan p = make_plan(O / groups, (C / groups) * KH * KW, true);
  return dpk_align_up(static_cast<size_t>(n * groups * p.tiles_m * p.tiles_n) * sizeof(float), 256);
}

namespace {
int conv_gs(const char* who, const void* x, const void* b, int in_dtype, void* gs, int gs_dtype,
            float* sumsq, int64_t n, int64_t C, const Depth& z, int64_t H, int64_t W, int64_t O,
            int64_t KH, int64_t KW, int64_t sh, int64_t sw, int64_t ph_lo, int64_t ph_hi, int64_t pw_lo,
            int64_t pw_hi, int64_t dh, int64_t dw, int64_t groups, float scale, void* ws, size_t ws_bytes,
            dpk_stream_t stream) {
  DPK_REQUIRE(n >= 0 && C >= 1 && H >= 1 && W >= 1 && O >= 1 && KH >= 1 && KW >= 1 && z.D >= 1 && z.KD >= 1,
              DPK_E_SHAPE, "%s: bad tensor sizes", who);
  DPK_REQUIRE(sh >= 1 && sw >= 1 && dh >= 1 && dw >= 1 && ph_lo >= 0 && ph_hi >= 0 && pw_lo >= 0 &&
                  pw_hi >= 0 && groups >= 1 && z.sd >= 1 && z.dd >= 1 && z.pd_lo >= 0 && z.pd_hi >= 0,
              DPK_E_SHAPE, "%s: bad geometry", who);
  DPK_REQUIRE(C % groups == 0 && O % groups == 0, DPK_E_SHAPE,
              "%s: groups=%lld does not divide C=%lld and O=%lld", who, (long long)groups,
              (long long)C, (long long)O);
  if (n == 0) return DPK_OK;
  const int64_t eh = H + ph_lo + ph_hi - (dh * (KH - 1) + 1), ew = W + pw_lo + pw_hi - (dw * (KW - 1) + 1);
  const int64_t ed = z.D + z.pd_lo + z.pd_hi - (z.dd * (z.KD - 1) + 1);
  DPK_REQUIRE(eh >= 0 && ew >= 0 && ed >= 0, DPK_E_SHAPE, "%s: kernel larger than the padded input", who);
  const int64_t OH = eh / sh + 1, OW = ew / sw + 1, OD = ed / z.sd + 1;
  const int64_t Q = OD * OH * OW, Pg = (C / groups) * z.KD * KH * KW;
  DPK_REQUIRE(C * z.D * H * W < (1LL << 31) && O * Q < (1LL << 31) && O * Pg < (1LL << 31), DPK_E_SHAPE,
              "%s: one sample exceeds 2^31 elements", who);
  DPK_REQUIRE(x && b && gs, DPK_E_ARG, "%s: NULL tensor", who);
  DPK_REQUIRE(dpk_dtype_ok(in_dtype) && dpk_dtype_ok(gs_dtype), DPK_E_DTYPE, "%s: dtypes %d,%d", who,
              in_dtype, gs_dtype);
  DPK_REQUIRE(dpk_aligned(x, dpk_elsize(in_dtype)) && dpk_aligned(b, dpk_elsize(in_dtype)) &&
                  dpk_aligned(gs, dpk_elsize(gs_dtype)),
              DPK_E_ALIGN, "%s: misaligned tensor", who);
  ConvGeom g;
  g.H = (int)H; g.W = (int)W; g.OW = (int)OW; g.Q = (int)Q;
  g.KH = (int)KH; g.KW = (int)KW; g.Pg = (int)Pg;
  g.sh = (int)sh; g.sw = (int)sw; g.dh = (int)dh; g.dw = (int)dw;
  g.ph = (int)ph_lo; g.pw = (int)pw_lo;
  g.Dd = (int)z.D; g.KD = (int)z.KD; g.sd = (int)z.sd; g.dd = (int)z.dd; g.pd = (int)z.pd_lo;
  g.OHW = (int)(OH * OW);
  const int64_t Hp = H + ph_lo + ph_hi, Wp = W + pw_lo + pw_hi;
  const bool flat = z.D == 1 && z.KD == 1 && z.pd_lo == 0 && z.pd_hi == 0;  // the LDS patch is two-dimensional
  const size_t patch_bytes =
      flat && Hp * Wp < (1 << 20) ? patch_lds_bytes(g, (int)(C / groups), (int)Hp, (int)Wp) : 0;
  const Plan p = make_plan(O / groups, Pg, patch_bytes > 0);
  const int64_t blocks = n * groups * p.tiles_m * p.tiles_n;
  DPK_REQUIRE(blocks <= DPK_MAX_GRID_X, DPK_E_SHAPE, "%s: %lld blocks exceed the grid limit", who,
              (long long)blocks);
  float* partials = nullptr;
  if (sumsq) {
    const size_t need = static_cast<size_t>(blocks) * sizeof(float);
    DPK_REQUIRE(ws && ws_bytes >= need, DPK_E_WORKSPACE, "%s: workspace %zu < %zu bytes", who,
                ws_bytes, need);
    DPK_REQUIRE(dpk_aligned(ws, 4), DPK_E_ALIGN, "%s: workspace misaligned", who);
    partials = static_cast<float*>(ws);
  }
  const bool vec = Q % 4 == 0 && dpk_aligned(b, in_dtype == DPK_BF16 ? 8 : 16);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (in_dtype == DPK_F32 && gs_dtype == DPK_F32)
    launch<float, float>(p, vec, x, b, gs, partials, g, n, (int)C, (int)O, (int)groups, scale, s, patch_bytes,
                       (int)Hp, (int)Wp);
  else if (in_dtype == DPK_BF16 && gs_dtype == DPK_BF16)
    launch<bf16_t, bf16_t>(p, vec, x, b, gs, partials, g, n, (int)C, (int)O, (int)groups, scale, s, patch_bytes,
                         (int)Hp, (int)Wp);
  else if (in_dtype == DPK_BF16 && gs_dtype == DPK_F32)
    launch<bf16_t, float>(p, vec, x, b, gs, partials, g, n, (int)C, (int)O, (int)groups, scale, s, patch_bytes,
                        (int)Hp, (int)Wp);
  else
    launch<float, bf16_t>(p, vec, x, b, gs, partials, g, n, (int)C, (int)O, (int)groups, scale, s, patch_bytes,
                        (int)Hp, (int)Wp);
  DPK_LAUNCH_CHECK(who);
  if (sumsq) {
    dpk_launch_reduce_rows(partials, n, static_cast<int64_t>(groups) * p.tiles_m * p.tiles_n, sumsq, 0,
                           1.f, s);
    DPK_LAUNCH_CHECK(who);
  }
  return DPK_OK;
}
}  // namespace

extern "C" int dpk_conv2d_gs(const void* x, const void* b, int in_dtype, void* gs, int gs_dtype,
                             float* sumsq, int64_t n, int64_t C, int64_t H, int64_t W, int64_t O,
                             int64_t KH, int64_t KW, int64_t sh, int64_t sw, int64_t ph_lo,
                             int64_t ph_hi, int64_t pw_lo, int64_t pw_hi, int64_t dh, int64_t dw,
                             int64_t groups, float scale, void* ws, size_t ws_bytes,
                             dpk_stream_t stream) {
  const Depth flat = {1, 1, 1, 0, 0, 1};
  return conv_gs("dpk_conv2d_gs", x, b, in_dtype, gs, gs_dtype, sumsq, n, C, flat, H, W, O, KH, KW, sh, sw,
                 ph_lo, ph_hi, pw_lo, pw_hi, dh, dw, groups, scale, ws, ws_bytes, stream);
}

extern "C" size_t dpk_conv3d_gs_workspace_bytes(int64_t n, int64_t C, int64_t O, int64_t KD, int64_t KH,
                                                int64_t KW, int64_t groups) {
  if (KD <= 0) return 0;
  return dpk_conv2d_gs_workspace_bytes(n, C, O, KD * KH, KW, groups);
}

extern "C" int dpk_conv3d_gs(const void* x, const void* b, int in_dtype, void* gs, int gs_dtype,
                             float* sumsq, int64_t n, int64_t C, int64_t D, int64_t H, int64_t W,
                             int64_t O, const int64_t* kernel, const int64_t* stride,
                             const int64_t* pad_lo, const int64_t* pad_hi, const int64_t* dilation,
                             int64_t groups, float scale, void* ws, size_t ws_bytes,
                             dpk_stream_t stream) {
  const char* who = "dpk_conv3d_gs";
  DPK_REQUIRE(kernel && stride && pad_lo && pad_hi && dilation, DPK_E_ARG, "%s: NULL geometry array", who);
  const Depth z = {D, kernel[0], stride[0], pad_lo[0], pad_hi[0], dilation[0]};
  return conv_gs(who, x, b, in_dtype, gs, gs_dtype, sumsq, n, C, z, H, W, O, kernel[1], kernel[2], stride[1],
                 stride[2], pad_lo[1], pad_hi[1], pad_lo[2], pad_hi[2], dilation[1], dilation[2], groups, scale,
                 ws, ws_bytes, stream);
}
