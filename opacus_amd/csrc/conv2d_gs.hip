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
#include <cstring>
#include <mutex>
#include <type_traits>

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
  // block order: 1 = each XCD works through a contiguous range of (sample, tile) units, so
  // that a sample's inputs are fetched into one L2 only; 0 = the hardware's round-robin
  int xcd_order;
};

// Element (k = q, col = p) of the unfolded activation, staged as S[k][p].
// D3: the input has a depth dimension as well (nn.Conv3d), p = (c, kd, kh, kw) and
// q = (od, oh, ow).
// The padded patch in LDS: Hp x Wp cells per channel, laid out with a row stride rs >= Wp and
// a channel stride cs >= Hp * rs chosen so that the cells one wave reads at a time fall into
// different LDS banks.
struct PatchDims {
  int Hp, Wp, rs, cs;
};

template <int BN, typename T, bool D3 = false>
struct LoaderIm2col {
  static constexpr int R = mf32::BK * BN / mf32::NTHREADS;
  static constexpr int PSTEP = mf32::NTHREADS / mf32::BK;
  const T* x;  // first channel of this sample's group
  ConvGeom g;
  int qend;  // positions from here on read as zeros (the end of this block's share of the contraction)
  int kq, pl0;
  int off[R], dy[R], dx[R], dz[D3 ? R : 1];
  float st[R];
  __device__ __forceinline__ LoaderIm2col(const T* x_, const ConvGeom& g_, int p0, int qend_) : x(x_), g(g_), qend(qend_) {
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
    const bool inq = q < qend;
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

// ksplit > 1: the contraction over the output positions is cut into ksplit pieces of kchunk
// positions (a multiple of the k tile), one block each; the raw tiles go to
// split_out[piece, n, O, Pg] and conv_split_reduce_kernel adds them. A layer with few, long
// blocks (a network's first convolution: three column tiles and 12,544 positions) fills the
// device that way. gs == NULL (norm only): nothing is stored, the squares are still summed.
template <int BM, int BN, typename TIN, typename TOUT, bool VEC, bool D3>
__global__ __launch_bounds__(kThreads) void conv2d_gs_kernel(
    const TIN* __restrict__ x, const TIN* __restrict__ b, TOUT* __restrict__ gs,
    float* __restrict__ partials, ConvGeom g, int C, int O, int groups, float scale, int tiles_m,
    int tiles_n, int ksplit, int kchunk, float* __restrict__ split_out, int64_t n) {
  __shared__ mf32::Smem<BM, BN> sm;
  __shared__ float red[kWaves];
  const int Og = O / groups, Cg = C / groups;
  // a sample's tiles run on one XCD (if the host asks), so that what they share is fetched into one L2 only
  const uint32_t unit = g.xcd_order ? xcd_contiguous_id(blockIdx.x, gridDim.x) : blockIdx.x;
  int64_t bid = unit;
  const int piece = static_cast<int>(bid % ksplit);
  bid /= ksplit;
  const int tn = static_cast<int>(bid % tiles_n);
  bid /= tiles_n;
  const int tm = static_cast<int>(bid % tiles_m);
  bid /= tiles_m;
  const int grp = static_cast<int>(bid % groups);
  const int64_t sample = bid / groups;
  const int m0 = tm * BM, p0 = tn * BN;
  const int kb = piece * kchunk;
  const int ke = kb + kchunk < g.Q ? kb + kchunk : g.Q;
  const TIN* bg = b + (sample * O + static_cast<int64_t>(grp) * Og) * g.Q;
  const TIN* xg = x + (sample * C + static_cast<int64_t>(grp) * Cg) * g.Dd * g.H * g.W;
  mf32::LoaderKContig<BM, TIN, VEC> la(bg, g.Q, m0, Og, ke);
  LoaderIm2col<BN, TIN, D3> lb(xg, g, p0, ke);
  mf32::Tile<BM, BN> tile;
  tile.clear();
  mf32::mainloop<BM, BN>(tile, sm, la, lb, kb, ke);
  if (split_out) {
    float* out = split_out + ((static_cast<int64_t>(piece) * n + sample) * O + static_cast<int64_t>(grp) * Og) * g.Pg;
    tile.for_each([&](int r, int c, float v) {
      const int m = m0 + r, p = p0 + c;
      if (m < Og && p < g.Pg) out[static_cast<int64_t>(m) * g.Pg + p] = v;
    });
    return;
  }
  TOUT* out = gs + (sample * O + static_cast<int64_t>(grp) * Og) * g.Pg;
  float ss = 0.f;
  tile.for_each([&](int r, int c, float v) {
    const int m = m0 + r, p = p0 + c;
    if (m < Og && p < g.Pg) {
      const float val = v * scale;
      if (gs) dpk_io<TOUT>::store(out + static_cast<int64_t>(m) * g.Pg + p, val);
      ss = fmaf(val, val, ss);
    }
  });
  if (partials) {
    const float s = block_sum<kWaves>(ss, red);
    if (threadIdx.x == 0) partials[unit] = s;
  }
}

// gs[sample, i] = scale * sum over the pieces of split[piece, sample, i], i < O * Pg, and the
// block's sum of squares of what it wrote. grid = n * chunks, kSplitChunk elements a block.
constexpr int kSplitChunk = 4096;
template <typename TOUT>
__global__ __launch_bounds__(kThreads) void conv_split_reduce_kernel(const float* __restrict__ split,
                                                                      TOUT* __restrict__ gs,
                                                                      float* __restrict__ partials, int64_t n,
                                                                      int64_t OP, int ksplit, int chunks, float scale) {
  __shared__ float red[kWaves];
  const int64_t sample = blockIdx.x / chunks;
  const int64_t i0 = static_cast<int64_t>(blockIdx.x % chunks) * kSplitChunk;
  float ss = 0.f;
  for (int64_t i = i0 + threadIdx.x; i < i0 + kSplitChunk && i < OP; i += kThreads) {
    float v = 0.f;
    for (int s = 0; s < ksplit; ++s) v += split[(static_cast<int64_t>(s) * n + sample) * OP + i];
    v *= scale;
    if (gs) dpk_io<TOUT>::store(gs + sample * OP + i, v);
    ss = fmaf(v, v, ss);
  }
  if (partials) {
    const float t = block_sum<kWaves>(ss, red);
    if (threadIdx.x == 0) partials[blockIdx.x] = t;
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
// take; here the k loop is MFMAs, LDS reads of the patch and register loads of the
// backprops.
// 4 consecutive elements / one element at a byte offset of a buffer descriptor (zeros past
// its end); the fp32 patch kernel serves fp32 input only (bf16 input has its own kernel)
template <typename T> __device__ __forceinline__ float4 buffer_load4(__amdgpu_buffer_rsrc_t r, uint32_t off);
template <> __device__ __forceinline__ float4 buffer_load4<float>(__amdgpu_buffer_rsrc_t r, uint32_t off) {
  typedef int vi4 __attribute__((ext_vector_type(4)));
  const vi4 v = __builtin_amdgcn_raw_buffer_load_b128(r, off, 0, 0);
  return make_float4(__int_as_float(v.x), __int_as_float(v.y), __int_as_float(v.z), __int_as_float(v.w));
}
template <typename T> __device__ __forceinline__ float buffer_load1(__amdgpu_buffer_rsrc_t r, uint32_t off);
template <> __device__ __forceinline__ float buffer_load1<float>(__amdgpu_buffer_rsrc_t r, uint32_t off) {
  return __int_as_float(__builtin_amdgcn_raw_buffer_load_b32(r, off, 0, 0));
}

constexpr int kPatchDepth = 4;                        // backprop k-tiles in flight per lane
constexpr int kPatchTrip = kPatchDepth * mf32::BK;    // k extent of one trip of the k loop

// ---- staging of the padded patch, shared by the two patch kernels ----------------------------
// CELL is what the patch holds: float (the fp32 kernel widens its input) or uint16_t (the bf16
// kernel keeps bf16 as it is). The table entry of an output position is the cell offset of its
// first patch cell times qmul (the bf16 kernel addresses bytes).
template <typename TIN, typename CELL>
struct PatchCell;
template <typename TIN>
struct PatchCell<TIN, float> {
  typedef typename dpk_io<TIN>::raw4 raw4;
  static __device__ __forceinline__ raw4 load4(const TIN* p) { return dpk_io<TIN>::load4_raw(p); }
  static __device__ __forceinline__ void put4(float* dst, raw4 r) {
    const float4 v = dpk_io<TIN>::unpack4(r);
    dst[0] = v.x;
    dst[1] = v.y;
    dst[2] = v.z;
    dst[3] = v.w;
  }
  static __device__ __forceinline__ float load1(const TIN* p) { return dpk_io<TIN>::load(p); }
};
template <>
struct PatchCell<bf16_t, uint16_t> {
  typedef dpk_vu2 raw4;
  static __device__ __forceinline__ raw4 load4(const bf16_t* p) { return dpk_io<bf16_t>::load4_raw(p); }
  static __device__ __forceinline__ void put4(uint16_t* dst, raw4 r) {
    dst[0] = static_cast<uint16_t>(r.x);
    dst[1] = static_cast<uint16_t>(r.x >> 16);
    dst[2] = static_cast<uint16_t>(r.y);
    dst[3] = static_cast<uint16_t>(r.y >> 16);
  }
  static __device__ __forceinline__ uint16_t load1(const bf16_t* p) { return *p; }
};

// Stages nch channels of the image at xg into xs (zero outside the image) and fills the table.
// A wave takes whole rows of the padded patch, lane = column, so no index is ever divided:
// (channel, row) advance by additions; 32 rows are loaded before any of them is stored (the
// staging is bound by global latency). When image rows are whole, aligned 4-element chunks
// (xvec) the interior is instead fetched as such chunks, eight per thread all in flight at once
// - one round trip per block - after the patch has been zeroed for its padding. The caller's
// barrier publishes both.
template <typename TIN, typename CELL>
__device__ __forceinline__ void stage_patch(CELL* __restrict__ xs, int* __restrict__ qtab,
                                            const TIN* __restrict__ xg, const ConvGeom& g, PatchDims pd,
                                            int nch, int xvec, int Qpad, int qmul) {
  typedef PatchCell<TIN, CELL> PC;
  const int Hp = pd.Hp, Wp = pd.Wp, RS = pd.rs, CS = pd.cs;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  const int rows = nch * Hp;
  if (xvec) {
    constexpr int kPer16 = 16 / static_cast<int>(sizeof(CELL));
    const int total16 = nch * CS / kPer16;  // the patch starts 16-byte aligned; a ragged tail is zeroed below
    for (int i = threadIdx.x; i < total16; i += kThreads)
      reinterpret_cast<uint4*>(xs)[i] = make_uint4(0u, 0u, 0u, 0u);
    for (int i = total16 * kPer16 + threadIdx.x; i < nch * CS; i += kThreads) xs[i] = static_cast<CELL>(0);
    __syncthreads();
    const int W4 = g.W / 4, chunks = nch * g.H * W4;
    constexpr int kChunksInFlight = 8;
    for (int i0 = threadIdx.x; i0 < chunks; i0 += kThreads * kChunksInFlight) {
      typename PC::raw4 v[kChunksInFlight];
#pragma unroll
      for (int u = 0; u < kChunksInFlight; ++u) {
        const int i = i0 + u * kThreads;
        v[u] = PC::load4(xg + static_cast<int64_t>(i < chunks ? i : 0) * 4);
      }
#pragma unroll
      for (int u = 0; u < kChunksInFlight; ++u) {
        const int i = i0 + u * kThreads;
        if (i < chunks) {
          const int r = i / W4, x4 = i - r * W4;  // r = c * H + iy
          const int c = r / g.H, iy = r - c * g.H;
          PC::put4(xs + c * CS + (iy + g.ph) * RS + g.pw + x4 * 4, v[u]);
        }
      }
    }
  } else {
    constexpr int kRowsInFlight = 32;
    for (int x0 = 0; x0 < Wp; x0 += DPK_WAVE) {
      const int xx = x0 + lane, ix = xx - g.pw;
      const bool col_ok = xx < Wp && static_cast<unsigned>(ix) < static_cast<unsigned>(g.W);
      int c = 0, y = wave;  // of the next row this wave stages
      while (y >= Hp) {
        y -= Hp;
        ++c;
      }
      for (int row = wave; row < rows; row += kWaves * kRowsInFlight) {
        CELL v[kRowsInFlight];
        const int c_first = c, y_first = y;
#pragma unroll
        for (int u = 0; u < kRowsInFlight; ++u) {
          const int iy = y - g.ph;
          const bool in = col_ok && row + u * kWaves < rows && static_cast<unsigned>(iy) < static_cast<unsigned>(g.H);
          v[u] = in ? PC::load1(xg + (static_cast<int64_t>(c) * g.H + iy) * g.W + ix) : static_cast<CELL>(0);
          y += kWaves;
          while (y >= Hp) {
            y -= Hp;
            ++c;
          }
        }
        // the same walk again for the cells (wave-uniform, a few scalar additions per row)
        int cs_ = c_first, ys_ = y_first;
#pragma unroll
        for (int u = 0; u < kRowsInFlight; ++u) {
          const int r = row + u * kWaves;
          if (r < rows && xx < Wp) xs[cs_ * CS + ys_ * RS + xx] = v[u];
          ys_ += kWaves;
          while (ys_ >= Hp) {
            ys_ -= Hp;
            ++cs_;
          }
        }
      }
    }
  }
  for (int q = threadIdx.x; q < Qpad; q += kThreads) {
    const int oh = q / g.OW, ow = q - oh * g.OW;
    qtab[q] = q < g.Q ? (oh * g.sh * RS + ow * g.sw) * qmul : 0;
  }
}

// RK (8, 4 or 0): the eight positions a half-wave takes of a k-tile fall into aligned runs of RK
// positions that lie in one output row at unit stride (stride 1 along the row, output width a
// multiple of RK), so a run's patch cells are consecutive: one table read and one address per
// run, the LDS reads at immediate offsets. 0: every position has its own table entry.
// Every vector instruction issued between the MFMAs of a wave costs MFMA time on this device
// (measured: 4 independent VALU instructions per 64-cycle fp32 MFMA stretch a loop by 23 % with
// three waves per SIMD), so the k loop keeps its address arithmetic to a minimum.
template <int BM, int BN, typename TIN, typename TOUT, bool VEC, int RK>
__global__ __launch_bounds__(kThreads) void conv2d_gs_patch_kernel(
    const TIN* __restrict__ x, const TIN* __restrict__ b, TOUT* __restrict__ gs,
    float* __restrict__ partials, ConvGeom g, int C, int O, int groups, float scale, int tiles_m,
    int tiles_n, PatchDims pd, int xvec, int nch_max) {
  const int RS = pd.rs, CS = pd.cs;
  using Tile = mf32::Tile<BM, BN>;
  extern __shared__ __align__(16) unsigned char dyn_lds[];
  // layout: qtab | patch. The k loop runs in trips of kPatchDepth k-tiles, all of them
  // unconditional: past the end the backprops read as zeros and the table points at the
  // patch's first element.
  const int Qpad = (g.Q + kPatchTrip - 1) / kPatchTrip * kPatchTrip;
  int* qtab = reinterpret_cast<int*>(dyn_lds);
  float* xs = reinterpret_cast<float*>(qtab + Qpad);
  __shared__ float red[kWaves];

  const int Og = O / groups, Cg = C / groups;
  // a sample's tiles run on one XCD (if the host asks), so that its backprops are fetched into one L2 only
  const uint32_t unit = g.xcd_order ? xcd_contiguous_id(blockIdx.x, gridDim.x) : blockIdx.x;
  int64_t bid = unit;
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

  const TIN* xg = x + ((sample * C + static_cast<int64_t>(grp) * Cg + c_lo) * g.H) * g.W;
  stage_patch<TIN, float>(xs, qtab, xg, g, pd, nch, xvec, Qpad, 1);
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
      base_p[j] = (c - c_lo) * CS + kh * g.dh * RS + kw * g.dw;
    } else {
      base_p[j] = 0;  // result discarded below; any address inside the patch will do
    }
  }
  (void)nch_max;

  // The backprop operand goes from global memory straight into registers. The instruction
  // contracts two k per step, one from each half of the wave; which k of the tile a half
  // takes is free, so half kk takes k = 8 kk .. 8 kk + 7: eight consecutive backprops of
  // the lane's output channel, two 16-byte loads. Nothing is staged in LDS and the k loop
  // has no barrier: every wave runs at its own pace, with kPatchDepth tiles of loads in
  // flight, while the gathered operand of the next tile (a table read, then a patch read
  // that depends on it) is asked for during the MFMAs of the current one.
  constexpr int D = kPatchDepth;
  constexpr int K2 = mf32::BK / 2;
  static_assert(K2 == 8, "two 4-element loads per lane and k-tile");
  const TIN* bg = b + (sample * O + static_cast<int64_t>(grp) * Og) * g.Q;
  // loads through a buffer descriptor over the group's Og x Q backprops: a lane whose row
  // or k lies outside gets an offset past the descriptor's end and reads zeros
  const __amdgpu_buffer_rsrc_t brs = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<TIN*>(bg), 0, Og * g.Q * static_cast<int>(sizeof(TIN)), 0x00020000);
  constexpr uint32_t kOutside = 0x7fffffffu;
  uint32_t row_off[Tile::TM];  // byte offset of (row, k = 8 kk), or past the end for a row outside
#pragma unroll
  for (int i = 0; i < Tile::TM; ++i) {
    const int m = m0 + wm0 + i * 32 + l32;
    row_off[i] = m < Og ? static_cast<uint32_t>(m * g.Q + kk * K2) * static_cast<uint32_t>(sizeof(TIN)) : kOutside;
  }
  auto fetch = [&](int kt, float (&a)[Tile::TM][K2]) {
    const int k = kt * mf32::BK + kk * K2;
    const bool tail = (kt + 1) * mf32::BK > g.Q;  // uniform: only the last tiles compare positions
#pragma unroll
    for (int i = 0; i < Tile::TM; ++i) {
      if (VEC) {
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          uint32_t off = row_off[i] + static_cast<uint32_t>(kt * mf32::BK + 4 * h) * static_cast<uint32_t>(sizeof(TIN));
          if (tail) {
            asm volatile("" ::: "memory");  // a branch, not a select: the steady loop skips the compare
            if (k + 4 * h >= g.Q) off = kOutside;
          }
          const float4 v = buffer_load4<TIN>(brs, off);
          a[i][4 * h + 0] = v.x;
          a[i][4 * h + 1] = v.y;
          a[i][4 * h + 2] = v.z;
          a[i][4 * h + 3] = v.w;
        }
      } else {
#pragma unroll
        for (int e = 0; e < K2; ++e) {
          uint32_t off = row_off[i] + static_cast<uint32_t>(kt * mf32::BK + e) * static_cast<uint32_t>(sizeof(TIN));
          if (tail) {
            asm volatile("" ::: "memory");
            if (k + e >= g.Q) off = kOutside;
          }
          a[i][e] = buffer_load1<TIN>(brs, off);
        }
      }
    }
  };
  constexpr int RUN = RK ? RK : 1;   // positions per table entry
  constexpr int NQ = K2 / RUN;       // table entries a half-wave needs per k-tile
  float av[D][Tile::TM][K2], bv[2][K2][Tile::TN];
  int qo[2][NQ];
  const int nk = Qpad / mf32::BK;  // a multiple of D
  auto read_q = [&](int kt, int (&q)[NQ]) {
    const int* qt = qtab + (kt < nk ? kt : 0) * mf32::BK + kk * K2;  // past the end: any valid entries
#pragma unroll
    for (int k2 = 0; k2 < NQ; ++k2) q[k2] = qt[k2 * RUN];
  };
  auto read_b = [&](const int (&q)[NQ], float (&bb)[K2][Tile::TN]) {
    if constexpr (RK != 0) {
#pragma unroll
      for (int j = 0; j < Tile::TN; ++j)
#pragma unroll
        for (int r = 0; r < NQ; ++r) {
          const float* cells = xs + (base_p[j] + q[r]);
#pragma unroll
          for (int e = 0; e < RUN; ++e) bb[r * RUN + e][j] = cells[e];
        }
    } else {
#pragma unroll
      for (int k2 = 0; k2 < K2; ++k2)
#pragma unroll
        for (int j = 0; j < Tile::TN; ++j) bb[k2][j] = xs[base_p[j] + q[k2]];
    }
  };
  Tile tile;
  tile.clear();
#pragma unroll
  for (int d = 0; d < D - 1; ++d) fetch(d, av[d]);
  __syncthreads();  // publishes the patch and qtab; the only barrier of the kernel body
  read_q(0, qo[0]);
  read_b(qo[0], bv[0]);
  read_q(1, qo[1]);
  for (int kt0 = 0; kt0 < nk; kt0 += D) {
#pragma unroll
    for (int d = 0; d < D; ++d) {
      const int kt = kt0 + d;
      const int cur = d & 1, nxt = cur ^ 1;
      fetch(kt + D - 1, av[(d + D - 1) % D]);
      read_b(qo[nxt], bv[nxt]);
      read_q(kt + 2, qo[cur]);  // tile kt's offsets were consumed one step ago
      // keep the requests above ahead of the MFMAs below: left to itself the scheduler
      // sinks each LDS read to just before the MFMA that uses it
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int k2 = 0; k2 < K2; ++k2)
#pragma unroll
        for (int i = 0; i < Tile::TM; ++i)
#pragma unroll
          for (int j = 0; j < Tile::TN; ++j)
            tile.acc[i][j] =
                __builtin_amdgcn_mfma_f32_32x32x2f32(av[d][i][k2], bv[cur][k2][j], tile.acc[i][j], 0, 0, 0);
    }
  }
  TOUT* out = gs + (sample * O + static_cast<int64_t>(grp) * Og) * g.Pg;
  float ss = 0.f;
  tile.for_each([&](int r, int c, float v) {
    const int m = m0 + r, p = p0 + c;
    if (m < Og && p < g.Pg) {
      const float val = v * scale;
      if (gs) dpk_io<TOUT>::store(out + static_cast<int64_t>(m) * g.Pg + p, val);
      ss = fmaf(val, val, ss);
    }
  });
  if (partials) {
    const float s = block_sum<kWaves>(ss, red);
    if (threadIdx.x == 0) partials[unit] = s;
  }
}

// ---- the patch kernel for bf16 input: v_mfma_f32_32x32x16_bf16 ---------------------------
// Same plan as above (padded patch in LDS, backprops from global memory into registers, a
// table of patch offsets per output position), with the operands left in bf16. The
// instruction wants, per lane, 8 consecutive k of one row: half kk of the wave holds
// k = 8 kk .. 8 kk + 7, which for the backprops is 16 contiguous bytes of global memory and
// for the gathered operand eight 2-byte LDS reads at table offsets. One MFMA now does the work
// of eight fp32 ones, so a k-tile's loads no longer hide behind its own arithmetic: the loop
// runs in trips of kP16Tiles k-tiles and asks for everything of the next trip (offsets two
// trips ahead) before the MFMAs of the current one.
constexpr int kP16Tiles = 4;
constexpr int kP16BK = 16;
constexpr int kP16TripK = kP16Tiles * kP16BK;
static_assert(kP16TripK == kPatchTrip, "both patch kernels pad the offset table alike");
// a row of a trip's backprops in LDS: 64 k and 16 bytes of padding (rows 36 words apart: the
// 16-byte fragment reads of 8 consecutive rows cover all 32 banks)
constexpr int kP16RowBytes = kP16TripK * 2 + 16;
constexpr size_t p16_stage_bytes(int bm) { return static_cast<size_t>(2) * bm * kP16RowBytes; }

// RK as in the fp32 patch kernel: a half-wave's eight positions of a k-tile come as aligned runs
// of RK consecutive cells of the patch (8, 4, or 0 for no such structure).
template <int BM, int BN, typename TOUT, bool VEC, int RK>
__global__ __launch_bounds__(kThreads) void conv2d_gs_patch16_kernel(
    const bf16_t* __restrict__ x, const bf16_t* __restrict__ b, TOUT* __restrict__ gs,
    float* __restrict__ partials, ConvGeom g, int C, int O, int groups, float scale, int tiles_m,
    int tiles_n, PatchDims pd, int xvec, int a_off) {
  const int RS = pd.rs, CS = pd.cs;
  using Tile = mf32::Tile<BM, BN>;  // accumulator layout of a 32 x 32 MFMA tile: the same
  typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
  typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
  extern __shared__ __align__(16) unsigned char dyn_lds[];
  const int Qpad = (g.Q + kP16TripK - 1) / kP16TripK * kP16TripK;
  int* qtab = reinterpret_cast<int*>(dyn_lds);  // byte offsets into the patch
  uint16_t* xs = reinterpret_cast<uint16_t*>(qtab + Qpad);
  __shared__ float red[kWaves];

  const int Og = O / groups, Cg = C / groups;
  // a sample's tiles run on one XCD (if the host asks), so that its backprops are fetched into one L2 only
  const uint32_t unit = g.xcd_order ? xcd_contiguous_id(blockIdx.x, gridDim.x) : blockIdx.x;
  int64_t bid = unit;
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

  const bf16_t* xg = x + ((sample * C + static_cast<int64_t>(grp) * Cg + c_lo) * g.H) * g.W;
  stage_patch<bf16_t, uint16_t>(xs, qtab, xg, g, pd, nch, xvec, Qpad, 2);
  const int wm0 = (wave >> 1) * Tile::WM, wn0 = (wave & 1) * Tile::WN;
  const int kk = lane >> 5, l32 = lane & 31;
  // byte address inside the patch of this lane's patch element (its columns of the tile)
  const unsigned char* xsb = reinterpret_cast<const unsigned char*>(xs);
  int base_p[Tile::TN];
#pragma unroll
  for (int j = 0; j < Tile::TN; ++j) {
    const int p = p0 + wn0 + j * 32 + l32;
    if (p < g.Pg) {
      const int c = p / KK, rem = p - c * KK;
      const int kh = rem / g.KW, kw = rem - kh * g.KW;
      base_p[j] = ((c - c_lo) * CS + kh * g.dh * RS + kw * g.dw) * 2;
    } else {
      base_p[j] = 0;  // result discarded below; any address inside the patch will do
    }
  }
  // The backprop operand goes through LDS. Read straight into MFMA layout every lane would
  // fetch 8 bytes of a different row, 64 cache lines per load instruction, and the address
  // path of the CU (a line per cycle), not the MFMAs, would set the kernel's time. Here four
  // threads share a row: a trip's 64 k of one row are one 128-byte line, requested two trips
  // before they are used, written to LDS one trip before, and read back as 16-byte fragments.
  const bf16_t* bg = b + (sample * O + static_cast<int64_t>(grp) * Og) * g.Q;
  const __amdgpu_buffer_rsrc_t brs = __builtin_amdgcn_make_buffer_rsrc(
      const_cast<bf16_t*>(bg), 0, Og * g.Q * static_cast<int>(sizeof(bf16_t)), 0x00020000);
  constexpr uint32_t kOutside = 0x7fffffffu;
  constexpr int kRowPasses = BM / 64;  // 256 threads cover 64 rows at a time
  const int srow = threadIdx.x >> 2, sseg = threadIdx.x & 3;  // staging: row of the pass, 16 k of the trip
  uint32_t stage_b[kRowPasses];  // byte offset of (row, k = 16 sseg), or past the end for a row outside
#pragma unroll
  for (int r = 0; r < kRowPasses; ++r) {
    const int m = m0 + r * 64 + srow;
    stage_b[r] = m < Og ? static_cast<uint32_t>(m * g.Q + sseg * 16) * 2u : kOutside;
  }
  const int ntrips = Qpad / kP16TripK;
  const int nfull = g.Q / kP16TripK;  // trips whose every k is a real position
  unsigned char* As = dyn_lds + a_off;  // [2][BM][kP16RowBytes]

  uint32_t ga[2][kRowPasses][8];  // a trip's share of this thread, as loaded
  uint32_t bv[2][kP16Tiles][Tile::TN][4];
  constexpr int RUN = RK ? RK : 1;  // positions per table entry
  constexpr int NQ = 8 / RUN;       // table entries a half-wave needs per k-tile
  int qo[kP16Tiles][NQ];
  auto load_q = [&](int trip) {
    trip = trip < ntrips ? trip : ntrips - 1;
#pragma unroll
    for (int t = 0; t < kP16Tiles; ++t) {
      const int* q8 = qtab + (trip * kP16Tiles + t) * kP16BK + kk * 8;
      if constexpr (RK != 0) {
#pragma unroll
        for (int r = 0; r < NQ; ++r) qo[t][r] = q8[r * RUN];
      } else {
        const int4 lo = reinterpret_cast<const int4*>(q8)[0], hi = reinterpret_cast<const int4*>(q8)[1];
        qo[t][0] = lo.x; qo[t][1] = lo.y; qo[t][2] = lo.z; qo[t][3] = lo.w;
        qo[t][4] = hi.x; qo[t][5] = hi.y; qo[t][6] = hi.z; qo[t][7] = hi.w;
      }
    }
  };
  typedef uint16_t u16x2 __attribute__((ext_vector_type(2)));
  auto load_b = [&](uint32_t (&bb)[kP16Tiles][Tile::TN][4]) {
#pragma unroll
    for (int t = 0; t < kP16Tiles; ++t)
#pragma unroll
      for (int j = 0; j < Tile::TN; ++j) {
        if constexpr (RK != 0) {
          // RK consecutive 2-byte cells from a 2-byte aligned address: the aligned words around
          // them, shifted into place per lane (a wide read at 2-byte alignment, which the
          // compiler would make of the 2-byte reads, is several times slower on this device)
#pragma unroll
          for (int r = 0; r < NQ; ++r) {
            const uint32_t at = static_cast<uint32_t>(base_p[j] + qo[t][r]);
            const uint32_t* w = reinterpret_cast<const uint32_t*>(xsb + (at & ~3u));
            const uint32_t shift = at & 2u;  // bytes
            uint32_t word[RUN / 2 + 1];
#pragma unroll
            for (int e = 0; e <= RUN / 2; ++e) word[e] = w[e];
#pragma unroll
            for (int e = 0; e < RUN / 2; ++e)
              bb[t][j][r * (RUN / 2) + e] = __builtin_amdgcn_alignbyte(word[e + 1], word[e], shift);
          }
        } else {
#pragma unroll
          for (int e = 0; e < 4; ++e) {
            u16x2 pr;
            pr.x = *reinterpret_cast<const uint16_t*>(xsb + base_p[j] + qo[t][2 * e]);
            pr.y = *reinterpret_cast<const uint16_t*>(xsb + base_p[j] + qo[t][2 * e + 1]);
            bb[t][j][e] = __builtin_bit_cast(uint32_t, pr);
          }
        }
      }
  };
  // global -> registers: 16 k (32 bytes) of each of this thread's rows
  auto load_a = [&](int trip, uint32_t (&aa)[kRowPasses][8]) {
    trip = trip < ntrips ? trip : ntrips - 1;
    const bool tail = trip >= nfull;  // uniform
    const int k0 = trip * kP16TripK + sseg * 16;  // this thread's first k
#pragma unroll
    for (int r = 0; r < kRowPasses; ++r) {
      if (VEC) {
#pragma unroll
        for (int h = 0; h < 4; ++h) {
          uint32_t off = stage_b[r] + static_cast<uint32_t>(trip * kP16TripK + 4 * h) * 2u;
          if (tail && k0 + 4 * h >= g.Q) off = kOutside;
          typedef int vi2 __attribute__((ext_vector_type(2)));
          const vi2 v = __builtin_amdgcn_raw_buffer_load_b64(brs, off, 0, 0);
          aa[r][2 * h + 0] = static_cast<uint32_t>(v.x);
          aa[r][2 * h + 1] = static_cast<uint32_t>(v.y);
        }
      } else {
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          uint32_t o0 = stage_b[r] + static_cast<uint32_t>(trip * kP16TripK + 2 * e) * 2u, o1 = o0 + 2u;
          if (k0 + 2 * e >= g.Q) o0 = kOutside;
          if (k0 + 2 * e + 1 >= g.Q) o1 = kOutside;
          const uint32_t lo = static_cast<uint16_t>(__builtin_amdgcn_raw_buffer_load_b16(brs, o0, 0, 0));
          const uint32_t hi = static_cast<uint16_t>(__builtin_amdgcn_raw_buffer_load_b16(brs, o1, 0, 0));
          aa[r][e] = lo | (hi << 16);
        }
      }
    }
  };
  // registers -> LDS buffer buf
  auto store_a = [&](int buf, const uint32_t (&aa)[kRowPasses][8]) {
#pragma unroll
    for (int r = 0; r < kRowPasses; ++r) {
      uint4* dst = reinterpret_cast<uint4*>(As + (static_cast<size_t>(buf) * BM + r * 64 + srow) * kP16RowBytes + sseg * 32);
      dst[0] = make_uint4(aa[r][0], aa[r][1], aa[r][2], aa[r][3]);
      dst[1] = make_uint4(aa[r][4], aa[r][5], aa[r][6], aa[r][7]);
    }
  };
  Tile tile;
  tile.clear();
  load_a(0, ga[0]);
  load_a(1, ga[1]);
  store_a(0, ga[0]);
  load_a(2, ga[0]);
  __syncthreads();  // publishes the patch, the table and the first trip's backprops
  load_q(0);
  load_b(bv[0]);
  load_q(1);
  auto trip_body = [&](auto cur_c, int trip) {
    constexpr int cur = decltype(cur_c)::value, nxt = cur ^ 1;
    load_b(bv[nxt]);   // uses the offsets of trip + 1
    load_q(trip + 2);  // and frees them for trip + 2
    uint4 av[kP16Tiles][Tile::TM];
#pragma unroll
    for (int t = 0; t < kP16Tiles; ++t)
#pragma unroll
      for (int i = 0; i < Tile::TM; ++i)
        av[t][i] = *reinterpret_cast<const uint4*>(
            As + (static_cast<size_t>(cur) * BM + wm0 + i * 32 + l32) * kP16RowBytes + t * 32 + kk * 16);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int t = 0; t < kP16Tiles; ++t)
#pragma unroll
      for (int i = 0; i < Tile::TM; ++i)
#pragma unroll
        for (int j = 0; j < Tile::TN; ++j) {
          const u32x4 ar = {av[t][i].x, av[t][i].y, av[t][i].z, av[t][i].w};
          const u32x4 br = {bv[cur][t][j][0], bv[cur][t][j][1], bv[cur][t][j][2], bv[cur][t][j][3]};
          tile.acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
              __builtin_bit_cast(bf16x8, ar), __builtin_bit_cast(bf16x8, br), tile.acc[i][j], 0, 0, 0);
        }
    // trip + 1's backprops (asked for two trips ago) move to the other buffer, whose last
    // readers passed the barrier that ended the previous trip; trip + 3 takes their registers
    store_a(nxt, ga[nxt]);
    load_a(trip + 3, ga[nxt]);
    __syncthreads();
  };
  for (int trip = 0; trip < ntrips; trip += 2) {
    trip_body(std::integral_constant<int, 0>(), trip);
    if (trip + 1 < ntrips) trip_body(std::integral_constant<int, 1>(), trip + 1);
  }
  TOUT* out = gs + (sample * O + static_cast<int64_t>(grp) * Og) * g.Pg;
  float ss = 0.f;
  tile.for_each([&](int r, int c, float v) {
    const int m = m0 + r, p = p0 + c;
    if (m < Og && p < g.Pg) {
      const float val = v * scale;
      if (gs) dpk_io<TOUT>::store(out + static_cast<int64_t>(m) * g.Pg + p, val);
      ss = fmaf(val, val, ss);
    }
  });
  if (partials) {
    const float s = block_sum<kWaves>(ss, red);
    if (threadIdx.x == 0) partials[unit] = s;
  }
}


// Most LDS the patch kernel asks for. Above 64 KB a kernel must be told so once
// (hipFuncSetAttribute); one block then has a CU's LDS nearly to itself, which still beats
// gathering the operand from global memory (64 -> 64 channels, 3 x 3 on 56 x 56 images, whose
// patch is 107 KB: 228 us against 371 us).
constexpr size_t kPatchLdsLimit = 150 * 1024;  // of the CU's 160 KB

// Layout and LDS bytes of the patch kernels for a 64 x 64 tile; bytes == 0 if the geometry does
// not fit. At one position of the k loop the 32 lanes of a half-wave read the patch cells of
// 32 consecutive columns p = (c, kh, kw), at c * cs + kh * dh * rs + kw * dw: with rs = Wp and
// cs = Hp * Wp those land in a handful of the 32 banks (3 x 3 on a 34-wide patch: three and
// four to a bank). A few cells of padding per row and channel, searched here, spread them out.
struct PatchLayout {
  PatchDims d;
  size_t bytes;
  int a_off;  // bf16 kernel: where the staged backprops start
};
PatchLayout search_patch_layout(const ConvGeom& g, int Cg, int Hp, int Wp, size_t elsize, size_t a_bytes);

// The search costs tens of microseconds, a model calls with the same few geometries step
// after step: the last results are kept.
PatchLayout patch_layout(const ConvGeom& g, int Cg, int Hp, int Wp, size_t elsize, size_t a_bytes) {
  struct Entry {
    int key[10];
    PatchLayout value;
  };
  static std::mutex mu;
  static Entry cache[32];
  static int used = 0, next = 0;
  const int key[10] = {g.KH, g.KW, g.dh, g.dw, g.Q, Cg, Hp, Wp, static_cast<int>(elsize), static_cast<int>(a_bytes)};
  {
    std::lock_guard<std::mutex> lock(mu);
    for (int i = 0; i < used; ++i)
      if (std::memcmp(cache[i].key, key, sizeof(key)) == 0) return cache[i].value;
  }
  const PatchLayout v = search_patch_layout(g, Cg, Hp, Wp, elsize, a_bytes);
  std::lock_guard<std::mutex> lock(mu);
  Entry& e = cache[next];
  std::memcpy(e.key, key, sizeof(key));
  e.value = v;
  next = (next + 1) % 32;
  if (used < 32) ++used;
  return v;
}

PatchLayout search_patch_layout(const ConvGeom& g, int Cg, int Hp, int Wp, size_t elsize, size_t a_bytes) {
  const int KK = g.KH * g.KW;
  int nch = (64 + KK - 2) / KK + 1;  // channels a run of 64 columns can touch
  if (nch > Cg) nch = Cg;
  const size_t q_bytes = static_cast<size_t>((g.Q + kPatchTrip - 1) / kPatchTrip * kPatchTrip) * sizeof(int);
  PatchLayout best;
  best.d = PatchDims{Hp, Wp, Wp, Hp * Wp};
  best.bytes = 0;
  best.a_off = 0;
  long best_cost = -1;
  for (int padr = 0; padr < 8; ++padr) {
    for (int padc = 0; padc < 32; ++padc) {
      const int rs = Wp + padr, cs = Hp * rs + padc;
      const size_t bytes = q_bytes + dpk_align_up(static_cast<size_t>(nch) * cs * elsize, 16) + a_bytes;
      if (bytes > kPatchLdsLimit) continue;
      // most distinct 4-byte words any bank serves, summed over the two half-tiles of columns
      long cost = 0;
      for (int p0 = 0; p0 < 64; p0 += 32) {
        long word_of[32][8];
        int served[32] = {0};
        for (int l = 0; l < 32; ++l) {
          const int p = p0 + l, c = p / KK, rem = p - c * KK, kh = rem / g.KW, kw = rem - kh * g.KW;
          if (c >= nch) continue;
          const long word = (static_cast<long>(c) * cs + kh * g.dh * rs + kw * g.dw) * static_cast<long>(elsize) / 4;
          const int bank = static_cast<int>(word % 32);
          bool seen = false;
          for (int k = 0; k < served[bank] && k < 8; ++k) seen = seen || word_of[bank][k] == word;
          if (!seen) {
            if (served[bank] < 8) word_of[bank][served[bank]] = word;
            ++served[bank];
          }
        }
        int worst = 0;
        for (int k = 0; k < 32; ++k) worst = served[k] > worst ? served[k] : worst;
        cost += worst;
      }
      // fewer conflicts first, then the smaller patch (more blocks per CU)
      if (best_cost < 0 || cost < best_cost || (cost == best_cost && bytes < best.bytes)) {
        best_cost = cost;
        best.d = PatchDims{Hp, Wp, rs, cs};
        best.bytes = bytes;
        best.a_off = static_cast<int>(bytes - a_bytes);
      }
    }
  }
  return best;
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

// One variant of the patch kernels (vector loads of the backprops or not, run length of
// consecutive cells). Above 64 KB of LDS the kernel must be told so: per device and cheap, so it is
// said again at every such launch rather than remembered; false if that is refused.
template <typename TIN, typename TOUT, bool V, int RK>
bool launch_patch(const Plan& p, dim3 grid, dim3 block, size_t patch_bytes, hipStream_t s, const TIN* xp,
                  const TIN* bp, TOUT* gp, float* partials, const ConvGeom& g, int C, int O, int groups,
                  float scale, PatchDims pd, int xvec, int a_off) {
  auto prepare = [&](const void* fn) {
    if (patch_bytes <= 64 * 1024 - 64) return true;
    if (hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, static_cast<int>(kPatchLdsLimit)) ==
        hipSuccess)
      return true;
    (void)hipGetLastError();  // the refusal is handled here, not reported by the next launch check
    return false;
  };
  if constexpr (std::is_same<TIN, bf16_t>::value) {
    if (p.bm == 128) {
      if (!prepare(reinterpret_cast<const void*>(&conv2d_gs_patch16_kernel<128, 64, TOUT, V, RK>))) return false;
      hipLaunchKernelGGL((conv2d_gs_patch16_kernel<128, 64, TOUT, V, RK>), grid, block, patch_bytes, s, xp, bp, gp,
                         partials, g, C, O, groups, scale, p.tiles_m, p.tiles_n, pd, xvec, a_off);
    } else {
      if (!prepare(reinterpret_cast<const void*>(&conv2d_gs_patch16_kernel<64, 64, TOUT, V, RK>))) return false;
      hipLaunchKernelGGL((conv2d_gs_patch16_kernel<64, 64, TOUT, V, RK>), grid, block, patch_bytes, s, xp, bp, gp,
                         partials, g, C, O, groups, scale, p.tiles_m, p.tiles_n, pd, xvec, a_off);
    }
  } else {
    if (!prepare(reinterpret_cast<const void*>(&conv2d_gs_patch_kernel<64, 64, TIN, TOUT, V, RK>))) return false;
    hipLaunchKernelGGL((conv2d_gs_patch_kernel<64, 64, TIN, TOUT, V, RK>), grid, block, patch_bytes, s, xp, bp, gp,
                       partials, g, C, O, groups, scale, p.tiles_m, p.tiles_n, pd, xvec, 0);
  }
  return true;
}

// (the plan comes back as the kernel that ran used it: a refused patch launch falls back to 64 x 64 tiles)
template <typename TIN, typename TOUT>
void launch(Plan& p, bool vec, const void* x, const void* b, void* gs, float* partials,
            const ConvGeom& g, int64_t n, int C, int O, int groups, float scale, hipStream_t s,
            size_t patch_bytes, PatchDims pd, int a_off, int ksplit, int kchunk, float* split_out) {
  dim3 grid(static_cast<unsigned>(n * groups * p.tiles_m * p.tiles_n * ksplit)), block(kThreads);
  const TIN* xp = static_cast<const TIN*>(x);
  const TIN* bp = static_cast<const TIN*>(b);
  TOUT* gp = static_cast<TOUT*>(gs);
  if (patch_bytes > 0) {
    // aligned runs of this many positions lie in one output row at unit stride
    const int run = g.sw != 1 ? 0 : g.OW % 8 == 0 ? 8 : g.OW % 4 == 0 ? 4 : 0;
    // image rows made of whole, aligned 4-element chunks: the patch interior is staged with vector loads
    const int xvec = (g.W % 4 == 0 && dpk_aligned(x, sizeof(TIN) == 2 ? 8 : 16)) ? 1 : 0;
    bool done;
#define DPK_PATCH(V, RK)                                                                                  \
  done = launch_patch<TIN, TOUT, V, RK>(p, grid, block, patch_bytes, s, xp, bp, gp, partials, g, C, O, groups, \
                                        scale, pd, xvec, a_off)
    if (vec && run == 8) DPK_PATCH(true, 8);
    else if (vec && run == 4) DPK_PATCH(true, 4);
    else if (vec) DPK_PATCH(true, 0);
    else DPK_PATCH(false, 0);
#undef DPK_PATCH
    if (done) return;
    // refused (more LDS than the device or runtime grants): the gather kernel on 64 x 64 tiles
    p.bm = p.bn = 64;
    p.tiles_m = static_cast<int>(dpk_cdiv(O / groups, 64));
    p.tiles_n = static_cast<int>(dpk_cdiv(g.Pg, 64));
    grid = dim3(static_cast<unsigned>(n * groups * p.tiles_m * p.tiles_n * ksplit));
  }
#define DPK_CONV_LAUNCH(BM, BN, V, D3)                                                            \
  hipLaunchKernelGGL((conv2d_gs_kernel<BM, BN, TIN, TOUT, V, D3>), grid, block, 0, s, xp, bp, gp, \
                     partials, g, C, O, groups, scale, p.tiles_m, p.tiles_n, ksplit, kchunk, split_out, n)
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

namespace {
// Pieces the contraction over Q output positions is cut into: only for the gather kernel's
// plan, when its blocks would leave most of the device idle and every piece keeps at least
// kSplitMinK positions.
constexpr int kSplitMax = 8, kSplitMinK = 512;
int split_pieces(int64_t blocks, int64_t Q, int cus) {
  if (cus <= 0 || blocks >= 2 * cus || Q < 2 * kSplitMinK) return 1;
  int64_t s = dpk_cdiv(4 * static_cast<int64_t>(cus), blocks);
  if (s > kSplitMax) s = kSplitMax;
  if (s > Q / kSplitMinK) s = Q / kSplitMinK;
  return s < 2 ? 1 : static_cast<int>(s);
}
struct ConvWs {
  size_t partials_bytes, total;  // block sums of squares first, then the pieces' raw tiles
};
ConvWs conv_ws(int64_t n, int64_t Og, int64_t Pg, int64_t groups, int64_t O, int pieces_max) {
  const Plan p = make_plan(Og, Pg, true);
  int64_t slots = n * groups * p.tiles_m * p.tiles_n;
  const int64_t chunks = n * dpk_cdiv(O * Pg, kSplitChunk);
  if (pieces_max > 1 && chunks > slots) slots = chunks;
  ConvWs w;
  w.partials_bytes = dpk_align_up(static_cast<size_t>(slots) * sizeof(float), 256);
  w.total = w.partials_bytes;
  if (pieces_max > 1) w.total += dpk_align_up(static_cast<size_t>(pieces_max) * n * O * Pg * sizeof(float), 256);
  return w;
}
}  // namespace

extern "C" size_t dpk_conv2d_gs_workspace_bytes(int64_t n, int64_t C, int64_t O, int64_t KH,
                                                int64_t KW, int64_t groups, int64_t Q) {
  if (n <= 0 || C <= 0 || O <= 0 || KH <= 0 || KW <= 0 || groups <= 0) return 0;
  if (C % groups != 0 || O % groups != 0) return 0;
  const int64_t Og = O / groups, Pg = (C / groups) * KH * KW;
  // the pieces of a split contraction (decided at call time from the device's size) need room
  // for their raw tiles; Q <= 0: the caller does not want the split
  // (the current device's CU count, as the call will use it: ask on the device the call is made on)
  const Plan p = make_plan(Og, Pg, false);
  int cus = dpk_device_cus();
  if (cus <= 0) cus = 256;
  const int pieces = Q > 0 ? split_pieces(n * groups * p.tiles_m * p.tiles_n, Q, cus) : 1;
  return conv_ws(n, Og, Pg, groups, O, pieces > 1 ? kSplitMax : 1).total;
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
  DPK_REQUIRE(x && b && (gs || sumsq), DPK_E_ARG, "%s: NULL tensor", who);
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
  // worth it when the tiles of a sample re-read enough input (measured: fetches of the C4 layer
  // 614 -> 135 MB, its kernel 4 % faster, a 7 x 7 / 2 stem 508 -> 393 us); with a few dozen output
  // positions per sample the kernel is a stream of stores, which ran 25 % slower in this order
  g.xcd_order = Q >= 256 ? 1 : 0;
  const int64_t Hp = H + ph_lo + ph_hi, Wp = W + pw_lo + pw_hi;
  const bool flat = z.D == 1 && z.KD == 1 && z.pd_lo == 0 && z.pd_hi == 0;  // the LDS patch is two-dimensional
  PatchLayout pl;
  pl.d = PatchDims{(int)Hp, (int)Wp, (int)Wp, (int)(Hp * Wp)};
  pl.bytes = 0;
  pl.a_off = 0;
  int bm16 = 64;
  if (flat && Hp * Wp < (1 << 20) && (O / groups) * Q * 4 < (1LL << 30)) {
    // bf16 input: 128 output channels per block where the layer has them (each gathered
    // fragment then feeds two MFMAs), if the staged backprops of 128 rows still fit
    if (in_dtype == DPK_BF16 && O / groups >= 128) {
      pl = patch_layout(g, (int)(C / groups), (int)Hp, (int)Wp, 2, p16_stage_bytes(128));
      bm16 = pl.bytes > 0 ? 128 : 64;
    }
    if (pl.bytes == 0)
      pl = patch_layout(g, (int)(C / groups), (int)Hp, (int)Wp, in_dtype == DPK_BF16 ? 2 : 4,
                        in_dtype == DPK_BF16 ? p16_stage_bytes(64) : 0);
  }
  const size_t patch_bytes = pl.bytes;
  Plan p = make_plan(O / groups, Pg, patch_bytes > 0);
  if (patch_bytes > 0 && bm16 == 128) {
    p.bm = 128;
    p.tiles_m = static_cast<int>(dpk_cdiv(O / groups, 128));
  }
  const int64_t blocks = n * groups * p.tiles_m * p.tiles_n;
  // few long blocks on the gather kernel: cut the contraction over the positions into pieces,
  // if the caller's workspace has room for their raw tiles
  int cus = dpk_device_cus();
  if (cus <= 0) cus = 256;
  int ksplit = patch_bytes > 0 ? 1 : split_pieces(blocks, Q, cus);
  ConvWs wl = conv_ws(n, O / groups, Pg, groups, O, ksplit);
  if (ksplit > 1 && !(ws && ws_bytes >= wl.total && dpk_aligned(ws, 256))) {
    ksplit = 1;  // no room for the pieces: one piece, and the (smaller) layout that goes with it
    wl = conv_ws(n, O / groups, Pg, groups, O, 1);
  }
  const int kchunk = ksplit > 1 ? static_cast<int>(dpk_cdiv(dpk_cdiv(Q, ksplit), mf32::BK) * mf32::BK) : static_cast<int>(Q);
  DPK_REQUIRE(blocks * ksplit <= DPK_MAX_GRID_X, DPK_E_SHAPE, "%s: %lld blocks exceed the grid limit", who,
              (long long)(blocks * ksplit));
  float* partials = nullptr;
  float* split_out = nullptr;
  if (sumsq) {
    // room for the plan with the most blocks: a refused patch launch falls back to it
    const size_t need = ksplit > 1 ? wl.total : wl.partials_bytes;
    DPK_REQUIRE(ws && ws_bytes >= need, DPK_E_WORKSPACE, "%s: workspace %zu < %zu bytes", who,
                ws_bytes, need);
    DPK_REQUIRE(dpk_aligned(ws, 4), DPK_E_ALIGN, "%s: workspace misaligned", who);
    partials = static_cast<float*>(ws);
  }
  if (ksplit > 1) split_out = reinterpret_cast<float*>(static_cast<char*>(ws) + wl.partials_bytes);
  // 16-byte (8-byte for bf16) loads of 4 backprops
  const bool vec = Q % 4 == 0 && dpk_aligned(b, in_dtype == DPK_BF16 ? 8 : 16);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (in_dtype == DPK_F32 && gs_dtype == DPK_F32)
    launch<float, float>(p, vec, x, b, gs, partials, g, n, (int)C, (int)O, (int)groups, scale, s, patch_bytes,
                       pl.d, pl.a_off, ksplit, kchunk, split_out);
  else if (in_dtype == DPK_BF16 && gs_dtype == DPK_BF16)
    launch<bf16_t, bf16_t>(p, vec, x, b, gs, partials, g, n, (int)C, (int)O, (int)groups, scale, s, patch_bytes,
                         pl.d, pl.a_off, ksplit, kchunk, split_out);
  else if (in_dtype == DPK_BF16 && gs_dtype == DPK_F32)
    launch<bf16_t, float>(p, vec, x, b, gs, partials, g, n, (int)C, (int)O, (int)groups, scale, s, patch_bytes,
                        pl.d, pl.a_off, ksplit, kchunk, split_out);
  else
    launch<float, bf16_t>(p, vec, x, b, gs, partials, g, n, (int)C, (int)O, (int)groups, scale, s, patch_bytes,
                        pl.d, pl.a_off, ksplit, kchunk, split_out);
  DPK_LAUNCH_CHECK(who);
  int64_t cols = static_cast<int64_t>(groups) * p.tiles_m * p.tiles_n;
  if (ksplit > 1) {
    // add the pieces, scale, store (unless only the norms are wanted) and square
    const int64_t OP = O * Pg;
    const int chunks = static_cast<int>(dpk_cdiv(OP, kSplitChunk));
    const dim3 grid(static_cast<unsigned>(n * chunks)), block(kThreads);
    if (gs_dtype == DPK_F32)
      hipLaunchKernelGGL(conv_split_reduce_kernel<float>, grid, block, 0, s, split_out, static_cast<float*>(gs), partials,
                         n, OP, ksplit, chunks, scale);
    else
      hipLaunchKernelGGL(conv_split_reduce_kernel<bf16_t>, grid, block, 0, s, split_out, static_cast<bf16_t*>(gs),
                         partials, n, OP, ksplit, chunks, scale);
    DPK_LAUNCH_CHECK(who);
    cols = chunks;
  }
  if (sumsq) {
    dpk_launch_reduce_rows(partials, n, cols, sumsq, 0, 1.f, s);
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
                                                int64_t KW, int64_t groups, int64_t Q) {
  if (KD <= 0) return 0;
  return dpk_conv2d_gs_workspace_bytes(n, C, O, KD * KH, KW, groups, Q);
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
