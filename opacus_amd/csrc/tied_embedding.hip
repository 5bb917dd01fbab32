// Ghost clipping for an embedding table tied to the output projection: the cross term.
//
// With weight W shared by nn.Embedding (ids -> rows of W) and nn.Linear (a -> a W^T), a
// sample's gradient is G = G_emb + G_head and
//   |G|^2 = |G_emb|^2 + |G_head|^2 + 2 <G_emb, G_head>.
// The first two are the ghost norms of the two layers. The reference stops here: it refuses
// tied parameters under ghost clipping
// (opacus/grad_sample/grad_sample_module_fast_gradient_clipping.py:172-179). The third is
//   <G_emb, G_head> = sum_t < e_t , G_head[ids_t, :] >
//                   = sum_t < e_t , sum_t' g[t', ids_t] a_t' >
// with e_t the backprops of the embedding output, a_t' the inputs of the head and g the
// backprops of its output: only the <= T rows of G_head that the sample's ids name are
// needed. Regrouped, cross = sum_{t', t} g[t', ids_t] (a_t' . e_t): a tile of the T' x T product
// a e^T (both operands contiguous along D, the layout of the ghost norm's Gram kernel) is
// formed in MFMA accumulators and multiplied, element by element, by the entries of g the
// ids name, read straight from g; neither the gathered matrix nor the product is stored.
// Shapes that kernel does not take go through three steps instead:
//   1. N[t', t] = g[t', ids_t]                       (gather, this file)
//   2. R[t, :]  = sum_t' N[t', t] a_t'               (the per-sample Linear contraction)
//   3. cross    = sum_{t,d} e[t,d] R[t,d]            (row dot product, this file)
#include "dpk_common.h"
#include "mfma_bf16_dlds.h"

namespace {

constexpr int kThreads = 256;
constexpr int kWaves = kThreads / DPK_WAVE;
constexpr int64_t kDotChunk = 8192;  // elements of one row per block of the dot kernel

// out[(s * T2 + t2) * T + t] = g[(s * T2 + t2) * V + ids[s * T + t]], zero for an id
// outside [0, V). grid = (T2, n); a block walks the T ids of its sample: contiguous
// writes, reads scattered inside one row of g.
template <typename TG>
__global__ __launch_bounds__(kThreads) void gather_columns_kernel(const TG* __restrict__ g,
                                                                   const int64_t* __restrict__ ids,
                                                                   TG* __restrict__ out, int64_t T,
                                                                   int64_t T2, int64_t V) {
  const int64_t s = blockIdx.y, t2 = blockIdx.x;
  const TG* row = g + (s * T2 + t2) * V;
  const int64_t* id = ids + s * T;
  TG* o = out + (s * T2 + t2) * T;
  for (int64_t t = threadIdx.x; t < T; t += kThreads) {
    const int64_t v = id[t];
    o[t] = (v >= 0 && v < V) ? row[v] : static_cast<TG>(0);
  }
}

// partial[s * chunks + c] = sum over chunk c of row s of x * y
template <typename TX>
__global__ __launch_bounds__(kThreads) void dot_partial_kernel(const TX* __restrict__ x,
                                                                const float* __restrict__ y, int64_t P,
                                                                float* __restrict__ partial) {
  __shared__ float red[kWaves];
  const int64_t s = blockIdx.y, c = blockIdx.x;
  const int64_t lo = c * kDotChunk;
  const int64_t hi = lo + kDotChunk < P ? lo + kDotChunk : P;
  const TX* xr = x + s * P;
  const float* yr = y + s * P;
  float a0 = 0.f, a1 = 0.f;
  int64_t i = lo + threadIdx.x;
  for (; i + kThreads < hi; i += 2 * kThreads) {
    a0 = fmaf(dpk_io<TX>::load(xr + i), yr[i], a0);
    a1 = fmaf(dpk_io<TX>::load(xr + i + kThreads), yr[i + kThreads], a1);
  }
  if (i < hi) a0 = fmaf(dpk_io<TX>::load(xr + i), yr[i], a0);
  const float v = block_sum<kWaves>(a0 + a1, red);
  if (threadIdx.x == 0) partial[s * gridDim.x + c] = v;
}

// one wave per sample: cross[s] = scale * sum_c partial[s, c], in a fixed order
__global__ __launch_bounds__(kThreads) void dot_final_kernel(const float* __restrict__ partial,
                                                              int64_t n, int64_t chunks, float scale,
                                                              float* __restrict__ cross) {
  const int64_t s = (static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x) / DPK_WAVE;
  const int lane = threadIdx.x & (DPK_WAVE - 1);
  if (s >= n) return;
  float v = 0.f;
  for (int64_t c = lane; c < chunks; c += DPK_WAVE) v += partial[s * chunks + c];
  v = wave_sum(v);
  if (lane == 0) cross[s] = scale * v;
}

// One 128 x 128 tile (rows: head positions t', columns: embedding positions t) of one sample.
// partial[unit] = sum over the tile of g[t', ids_t] * (a_t' . e_t).
using CrossCfg = mb16d::Config<2, 2, 2, 64>;

template <typename TE>
__global__ __launch_bounds__(CrossCfg::kThreads) void tied_cross_tile_kernel(
    const int64_t* __restrict__ ids, const TE* __restrict__ e, const TE* __restrict__ a, const TE* __restrict__ g,
    float* __restrict__ partial, int64_t T, int64_t T2, int64_t D, int64_t V, int tiles_t, int tiles_t2,
    uint32_t nunits) {
  using C = CrossCfg;
  __shared__ mb16d::Smem<C> sm;
  __shared__ float red[C::kWaves];
  __shared__ int64_t s_ids[C::BN];
  const uint32_t unit = xcd_contiguous_id(blockIdx.x, nunits);
  const uint32_t per_sample = static_cast<uint32_t>(tiles_t) * tiles_t2;
  const int64_t sample = unit / per_sample;
  const uint32_t rest = unit % per_sample;
  const int64_t r0 = static_cast<int64_t>(rest / tiles_t) * C::BM;  // first head position t'
  const int64_t c0 = static_cast<int64_t>(rest % tiles_t) * C::BN;  // first embedding position t
  const int wave = threadIdx.x >> 6, lane = threadIdx.x & 63;
  const int kh = lane >> 5, l32 = lane & 31;
  const int wm0 = (wave / C::kWaveCols) * 64, wn0 = (wave % C::kWaveCols) * 64;
  if (threadIdx.x < C::BN) {
    const int64_t t = c0 + threadIdx.x;
    const int64_t id = t < T ? ids[sample * T + t] : -1;
    s_ids[threadIdx.x] = (id >= 0 && id < V) ? id : -1;  // outside the table: contributes nothing
  }
  __syncthreads();
  // The 64 entries of g this lane's part of the tile meets are requested before the main loop
  // and used after it: scattered two-byte reads, whose latency the contraction covers.
  const TE* gs = g + sample * T2 * V;
  TE gv[2][2][16];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int64_t id = s_ids[wn0 + j * 32 + l32];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int v = 0; v < 16; ++v) {
        const int64_t row = r0 + wm0 + i * 32 + (v >> 2) * 8 + kh * 4 + (v & 3);
        gv[i][j][v] = (id >= 0 && row < T2) ? gs[row * V + id] : static_cast<TE>(0);
      }
  }
  mb16d::Tile tile;
  tile.clear();
  mb16d::mainloop<C, TE>(tile, sm, a + sample * T2 * D, e + sample * T * D, D, r0, c0, T2, T, D, wm0, wn0);
  float sum = 0.f;
#pragma unroll
  for (int j = 0; j < 2; ++j)
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int v = 0; v < 16; ++v) sum = fmaf(dpk_io<TE>::load(&gv[i][j][v]), tile.acc[i][j][v], sum);
  const float t = block_sum<C::kWaves>(sum, red);
  if (threadIdx.x == 0) partial[unit] = t;
}

struct CrossLayout {
  size_t gathered, product, partial, linear, total;
};

CrossLayout cross_layout(int64_t n, int64_t T, int64_t T2, int64_t D, int head_dtype) {
  CrossLayout l;
  l.gathered = 0;
  l.product = dpk_align_up(static_cast<size_t>(n) * T2 * T * dpk_elsize(head_dtype), 256);
  l.partial = l.product + dpk_align_up(static_cast<size_t>(n) * T * D * sizeof(float), 256);
  l.linear = l.partial + dpk_align_up(static_cast<size_t>(n) * dpk_cdiv(T * D, kDotChunk) * sizeof(float), 256);
  l.total = l.linear + dpk_align_up(dpk_linear_gs_workspace_bytes(n, T2, T, D), 256);
  return l;
}

}  // namespace

extern "C" size_t dpk_tied_embedding_cross_workspace_bytes(int64_t n, int64_t T, int64_t T2, int64_t D,
                                                           int head_dtype) {
  if (n <= 0 || T <= 0 || T2 <= 0 || D <= 0) return 0;
  return cross_layout(n, T, T2, D, head_dtype).total;
}

extern "C" int dpk_tied_embedding_cross(const int64_t* ids, const void* e, int emb_dtype, const void* a,
                                        const void* g, int head_dtype, float* cross, int64_t n, int64_t T,
                                        int64_t T2, int64_t D, int64_t V, float scale, void* ws,
                                        size_t ws_bytes, dpk_stream_t stream) {
  const char* who = "dpk_tied_embedding_cross";
  DPK_REQUIRE(n >= 0 && T >= 1 && T2 >= 1 && D >= 1 && V >= 1, DPK_E_SHAPE,
              "%s: n=%lld T=%lld T2=%lld D=%lld V=%lld", who, (long long)n, (long long)T, (long long)T2,
              (long long)D, (long long)V);
  if (n == 0) return DPK_OK;
  DPK_REQUIRE(ids && e && a && g && cross, DPK_E_ARG, "%s: NULL argument", who);
  DPK_REQUIRE(dpk_dtype_ok(emb_dtype) && dpk_dtype_ok(head_dtype), DPK_E_DTYPE, "%s: dtypes %d,%d", who,
              emb_dtype, head_dtype);
  DPK_REQUIRE(dpk_aligned(ids, 8) && dpk_aligned(e, dpk_elsize(emb_dtype)) &&
                  dpk_aligned(a, dpk_elsize(head_dtype)) && dpk_aligned(g, dpk_elsize(head_dtype)) &&
                  dpk_aligned(cross, 4),
              DPK_E_ALIGN, "%s: misaligned argument", who);
  DPK_REQUIRE(T2 <= DPK_MAX_GRID_X && n <= DPK_MAX_GRID_YZ, DPK_E_SHAPE, "%s: grid limit (T2=%lld, n=%lld)", who,
              (long long)T2, (long long)n);
  const CrossLayout l = cross_layout(n, T, T2, D, head_dtype);
  DPK_REQUIRE(ws && ws_bytes >= l.total, DPK_E_WORKSPACE, "%s: workspace %zu < %zu bytes", who, ws_bytes, l.total);
  DPK_REQUIRE(dpk_aligned(ws, 256), DPK_E_ALIGN, "%s: workspace must be 256-byte aligned", who);
  char* base = static_cast<char*>(ws);
  {
    // the tile kernel: one element type, whole 128-byte stage rows, 32-bit offsets inside a sample
    const int64_t es = dpk_elsize(head_dtype), widest = T > T2 ? T : T2;
    const int64_t tiles_t = dpk_cdiv(T, CrossCfg::BN), tiles_t2 = dpk_cdiv(T2, CrossCfg::BM);
    const int64_t units = n * tiles_t * tiles_t2;
    if (emb_dtype == head_dtype && D % (128 / es) == 0 && dpk_aligned(e, 16) && dpk_aligned(a, 16) &&
        widest * D * es < (int64_t{1} << 32) && units <= DPK_MAX_GRID_X && units * 4 <= (int64_t)(l.total - l.partial)) {
      hipStream_t s = static_cast<hipStream_t>(stream);
      float* part = reinterpret_cast<float*>(base + l.partial);
      const dim3 grid(static_cast<unsigned>(units)), block(CrossCfg::kThreads);
      if (head_dtype == DPK_F32)
        hipLaunchKernelGGL(tied_cross_tile_kernel<float>, grid, block, 0, s, ids, static_cast<const float*>(e),
                           static_cast<const float*>(a), static_cast<const float*>(g), part, T, T2, D, V, (int)tiles_t,
                           (int)tiles_t2, static_cast<uint32_t>(units));
      else
        hipLaunchKernelGGL(tied_cross_tile_kernel<bf16_t>, grid, block, 0, s, ids, static_cast<const bf16_t*>(e),
                           static_cast<const bf16_t*>(a), static_cast<const bf16_t*>(g), part, T, T2, D, V, (int)tiles_t,
                           (int)tiles_t2, static_cast<uint32_t>(units));
      DPK_LAUNCH_CHECK(who);
      hipLaunchKernelGGL(dot_final_kernel, dim3(static_cast<unsigned>(dpk_cdiv(n * DPK_WAVE, kThreads))), dim3(kThreads),
                         0, s, part, n, tiles_t * tiles_t2, scale, cross);
      DPK_LAUNCH_CHECK(who);
      return DPK_OK;
    }
  }
  void* gathered = base + l.gathered;
  float* product = reinterpret_cast<float*>(base + l.product);
  float* partial = reinterpret_cast<float*>(base + l.partial);
  hipStream_t s = static_cast<hipStream_t>(stream);

  const dim3 ggrid(static_cast<unsigned>(T2), static_cast<unsigned>(n));
  if (head_dtype == DPK_F32)
    hipLaunchKernelGGL((gather_columns_kernel<float>), ggrid, dim3(kThreads), 0, s, static_cast<const float*>(g),
                       ids, static_cast<float*>(gathered), T, T2, V);
  else
    hipLaunchKernelGGL((gather_columns_kernel<bf16_t>), ggrid, dim3(kThreads), 0, s, static_cast<const bf16_t*>(g),
                       ids, static_cast<bf16_t*>(gathered), T, T2, V);
  DPK_LAUNCH_CHECK(who);

  // R[s, t, :] = sum_t2 N[s, t2, t] * a[s, t2, :]: the Linear per-sample contraction with
  // "out" = T and the sum over the T2 head positions
  const int rc = dpk_linear_gs(gathered, a, head_dtype, product, DPK_F32, nullptr, n, T2, T, D, 1.0f,
                               DPK_TILE_AUTO, base + l.linear, l.total - l.linear, stream);
  if (rc != DPK_OK) return rc;

  const int64_t P = T * D, chunks = dpk_cdiv(P, kDotChunk);
  DPK_REQUIRE(chunks <= DPK_MAX_GRID_X, DPK_E_SHAPE, "%s: T*D too large", who);
  const dim3 dgrid(static_cast<unsigned>(chunks), static_cast<unsigned>(n));
  if (emb_dtype == DPK_F32)
    hipLaunchKernelGGL((dot_partial_kernel<float>), dgrid, dim3(kThreads), 0, s, static_cast<const float*>(e),
                       product, P, partial);
  else
    hipLaunchKernelGGL((dot_partial_kernel<bf16_t>), dgrid, dim3(kThreads), 0, s, static_cast<const bf16_t*>(e),
                       product, P, partial);
  hipLaunchKernelGGL(dot_final_kernel, dim3(static_cast<unsigned>(dpk_cdiv(n * DPK_WAVE, kThreads))), dim3(kThreads),
                     0, s, partial, n, chunks, scale, cross);
  DPK_LAUNCH_CHECK(who);
  return DPK_OK;
}
