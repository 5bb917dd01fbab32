// DPOptimizer.add_noise + scale_grad (opacus/optimizers/optimizer.py:477-504)
// with _generate_noise (optimizer.py:104-169) folded in: one pass that reads
// summed_grad, draws Gaussian noise from a counter-based generator in registers,
// adds, divides and writes grad: 2 * P * elsize bytes of HBM traffic, against about a
// hundred ALU instructions per four elements for the generator.
//
// Generator: Philox4x32-10 (Salmon et al., SC'11), key = seed, counter =
// (group index lo, hi, offset lo, hi) where a group is 4 consecutive elements.
// The four 32-bit outputs make two Box-Muller pairs, i.e. the four normals of
// the group. The stream therefore depends only on (seed, offset, element
// index), never on the launch shape.
#include "dpk_common.h"
#include "philox_normal.h"

namespace {

constexpr int kThreads = 256;

using dpk_noise::noise4;

// A block covers kGroupsPerBlock consecutive 4-element groups of one tensor, thread t
// taking groups t, t + 256, ... so that a wave's accesses stay contiguous.
constexpr int kUnroll = 4;
constexpr int kGroupsPerBlock = kThreads * kUnroll;

struct NoiseArgs {
  const void* summed[DPK_MULTI_MAX];  // NULL: the tensor counts as zeros
  void* grad[DPK_MULTI_MAX];
  int64_t P[DPK_MULTI_MAX];
  int64_t gprefix[DPK_MULTI_MAX + 1];   // groups before tensor k: its base in the counter space
  uint32_t bprefix[DPK_MULTI_MAX + 1];  // blocks before tensor k
  int K;
};

// Tensor k's element i uses Philox group gprefix[k] + i / 4: the tensors draw from one
// stream laid end to end, whatever the launch shape. Blocks never straddle tensors.
template <typename TI, typename TO>
__global__ __launch_bounds__(kThreads) void add_noise_kernel(NoiseArgs a, float std, float denom,
                                                               uint64_t seed, uint64_t offset,
                                                               int draws) {
  // the tensor this block belongs to: last k with bprefix[k] <= blockIdx.x (uniform, scalar)
  int lo = 0, hi = a.K - 1;
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (a.bprefix[mid] <= blockIdx.x) lo = mid;
    else hi = mid - 1;
  }
  const int k = lo;
  const int64_t P = a.P[k];
  const TI* summed = static_cast<const TI*>(a.summed[k]);
  TO* grad = static_cast<TO*>(a.grad[k]);
  const uint64_t gbase = static_cast<uint64_t>(a.gprefix[k]);
  const bool aligned =
      ((reinterpret_cast<uintptr_t>(summed) | reinterpret_cast<uintptr_t>(grad)) & 15) == 0;
  const float inv = 1.0f / denom;
  const bool exact_div = std == 0.f;  // a pure rescale stays a correctly rounded division
  const int64_t g0 = static_cast<int64_t>(blockIdx.x - a.bprefix[k]) * kGroupsPerBlock + threadIdx.x;
#pragma unroll
  for (int u = 0; u < kUnroll; ++u) {
    const int64_t g = g0 + u * kThreads;
    const int64_t i = g * 4;
    if (i >= P) break;
    float4 z = make_float4(0.f, 0.f, 0.f, 0.f);
    if (std != 0.f) {
      z = noise4(gbase + static_cast<uint64_t>(g), seed, offset, draws);
      z.x *= std;
      z.y *= std;
      z.z *= std;
      z.w *= std;
    }
    if (aligned && i + 4 <= P) {
      float4 v = summed ? dpk_io<TI>::load4(summed + i) : make_float4(0.f, 0.f, 0.f, 0.f);
      if (exact_div) {
        v = make_float4(v.x / denom, v.y / denom, v.z / denom, v.w / denom);
      } else {
        v = make_float4((v.x + z.x) * inv, (v.y + z.y) * inv, (v.z + z.z) * inv, (v.w + z.w) * inv);
      }
      dpk_io<TO>::store4(grad + i, v);
    } else {
      const float zz[4] = {z.x, z.y, z.z, z.w};
      for (int e = 0; e < 4 && i + e < P; ++e) {
        const float v = summed ? dpk_io<TI>::load(summed + i + e) : 0.f;
        dpk_io<TO>::store(grad + i + e, exact_div ? v / denom : (v + zz[e]) * inv);
      }
    }
  }
}

int launch(const char* who, const NoiseArgs& a, unsigned blocks, int in_dtype, int out_dtype, float std,
           float denom, uint64_t seed, uint64_t offset, int draws, hipStream_t s) {
  const dim3 grid(blocks), block(kThreads);
#define DPK_NM(TI, TO) \
  hipLaunchKernelGGL((add_noise_kernel<TI, TO>), grid, block, 0, s, a, std, denom, seed, offset, draws)
  if (in_dtype == DPK_F32 && out_dtype == DPK_F32) DPK_NM(float, float);
  else if (in_dtype == DPK_F32 && out_dtype == DPK_BF16) DPK_NM(float, bf16_t);
  else if (in_dtype == DPK_BF16 && out_dtype == DPK_F32) DPK_NM(bf16_t, float);
  else DPK_NM(bf16_t, bf16_t);
#undef DPK_NM
  DPK_LAUNCH_CHECK(who);
  return DPK_OK;
}

// Fills slot k; returns false when the block count would overflow the grid.
bool add_tensor(NoiseArgs& a, int k, const void* summed, void* grad, int64_t P) {
  a.summed[k] = summed;
  a.grad[k] = grad;
  a.P[k] = P;
  const int64_t groups = dpk_cdiv(P, 4);
  a.gprefix[k + 1] = a.gprefix[k] + groups;
  const int64_t nb = static_cast<int64_t>(a.bprefix[k]) + dpk_cdiv(groups, kGroupsPerBlock);
  if (nb > DPK_MAX_GRID_X) return false;
  a.bprefix[k + 1] = static_cast<uint32_t>(nb);
  return true;
}

}  // namespace

extern "C" int dpk_add_noise(const void* summed, int in_dtype, void* grad, int out_dtype, int64_t P,
                             float std, float denom, uint64_t seed, uint64_t offset, int draws,
                             dpk_stream_t stream) {
  const char* who = "dpk_add_noise";
  DPK_REQUIRE(P >= 0, DPK_E_SHAPE, "%s: P=%lld", who, (long long)P);
  if (P == 0) return DPK_OK;
  DPK_REQUIRE(summed && grad, DPK_E_ARG, "%s: NULL tensor", who);
  DPK_REQUIRE(dpk_dtype_ok(in_dtype) && dpk_dtype_ok(out_dtype), DPK_E_DTYPE, "%s: dtypes %d,%d", who,
              in_dtype, out_dtype);
  DPK_REQUIRE(draws == 1 || draws == 4, DPK_E_ARG, "%s: draws=%d (1 or 4)", who, draws);
  DPK_REQUIRE(std >= 0.f && denom != 0.f, DPK_E_ARG, "%s: std=%g denom=%g", who, (double)std,
              (double)denom);
  DPK_REQUIRE(dpk_aligned(summed, dpk_elsize(in_dtype)) && dpk_aligned(grad, dpk_elsize(out_dtype)),
              DPK_E_ALIGN, "%s: misaligned tensor", who);
  NoiseArgs a;
  a.K = 1;
  a.gprefix[0] = 0;
  a.bprefix[0] = 0;
  DPK_REQUIRE(add_tensor(a, 0, summed, grad, P), DPK_E_SHAPE, "%s: P too large", who);
  return launch(who, a, a.bprefix[1], in_dtype, out_dtype, std, denom, seed, offset, draws,
                static_cast<hipStream_t>(stream));
}

extern "C" int dpk_fill_normal(float* out, int64_t P, float std, uint64_t seed, uint64_t offset,
                               dpk_stream_t stream) {
  const char* who = "dpk_fill_normal";
  DPK_REQUIRE(P >= 0, DPK_E_SHAPE, "%s: P=%lld", who, (long long)P);
  if (P == 0) return DPK_OK;
  DPK_REQUIRE(out, DPK_E_ARG, "%s: NULL tensor", who);
  DPK_REQUIRE(std >= 0.f, DPK_E_ARG, "%s: std=%g", who, (double)std);
  DPK_REQUIRE(dpk_aligned(out, 4), DPK_E_ALIGN, "%s: misaligned tensor", who);
  NoiseArgs a;
  a.K = 1;
  a.gprefix[0] = 0;
  a.bprefix[0] = 0;
  DPK_REQUIRE(add_tensor(a, 0, nullptr, out, P), DPK_E_SHAPE, "%s: P too large", who);
  return launch(who, a, a.bprefix[1], DPK_F32, DPK_F32, std, 1.0f, seed, offset, 1,
                static_cast<hipStream_t>(stream));
}

extern "C" int dpk_add_noise_multi(const void* const* summed, void* const* grad, const int64_t* P,
                                   int64_t K, int in_dtype, int out_dtype, float std, float denom,
                                   uint64_t seed, uint64_t offset, int draws, dpk_stream_t stream) {
  const char* who = "dpk_add_noise_multi";
  DPK_REQUIRE(summed && grad && P, DPK_E_ARG, "%s: NULL pointer table", who);
  DPK_REQUIRE(K >= 1 && K <= DPK_MULTI_MAX, DPK_E_SHAPE, "%s: K=%lld not in [1,%d]", who, (long long)K,
              DPK_MULTI_MAX);
  DPK_REQUIRE(dpk_dtype_ok(in_dtype) && dpk_dtype_ok(out_dtype), DPK_E_DTYPE, "%s: dtypes %d,%d", who,
              in_dtype, out_dtype);
  DPK_REQUIRE(draws == 1 || draws == 4, DPK_E_ARG, "%s: draws=%d (1 or 4)", who, draws);
  DPK_REQUIRE(std >= 0.f && denom != 0.f, DPK_E_ARG, "%s: std=%g denom=%g", who, (double)std, (double)denom);
  NoiseArgs a;
  a.K = static_cast<int>(K);
  a.gprefix[0] = 0;
  a.bprefix[0] = 0;
  for (int k = 0; k < K; ++k) {
    DPK_REQUIRE(P[k] >= 1, DPK_E_SHAPE, "%s: P[%d]=%lld", who, k, (long long)P[k]);
    DPK_REQUIRE(summed[k] && grad[k], DPK_E_ARG, "%s: tensor %d is NULL", who, k);
    DPK_REQUIRE(dpk_aligned(summed[k], dpk_elsize(in_dtype)) && dpk_aligned(grad[k], dpk_elsize(out_dtype)),
                DPK_E_ALIGN, "%s: tensor %d misaligned", who, k);
    DPK_REQUIRE(add_tensor(a, k, summed[k], grad[k], P[k]), DPK_E_SHAPE, "%s: too many blocks", who);
  }
  return launch(who, a, a.bprefix[K], in_dtype, out_dtype, std, denom, seed, offset, draws,
                static_cast<hipStream_t>(stream));
}
