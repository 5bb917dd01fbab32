// DPOptimizer.add_noise + scale_grad (opacus/optimizers/optimizer.py:477-504)
// with _generate_noise (optimizer.py:104-169) folded in: one pass that reads
// summed_grad, draws Gaussian noise from a counter-based generator in registers,
// adds, divides and writes grad. HBM-bound: 2 * P * elsize bytes.
//
// Generator: Philox4x32-10 (Salmon et al., SC'11), key = seed, counter =
// (group index lo, hi, offset lo, hi) where a group is 4 consecutive elements.
// The four 32-bit outputs make two Box-Muller pairs, i.e. the four normals of
// the group. The stream therefore depends only on (seed, offset, element
// index), never on the launch shape.
#include "dpk_common.h"

namespace {

constexpr int kThreads = 256;

__device__ __forceinline__ uint4 philox4x32_10(uint4 c, uint2 k) {
  constexpr uint32_t M0 = 0xD2511F53u, M1 = 0xCD9E8D57u, W0 = 0x9E3779B9u, W1 = 0xBB67AE85u;
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    const uint32_t hi0 = __umulhi(M0, c.x), lo0 = M0 * c.x;
    const uint32_t hi1 = __umulhi(M1, c.z), lo1 = M1 * c.z;
    c = make_uint4(hi1 ^ c.y ^ k.x, lo1, hi0 ^ c.w ^ k.y, lo0);
    k.x += W0;
    k.y += W1;
  }
  return c;
}

// Uniform in (0, 1]: 32 random bits placed at the centre of their 2^-32 cell.
__device__ __forceinline__ float u01(uint32_t x) {
  return static_cast<float>(x) * 2.3283064365386963e-10f + 1.1641532182693481e-10f;
}

__device__ __forceinline__ float4 normal4(uint64_t group, uint64_t seed, uint64_t offset) {
  const uint4 r = philox4x32_10(
      make_uint4(static_cast<uint32_t>(group), static_cast<uint32_t>(group >> 32),
                 static_cast<uint32_t>(offset), static_cast<uint32_t>(offset >> 32)),
      make_uint2(static_cast<uint32_t>(seed), static_cast<uint32_t>(seed >> 32)));
  const float r0 = sqrtf(-2.0f * logf(u01(r.x)));
  const float r1 = sqrtf(-2.0f * logf(u01(r.z)));
  float s0, c0, s1, c1;
  sincosf(6.2831853071795865f * u01(r.y), &s0, &c0);
  sincosf(6.2831853071795865f * u01(r.w), &s1, &c1);
  return make_float4(r0 * c0, r0 * s0, r1 * c1, r1 * s1);
}

__device__ __forceinline__ float4 noise4(uint64_t group, uint64_t seed, uint64_t offset, int draws) {
  float4 z = normal4(group, seed, offset);
  if (draws == 4) {
    // The reference's secure mode: four independent normals summed and halved
    // (variance 4/4 = 1), optimizer.py:150-160.
    for (int d = 1; d < 4; ++d) {
      float4 y = normal4(group, seed, offset + d);
      z.x += y.x;
      z.y += y.y;
      z.z += y.z;
      z.w += y.w;
    }
    z.x *= 0.5f;
    z.y *= 0.5f;
    z.z *= 0.5f;
    z.w *= 0.5f;
  }
  return z;
}

template <typename TI, typename TO, bool VEC>
__global__ __launch_bounds__(kThreads) void add_noise_kernel(const TI* __restrict__ summed,
                                                               TO* __restrict__ grad, int64_t P,
                                                               float std, float denom,
                                                               uint64_t seed, uint64_t offset,
                                                               int draws) {
  const int64_t g = static_cast<int64_t>(blockIdx.x) * kThreads + threadIdx.x;
  const int64_t i = g * 4;
  if (i >= P) return;
  float4 z = make_float4(0.f, 0.f, 0.f, 0.f);
  if (std != 0.f) {
    z = noise4(static_cast<uint64_t>(g), seed, offset, draws);
    z.x *= std;
    z.y *= std;
    z.z *= std;
    z.w *= std;
  }
  if (VEC && i + 4 <= P) {
    float4 v = summed ? dpk_io<TI>::load4(summed + i) : make_float4(0.f, 0.f, 0.f, 0.f);
    v.x = (v.x + z.x) / denom;
    v.y = (v.y + z.y) / denom;
    v.z = (v.z + z.z) / denom;
    v.w = (v.w + z.w) / denom;
    dpk_io<TO>::store4(grad + i, v);
  } else {
    const float zz[4] = {z.x, z.y, z.z, z.w};
    for (int e = 0; e < 4 && i + e < P; ++e) {
      const float v = summed ? dpk_io<TI>::load(summed + i + e) : 0.f;
      dpk_io<TO>::store(grad + i + e, (v + zz[e]) / denom);
    }
  }
}

template <typename TI, typename TO>
void launch(const void* summed, void* grad, int64_t P, float std, float denom, uint64_t seed,
            uint64_t offset, int draws, bool vec, hipStream_t s) {
  const unsigned blocks = static_cast<unsigned>(dpk_cdiv(dpk_cdiv(P, 4), kThreads));
  if (vec)
    hipLaunchKernelGGL((add_noise_kernel<TI, TO, true>), dim3(blocks), dim3(kThreads), 0, s,
                       static_cast<const TI*>(summed), static_cast<TO*>(grad), P, std, denom, seed,
                       offset, draws);
  else
    hipLaunchKernelGGL((add_noise_kernel<TI, TO, false>), dim3(blocks), dim3(kThreads), 0, s,
                       static_cast<const TI*>(summed), static_cast<TO*>(grad), P, std, denom, seed,
                       offset, draws);
}

struct NoiseMulti {
  const void* summed[DPK_MULTI_MAX];
  void* grad[DPK_MULTI_MAX];
  int64_t P[DPK_MULTI_MAX];
  int64_t gprefix[DPK_MULTI_MAX + 1];  // 4-element groups before tensor k: block and counter base
  int K;
};

// All parameters of an optimizer in one launch. Tensor k's element i uses Philox
// group gprefix[k] + i / 4, i.e. the tensors draw from one stream laid end to end.
// Blocks never straddle tensors (each tensor's groups are padded to whole blocks
// in the grid, not in the counter space).
template <typename TI, typename TO>
__global__ __launch_bounds__(kThreads) void add_noise_multi_kernel(NoiseMulti a, float std, float denom,
                                                                     uint64_t seed, uint64_t offset,
                                                                     int draws) {
  // Which tensor this block belongs to: tensor k owns ceil(groups_k / kThreads) blocks.
  int k = 0;
  int64_t b0 = 0;
  for (;;) {
    const int64_t nb = ((a.gprefix[k + 1] - a.gprefix[k]) + kThreads - 1) / kThreads;
    if (static_cast<int64_t>(blockIdx.x) < b0 + nb || k + 1 >= a.K) break;
    b0 += nb;
    ++k;
  }
  const int64_t g = (static_cast<int64_t>(blockIdx.x) - b0) * kThreads + threadIdx.x;
  const int64_t i = g * 4, P = a.P[k];
  if (i >= P) return;
  const TI* summed = static_cast<const TI*>(a.summed[k]);
  TO* grad = static_cast<TO*>(a.grad[k]);
  float4 z = make_float4(0.f, 0.f, 0.f, 0.f);
  if (std != 0.f) {
    z = noise4(static_cast<uint64_t>(a.gprefix[k] + g), seed, offset, draws);
    z.x *= std;
    z.y *= std;
    z.z *= std;
    z.w *= std;
  }
  const bool vec = i + 4 <= P && ((reinterpret_cast<uintptr_t>(summed) | reinterpret_cast<uintptr_t>(grad)) & 15) == 0;
  if (vec) {
    float4 v = dpk_io<TI>::load4(summed + i);
    v.x = (v.x + z.x) / denom;
    v.y = (v.y + z.y) / denom;
    v.z = (v.z + z.z) / denom;
    v.w = (v.w + z.w) / denom;
    dpk_io<TO>::store4(grad + i, v);
  } else {
    const float zz[4] = {z.x, z.y, z.z, z.w};
    for (int e = 0; e < 4 && i + e < P; ++e)
      dpk_io<TO>::store(grad + i + e, (dpk_io<TI>::load(summed + i + e) + zz[e]) / denom);
  }
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
  DPK_REQUIRE(dpk_cdiv(dpk_cdiv(P, 4), kThreads) <= DPK_MAX_GRID_X, DPK_E_SHAPE, "%s: P too large", who);
  const bool vec = dpk_aligned(summed, in_dtype == DPK_BF16 ? 8 : 16) &&
                   dpk_aligned(grad, out_dtype == DPK_BF16 ? 8 : 16);
  hipStream_t s = static_cast<hipStream_t>(stream);
  if (in_dtype == DPK_F32 && out_dtype == DPK_F32)
    launch<float, float>(summed, grad, P, std, denom, seed, offset, draws, vec, s);
  else if (in_dtype == DPK_F32 && out_dtype == DPK_BF16)
    launch<float, bf16_t>(summed, grad, P, std, denom, seed, offset, draws, vec, s);
  else if (in_dtype == DPK_BF16 && out_dtype == DPK_F32)
    launch<bf16_t, float>(summed, grad, P, std, denom, seed, offset, draws, vec, s);
  else
    launch<bf16_t, bf16_t>(summed, grad, P, std, denom, seed, offset, draws, vec, s);
  DPK_LAUNCH_CHECK(who);
  return DPK_OK;
}

extern "C" int dpk_fill_normal(float* out, int64_t P, float std, uint64_t seed, uint64_t offset,
                               dpk_stream_t stream) {
  const char* who = "dpk_fill_normal";
  DPK_REQUIRE(P >= 0, DPK_E_SHAPE, "%s: P=%lld", who, (long long)P);
  if (P == 0) return DPK_OK;
  DPK_REQUIRE(out, DPK_E_ARG, "%s: NULL tensor", who);
  DPK_REQUIRE(dpk_aligned(out, 4), DPK_E_ALIGN, "%s: misaligned tensor", who);
  DPK_REQUIRE(dpk_cdiv(dpk_cdiv(P, 4), kThreads) <= DPK_MAX_GRID_X, DPK_E_SHAPE, "%s: P too large", who);
  launch<float, float>(nullptr, out, P, std, 1.0f, seed, offset, 1, dpk_aligned(out, 16),
                       static_cast<hipStream_t>(stream));
  DPK_LAUNCH_CHECK(who);
  return DPK_OK;
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
  NoiseMulti a;
  a.K = static_cast<int>(K);
  a.gprefix[0] = 0;
  int64_t blocks = 0;
  for (int k = 0; k < K; ++k) {
    DPK_REQUIRE(P[k] >= 1, DPK_E_SHAPE, "%s: P[%d]=%lld", who, k, (long long)P[k]);
    DPK_REQUIRE(summed[k] && grad[k], DPK_E_ARG, "%s: tensor %d is NULL", who, k);
    DPK_REQUIRE(dpk_aligned(summed[k], dpk_elsize(in_dtype)) && dpk_aligned(grad[k], dpk_elsize(out_dtype)),
                DPK_E_ALIGN, "%s: tensor %d misaligned", who, k);
    a.summed[k] = summed[k];
    a.grad[k] = grad[k];
    a.P[k] = P[k];
    const int64_t groups = dpk_cdiv(P[k], 4);
    a.gprefix[k + 1] = a.gprefix[k] + groups;
    blocks += dpk_cdiv(groups, kThreads);
  }
  DPK_REQUIRE(blocks <= DPK_MAX_GRID_X, DPK_E_SHAPE, "%s: too many blocks", who);
  hipStream_t s = static_cast<hipStream_t>(stream);
  const dim3 grid(static_cast<unsigned>(blocks)), block(kThreads);
#define DPK_NM(TI, TO) \
  hipLaunchKernelGGL((add_noise_multi_kernel<TI, TO>), grid, block, 0, s, a, std, denom, seed, offset, draws)
  if (in_dtype == DPK_F32 && out_dtype == DPK_F32) DPK_NM(float, float);
  else if (in_dtype == DPK_F32 && out_dtype == DPK_BF16) DPK_NM(float, bf16_t);
  else if (in_dtype == DPK_BF16 && out_dtype == DPK_F32) DPK_NM(bf16_t, float);
  else DPK_NM(bf16_t, bf16_t);
#undef DPK_NM
  DPK_LAUNCH_CHECK(who);
  return DPK_OK;
}
