// Counter-based Gaussian noise for DPOptimizer.add_noise (opacus/optimizers/optimizer.py:104-169,
// 477-493), shared by the kernels that add it.
//
// Generator: Philox4x32-10 (Salmon et al., SC'11), key = seed, counter =
// (group index lo, hi, offset lo, hi) where a group is 4 consecutive elements of the stream.
// The four 32-bit outputs make two Box-Muller pairs, i.e. the four normals of the group. The
// stream depends only on (seed, offset, element index), never on the launch shape.
#pragma once

#include "dpk_common.h"

namespace dpk_noise {

__device__ __forceinline__ uint4 philox4x32_10(uint4 c, uint2 k) {
  constexpr uint32_t M0 = 0xD2511F53u, M1 = 0xCD9E8D57u, W0 = 0x9E3779B9u, W1 = 0xBB67AE85u;
#pragma unroll
  for (int r = 0; r < 10; ++r) {
    // one 32 x 32 -> 64 bit multiply per product (v_mad_u64_u32) instead of a low and a
    // high multiply: the integer multiplies are what bounds this generator
    const uint64_t p0 = static_cast<uint64_t>(M0) * c.x, p1 = static_cast<uint64_t>(M1) * c.z;
    const uint32_t hi0 = static_cast<uint32_t>(p0 >> 32), lo0 = static_cast<uint32_t>(p0);
    const uint32_t hi1 = static_cast<uint32_t>(p1 >> 32), lo1 = static_cast<uint32_t>(p1);
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
  // Box-Muller on the hardware transcendentals: v_log_f32 is log2, v_sin/v_cos take
  // their argument in revolutions, so cos(2 pi u) is one instruction. The kernel is
  // otherwise bound by these, not by memory.
  constexpr float kNeg2Ln2 = -1.3862943611198906f;
  const float r0 = __builtin_amdgcn_sqrtf(kNeg2Ln2 * __builtin_amdgcn_logf(u01(r.x)));
  const float r1 = __builtin_amdgcn_sqrtf(kNeg2Ln2 * __builtin_amdgcn_logf(u01(r.z)));
  const float t0 = u01(r.y), t1 = u01(r.w);
  return make_float4(r0 * __builtin_amdgcn_cosf(t0), r0 * __builtin_amdgcn_sinf(t0),
                     r1 * __builtin_amdgcn_cosf(t1), r1 * __builtin_amdgcn_sinf(t1));
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

}  // namespace dpk_noise
