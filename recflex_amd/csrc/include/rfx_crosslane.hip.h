// Cross-lane butterfly steps for 64-lane wavefronts on gfx950, without going through LDS
// memory: DPP modifiers for lane distances 1, 2, 4, 8; ds_swizzle (crossbar only) for 16;
// v_permlane32_swap for 32.
//
// Reference counterpart: the shared-memory tree with __syncwarp/__syncthreads in
// examples/csrc/include/one_block_multi_sample_kernel.cuh:78-98 (and the 32-lane warp
// assumption `32 % VBLOCK_DIM_XY` there).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace rfx {

// v + (value of v held by lane ^ S).  Every lane of the pair must be active.
template <int S> __device__ __forceinline__ float add_xor(float v) {
  static_assert(S == 1 || S == 2 || S == 4 || S == 8 || S == 16 || S == 32, "lane distance");
  const int i = __float_as_int(v);
  if constexpr (S == 1) {
    // quad_perm:[1,0,3,2]
    return v + __int_as_float(__builtin_amdgcn_update_dpp(i, i, 0xB1, 0xf, 0xf, false));
  } else if constexpr (S == 2) {
    // quad_perm:[2,3,0,1]
    return v + __int_as_float(__builtin_amdgcn_update_dpp(i, i, 0x4E, 0xf, 0xf, false));
  } else if constexpr (S == 4) {
    // banks 0 and 2 of each 16-lane row read lane+4 (row_shl:4), banks 1 and 3 read lane-4
    // (row_shr:4)
    int r = __builtin_amdgcn_update_dpp(i, i, 0x104, 0xf, 0x5, false);
    r = __builtin_amdgcn_update_dpp(r, i, 0x114, 0xf, 0xA, false);
    return v + __int_as_float(r);
  } else if constexpr (S == 8) {
    // row_ror:8 inside a 16-lane row is lane ^ 8
    return v + __int_as_float(__builtin_amdgcn_update_dpp(i, i, 0x128, 0xf, 0xf, false));
  } else if constexpr (S == 16) {
    // bit-mask mode: and_mask 0x1f, or_mask 0, xor_mask 0x10
    return v + __int_as_float(__builtin_amdgcn_ds_swizzle(i, 0x401F));
  } else {
    // r[0] = {lanes 0-31: own, lanes 32-63: value of lane-32}
    // r[1] = {lanes 0-31: value of lane+32, lanes 32-63: own}
    const auto r = __builtin_amdgcn_permlane32_swap(i, i, false, false);
    return __int_as_float(r[0]) + __int_as_float(r[1]);
  }
}

// Sum over the lanes {lane ^ (k*X) : k} of a team of T = X*Y consecutive lanes (X, Y powers of
// two, T <= 64): afterwards every lane holds the total of its column over the Y lookup lanes.
template <int X, int T> __device__ __forceinline__ float reduce_over_y(float v) {
  if constexpr (X <= 1 && T > 1) v = add_xor<1>(v);
  if constexpr (X <= 2 && T > 2) v = add_xor<2>(v);
  if constexpr (X <= 4 && T > 4) v = add_xor<4>(v);
  if constexpr (X <= 8 && T > 8) v = add_xor<8>(v);
  if constexpr (X <= 16 && T > 16) v = add_xor<16>(v);
  if constexpr (X <= 32 && T > 32) v = add_xor<32>(v);
  return v;
}

} // namespace rfx
