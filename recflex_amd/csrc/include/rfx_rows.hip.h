// Row formats, 16-byte row vectors and the fp32 decode/accumulate step for the three table
// element types of the fused embedding kernel (gfx950, wave64).
//
// Reference counterpart: examples/csrc/include/aligned_vector.cuh:8-136 (AlignedVector<T,N>,
// fp32 only, 1/2/4-float vectors).  Here a row vector is always the widest power-of-two byte
// packet (16/8/4 B) that divides the row payload, so one lane moves 4 fp32, 8 fp16 or 16 int8
// elements per global_load_dwordx4.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace rfx {

// table element types (MetaData.data_type in the Python emitter: "float" / "half" / "int8")
constexpr int F32 = 0;
constexpr int F16 = 1;
// I8: row = D unsigned 8-bit codes, then one fp16 scale and one fp16 bias, padded so that the
// row stride is a multiple of 16 B.  value = code * scale + bias.
constexpr int I8 = 2;

__host__ __device__ constexpr int ceil_div(int a, int b) { return (a + b - 1) / b; }
__host__ __device__ constexpr int round_up(int a, int b) { return ceil_div(a, b) * b; }

template <int DT, int D> struct Row {
  static constexpr int ESZ = DT == F32 ? 4 : (DT == F16 ? 2 : 1);
  static constexpr int PAYLOAD = D * ESZ;
  static_assert(PAYLOAD % 4 == 0, "row payload must be a whole number of dwords");
  // bytes between consecutive rows
  static constexpr int STRIDE = DT == I8 ? round_up(PAYLOAD + 4, 16) : PAYLOAD;
  // bytes one lane moves per load
  static constexpr int VB = PAYLOAD % 16 == 0 ? 16 : (PAYLOAD % 8 == 0 ? 8 : 4);
  // vectors per row, elements per vector
  static constexpr int V = PAYLOAD / VB;
  static constexpr int EPV = VB / ESZ;
};

typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));

// the two fp16 halves of a dword as fp32 (x = low half)
__device__ __forceinline__ f32x2 unpack_half2(uint32_t w) {
  const f16x2 h = __builtin_bit_cast(f16x2, w);
  f32x2 r; r.x = static_cast<float>(h.x); r.y = static_cast<float>(h.y);
  return r;
}

template <int VB> struct Vec {
  uint32_t w[VB / 4];
};

template <int VB> __device__ __forceinline__ Vec<VB> load_vec(const char *__restrict__ p) {
  Vec<VB> r;
  if constexpr (VB == 16) {
    const u32x4 t = *reinterpret_cast<const u32x4 *>(p);
    r.w[0] = t.x; r.w[1] = t.y; r.w[2] = t.z; r.w[3] = t.w;
  } else if constexpr (VB == 8) {
    const u32x2 t = *reinterpret_cast<const u32x2 *>(p);
    r.w[0] = t.x; r.w[1] = t.y;
  } else {
    r.w[0] = *reinterpret_cast<const uint32_t *>(p);
  }
  return r;
}

// scale (x) and bias (y) of an I8 row, stored as two fp16 right after the codes
template <int D> __device__ __forceinline__ f32x2 load_scale_bias(const char *__restrict__ row) {
  return unpack_half2(*reinterpret_cast<const uint32_t *>(row + D));
}

// acc[0..EPV) += decode(v).  For I8 only code*scale is added here; the bias is summed once per
// lookup by the caller and added to every column after the bag is finished.
#ifndef RFX_F16_FMA_MIX
#define RFX_F16_FMA_MIX 1
#endif

// acc + (the fp16 value in the low (HI == 0) or high (HI == 1) half of w), rounded once
template <int HI> __device__ __forceinline__ float add_half(float acc, uint32_t w) {
  if constexpr (HI == 0)
    asm("v_fma_mix_f32 %0, %1, 1.0, %0 op_sel_hi:[1,0,0]" : "+v"(acc) : "v"(w));
  else
    asm("v_fma_mix_f32 %0, %1, 1.0, %0 op_sel:[1,0,0] op_sel_hi:[1,0,0]" : "+v"(acc) : "v"(w));
  return acc;
}

template <int DT, int VB>
__device__ __forceinline__ void accumulate(float *acc, const Vec<VB> &v, float scale) {
  if constexpr (DT == F32) {
#pragma unroll
    for (int i = 0; i < VB / 4; ++i) acc[i] += __uint_as_float(v.w[i]);
  } else if constexpr (DT == F16) {
#pragma unroll
    for (int i = 0; i < VB / 4; ++i) {
#if RFX_F16_FMA_MIX
      // acc += half: one v_fma_mix_f32 (half * 1.0 + acc, the half taken straight from the low or
      // high 16 bits of the loaded dword) instead of a conversion and an add; same rounding
      acc[2 * i] = add_half<0>(acc[2 * i], v.w[i]);
      acc[2 * i + 1] = add_half<1>(acc[2 * i + 1], v.w[i]);
#else
      const f32x2 f = unpack_half2(v.w[i]);
      acc[2 * i] += f.x;
      acc[2 * i + 1] += f.y;
#endif
    }
  } else {
#pragma unroll
    for (int i = 0; i < VB / 4; ++i) {
      const uint32_t w = v.w[i];
      acc[4 * i + 0] = fmaf(static_cast<float>(w & 0xffu), scale, acc[4 * i + 0]);
      acc[4 * i + 1] = fmaf(static_cast<float>((w >> 8) & 0xffu), scale, acc[4 * i + 1]);
      acc[4 * i + 2] = fmaf(static_cast<float>((w >> 16) & 0xffu), scale, acc[4 * i + 2]);
      acc[4 * i + 3] = fmaf(static_cast<float>(w >> 24), scale, acc[4 * i + 3]);
    }
  }
}

// One store to the pooled output.  Output elements are written once and never read back by the
// kernel; with the non-temporal hint they do not compete with the table rows for the L2
// (measured against plain stores: 2-3 % less kernel time on the 100-, 200- and 400-feature
// models, identical bits).
template <typename T> __device__ __forceinline__ void store_streaming(T *p, const T v) {
  __builtin_nontemporal_store(v, p);
}

// Store n fp32 values to the pooled output.  OVEC = widest store (in floats) the output
// column offset of this feature allows: 4 -> global_store_dwordx4.
template <int N, int OVEC>
__device__ __forceinline__ void store_floats(float *__restrict__ dst, const float *src) {
  if constexpr (OVEC == 4 && N % 4 == 0) {
#pragma unroll
    for (int i = 0; i < N; i += 4) {
      f32x4 t; t.x = src[i]; t.y = src[i + 1]; t.z = src[i + 2]; t.w = src[i + 3];
      store_streaming(reinterpret_cast<f32x4 *>(dst + i), t);
    }
  } else if constexpr (OVEC >= 2 && N % 2 == 0) {
#pragma unroll
    for (int i = 0; i < N; i += 2) {
      f32x2 t; t.x = src[i]; t.y = src[i + 1];
      store_streaming(reinterpret_cast<f32x2 *>(dst + i), t);
    }
  } else {
#pragma unroll
    for (int i = 0; i < N; ++i) store_streaming(dst + i, src[i]);
  }
}

} // namespace rfx
