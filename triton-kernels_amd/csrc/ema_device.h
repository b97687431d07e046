// Device-side helpers shared by the EMA kernels (gfx950, wave64).
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace ema {

typedef __bf16 bf16_t;
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

constexpr int kWave = 64;
#define EMA_MAX_CHUNK_DEV 1024

// One descriptor per sequence tensor: element strides of (batch, position, head); the
// feature axis has unit stride.
struct SeqStrides {
  int64_t sb, sl, sh;
};

// ------------------------------------------------------------------ wave primitives

// v of the lane selected by a DPP control, or 0 where the control has no source lane or
// the row is masked out.
template <int CTRL, int ROW_MASK>
__device__ __forceinline__ float dpp_or_zero(float v) {
  return __int_as_float(
      __builtin_amdgcn_update_dpp(0, __float_as_int(v), CTRL, ROW_MASK, 0xf, false));
}

// Inclusive prefix sum over the 64 lanes of a wave with DPP row shifts and row broadcasts
// (no LDS traffic).
__device__ __forceinline__ float wave_inclusive_scan(float v) {
  v += dpp_or_zero<0x111, 0xf>(v);  // row_shr:1
  v += dpp_or_zero<0x112, 0xf>(v);  // row_shr:2
  v += dpp_or_zero<0x114, 0xf>(v);  // row_shr:4
  v += dpp_or_zero<0x118, 0xf>(v);  // row_shr:8
  v += dpp_or_zero<0x142, 0xa>(v);  // row_bcast:15 into rows 1 and 3
  v += dpp_or_zero<0x143, 0xc>(v);  // row_bcast:31 into rows 2 and 3
  return v;
}

// Exclusive prefix sum over the 64 lanes: the inclusive sum of the lane before, 0 in lane 0.
// Formed by a shift and not as `inclusive - own value`, which is NaN for an infinite term (a
// log-decay of -inf marks a state reset and must stay -inf in every later sum).
__device__ __forceinline__ float wave_exclusive_scan(float v) {
  const float up = __shfl_up(wave_inclusive_scan(v), 1, 64);
  return (threadIdx.x & 63) == 0 ? 0.f : up;
}

// Sum over the 64 lanes, returned in every lane.
__device__ __forceinline__ float wave_sum(float v) {
  v = wave_inclusive_scan(v);
  return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}

// ------------------------------------------------------------------ 16-byte vectors

template <typename T>
struct Vec16;  // 16 bytes of T
template <>
struct Vec16<float> {
  static constexpr int N = 4;
  float4 raw;
  __device__ __forceinline__ float get(int i) const {
    return i == 0 ? raw.x : i == 1 ? raw.y : i == 2 ? raw.z : raw.w;
  }
  __device__ __forceinline__ void set(int i, float f) {
    if (i == 0) raw.x = f;
    else if (i == 1) raw.y = f;
    else if (i == 2) raw.z = f;
    else raw.w = f;
  }
  __device__ __forceinline__ void put(int i, float f) { set(i, f); }
  __device__ __forceinline__ void set_all(const float* f) { raw = make_float4(f[0], f[1], f[2], f[3]); }
  __device__ __forceinline__ void zero() { raw = make_float4(0.f, 0.f, 0.f, 0.f); }
};
template <>
struct Vec16<bf16_t> {
  static constexpr int N = 8;
  bf16x8 raw;
  __device__ __forceinline__ float get(int i) const { return (float)raw[i]; }
  __device__ __forceinline__ void set(int i, float f) { raw[i] = (bf16_t)f; }
  __device__ __forceinline__ void put(int i, bf16_t f) { raw[i] = f; }
  // all eight elements from floats, converted two at a time (one packed conversion per pair
  // instead of a conversion and a byte permute per element)
  __device__ __forceinline__ void set_all(const float* f) {
    typedef float f32x2 __attribute__((ext_vector_type(2)));
    typedef bf16_t b16x2 __attribute__((ext_vector_type(2)));
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const f32x2 p = {f[2 * i], f[2 * i + 1]};
      const b16x2 q = __builtin_convertvector(p, b16x2);
      raw[2 * i] = q[0];
      raw[2 * i + 1] = q[1];
    }
  }
  __device__ __forceinline__ void zero() {
#pragma unroll
    for (int i = 0; i < 8; ++i) raw[i] = (bf16_t)0.0f;
  }
};

template <typename T>
__device__ __forceinline__ Vec16<T> load16(const T* p) {
  Vec16<T> v;
  v.raw = *reinterpret_cast<const decltype(v.raw)*>(p);
  return v;
}
template <typename T>
__device__ __forceinline__ void store16(T* p, const Vec16<T>& v) {
  *reinterpret_cast<decltype(v.raw)*>(p) = v.raw;
}

// The same with the non-temporal hint, for global data that the kernel touches once and no other
// workgroup is about to read through the same L2.
typedef float f32x4_t __attribute__((ext_vector_type(4)));
__device__ __forceinline__ Vec16<float> load16_stream(const float* p) {
  const f32x4_t t = __builtin_nontemporal_load(reinterpret_cast<const f32x4_t*>(p));
  Vec16<float> v;
  v.raw = make_float4(t[0], t[1], t[2], t[3]);
  return v;
}
__device__ __forceinline__ Vec16<bf16_t> load16_stream(const bf16_t* p) {
  Vec16<bf16_t> v;
  v.raw = __builtin_nontemporal_load(reinterpret_cast<const bf16x8*>(p));
  return v;
}
__device__ __forceinline__ void store16_stream(float* p, const Vec16<float>& v) {
  const f32x4_t t = {v.raw.x, v.raw.y, v.raw.z, v.raw.w};
  __builtin_nontemporal_store(t, reinterpret_cast<f32x4_t*>(p));
}
__device__ __forceinline__ void store16_stream(bf16_t* p, const Vec16<bf16_t>& v) {
  __builtin_nontemporal_store(v.raw, reinterpret_cast<bf16x8*>(p));
}

// ------------------------------------------------------------------ MFMA groups
// One "group" multiplies a 32 x KG tile by a KG x 32 tile, KG = 2 * Vec16<T>::N.  A lane
// holds Vec16<T>::N consecutive k of row (lane % 32), starting at k = N * (lane / 32),
// for both operands; the accumulator of lane l, register v, is element
// (8 * (v / 4) + 4 * (l / 32) + v % 4,  l % 32) of the 32 x 32 result.
__device__ __forceinline__ void mma_group(const Vec16<bf16_t>& a, const Vec16<bf16_t>& b,
                                          floatx16& acc) {
  acc = __builtin_amdgcn_mfma_f32_32x32x16_bf16(a.raw, b.raw, acc, 0, 0, 0);
}
__device__ __forceinline__ void mma_group(const Vec16<float>& a, const Vec16<float>& b,
                                          floatx16& acc) {
  acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.raw.x, b.raw.x, acc, 0, 0, 0);
  acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.raw.y, b.raw.y, acc, 0, 0, 0);
  acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.raw.z, b.raw.z, acc, 0, 0, 0);
  acc = __builtin_amdgcn_mfma_f32_32x32x2f32(a.raw.w, b.raw.w, acc, 0, 0, 0);
}

// B operand of a bf16 MFMA group from a row-major LDS tile t[k][col] (pitch in elements):
// lane l receives t[k0 + 8*(l/32) + e][col0 + l%32], e = 0..7, through two transposing
// 64-bit LDS reads.  In each group of 16 lanes, lane i supplies the address of four
// consecutive columns of row i/4 and receives, for column i of the 16-column strip, the
// four rows of the group.
typedef bf16_t bf16x4 __attribute__((ext_vector_type(4)));
__device__ __forceinline__ Vec16<bf16_t> lds_read_kmajor(const bf16_t* t, int pitch, int k0,
                                                         int col0, int lane) {
  const int i = lane & 15;
  const int row = k0 + 8 * (lane >> 5) + (i >> 2);
  const int col = col0 + 16 * ((lane >> 4) & 1) + 4 * (i & 3);
  const bf16_t* p = t + row * pitch + col;
  typedef __attribute__((address_space(3))) bf16x4 lds_bf16x4;
  const bf16x4 lo = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_bf16x4*)p);
  const bf16x4 hi = __builtin_amdgcn_ds_read_tr16_b64_v4bf16((lds_bf16x4*)(p + 4 * pitch));
  Vec16<bf16_t> r;
  r.raw = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
  return r;
}

__device__ __forceinline__ int acc_row(int v, int lane) {
  return 8 * (v >> 2) + 4 * (lane >> 5) + (v & 3);
}

}  // namespace ema
