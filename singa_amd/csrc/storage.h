// Storage types of the bandwidth-bound kernels.  Arithmetic is always fp32; a storage type says
// how 16 bytes of a tensor turn into floats and back: fp32 (4 elements), IEEE binary16 and
// bfloat16 (8 elements, carried as uint16_t).  Stores round to nearest, ties to even.
#ifndef SINGA_AMD_CSRC_STORAGE_H_
#define SINGA_AMD_CSRC_STORAGE_H_

#include <hip/hip_runtime.h>
#include <stdint.h>

typedef float sgh_v4f __attribute__((ext_vector_type(4)));
typedef unsigned int sgh_v4u __attribute__((ext_vector_type(4)));

__device__ __forceinline__ float sgh_f16_to_f32(uint16_t b) {
  _Float16 h;
  __builtin_memcpy(&h, &b, 2);
  return float(h);
}
__device__ __forceinline__ uint16_t sgh_f32_to_f16(float f) {
  const _Float16 h = _Float16(f);  // v_cvt_f16_f32: round to nearest even
  uint16_t b;
  __builtin_memcpy(&b, &h, 2);
  return b;
}
__device__ __forceinline__ float sgh_bf16_to_f32(uint16_t b) { return __builtin_bit_cast(float, unsigned(b) << 16); }
__device__ __forceinline__ uint16_t sgh_f32_to_bf16(float f) {
  const __bf16 h = __bf16(f);  // v_cvt_pk_bf16_f32: round to nearest even, NaN stays a (quiet) NaN
  uint16_t b;
  __builtin_memcpy(&b, &h, 2);
  return b;
}

// two results rounded and packed into a dword (low half first) by one instruction: v_cvt_pk_f16_f32 /
// v_cvt_pk_bf16_f32, the same roundings as the single conversions above
typedef float sgh_v2f __attribute__((ext_vector_type(2)));
__device__ __forceinline__ unsigned sgh_pack2_f16(float lo, float hi) {
  typedef _Float16 h2 __attribute__((ext_vector_type(2)));
  const h2 h = __builtin_convertvector(sgh_v2f{lo, hi}, h2);
  return __builtin_bit_cast(unsigned, h);
}
__device__ __forceinline__ unsigned sgh_pack2_bf16(float lo, float hi) {
  typedef __bf16 b2 __attribute__((ext_vector_type(2)));
  const b2 h = __builtin_convertvector(sgh_v2f{lo, hi}, b2);
  return __builtin_bit_cast(unsigned, h);
}

struct StF32 {
  typedef float elem;
  static constexpr int VEC = 4;
  static __device__ __forceinline__ float ld(const elem *p) { return *p; }
  static __device__ __forceinline__ void st(elem *p, float v) { *p = v; }
  static __device__ __forceinline__ float stored(float v) { return v; }  // the value a store keeps
  static __device__ __forceinline__ bool stored_positive(float v) { return v > 0.f; }
  template <bool NT>
  static __device__ __forceinline__ void load16(const elem *p, float *out) {
    const sgh_v4f v = NT ? __builtin_nontemporal_load(reinterpret_cast<const sgh_v4f *>(p))
                         : *reinterpret_cast<const sgh_v4f *>(p);
    out[0] = v[0];
    out[1] = v[1];
    out[2] = v[2];
    out[3] = v[3];
  }
  static __device__ __forceinline__ void store16(elem *p, const float *in) {
    *reinterpret_cast<sgh_v4f *>(p) = sgh_v4f{in[0], in[1], in[2], in[3]};
  }
};

// TINY: the largest float that the store rounds to zero (half of the smallest subnormal of the
// 16-bit type: a tie, and ties go to the even neighbour 0), so "the stored value is > 0" is v > TINY.
// HALFVEC: the vector accesses move 8 bytes (4 elements) instead of 16, for tensors whose rows are
// 8- but not 16-byte aligned (e.g. 14 x 14 planes).
template <float (*LD)(uint16_t), uint16_t (*ST)(float), unsigned TINY_BITS, bool HALFVEC = false>
struct St16 {
  typedef uint16_t elem;
  static constexpr int VEC = HALFVEC ? 4 : 8;
  static __device__ __forceinline__ float ld(const elem *p) { return LD(*p); }
  static __device__ __forceinline__ void st(elem *p, float v) { *p = ST(v); }
  static __device__ __forceinline__ float stored(float v) { return LD(ST(v)); }  // the value a store keeps
  static __device__ __forceinline__ bool stored_positive(float v) { return v > __builtin_bit_cast(float, TINY_BITS); }
  template <bool NT>
  static __device__ __forceinline__ void load16(const elem *p, float *out) {   // one vector access: VEC elements
    typedef unsigned int vec __attribute__((ext_vector_type(VEC / 2)));
    const vec v = NT ? __builtin_nontemporal_load(reinterpret_cast<const vec *>(p)) : *reinterpret_cast<const vec *>(p);
#pragma unroll
    for (int j = 0; j < VEC / 2; ++j) {
      out[2 * j] = LD(uint16_t(v[j] & 0xffffu));
      out[2 * j + 1] = LD(uint16_t(v[j] >> 16));
    }
  }
  static __device__ __forceinline__ void store16(elem *p, const float *in) {
    typedef unsigned int vec __attribute__((ext_vector_type(VEC / 2)));
    vec r;
#pragma unroll
    for (int j = 0; j < VEC / 2; ++j) {
      if constexpr (ST == sgh_f32_to_f16) r[j] = sgh_pack2_f16(in[2 * j], in[2 * j + 1]);
      else if constexpr (ST == sgh_f32_to_bf16) r[j] = sgh_pack2_bf16(in[2 * j], in[2 * j + 1]);
      else r[j] = unsigned(ST(in[2 * j])) | (unsigned(ST(in[2 * j + 1])) << 16);
    }
    *reinterpret_cast<vec *>(p) = r;
  }
};

// binary16: smallest subnormal 2^-24, so 2^-25 (0x33000000) and below store as 0;
// bfloat16: smallest subnormal 2^-133, so 2^-134 (fp32 subnormal 0x00008000) and below store as 0
typedef St16<sgh_f16_to_f32, sgh_f32_to_f16, 0x33000000u> StF16;
typedef St16<sgh_bf16_to_f32, sgh_f32_to_bf16, 0x00008000u> StBF16;
typedef St16<sgh_f16_to_f32, sgh_f32_to_f16, 0x33000000u, true> StF16x4;
typedef St16<sgh_bf16_to_f32, sgh_f32_to_bf16, 0x00008000u, true> StBF16x4;

#endif  // SINGA_AMD_CSRC_STORAGE_H_
