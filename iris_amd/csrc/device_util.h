// Device helpers shared by the kernels of libiris_hip: heap-slot address translation, 16-bit float
// conversions, element-type traits and atomic adds.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "iris_hip.h"

// Address of `p` (a pointer into slot `from`) in slot `to`.
__device__ __forceinline__ char* slot_ptr(const long long* heap_bases, const void* p, int from, int to) {
  unsigned long long off = (unsigned long long)p - (unsigned long long)heap_bases[from];
  return (char*)((unsigned long long)heap_bases[to] + off);
}

__device__ __forceinline__ float bf16_bits_to_float(unsigned short b) { return __uint_as_float(((unsigned)b) << 16); }

__device__ __forceinline__ unsigned short float_to_bf16_bits(float f) {
  __bf16 h = (__bf16)f;  // round to nearest even; v_cvt_pk_bf16_f32 on gfx950
  return __builtin_bit_cast(unsigned short, h);
}
__device__ __forceinline__ unsigned short float_to_f16_bits(float f) {
  _Float16 h = (_Float16)f;
  return __builtin_bit_cast(unsigned short, h);
}
__device__ __forceinline__ float f16_bits_to_float(unsigned short b) {
  return (float)__builtin_bit_cast(_Float16, b);
}

// Two floats rounded (to nearest even) and packed into one word, `lo` in the low half: one
// v_cvt_pk_bf16_f32 / v_cvt_pk_f16_f32 instead of two conversions and a merge.
typedef __attribute__((ext_vector_type(2))) float f32x2_t;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
typedef __attribute__((ext_vector_type(2))) _Float16 half2_t;
__device__ __forceinline__ unsigned pack_bf16(float lo, float hi) {
  f32x2_t v = {lo, hi};
  return __builtin_bit_cast(unsigned, __builtin_convertvector(v, bf16x2_t));
}
__device__ __forceinline__ unsigned pack_f16(float lo, float hi) {
  f32x2_t v = {lo, hi};
  return __builtin_bit_cast(unsigned, __builtin_convertvector(v, half2_t));
}

// Output element kinds of the 16-bit epilogue.
struct OutBF16 {
  static __device__ __forceinline__ float to_float(unsigned short b) { return bf16_bits_to_float(b); }
  static __device__ __forceinline__ unsigned short from_float(float f) { return float_to_bf16_bits(f); }
  static __device__ __forceinline__ unsigned pack(float lo, float hi) { return pack_bf16(lo, hi); }
  static constexpr bool kFp32SumInReference = false;
};
struct OutF16 {
  static __device__ __forceinline__ float to_float(unsigned short b) { return f16_bits_to_float(b); }
  static __device__ __forceinline__ unsigned short from_float(float f) { return float_to_f16_bits(f); }
  static __device__ __forceinline__ unsigned pack(float lo, float hi) { return pack_f16(lo, hi); }
  static constexpr bool kFp32SumInReference = true;
};

// Atomically add two packed 16-bit floats (one 32-bit word) to memory.
typedef __attribute__((ext_vector_type(2))) short s16x2_t;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2_t;
template <class Out>
__device__ __forceinline__ void atomic_add_packed(char* addr, unsigned word) {
  if constexpr (Out::kFp32SumInReference)  // float16
    __builtin_amdgcn_global_atomic_fadd_v2f16((__attribute__((address_space(1))) f16x2_t*)addr,
                                              __builtin_bit_cast(f16x2_t, word));
  else
    __builtin_amdgcn_global_atomic_fadd_v2bf16((__attribute__((address_space(1))) s16x2_t*)addr,
                                               __builtin_bit_cast(s16x2_t, word));
}

__device__ __forceinline__ float load_scalar_as_float(const char* base, long long idx, int dtype) {
  if (dtype == IRIS_HIP_FP32) return ((const float*)base)[idx];
  unsigned short b = ((const unsigned short*)base)[idx];
  return dtype == IRIS_HIP_BF16 ? bf16_bits_to_float(b) : f16_bits_to_float(b);
}

// Atomic add of one 16-bit float: compare-and-swap on the aligned 32-bit word that contains it.
template <class E>
__device__ __forceinline__ void atomic_add_half(char* p, float f) {
  unsigned* word = (unsigned*)((unsigned long long)p & ~3ull);
  const int shift = ((unsigned long long)p & 2) ? 16 : 0;
  unsigned old = *word, assumed;
  do {
    assumed = old;
    unsigned short cur = (unsigned short)(assumed >> shift);
    float sum = E::load((const char*)&cur) + f;
    unsigned short nv;
    E::store((char*)&nv, sum);
    const unsigned repl = (assumed & ~(0xFFFFu << shift)) | ((unsigned)nv << shift);
    old = atomicCAS(word, assumed, repl);
  } while (old != assumed);
}

struct ElemBF16 {
  static constexpr int size = 2;
  static __device__ __forceinline__ float load(const char* p) { return bf16_bits_to_float(*(const unsigned short*)p); }
  static __device__ __forceinline__ void store(char* p, float f) { *(unsigned short*)p = float_to_bf16_bits(f); }
  static __device__ __forceinline__ float round(float f) { return bf16_bits_to_float(float_to_bf16_bits(f)); }
  static __device__ __forceinline__ void atomic_add(char* p, float f) { atomic_add_half<ElemBF16>(p, f); }
  static constexpr bool kFp32SumInReference = false;
};
struct ElemF16 {
  static constexpr int size = 2;
  static __device__ __forceinline__ float load(const char* p) { return f16_bits_to_float(*(const unsigned short*)p); }
  static __device__ __forceinline__ void store(char* p, float f) { *(unsigned short*)p = float_to_f16_bits(f); }
  static __device__ __forceinline__ float round(float f) { return f16_bits_to_float(float_to_f16_bits(f)); }
  static __device__ __forceinline__ void atomic_add(char* p, float f) { atomic_add_half<ElemF16>(p, f); }
  static constexpr bool kFp32SumInReference = true;
};
struct ElemF32 {
  static constexpr int size = 4;
  static __device__ __forceinline__ float load(const char* p) { return *(const float*)p; }
  static __device__ __forceinline__ void store(char* p, float f) { *(float*)p = f; }
  static __device__ __forceinline__ float round(float f) { return f; }
  static __device__ __forceinline__ void atomic_add(char* p, float f) { atomicAdd((float*)p, f); }
  static constexpr bool kFp32SumInReference = false;  // fp32 data sums in fp32 either way
};
struct ElemFP8 {
  static constexpr int size = 1;
  static __device__ __forceinline__ float load(const char* p) {
    return __builtin_amdgcn_cvt_f32_fp8((int)*(const unsigned char*)p, 0);
  }
};

