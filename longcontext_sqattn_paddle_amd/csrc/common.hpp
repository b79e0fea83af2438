// Shared host/device helpers of libsqattn_hip.so (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <string.h>

#include <type_traits>

#include "sqattn.h"

namespace sq {

// ------------------------------------------------------------------------------------------ errors
void set_error(const char* fmt, ...);  // stores a thread-local message, defined in capi.hip

#define SQ_FAIL(code, ...)        \
  do {                            \
    ::sq::set_error(__VA_ARGS__); \
    return (code);                \
  } while (0)

#define SQ_REQUIRE(cond, code, ...)          \
  do {                                       \
    if (!(cond)) SQ_FAIL(code, __VA_ARGS__); \
  } while (0)

#define SQ_HIP(call)                                                                        \
  do {                                                                                      \
    hipError_t e__ = (call);                                                                \
    if (e__ != hipSuccess) SQ_FAIL(SQ_EHIP, "%s failed: %s", #call, hipGetErrorString(e__)); \
  } while (0)

// ------------------------------------------------------------------------------------ tensor views
enum class DType { BF16, F16, F32, I32, OTHER };

inline DType dtype_of(const DLTensor* t) {
  if (t->dtype.lanes != 1) return DType::OTHER;
  if (t->dtype.code == kDLBfloat && t->dtype.bits == 16) return DType::BF16;
  if (t->dtype.code == kDLFloat && t->dtype.bits == 16) return DType::F16;
  if (t->dtype.code == kDLFloat && t->dtype.bits == 32) return DType::F32;
  if (t->dtype.code == kDLInt && t->dtype.bits == 32) return DType::I32;
  return DType::OTHER;
}

inline int dtype_bytes(DType d) { return (d == DType::BF16 || d == DType::F16) ? 2 : 4; }

inline bool on_gpu(const DLTensor* t) {
  return t->device.device_type == kDLROCM || t->device.device_type == kDLCUDA;
}

inline int64_t stride_of(const DLTensor* t, int dim) {
  if (t->strides) return t->strides[dim];
  int64_t s = 1;
  for (int i = t->ndim - 1; i > dim; --i) s *= t->shape[i];
  return s;
}

inline char* data_of(const DLTensor* t) { return static_cast<char*>(t->data) + t->byte_offset; }

inline int64_t numel_of(const DLTensor* t) {
  int64_t n = 1;
  for (int i = 0; i < t->ndim; ++i) n *= t->shape[i];
  return n;
}

inline bool is_compact(const DLTensor* t) {
  int64_t s = 1;
  for (int i = t->ndim - 1; i >= 0; --i) {
    if (t->shape[i] != 1 && stride_of(t, i) != s) return false;
    s *= t->shape[i];
  }
  return true;
}

// Common checks of one tensor argument: non-null, on a GPU, expected rank, last dim contiguous,
// 16-byte aligned base.  Returns SQ_OK or an error code with the message set.
int check_tensor(const DLTensor* t, const char* name, int ndim, int device_id);

// ------------------------------------------------------------------------------------ device utils
#if defined(__HIPCC__)
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8_t;
typedef __attribute__((ext_vector_type(8))) _Float16 f16x8_t;
typedef __attribute__((ext_vector_type(4))) _Float16 f16x4_t;
typedef __attribute__((ext_vector_type(4))) float f32x4_t;
typedef __attribute__((ext_vector_type(16))) float f32x16_t;
typedef __attribute__((ext_vector_type(4))) int i32x4_t;
typedef __attribute__((ext_vector_type(2))) int i32x2_t;

__device__ __forceinline__ float bf16_bits_to_f32(uint32_t bits16) { return __uint_as_float(bits16 << 16); }

// round-to-nearest-even fp32 -> bf16 bit pattern (finite inputs)
// fp32 -> bf16, round to nearest even: gfx950 converts in hardware (v_cvt_pk_bf16_f32, two values per instruction),
// with the same bits as the add-0x7fff-plus-lsb sequence for every finite input
__device__ __forceinline__ uint32_t f32_to_bf16_bits(float x) {
  return (uint32_t)__builtin_bit_cast(uint16_t, (__bf16)x);
}
__device__ __forceinline__ uint32_t pack_bf16x2(float lo, float hi) {
  typedef __attribute__((ext_vector_type(2))) float f32x2_t;
  typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(f32x2_t{lo, hi}, bf16x2_t));
}

// e4m3 (OCP, max 448) round trip of a non-negative value <= 448: fp32 -> fp8 (RNE) -> fp32
__device__ __forceinline__ float e4m3_roundtrip(float x) {
  int pk = __builtin_amdgcn_cvt_pk_fp8_f32(x, x, 0, false);
  return __builtin_amdgcn_cvt_f32_fp8(pk, 0);
}

__device__ __forceinline__ float wave_xor_max(float v, int mask) { return fmaxf(v, __shfl_xor(v, mask)); }

// ---- division by a divisor that many dividends share.  A correctly rounded fp32 division is, on this hardware, a
// reciprocal estimate refined once, a first quotient and two residual corrections, wrapped in a range pre-scaling and
// a fix-up of special operands (zero, infinite, denormal divisors; quotients near the ends of the exponent range).
// Here the refined reciprocal is formed once per divisor and the wrapping is left out: the result equals n / d bit
// for bit as long as d is a normal number well inside the exponent range, and so are the quotients (callers state
// their ranges); n = +-0 gives +-0.
struct Divisor {
  float d, rcp;
};
__device__ __forceinline__ Divisor make_divisor(float d) {
#pragma clang fp contract(off)
  const float y0 = __builtin_amdgcn_rcpf(d);
  const float e = __builtin_fmaf(-d, y0, 1.0f);
  return Divisor{d, __builtin_fmaf(e, y0, y0)};
}
__device__ __forceinline__ float divide(float n, const Divisor& s) {
#pragma clang fp contract(off)
  const float q0 = n * s.rcp;
  const float r0 = __builtin_fmaf(-s.d, q0, n);
  const float q1 = __builtin_fmaf(r0, s.rcp, q0);
  const float r1 = __builtin_fmaf(-s.d, q1, n);
  return __builtin_fmaf(r1, s.rcp, q1);
}

// ---- x / d for x < 2^31 and a divisor fixed per launch, as one multiply-high, one add and one shift (d >= 1):
// m = ceil(2^(32+s) / d) - 2^32 with s = ceil(log2 d), set up on the host.  An integer division by a kernel argument is
// otherwise a software routine: some 30 vector instructions in 32 bits, a few hundred in 64.
struct FastDiv {
  uint32_t m, s, d;
};
inline FastDiv make_fastdiv(uint32_t d) {
  FastDiv f;
  f.d = d;
  f.s = 0;
  while ((1ull << f.s) < d) ++f.s;
  f.m = (uint32_t)((((1ull << (32 + f.s)) + d - 1) / d) - (1ull << 32));
  return f;
}
__device__ __forceinline__ uint32_t fastdiv(uint32_t x, const FastDiv& f) { return (__umulhi(x, f.m) + x) >> f.s; }

// ---- hand-scheduled LDS reads.  The compiler cannot tell that a ds_read never touches the buffers that
// global_load_lds copies are still filling, so it would stall every tile on vmcnt(0); reads issued through
// these helpers are invisible to that logic, and the data dependence is carried by lds_wait instead.
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4_t;
template <int OFF>
__device__ __forceinline__ u32x4_t lds_read128(uint32_t addr) {
  u32x4_t r;
  asm volatile("ds_read_b128 %0, %1 offset:%2" : "=v"(r) : "v"(addr), "n"(OFF));
  return r;
}
// wait until at most N LDS reads issued after the one that produced x (and y) are outstanding; LDS reads
// return in order, so x (and y) have landed afterwards
template <int N>
__device__ __forceinline__ void lds_wait(u32x4_t& x) {
  asm volatile("s_waitcnt lgkmcnt(%1)" : "+v"(x) : "n"(N));
}
template <int N>
__device__ __forceinline__ void lds_wait(u32x4_t& x, u32x4_t& y) {
  asm volatile("s_waitcnt lgkmcnt(%2)" : "+v"(x), "+v"(y) : "n"(N));
}
template <int I, int N, class F>
__device__ __forceinline__ void static_for(F&& f) {
  if constexpr (I < N) {
    f(std::integral_constant<int, I>{});
    static_for<I + 1, N>(f);
  }
}
#endif

}  // namespace sq
