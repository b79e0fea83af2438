// Measurement aid for gfx950 (MI355X), no counterpart in the reference: the rate the matrix cores sustain when a kernel
// issues nothing but MFMAs, with operands the caller supplies.  The published peaks (2.5 PFLOP/s bf16, 5.0 PFLOP/s fp8)
// hold for operands that do not change; with operands like the attention kernels' (random bf16 / e4m3 values) the chip
// lowers its clock under the matrix cores' switching power and the same loop runs a quarter slower.  bench.py reports
// that rate next to the published peak, so that a kernel's distance from the peak can be split into what the machine
// gives up on such data and what the kernel gives up.
//
// One workgroup of eight waves per CU (two per SIMD, as the prefill kernel runs), every lane loads four operand sets of
// 64 bytes once and then issues `iters` x 16 MFMAs on four accumulators: v_mfma_f32_32x32x16_bf16 (kind 0, a set = 16
// bytes of A + 16 of B, the rest unused) or v_mfma_f32_32x32x64_f8f6f4 on e4m3 (kind 1, 32 bytes of A + 32 of B).  The
// sums go to `sink` so that the loop cannot be removed; nothing else is written.
//
// Built into a library of its own, libsqattn_probe.so, next to the product library: it is loaded by the benchmark and
// its test only and is not part of the C ABI a maintainer binds.  Entry points:
//   size_t  sq_probe_mfma_operand_bytes(void)              bytes `operands` must hold (64 per lane and set, four sets per lane)
//   int64_t sq_probe_mfma_flops(int32_t kind, int32_t iters)  floating-point operations of one launch
//   int     sq_probe_mfma_rate(int32_t kind, const DLTensor* operands, DLTensor* sink, int32_t iters, void* stream)
//           kind 0 = v_mfma_f32_32x32x16_bf16, 1 = v_mfma_f32_32x32x64_f8f6f4 on e4m3; sink: fp32, at least 131072 elements;
//           iters at most kProbeMaxIters, which keeps one launch well under a second
#include "common.hpp"

namespace sq {
namespace {

typedef __attribute__((ext_vector_type(8))) int i32x8_t;
constexpr int kProbeGroups = 256, kProbeThreads = 512, kProbeSets = 4, kProbeSetBytes = 64;
constexpr int kProbeMaxIters = 1 << 18;   // 4 M MFMAs per wave: about 0.15 s per launch

template <int KIND>
__global__ __launch_bounds__(kProbeThreads) void probe_mfma_kernel(const uint32_t* src, float* sink, int iters) {
  u32x4_t a[kProbeSets], b[kProbeSets];
  i32x8_t a8[kProbeSets], b8[kProbeSets];
#pragma unroll
  for (int s = 0; s < kProbeSets; ++s) {
    const uint32_t* p = src + ((size_t)(blockIdx.x * kProbeThreads + threadIdx.x) * kProbeSets + s) * (kProbeSetBytes / 4);
    a[s] = *(const u32x4_t*)p;
    b[s] = *(const u32x4_t*)(p + 4);
#pragma unroll
    for (int i = 0; i < 8; ++i) {
      a8[s][i] = (int)p[i];
      b8[s][i] = (int)p[8 + i];
    }
  }
  f32x16_t acc[4];
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int i = 0; i < 16; ++i) acc[j][i] = 0.f;
  for (int it = 0; it < iters; ++it) {
#pragma unroll
    for (int s = 0; s < 16; ++s) {
      if constexpr (KIND == 0)
        asm volatile("v_mfma_f32_32x32x16_bf16 %0, %1, %2, %0" : "+v"(acc[s & 3]) : "v"(a[s & 3]), "v"(b[(s >> 2) & 3]));
      else
        asm volatile("v_mfma_f32_32x32x64_f8f6f4 %0, %1, %2, %0" : "+v"(acc[s & 3]) : "v"(a8[s & 3]), "v"(b8[(s >> 2) & 3]));
    }
  }
  // The MFMAs above are opaque asm statements, so the compiler does not know that the matrix pipe is still writing the
  // accumulators: the wait states between the last MFMA and the first read are supplied by hand (a 16-pass MFMA needs
  // fewer than 32).
#pragma unroll
  for (int j = 0; j < 4; ++j) asm volatile("s_nop 15\n\ts_nop 15" : "+v"(acc[j]));
  float r = 0.f;
#pragma unroll
  for (int j = 0; j < 4; ++j)
#pragma unroll
    for (int i = 0; i < 16; ++i) r += acc[j][i];
  sink[blockIdx.x * kProbeThreads + threadIdx.x] = r;
}

}  // namespace
}  // namespace sq

using namespace sq;

extern "C" size_t sq_probe_mfma_operand_bytes(void) { return (size_t)kProbeGroups * kProbeThreads * kProbeSets * kProbeSetBytes; }

extern "C" int64_t sq_probe_mfma_flops(int32_t kind, int32_t iters) {
  return (int64_t)kProbeGroups * (kProbeThreads / 64) * iters * 16 * (kind == 1 ? 131072 : 32768);
}

extern "C" int sq_probe_mfma_rate(int32_t kind, const DLTensor* operands, DLTensor* sink, int32_t iters, void* stream) {
  const char* fn = "sq_probe_mfma_rate";
  SQ_REQUIRE(kind == 0 || kind == 1, SQ_EINVAL, "%s: kind must be 0 (bf16 32x32x16) or 1 (e4m3 32x32x64), got %d", fn, (int)kind);
  SQ_REQUIRE(operands && sink, SQ_EINVAL, "%s: null tensor argument", fn);
  SQ_REQUIRE(iters > 0 && iters <= kProbeMaxIters, SQ_EINVAL, "%s: iters must be in 1 .. %d (got %d)", fn, kProbeMaxIters, (int)iters);
  int rc;
  if ((rc = check_tensor(operands, "operands", 1, operands->device.device_id))) return rc;
  const int dev = operands->device.device_id;
  if ((rc = check_tensor(sink, "sink", 1, dev))) return rc;
  const int64_t need = (int64_t)sq_probe_mfma_operand_bytes();
  SQ_REQUIRE(operands->dtype.lanes == 1 && operands->shape[0] * (operands->dtype.bits / 8) >= need && stride_of(operands, 0) == 1, SQ_ESHAPE,
             "%s: operands must be a contiguous tensor of at least %lld bytes", fn, (long long)need);
  SQ_REQUIRE(dtype_of(sink) == DType::F32 && sink->shape[0] >= kProbeGroups * kProbeThreads && stride_of(sink, 0) == 1, SQ_ESHAPE,
             "%s: sink must be a contiguous fp32 tensor of at least %d elements", fn, kProbeGroups * kProbeThreads);
  int cur = -1;
  SQ_HIP(hipGetDevice(&cur));
  SQ_REQUIRE(cur == dev, SQ_EDEVICE, "%s: tensors live on device %d but the current device is %d", fn, dev, cur);
  const uint32_t* src = (const uint32_t*)data_of(operands);
  float* out = (float*)data_of(sink);
  if (kind == 0) hipLaunchKernelGGL(probe_mfma_kernel<0>, dim3(kProbeGroups), dim3(kProbeThreads), 0, (hipStream_t)stream, src, out, (int)iters);
  else hipLaunchKernelGGL(probe_mfma_kernel<1>, dim3(kProbeGroups), dim3(kProbeThreads), 0, (hipStream_t)stream, src, out, (int)iters);
  SQ_HIP(hipGetLastError());
  return SQ_OK;
}
