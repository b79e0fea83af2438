// The three element-wise passes a decoder layer runs around the attention call, for gfx950 (MI355X).  They replace
// the tensor-expression helpers of the reference's model_hub/utils.py, each of which launches one kernel per
// operator and materialises every intermediate:
//   rmsnorm                                (utils.py:15-19, used by layernorm, model_hub/qwen.py:345-350)
//   silu_and_mul                           (utils.py:4-13,  used by mlp,       model_hub/qwen.py:319-326)
//   apply_rope_with_cos_sin_cache_inplace  (utils.py:21-106, used by apply_rotary_pos_emb, qwen.py:352-367)
// Each is one pass here: 16-byte loads, the arithmetic in registers with the reference's rounding points (every
// tensor operator of the reference rounds its result to the tensor dtype; the products with the fp32 cos/sin table
// are fp32), 16-byte stores.  All three are HBM-bound; algorithmic bytes = inputs read once + output written once.
#include "common.hpp"

namespace sq {
namespace {

template <bool BF16>
__device__ __forceinline__ float ld(uint32_t bits16) {
  if constexpr (BF16) return bf16_bits_to_f32(bits16);
  else return (float)__builtin_bit_cast(_Float16, (uint16_t)bits16);
}
// round an fp32 value to the tensor dtype and back (the rounding a tensor operator's output undergoes)
template <bool BF16>
__device__ __forceinline__ float rnd(float x) {
  if constexpr (BF16) return bf16_bits_to_f32(f32_to_bf16_bits(x));
  else return (float)(_Float16)x;
}
template <bool BF16>
__device__ __forceinline__ uint32_t st(float x) {
  if constexpr (BF16) return f32_to_bf16_bits(x);
  else return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)x);
}
template <bool BF16>
__device__ __forceinline__ void unpack8(const u32x4_t& w, float (&f)[8]) {
#pragma unroll
  for (int j = 0; j < 4; ++j) {
    f[2 * j] = ld<BF16>(w[j] & 0xffffu);
    f[2 * j + 1] = ld<BF16>(w[j] >> 16);
  }
}
template <bool BF16>
__device__ __forceinline__ u32x4_t pack8(const float (&f)[8]) {
  u32x4_t w;
#pragma unroll
  for (int j = 0; j < 4; ++j) w[j] = st<BF16>(f[2 * j]) | (st<BF16>(f[2 * j + 1]) << 16);
  return w;
}

// ---------------------------------------------------------------------------------------------- RMSNorm
// out = (x * rsqrt(mean(x^2) + eps)) * weight with the reference's five tensor operators (utils.py:17-19):
// square, mean (fp32 accumulation), + eps, rsqrt, x * r, * weight -- each rounded to the tensor dtype.
constexpr int kNormThreads = 256;    // four waves, each normalises one row: no LDS, no barrier
constexpr int kNormMaxChunks = 16;   // 16-byte chunks per lane held in registers: rows up to 8192 elements

struct NormArgs {
  const char* x;
  const char* w;
  char* out;
  int64_t x_sr, o_sr;   // row strides in bytes
  int64_t rows;
  int32_t dim;
  float eps;
};

template <bool BF16, int CHUNKS>   // CHUNKS = ceil(dim / 8 / 64): loads a lane keeps in flight
__global__ __launch_bounds__(kNormThreads) void rmsnorm_kernel(NormArgs a) {
  const int lane = threadIdx.x & 63;
  const int64_t row = (int64_t)blockIdx.x * (kNormThreads / 64) + (threadIdx.x >> 6);
  if (row >= a.rows) return;
  const int chunks = a.dim / 8;
  const char* xr = a.x + row * a.x_sr;
  u32x4_t v[CHUNKS];
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int ch = lane + c * 64;
    if (ch < chunks) v[c] = __builtin_nontemporal_load((const u32x4_t*)(xr + ch * 16));
  }
  // (the weight does not depend on the row's sum: requested here, it arrives while the lanes fold)
  u32x4_t wt[CHUNKS];
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int ch = lane + c * 64;
    if (ch < chunks) wt[c] = *(const u32x4_t*)(a.w + ch * 16);
  }
  // fixed association: the eight rounded squares of a chunk, the lane's chunk sums in ascending order, then the lanes
  // (the projections that carry this norm in front of them, linear_rows_kernel, form the same sums spread over waves)
  float sum = 0.f;
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    if (lane + c * 64 < chunks) {
      float f[8];
      unpack8<BF16>(v[c], f);
      float p = 0.f;
#pragma unroll
      for (int e = 0; e < 8; ++e) p += rnd<BF16>(f[e] * f[e]);
      sum += p;
    }
  }
#pragma unroll
  for (int m = 32; m > 0; m >>= 1) sum += __shfl_xor(sum, m);
  const float var = rnd<BF16>(sum / (float)a.dim);
  const float ve = rnd<BF16>(var + a.eps);
  const float r = rnd<BF16>(1.0f / sqrtf(ve));
  char* orow = a.out + row * a.o_sr;
#pragma unroll
  for (int c = 0; c < CHUNKS; ++c) {
    const int ch = lane + c * 64;
    if (ch < chunks) {
      float f[8], g[8];
      unpack8<BF16>(v[c], f);
      unpack8<BF16>(wt[c], g);
#pragma unroll
      for (int e = 0; e < 8; ++e) f[e] = rnd<BF16>(f[e] * r) * g[e];
      __builtin_nontemporal_store(pack8<BF16>(f), (u32x4_t*)(orow + ch * 16));
    }
  }
}

// ---------------------------------------------------------------------------------------------- SiLU * mul
// out = x2 * (x1 * sigmoid(x1)) for x = [x1 | x2] along the last dimension (utils.py:11-13): three tensor operators,
// each rounded to the tensor dtype.
struct ActArgs {
  const char* x;
  char* out;
  int64_t x_sr, o_sr;   // row strides in bytes
  int64_t rows;
  int32_t half_chunks;  // 16-byte chunks in one half of a row
};

template <bool BF16>
__global__ __launch_bounds__(256) void silu_mul_kernel(ActArgs a) {
  const int64_t total = a.rows * a.half_chunks;
  const int64_t stride = (int64_t)gridDim.x * blockDim.x;
  // two chunks per thread and iteration: four loads in flight before the arithmetic starts
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += 2 * stride) {
    u32x4_t w1[2], w2[2];
    int64_t off_out[2];
    bool live[2];
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      const int64_t ii = i + u * stride;
      live[u] = ii < total;
      const int64_t row = live[u] ? ii / a.half_chunks : 0;
      const int c = live[u] ? (int)(ii - row * a.half_chunks) : 0;
      const char* xr = a.x + row * a.x_sr;
      w1[u] = __builtin_nontemporal_load((const u32x4_t*)(xr + c * 16));
      w2[u] = __builtin_nontemporal_load((const u32x4_t*)(xr + (a.half_chunks + c) * 16));
      off_out[u] = row * a.o_sr + c * 16;
    }
#pragma unroll
    for (int u = 0; u < 2; ++u) {
      float f1[8], f2[8];
      unpack8<BF16>(w1[u], f1);
      unpack8<BF16>(w2[u], f2);
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        // v_exp_f32 and v_rcp_f32 (an ulp or two in fp32, far below the 16-bit rounding that follows)
        const float sg = rnd<BF16>(__builtin_amdgcn_rcpf(1.0f + __expf(-f1[e])));
        f1[e] = f2[e] * rnd<BF16>(f1[e] * sg);
      }
      if (live[u]) __builtin_nontemporal_store(pack8<BF16>(f1), (u32x4_t*)(a.out + off_out[u]));
    }
  }
}

// ---------------------------------------------------------------------------------------------- RoPE
// Rotation of the two halves of every head (utils.py:74-85) by the cos | sin rows of the token's position
// (:44-49): out1 = x1 cos - x2 sin, out2 = x1 sin + x2 cos, formed in fp32 (the table is fp32, so the reference's
// products and sums are fp32 tensor operators: no fused multiply-add) and rounded once to the tensor dtype.
struct RopeArgs {
  const char* q;
  const char* k;
  char* qo;
  char* ko;
  const void* pos;
  const float* table;   // [max_pos, head_dim]: cos in the first half of a row, sin in the second
  int64_t q_sr, k_sr, qo_sr, ko_sr;   // token strides in bytes
  int64_t tokens;
  int32_t q_heads, k_heads, half_chunks, max_pos, pos_is_i64;
};

constexpr int kRopeHeads = 4;   // heads per work item: one read of the cos/sin chunk serves four heads

template <bool BF16, typename IDX>   // IDX: 32-bit work-item index whenever the tensor allows it (cheaper divisions)
__global__ __launch_bounds__(256) void rope_kernel(RopeArgs a) {
  // work item = (token, group of up to four heads of q or of k, 16-byte chunk of a half head)
  const int q_groups = (a.q_heads + kRopeHeads - 1) / kRopeHeads, k_groups = (a.k_heads + kRopeHeads - 1) / kRopeHeads;
  const IDX per_token = (IDX)((q_groups + k_groups) * a.half_chunks);
  const IDX total = (IDX)a.tokens * per_token;
  const int half_bytes = a.half_chunks * 16;
  for (IDX i = (IDX)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (IDX)gridDim.x * blockDim.x) {
    const IDX t = i / per_token;
    const int j = (int)(i - t * per_token);
    const int gi = j / a.half_chunks, c = j - gi * a.half_chunks;
    const bool is_k = gi >= q_groups;
    const int h0 = (is_k ? gi - q_groups : gi) * kRopeHeads;
    const int nh = min(kRopeHeads, (is_k ? a.k_heads : a.q_heads) - h0);
    int64_t p = a.pos_is_i64 ? ((const int64_t*)a.pos)[t] : (int64_t)((const int32_t*)a.pos)[t];
    p = p < 0 ? 0 : (p >= a.max_pos ? a.max_pos - 1 : p);   // a position outside the table is the caller's error; the clamp keeps the read inside it
    const char* src = (is_k ? a.k + (int64_t)t * a.k_sr : a.q + (int64_t)t * a.q_sr) + (int64_t)h0 * 2 * half_bytes + c * 16;
    char* dst = (is_k ? a.ko + (int64_t)t * a.ko_sr : a.qo + (int64_t)t * a.qo_sr) + (int64_t)h0 * 2 * half_bytes + c * 16;
    u32x4_t w1[kRopeHeads], w2[kRopeHeads];
#pragma unroll
    for (int u = 0; u < kRopeHeads; ++u) {
      if (u < nh) {
        w1[u] = __builtin_nontemporal_load((const u32x4_t*)(src + u * 2 * half_bytes));
        w2[u] = __builtin_nontemporal_load((const u32x4_t*)(src + u * 2 * half_bytes + half_bytes));
      }
    }
    const float* row = a.table + p * (2 * 8 * a.half_chunks);
    float cs[8], sn[8];
    *(f32x4_t*)&cs[0] = *(const f32x4_t*)(row + 8 * c);
    *(f32x4_t*)&cs[4] = *(const f32x4_t*)(row + 8 * c + 4);
    *(f32x4_t*)&sn[0] = *(const f32x4_t*)(row + 8 * a.half_chunks + 8 * c);
    *(f32x4_t*)&sn[4] = *(const f32x4_t*)(row + 8 * a.half_chunks + 8 * c + 4);
#pragma unroll
    for (int u = 0; u < kRopeHeads; ++u) {
      if (u < nh) {
        float x1[8], x2[8];
        unpack8<BF16>(w1[u], x1);
        unpack8<BF16>(w2[u], x2);
        {
          // the reference's products and sums are separate fp32 operators: a fused multiply-add would round
          // differently (visibly so where the two products nearly cancel)
#pragma clang fp contract(off)
#pragma unroll
          for (int e = 0; e < 8; ++e) {
            const float a1 = x1[e] * cs[e], b1 = x2[e] * sn[e];
            const float a2 = x1[e] * sn[e], b2 = x2[e] * cs[e];
            x1[e] = a1 - b1;
            x2[e] = a2 + b2;
          }
        }
        __builtin_nontemporal_store(pack8<BF16>(x1), (u32x4_t*)(dst + u * 2 * half_bytes));
        __builtin_nontemporal_store(pack8<BF16>(x2), (u32x4_t*)(dst + u * 2 * half_bytes + half_bytes));
      }
    }
  }
}

int rows2d(const char* fn, const DLTensor* t, const char* name, int dev, DType dt, int64_t rows, int64_t cols) {
  int rc;
  if ((rc = check_tensor(t, name, 2, dev))) return rc;
  SQ_REQUIRE(dtype_of(t) == dt, SQ_EDTYPE, "%s: %s must have the dtype of the first tensor (bf16 or fp16)", fn, name);
  SQ_REQUIRE(t->shape[0] == rows && t->shape[1] == cols, SQ_ESHAPE, "%s: %s must be [%lld, %lld]", fn, name, (long long)rows, (long long)cols);
  SQ_REQUIRE(stride_of(t, 0) % 8 == 0 || rows == 1, SQ_ESHAPE, "%s: rows of %s are not 16-byte aligned", fn, name);
  return SQ_OK;
}

unsigned grid_for(int64_t items) {
  int64_t blocks = (items + 255) / 256;
  if (blocks > 256 * 16) blocks = 256 * 16;
  return (unsigned)(blocks < 1 ? 1 : blocks);
}

}  // namespace
}  // namespace sq

using namespace sq;

extern "C" int sq_rmsnorm(const DLTensor* x, const DLTensor* weight, DLTensor* out, float epsilon, void* stream) {
  const char* fn = "sq_rmsnorm";
  SQ_REQUIRE(x && weight && out, SQ_EINVAL, "%s: null tensor argument", fn);
  int rc;
  if ((rc = check_tensor(x, "x", 2, x->device.device_id))) return rc;
  const int dev = x->device.device_id;
  const DType dt = dtype_of(x);
  SQ_REQUIRE(dt == DType::BF16 || dt == DType::F16, SQ_EDTYPE, "%s: x must be bf16 or fp16", fn);
  const int64_t R = x->shape[0], dim = x->shape[1];
  SQ_REQUIRE(R > 0 && dim > 0, SQ_ESHAPE, "%s: empty tensor", fn);
  SQ_REQUIRE(dim % 8 == 0 && dim <= 8 * 64 * kNormMaxChunks, SQ_EUNSUPPORTED,
             "%s: the row length must be a multiple of 8 and at most %d (got %lld)", fn, 8 * 64 * kNormMaxChunks, (long long)dim);
  if ((rc = rows2d(fn, x, "x", dev, dt, R, dim)) || (rc = rows2d(fn, out, "out", dev, dt, R, dim))) return rc;
  if ((rc = check_tensor(weight, "weight", 1, dev))) return rc;
  SQ_REQUIRE(dtype_of(weight) == dt && weight->shape[0] == dim, SQ_ESHAPE, "%s: weight must be [%lld] of x's dtype", fn, (long long)dim);
  int cur = -1;
  SQ_HIP(hipGetDevice(&cur));
  SQ_REQUIRE(cur == dev, SQ_EDEVICE, "%s: tensors live on device %d but the current device is %d", fn, dev, cur);
  NormArgs a;
  a.x = data_of(x);
  a.w = data_of(weight);
  a.out = data_of(out);
  a.x_sr = stride_of(x, 0) * 2;
  a.o_sr = stride_of(out, 0) * 2;
  a.rows = R;
  a.dim = (int)dim;
  a.eps = epsilon;
  const int per_lane = (int)((dim / 8 + 63) / 64);
  const dim3 grid((unsigned)((R + kNormThreads / 64 - 1) / (kNormThreads / 64)));
  hipStream_t st = (hipStream_t)stream;
#define SQ_NORM_LAUNCH(C)                                                                                         \
  do {                                                                                                            \
    if (dt == DType::BF16) hipLaunchKernelGGL((rmsnorm_kernel<true, C>), grid, dim3(kNormThreads), 0, st, a);    \
    else hipLaunchKernelGGL((rmsnorm_kernel<false, C>), grid, dim3(kNormThreads), 0, st, a);                     \
  } while (0)
  if (per_lane <= 2) SQ_NORM_LAUNCH(2);
  else if (per_lane <= 4) SQ_NORM_LAUNCH(4);
  else if (per_lane <= 8) SQ_NORM_LAUNCH(8);
  else SQ_NORM_LAUNCH(16);
#undef SQ_NORM_LAUNCH
  SQ_HIP(hipGetLastError());
  return SQ_OK;
}

extern "C" int sq_silu_and_mul(const DLTensor* x, DLTensor* out, void* stream) {
  const char* fn = "sq_silu_and_mul";
  SQ_REQUIRE(x && out, SQ_EINVAL, "%s: null tensor argument", fn);
  int rc;
  if ((rc = check_tensor(x, "x", 2, x->device.device_id))) return rc;
  const int dev = x->device.device_id;
  const DType dt = dtype_of(x);
  SQ_REQUIRE(dt == DType::BF16 || dt == DType::F16, SQ_EDTYPE, "%s: x must be bf16 or fp16", fn);
  const int64_t R = x->shape[0], two = x->shape[1];
  SQ_REQUIRE(R > 0 && two > 0, SQ_ESHAPE, "%s: empty tensor", fn);
  SQ_REQUIRE(two % 16 == 0, SQ_EUNSUPPORTED, "%s: the row length must be a multiple of 16 (got %lld)", fn, (long long)two);
  if ((rc = rows2d(fn, x, "x", dev, dt, R, two)) || (rc = rows2d(fn, out, "out", dev, dt, R, two / 2))) return rc;
  int cur = -1;
  SQ_HIP(hipGetDevice(&cur));
  SQ_REQUIRE(cur == dev, SQ_EDEVICE, "%s: tensors live on device %d but the current device is %d", fn, dev, cur);
  ActArgs a;
  a.x = data_of(x);
  a.out = data_of(out);
  a.x_sr = stride_of(x, 0) * 2;
  a.o_sr = stride_of(out, 0) * 2;
  a.rows = R;
  a.half_chunks = (int)(two / 16);
  const unsigned grid = grid_for(R * a.half_chunks);
  if (dt == DType::BF16) hipLaunchKernelGGL(silu_mul_kernel<true>, dim3(grid), dim3(256), 0, (hipStream_t)stream, a);
  else hipLaunchKernelGGL(silu_mul_kernel<false>, dim3(grid), dim3(256), 0, (hipStream_t)stream, a);
  SQ_HIP(hipGetLastError());
  return SQ_OK;
}

extern "C" int sq_rope(const DLTensor* query, const DLTensor* key, DLTensor* query_out, DLTensor* key_out,
                       const DLTensor* position_ids, const DLTensor* cos_sin_cache, int32_t head_dim, void* stream) {
  const char* fn = "sq_rope";
  SQ_REQUIRE(query && key && query_out && key_out && position_ids && cos_sin_cache, SQ_EINVAL, "%s: null tensor argument", fn);
  int rc;
  if ((rc = check_tensor(query, "query", 2, query->device.device_id))) return rc;
  const int dev = query->device.device_id;
  const DType dt = dtype_of(query);
  SQ_REQUIRE(dt == DType::BF16 || dt == DType::F16, SQ_EDTYPE, "%s: query must be bf16 or fp16", fn);
  SQ_REQUIRE(head_dim > 0 && head_dim % 16 == 0, SQ_EUNSUPPORTED, "%s: head_dim must be a multiple of 16 (got %d)", fn, (int)head_dim);
  const int64_t T = query->shape[0], qd = query->shape[1];
  if ((rc = check_tensor(key, "key", 2, dev))) return rc;
  const int64_t kd = key->shape[1];
  SQ_REQUIRE(T > 0 && qd > 0 && kd > 0 && qd % head_dim == 0 && kd % head_dim == 0, SQ_ESHAPE,
             "%s: query [%lld, %lld] and key [.., %lld] must hold whole heads of %d", fn, (long long)T, (long long)qd, (long long)kd, (int)head_dim);
  if ((rc = rows2d(fn, query, "query", dev, dt, T, qd)) || (rc = rows2d(fn, key, "key", dev, dt, T, kd)) ||
      (rc = rows2d(fn, query_out, "query_out", dev, dt, T, qd)) || (rc = rows2d(fn, key_out, "key_out", dev, dt, T, kd)))
    return rc;
  SQ_REQUIRE(on_gpu(position_ids) && position_ids->device.device_id == dev && on_gpu(cos_sin_cache) && cos_sin_cache->device.device_id == dev,
             SQ_EDEVICE, "%s: position_ids and cos_sin_cache must live on the tensors' device", fn);
  const bool i64 = position_ids->dtype.code == kDLInt && position_ids->dtype.bits == 64 && position_ids->dtype.lanes == 1;
  SQ_REQUIRE((i64 || dtype_of(position_ids) == DType::I32) && numel_of(position_ids) == T && is_compact(position_ids), SQ_ESHAPE,
             "%s: position_ids must be a contiguous int32 or int64 tensor of %lld entries", fn, (long long)T);
  SQ_REQUIRE(dtype_of(cos_sin_cache) == DType::F32 && cos_sin_cache->ndim == 2 && cos_sin_cache->shape[1] == head_dim && is_compact(cos_sin_cache) &&
                 cos_sin_cache->shape[0] > 0 && cos_sin_cache->shape[0] < ((int64_t)1 << 31),
             SQ_ESHAPE, "%s: cos_sin_cache must be a contiguous fp32 [max_position, %d] table (cos | sin)", fn, (int)head_dim);
  SQ_REQUIRE(((uintptr_t)data_of(cos_sin_cache) & 15) == 0, SQ_ESHAPE, "%s: cos_sin_cache is not 16-byte aligned", fn);
  int cur = -1;
  SQ_HIP(hipGetDevice(&cur));
  SQ_REQUIRE(cur == dev, SQ_EDEVICE, "%s: tensors live on device %d but the current device is %d", fn, dev, cur);
  RopeArgs a;
  a.q = data_of(query);
  a.k = data_of(key);
  a.qo = data_of(query_out);
  a.ko = data_of(key_out);
  a.pos = data_of(position_ids);
  a.table = (const float*)data_of(cos_sin_cache);
  a.q_sr = stride_of(query, 0) * 2;
  a.k_sr = stride_of(key, 0) * 2;
  a.qo_sr = stride_of(query_out, 0) * 2;
  a.ko_sr = stride_of(key_out, 0) * 2;
  a.tokens = T;
  a.q_heads = (int)(qd / head_dim);
  a.k_heads = (int)(kd / head_dim);
  a.half_chunks = head_dim / 16;
  a.max_pos = (int)cos_sin_cache->shape[0];
  a.pos_is_i64 = i64 ? 1 : 0;
  const int64_t items = T * ((a.q_heads + kRopeHeads - 1) / kRopeHeads + (a.k_heads + kRopeHeads - 1) / kRopeHeads) * a.half_chunks;
  const unsigned grid = grid_for(items);
  const bool small = items < ((int64_t)1 << 30);
  hipStream_t st = (hipStream_t)stream;
  if (dt == DType::BF16) {
    if (small) hipLaunchKernelGGL((rope_kernel<true, uint32_t>), dim3(grid), dim3(256), 0, st, a);
    else hipLaunchKernelGGL((rope_kernel<true, int64_t>), dim3(grid), dim3(256), 0, st, a);
  } else {
    if (small) hipLaunchKernelGGL((rope_kernel<false, uint32_t>), dim3(grid), dim3(256), 0, st, a);
    else hipLaunchKernelGGL((rope_kernel<false, int64_t>), dim3(grid), dim3(256), 0, st, a);
  }
  SQ_HIP(hipGetLastError());
  return SQ_OK;
}
