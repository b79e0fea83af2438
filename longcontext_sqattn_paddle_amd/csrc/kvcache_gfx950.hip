// KV-cache row movement for gfx950 (MI355X): the two tensor updates of the reference's cache object,
// cache_hub/flash_attn_cache.py:
//   prefill_update_kv_cache (:153-232)  cache[layer][b, 0:n] = states[0, valid_start:valid_start+n]   (K and V)
//   decode_update_kv_cache  (:239-256)  cache[layer][b, valid_length[b]] = states[b, 0] for every b, and
//                                       valid_length += 1 after the last layer
// The cache of one layer is [B, max_length, Hkv, D] (token-major, "NHD", :60-81): a token is one contiguous row of
// Hkv*D elements (1 KB for 4 kv heads of 128 bf16), which is also what the decode attention kernel streams.
//
// Both are pure HBM row copies, done with 16-byte accesses, K and V in one launch:
//   * store: one 16-byte chunk per thread, grid-stride over rows x chunks; source rows may be strided (a view into
//     a fused projection output), cache rows are contiguous.  Algorithmic bytes: 2 tensors x n rows x row bytes,
//     each read once and written once.
//   * append: one workgroup per sequence copies the K row and the V row to position valid_length[b], then
//     publishes attend_length[b] = position + 1 (what the attention of this step covers) and, when `advance` is
//     set, valid_length[b] = position + 1.  No host synchronisation: the lengths never leave the device.
//   * reorder (no reference counterpart): a copy of a layer's cache with every kv head's rows permuted, e.g. into the
//     order of its k-means clusters, so that a selection of whole clusters reads runs of neighbouring rows instead
//     of scattered ones.
#include "common.hpp"

namespace sq {
namespace {

struct StoreArgs {
  const char* k_src;
  const char* v_src;
  char* k_dst;
  char* v_dst;
  int64_t k_sn, k_sh, v_sn, v_sh;   // source strides in bytes (token, head); the D elements of a head are contiguous
  int64_t n;                        // rows to copy
  int32_t heads, head_chunks;       // kv heads, 16-byte chunks per head (D * 2 / 16)
};

__global__ __launch_bounds__(256) void kv_store_kernel(StoreArgs a) {
  const int64_t row_chunks = (int64_t)a.heads * a.head_chunks;
  const int64_t total = 2 * a.n * row_chunks;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < total; i += (int64_t)gridDim.x * blockDim.x) {
    const bool is_v = i >= a.n * row_chunks;
    const int64_t j = is_v ? i - a.n * row_chunks : i;
    const int64_t row = j / row_chunks;
    const int c = (int)(j - row * row_chunks);
    const int h = c / a.head_chunks, cc = c - h * a.head_chunks;
    const char* src = is_v ? a.v_src + row * a.v_sn + h * a.v_sh : a.k_src + row * a.k_sn + h * a.k_sh;
    char* dst = (is_v ? a.v_dst : a.k_dst) + (row * row_chunks + c) * 16;
    const u32x4_t w = __builtin_nontemporal_load((const u32x4_t*)(src + cc * 16));   // streamed once: keep it out of L2's way
    __builtin_nontemporal_store(w, (u32x4_t*)dst);
  }
}

struct AppendArgs {
  const char* k_src;
  const char* v_src;
  char* k_dst;
  char* v_dst;
  int64_t k_sb, k_sh, v_sb, v_sh;   // source strides in bytes (sequence, head)
  int64_t kc_sb, vc_sb;             // cache strides in bytes per sequence
  int32_t* valid_length;            // [B]
  int32_t* attend_length;           // [B] or null
  int32_t max_length, heads, head_chunks, advance;
};

__global__ __launch_bounds__(128) void kv_append_kernel(AppendArgs a) {
  const int b = blockIdx.x;
  const int pos = a.valid_length[b];
  const int row_chunks = a.heads * a.head_chunks;
  const int64_t row_bytes = (int64_t)row_chunks * 16;
  if (pos >= 0 && pos < a.max_length) {   // a full sequence stays as it is; the host refuses the call before that
    for (int i = threadIdx.x; i < 2 * row_chunks; i += blockDim.x) {
      const bool is_v = i >= row_chunks;
      const int c = is_v ? i - row_chunks : i;
      const int h = c / a.head_chunks, cc = c - h * a.head_chunks;
      const char* src = is_v ? a.v_src + b * a.v_sb + h * a.v_sh : a.k_src + b * a.k_sb + h * a.k_sh;
      char* dst = is_v ? a.v_dst + b * a.vc_sb : a.k_dst + b * a.kc_sb;
      *(uint4*)(dst + pos * row_bytes + c * 16) = *(const uint4*)(src + cc * 16);
    }
  }
  __syncthreads();   // every thread has read valid_length[b] before it may change
  if (threadIdx.x == 0) {
    const int next = pos < a.max_length ? pos + 1 : pos;
    if (a.attend_length) a.attend_length[b] = next;
    if (a.advance) a.valid_length[b] = next;
  }
}

struct ReorderArgs {
  const char* k_src;
  const char* v_src;
  char* k_dst;
  char* v_dst;
  const int32_t* order;             // [B * heads, n]
  int64_t n, src_len;               // rows per head in the copy, rows per sequence in the source
  int32_t batch, heads, head_chunks;
};

// One 16-byte chunk per thread: chunk (b, p, h, cc) of the copy comes from row order[b * heads + h][p] of head h.
// Writes are contiguous; reads are one 256-byte head row per 16 lanes.  Ids outside [0, src_len) give zero rows.
__global__ __launch_bounds__(256) void kv_reorder_kernel(ReorderArgs a) {
  const int64_t row_chunks = (int64_t)a.heads * a.head_chunks;
  const int64_t per_tensor = (int64_t)a.batch * a.n * row_chunks;
  for (int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x; i < 2 * per_tensor; i += (int64_t)gridDim.x * blockDim.x) {
    const bool is_v = i >= per_tensor;
    const int64_t j = is_v ? i - per_tensor : i;
    const int64_t row = j / row_chunks;                 // b * n + p
    const int c = (int)(j - row * row_chunks);
    const int h = c / a.head_chunks;
    const int64_t b = row / a.n, p = row - b * a.n;
    const int32_t id = a.order[(b * a.heads + h) * a.n + p];
    u32x4_t w = {0u, 0u, 0u, 0u};
    if (id >= 0 && id < a.src_len) w = __builtin_nontemporal_load((const u32x4_t*)((is_v ? a.v_src : a.k_src) + ((b * a.src_len + id) * row_chunks + c) * 16));
    __builtin_nontemporal_store(w, (u32x4_t*)((is_v ? a.v_dst : a.k_dst) + j * 16));
  }
}

// states [B, T, Hkv, D] (any strides with contiguous D, 16-byte aligned heads); cache [B, L, Hkv, D] compact
int check_pair(const char* fn, const DLTensor* s, const char* sname, const DLTensor* c, const char* cname, int dev, DType dt) {
  int rc;
  if ((rc = check_tensor(s, sname, 4, dev)) || (rc = check_tensor(c, cname, 4, dev))) return rc;
  SQ_REQUIRE(dtype_of(s) == dt && dtype_of(c) == dt, SQ_EDTYPE, "%s: %s and %s must share one 16-bit dtype (bf16 or fp16)", fn, sname, cname);
  SQ_REQUIRE(s->shape[2] == c->shape[2] && s->shape[3] == c->shape[3], SQ_ESHAPE, "%s: %s and %s differ in heads or head_dim", fn, sname, cname);
  SQ_REQUIRE(is_compact(c), SQ_ESHAPE, "%s: %s must be contiguous [B, max_length, Hkv, D]", fn, cname);
  SQ_REQUIRE(s->shape[3] % 8 == 0, SQ_EUNSUPPORTED, "%s: head_dim must be a multiple of 8", fn);
  for (int d = 0; d < 3; ++d)
    SQ_REQUIRE(stride_of(s, d) % 8 == 0 || s->shape[d] == 1, SQ_ESHAPE, "%s: heads of %s are not 16-byte aligned", fn, sname);
  return SQ_OK;
}

}  // namespace
}  // namespace sq

using namespace sq;

extern "C" int sq_kv_cache_store(const DLTensor* key_states, const DLTensor* value_states, DLTensor* key_cache,
                                 DLTensor* value_cache, int32_t batch_index, int64_t valid_start, void* stream) {
  const char* fn = "sq_kv_cache_store";
  SQ_REQUIRE(key_states && value_states && key_cache && value_cache, SQ_EINVAL, "%s: null tensor argument", fn);
  int rc;
  if ((rc = check_tensor(key_states, "key_states", 4, key_states->device.device_id))) return rc;
  const int dev = key_states->device.device_id;
  const DType dt = dtype_of(key_states);
  SQ_REQUIRE(dt == DType::BF16 || dt == DType::F16, SQ_EDTYPE, "%s: key_states must be bf16 or fp16", fn);
  if ((rc = check_pair(fn, key_states, "key_states", key_cache, "key_cache", dev, dt)) ||
      (rc = check_pair(fn, value_states, "value_states", value_cache, "value_cache", dev, dt)))
    return rc;
  // "Multi-batch prefilling only support prefill single batch one by one" (flash_attn_cache.py:166-169)
  SQ_REQUIRE(key_states->shape[0] == 1 && value_states->shape[0] == 1, SQ_ESHAPE, "%s: prefill stores one sequence per call (batch %lld given)", fn,
             (long long)key_states->shape[0]);
  const int64_t T = key_states->shape[1], L = key_cache->shape[1], Bc = key_cache->shape[0];
  SQ_REQUIRE(value_states->shape[1] == T && value_states->shape[2] == key_states->shape[2] && value_states->shape[3] == key_states->shape[3],
             SQ_ESHAPE, "%s: key_states and value_states differ in shape", fn);
  SQ_REQUIRE(value_cache->shape[0] == Bc && value_cache->shape[1] == L, SQ_ESHAPE, "%s: key_cache and value_cache differ in shape", fn);
  SQ_REQUIRE(batch_index >= 0 && batch_index < Bc, SQ_EINVAL, "%s: batch index %d outside the cache's %lld sequences", fn, (int)batch_index, (long long)Bc);
  // "Prefilling sequence length exceeds max length" (:170-172)
  SQ_REQUIRE(T <= L, SQ_ESHAPE, "Prefilling sequence length %lld exceeds max length %lld.", (long long)T, (long long)L);
  SQ_REQUIRE(valid_start >= 0 && valid_start <= T, SQ_EINVAL, "%s: valid_start %lld outside [0, %lld]", fn, (long long)valid_start, (long long)T);
  int cur = -1;
  SQ_HIP(hipGetDevice(&cur));
  SQ_REQUIRE(cur == dev, SQ_EDEVICE, "%s: tensors live on device %d but the current device is %d", fn, dev, cur);
  const int64_t n = T - valid_start;
  if (n == 0) return SQ_OK;
  const int64_t H = key_states->shape[2], D = key_states->shape[3];
  StoreArgs a;
  a.k_sn = stride_of(key_states, 1) * 2;
  a.k_sh = stride_of(key_states, 2) * 2;
  a.v_sn = stride_of(value_states, 1) * 2;
  a.v_sh = stride_of(value_states, 2) * 2;
  a.k_src = data_of(key_states) + valid_start * a.k_sn;
  a.v_src = data_of(value_states) + valid_start * a.v_sn;
  a.k_dst = data_of(key_cache) + (int64_t)batch_index * L * H * D * 2;
  a.v_dst = data_of(value_cache) + (int64_t)batch_index * L * H * D * 2;
  a.n = n;
  a.heads = (int)H;
  a.head_chunks = (int)(D / 8);
  const int64_t chunks = 2 * n * H * (D / 8);
  int64_t blocks = (chunks + 1023) / 1024;   // about four chunks per thread, at most 32 workgroups per CU
  if (blocks > 8192) blocks = 8192;
  hipLaunchKernelGGL(kv_store_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, a);
  SQ_HIP(hipGetLastError());
  return SQ_OK;
}

extern "C" int sq_kv_cache_append(const DLTensor* key_states, const DLTensor* value_states, DLTensor* key_cache,
                                  DLTensor* value_cache, DLTensor* valid_length, DLTensor* attend_length, int32_t advance,
                                  void* stream) {
  const char* fn = "sq_kv_cache_append";
  SQ_REQUIRE(key_states && value_states && key_cache && value_cache && valid_length, SQ_EINVAL, "%s: null tensor argument", fn);
  int rc;
  if ((rc = check_tensor(key_states, "key_states", 4, key_states->device.device_id))) return rc;
  const int dev = key_states->device.device_id;
  const DType dt = dtype_of(key_states);
  SQ_REQUIRE(dt == DType::BF16 || dt == DType::F16, SQ_EDTYPE, "%s: key_states must be bf16 or fp16", fn);
  if ((rc = check_pair(fn, key_states, "key_states", key_cache, "key_cache", dev, dt)) ||
      (rc = check_pair(fn, value_states, "value_states", value_cache, "value_cache", dev, dt)))
    return rc;
  const int64_t B = key_cache->shape[0], L = key_cache->shape[1], H = key_cache->shape[2], D = key_cache->shape[3];
  SQ_REQUIRE(key_states->shape[0] == B && value_states->shape[0] == B && key_states->shape[1] == 1 && value_states->shape[1] == 1, SQ_ESHAPE,
             "%s: key_states and value_states must be [%lld, 1, Hkv, D] (one new token per cached sequence)", fn, (long long)B);
  SQ_REQUIRE(value_states->shape[2] == H && value_states->shape[3] == D && value_cache->shape[0] == B && value_cache->shape[1] == L, SQ_ESHAPE,
             "%s: key and value tensors differ in shape", fn);
  SQ_REQUIRE(L < ((int64_t)1 << 31) && B < 65536, SQ_EUNSUPPORTED, "%s: cache too large", fn);
  DLTensor* lens[2] = {valid_length, attend_length};
  for (int i = 0; i < 2; ++i) {
    const DLTensor* t = lens[i];
    if (!t) continue;
    SQ_REQUIRE(on_gpu(t) && t->device.device_id == dev, SQ_EDEVICE, "%s: length tensors must live on the cache's device", fn);
    SQ_REQUIRE(dtype_of(t) == DType::I32 && t->ndim == 1 && t->shape[0] == B && is_compact(t), SQ_ESHAPE,
               "%s: length tensors must be contiguous int32 [%lld]", fn, (long long)B);
  }
  int cur = -1;
  SQ_HIP(hipGetDevice(&cur));
  SQ_REQUIRE(cur == dev, SQ_EDEVICE, "%s: tensors live on device %d but the current device is %d", fn, dev, cur);
  AppendArgs a;
  a.k_src = data_of(key_states);
  a.v_src = data_of(value_states);
  a.k_dst = data_of(key_cache);
  a.v_dst = data_of(value_cache);
  a.k_sb = stride_of(key_states, 0) * 2;
  a.k_sh = stride_of(key_states, 2) * 2;
  a.v_sb = stride_of(value_states, 0) * 2;
  a.v_sh = stride_of(value_states, 2) * 2;
  a.kc_sb = L * H * D * 2;
  a.vc_sb = L * H * D * 2;
  a.valid_length = (int32_t*)data_of(valid_length);
  a.attend_length = attend_length ? (int32_t*)data_of(attend_length) : nullptr;
  a.max_length = (int)L;
  a.heads = (int)H;
  a.head_chunks = (int)(D / 8);
  a.advance = advance;
  hipLaunchKernelGGL(kv_append_kernel, dim3((unsigned)B), dim3(128), 0, (hipStream_t)stream, a);
  SQ_HIP(hipGetLastError());
  return SQ_OK;
}

extern "C" int sq_kv_cache_reorder(const DLTensor* key_cache, const DLTensor* value_cache, const DLTensor* order, DLTensor* key_out,
                                   DLTensor* value_out, void* stream) {
  const char* fn = "sq_kv_cache_reorder";
  SQ_REQUIRE(key_cache && value_cache && order && key_out && value_out, SQ_EINVAL, "%s: null tensor argument", fn);
  int rc;
  if ((rc = check_tensor(key_cache, "key_cache", 4, key_cache->device.device_id))) return rc;
  const int dev = key_cache->device.device_id;
  const DType dt = dtype_of(key_cache);
  SQ_REQUIRE(dt == DType::BF16 || dt == DType::F16, SQ_EDTYPE, "%s: key_cache must be bf16 or fp16", fn);
  const DLTensor* all[4] = {key_cache, value_cache, key_out, value_out};
  const char* names[4] = {"key_cache", "value_cache", "key_out", "value_out"};
  for (int i = 0; i < 4; ++i) {
    if ((rc = check_tensor(all[i], names[i], 4, dev))) return rc;
    SQ_REQUIRE(dtype_of(all[i]) == dt, SQ_EDTYPE, "%s: %s must have key_cache's dtype", fn, names[i]);
    SQ_REQUIRE(is_compact(all[i]), SQ_ESHAPE, "%s: %s must be contiguous [B, rows, Hkv, D]", fn, names[i]);
    SQ_REQUIRE(all[i]->shape[0] == key_cache->shape[0] && all[i]->shape[2] == key_cache->shape[2] && all[i]->shape[3] == key_cache->shape[3],
               SQ_ESHAPE, "%s: %s differs from key_cache in batch, heads or head_dim", fn, names[i]);
  }
  const int64_t B = key_cache->shape[0], L = key_cache->shape[1], H = key_cache->shape[2], D = key_cache->shape[3], n = key_out->shape[1];
  SQ_REQUIRE(value_cache->shape[1] == L && value_out->shape[1] == n, SQ_ESHAPE, "%s: key and value tensors differ in rows", fn);
  SQ_REQUIRE(D % 8 == 0, SQ_EUNSUPPORTED, "%s: head_dim must be a multiple of 8", fn);
  SQ_REQUIRE(on_gpu(order) && order->device.device_id == dev, SQ_EDEVICE, "%s: order must live on the cache's device", fn);
  SQ_REQUIRE(dtype_of(order) == DType::I32 && order->ndim == 2 && order->shape[0] == B * H && order->shape[1] == n && is_compact(order), SQ_ESHAPE,
             "%s: order must be contiguous int32 [%lld, %lld]", fn, (long long)(B * H), (long long)n);
  SQ_REQUIRE(L < ((int64_t)1 << 31) && n < ((int64_t)1 << 31), SQ_EUNSUPPORTED, "%s: cache too large", fn);
  int cur = -1;
  SQ_HIP(hipGetDevice(&cur));
  SQ_REQUIRE(cur == dev, SQ_EDEVICE, "%s: tensors live on device %d but the current device is %d", fn, dev, cur);
  if (n == 0 || B == 0) return SQ_OK;
  ReorderArgs a;
  a.k_src = data_of(key_cache);
  a.v_src = data_of(value_cache);
  a.k_dst = data_of(key_out);
  a.v_dst = data_of(value_out);
  a.order = (const int32_t*)data_of(order);
  a.n = n;
  a.src_len = L;
  a.batch = (int32_t)B;
  a.heads = (int32_t)H;
  a.head_chunks = (int32_t)(D / 8);
  const int64_t chunks = 2 * B * n * H * (D / 8);
  int64_t blocks = (chunks + 1023) / 1024;
  if (blocks > 8192) blocks = 8192;
  hipLaunchKernelGGL(kv_reorder_kernel, dim3((unsigned)blocks), dim3(256), 0, (hipStream_t)stream, a);
  SQ_HIP(hipGetLastError());
  return SQ_OK;
}
