// Calibration histograms for the window search (gfx950).
//
// The reference materialises the dense causal attention map of a layer, [Hq, N, N] in the model dtype
// (sqattn/attn_replacer.py:253-278, kept as `current_attention`, model_hub/qwen.py:38-41), and reduces every head's map
// to an "energy by distance" histogram with index tensors of the same size and a bincount
// (sqattn/window_search.py:20-87, 244-321).  Here the map never exists: one workgroup owns 128 query rows of a head,
// walks the key tiles below its diagonal twice with Q.K^T on the matrix cores (first for the softmax normaliser of
// each row, then for the probabilities themselves) and adds every probability, weighted, into a histogram in LDS;
// the LDS histogram is flushed into the fp64 result in HBM with one atomic per bin.  HBM traffic is Q once and K
// once per 128 rows; memory is O(N) instead of O(Hq N^2).
#include "common.hpp"

namespace sq {
namespace {

constexpr int kD = 128;          // head dimension (the host pads smaller heads with zeros)
constexpr int kBM = 128;         // query rows per workgroup: four waves of 32
constexpr int kBN = 64;          // keys per tile
constexpr int kKStride = 272;    // bytes per key row in LDS: 256 + 16 of padding against bank conflicts
constexpr int kMaxBins = 8192;   // LDS histogram of the relative kinds (32 KB)
constexpr int kWindow = kBM + kBN - 1;   // distinct distances inside one (query block, key tile) pair

struct HistArgs {
  const char* q;
  const char* k;
  double* hist;
  int64_t q_sb, q_sh, q_sn;   // byte strides of q [B, Hq, N, 128]
  int64_t k_sb, k_sh, k_sn;   // byte strides of k [B, Hkv, N, 128]
  int N, Hq, groups, bins, sink;
  float scale2;               // softmax scale times log2(e)
};

template <bool BF16>
__device__ __forceinline__ f32x16_t mfma32(const uint4& a, const uint4& b, f32x16_t c) {
  if constexpr (BF16)
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b), c, 0, 0, 0);
  else
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0, 0, 0);
}

// KIND 0: bin = i - j, weight p (i - j), distances >= bins dropped, keys below the sink excluded
//         (window_search.py:20-48 with sink 0, :283-321)
// KIND 1: bin = floor(bins (i - j) / max(i, 1)), weight p (i - j)                               (:51-87)
// KIND 2: keys below the sink excluded; rows i <= sink fall into bin 0; bin = floor(bins (i - j) / max(i - sink, 1)),
//         weight p (bins rel + 1)                                                               (:244-280)
// Bin indices are formed with the reference's fp32 expressions (divide, multiply, floor, clamp), one rounding each.
template <bool BF16, int KIND>
__global__ __launch_bounds__(256) void attn_histogram_kernel(HistArgs a) {
  __shared__ __align__(16) char ktile[kBN * kKStride];
  // KIND 0: a ring of 256 bins indexed by distance & 255.  One (query block, key tile) pair spans 191 distances, the
  // next tile's span lies 64 lower, so after a tile its top 64 distances are final: they are flushed and cleared,
  // and their slots are the ones the span reaches 128 distances later.
  __shared__ float hl[KIND == 0 ? 256 : kMaxBins];

  const int qb = gridDim.x - 1 - blockIdx.x;   // the longest rows first
  const int h = blockIdx.y, b = blockIdx.z, kvh = h / a.groups;
  const int tid = threadIdx.x, wave = tid >> 6, lane = tid & 63, c32 = lane & 31, g = lane >> 5;
  const int row = qb * kBM + wave * 32 + c32;   // this lane's query row i; its keys within a tile: 32 bn + 8 (e >> 2) + (e & 3) + 4 g
  const bool row_ok = row < a.N;
  const int wave_last_row = qb * kBM + wave * 32 + 31;

  // Q as the B operand of S^T = K Q^T: lane holds q[i][16 kk + 8 g .. + 7]
  uint4 qf[8];
  {
    const char* qrow = a.q + (int64_t)b * a.q_sb + (int64_t)h * a.q_sh + (int64_t)(row_ok ? row : a.N - 1) * a.q_sn;
#pragma unroll
    for (int kk = 0; kk < 8; ++kk) qf[kk] = *(const uint4*)(qrow + (2 * kk + g) * 16);
  }
  const int last_key = ((qb + 1) * kBM < a.N ? (qb + 1) * kBM : a.N) - 1;
  const int tiles = last_key / kBN + 1;
  const char* kbase = a.k + (int64_t)b * a.k_sb + (int64_t)kvh * a.k_sh;

  auto load_tile = [&](int jt) {   // 64 keys x 16 chunks of 16 bytes, four chunks per thread; keys past the end read as zero
#pragma unroll
    for (int r = 0; r < 4; ++r) {
      const int kr = (tid >> 4) + 16 * r, key = jt * kBN + kr;
      uint4 v = make_uint4(0, 0, 0, 0);
      if (key < a.N) v = *(const uint4*)(kbase + (int64_t)key * a.k_sn + (tid & 15) * 16);
      *(uint4*)(ktile + kr * kKStride + (tid & 15) * 16) = v;
    }
  };
  auto scores = [&](f32x16_t (&S)[2]) {
#pragma unroll
    for (int i = 0; i < 16; ++i) S[0][i] = S[1][i] = 0.f;
#pragma unroll
    for (int kk = 0; kk < 8; ++kk) {
      const uint4 a0 = *(const uint4*)(ktile + c32 * kKStride + (2 * kk + g) * 16);
      const uint4 a1 = *(const uint4*)(ktile + (32 + c32) * kKStride + (2 * kk + g) * 16);
      S[0] = mfma32<BF16>(a0, qf[kk], S[0]);
      S[1] = mfma32<BF16>(a1, qf[kk], S[1]);
    }
  };

  // ---- pass 1: row maximum and denominator (base-2 exponent domain)
  float m = -INFINITY, l = 0.f;
  for (int jt = 0; jt < tiles; ++jt) {
    __syncthreads();
    load_tile(jt);
    __syncthreads();
    if (jt * kBN > wave_last_row) continue;   // wave-uniform: the tile lies above all of this wave's rows
    f32x16_t S[2];
    scores(S);
    float tm = -INFINITY;
#pragma unroll
    for (int bn = 0; bn < 2; ++bn)
#pragma unroll
      for (int e = 0; e < 16; ++e) {
        const int key = jt * kBN + 32 * bn + 8 * (e >> 2) + (e & 3) + 4 * g;
        const float s = (key <= row) ? S[bn][e] * a.scale2 : -INFINITY;
        S[bn][e] = s;
        tm = fmaxf(tm, s);
      }
    if (tm > -INFINITY) {
      const float mn = fmaxf(m, tm);
      float sum = 0.f;
#pragma unroll
      for (int bn = 0; bn < 2; ++bn)
#pragma unroll
        for (int e = 0; e < 16; ++e) sum += __builtin_amdgcn_exp2f(S[bn][e] - mn);
      l = l * __builtin_amdgcn_exp2f(m - mn) + sum;
      m = mn;
    }
  }
  // the other 32 keys of every tile of this row live in lane ^ 32
  const float mo = __shfl_xor(m, 32), lo = __shfl_xor(l, 32);
  const float mt = fmaxf(m, mo);
  l = (m > -INFINITY ? l * __builtin_amdgcn_exp2f(m - mt) : 0.f) + (mo > -INFINITY ? lo * __builtin_amdgcn_exp2f(mo - mt) : 0.f);
  const float inv_l = 1.0f / l;

  // ---- pass 2: probabilities into the LDS histogram
  const float nbf = (float)a.bins;
  // one divisor per row: integers in [1, 2^24], quotients in [0, 2^24], so the shared-divisor division is exact IEEE
  const Divisor den = make_divisor((KIND == 1) ? (float)(row > 1 ? row : 1) : fmaxf((float)row - (float)a.sink, 1.0f));
  __syncthreads();
  for (int t = tid; t < (KIND == 0 ? 256 : a.bins); t += 256) hl[t] = 0.f;
  double* hist = a.hist + ((int64_t)b * a.Hq + h) * a.bins;
  // KIND 1, 2: a row's keys of one tile fall into one or two bins once the row index is large, and so do the rows of a
  // wave; each lane therefore sums in a register while the bin stays the same and goes to LDS only when it changes
  int cur_bin = -1;
  float cur_sum = 0.f;
  auto add_relative = [&](int bi, float w) {
    if (bi == cur_bin) {
      cur_sum += w;
    } else {
      if (cur_bin >= 0) atomicAdd(&hl[cur_bin], cur_sum);
      cur_bin = bi;
      cur_sum = w;
    }
  };
  for (int jt = 0; jt < tiles; ++jt) {
    __syncthreads();
    load_tile(jt);
    __syncthreads();
    const int base = qb * kBM - (jt * kBN + kBN - 1);   // smallest distance of this (query block, key tile) pair
    if (jt * kBN <= wave_last_row) {
      f32x16_t S[2];
      scores(S);
      if constexpr (KIND == 0) {
        // Pairs of equal distance lie on the diagonals of the wave's 32 x 64 block.  Element e of lane (g, c) has the
        // key offset ko = 8 (e >> 2) + (e & 3) + 4 g within its half tile, so rotating element e by ko lanes inside
        // each half wave brings every pair with row - key = Dw - 32 bn + t to lane t (Dw = the wave's first row minus
        // the tile's first key); pairs that wrap around belong 32 distances lower.  Three sums per lane instead of 32
        // LDS atomics.
        float acc[2][2] = {{0.f, 0.f}, {0.f, 0.f}};   // [bn][wrapped]
#pragma unroll
        for (int bn = 0; bn < 2; ++bn)
#pragma unroll
          for (int e = 0; e < 16; ++e) {
            const int ko = 8 * (e >> 2) + (e & 3) + 4 * g;
            const int key = jt * kBN + 32 * bn + ko;
            const int dist = row - key;
            const bool valid = row_ok && key <= row && key >= a.sink && dist < a.bins;
            const float p = __builtin_amdgcn_exp2f(S[bn][e] * a.scale2 - mt) * inv_l;
            const float w = valid ? p * (float)dist : 0.f;
            const float r = __shfl(w, (lane & 32) | ((c32 + ko) & 31));
            if (c32 + ko >= 32) acc[bn][1] += r;
            else acc[bn][0] += r;
          }
        float grp[3] = {acc[0][0], acc[0][1] + acc[1][0], acc[1][1]};   // distances Dw + t, Dw + t - 32, Dw + t - 64
        const int Dw = qb * kBM + wave * 32 - jt * kBN;
#pragma unroll
        for (int k = 0; k < 3; ++k) {
          const float v = grp[k] + __shfl_xor(grp[k], 32);   // the two halves of the wave hold different keys of the same rows
          const int d = Dw + c32 - 32 * k;
          if (g == (k & 1) && d >= 0 && v != 0.f) atomicAdd(&hl[d & 255], v);
        }
      } else {
#pragma unroll
      for (int bn = 0; bn < 2; ++bn)
#pragma unroll
        for (int e = 0; e < 16; ++e) {
#pragma clang fp contract(off)
          const int key = jt * kBN + 32 * bn + 8 * (e >> 2) + (e & 3) + 4 * g;
          if (!(row_ok && key <= row) || (KIND != 1 && key < a.sink)) continue;
          const float p = __builtin_amdgcn_exp2f(S[bn][e] * a.scale2 - mt) * inv_l;
          const int dist = row - key;
          if constexpr (KIND == 1) {
            const float sc = divide((float)dist, den) * nbf;
            int bi = (int)__builtin_floorf(sc);
            bi = bi < a.bins - 1 ? bi : a.bins - 1;
            add_relative(bi, p * (float)dist);
          } else {
            float sc = divide((float)dist, den) * nbf;
            if (row <= a.sink) sc = 0.f;
            int bi = (int)__builtin_floorf(sc);
            bi = bi < a.bins - 1 ? bi : a.bins - 1;
            add_relative(bi, p * (sc + 1.0f));
          }
        }
      }
    }
    if constexpr (KIND == 0) {
      __syncthreads();
      // after the last tile everything that is left, otherwise the 64 distances the next tile cannot reach
      const int lo = (jt == tiles - 1) ? base : base + kBM - 1;
      const int d = lo + tid;
      if (d <= base + kWindow - 1) {
        const float v = hl[d & 255];
        hl[d & 255] = 0.f;
        if (d >= 0 && d < a.bins && v != 0.f) atomicAdd(hist + d, (double)v);
      }
    }
  }
  if constexpr (KIND != 0) {
    if (cur_bin >= 0) atomicAdd(&hl[cur_bin], cur_sum);
    __syncthreads();
    for (int t = tid; t < a.bins; t += 256) {
      const float v = hl[t];
      if (v != 0.f) atomicAdd(hist + t, (double)v);
    }
  }
}

template <bool BF16>
void launch_histogram(int kind, dim3 grid, hipStream_t stream, const HistArgs& a) {
  if (kind == 0) hipLaunchKernelGGL((attn_histogram_kernel<BF16, 0>), grid, dim3(256), 0, stream, a);
  else if (kind == 1) hipLaunchKernelGGL((attn_histogram_kernel<BF16, 1>), grid, dim3(256), 0, stream, a);
  else hipLaunchKernelGGL((attn_histogram_kernel<BF16, 2>), grid, dim3(256), 0, stream, a);
}

}  // namespace
}  // namespace sq

using namespace sq;

extern "C" int sq_attention_histogram(const DLTensor* q, const DLTensor* k, DLTensor* hist, const sq_histogram_params* p, void* stream) {
  const char* fn = "sq_attention_histogram";
  SQ_REQUIRE(q && k && hist && p, SQ_EINVAL, "%s: null argument", fn);
  int rc;
  if ((rc = check_tensor(q, "q", 4, q->device.device_id))) return rc;
  const int dev = q->device.device_id;
  if ((rc = check_tensor(k, "k", 4, dev))) return rc;
  const DType dt = dtype_of(q);
  SQ_REQUIRE(dt == DType::BF16 || dt == DType::F16, SQ_EDTYPE, "%s: q must be bf16 or fp16", fn);
  SQ_REQUIRE(dtype_of(k) == dt, SQ_EDTYPE, "%s: q and k differ in dtype", fn);
  const int64_t B = q->shape[0], Hq = q->shape[1], N = q->shape[2], D = q->shape[3], Hkv = k->shape[1];
  SQ_REQUIRE(D == kD, SQ_EUNSUPPORTED, "%s: head_dim must be 128 (got %lld; pad with zeros)", fn, (long long)D);
  SQ_REQUIRE(k->shape[0] == B && k->shape[2] == N && k->shape[3] == D, SQ_ESHAPE, "%s: k must be [%lld, Hkv, %lld, %lld]", fn, (long long)B,
             (long long)N, (long long)D);
  SQ_REQUIRE(Hkv > 0 && Hq % Hkv == 0, SQ_ESHAPE, "%s: %lld query heads are not a multiple of %lld kv heads", fn, (long long)Hq, (long long)Hkv);
  SQ_REQUIRE(N >= 1 && N <= (1 << 24), SQ_EUNSUPPORTED, "%s: sequence length %lld outside [1, 2^24]", fn, (long long)N);
  SQ_REQUIRE(B >= 1 && B < 65536 && Hq < 65536, SQ_EUNSUPPORTED, "%s: batch or head count too large", fn);
  SQ_REQUIRE(p->kind >= 0 && p->kind <= 2, SQ_EINVAL, "%s: unknown histogram kind %d", fn, (int)p->kind);
  SQ_REQUIRE(p->bins >= 1, SQ_EINVAL, "%s: bins must be positive (got %d)", fn, (int)p->bins);
  SQ_REQUIRE(p->kind == 0 || p->bins <= kMaxBins, SQ_EUNSUPPORTED, "%s: at most %d relative bins (got %d)", fn, kMaxBins, (int)p->bins);
  SQ_REQUIRE(p->sink >= 0, SQ_EINVAL, "%s: sink must be >= 0 (got %d)", fn, (int)p->sink);
  SQ_REQUIRE(p->kind != 1 || p->sink == 0, SQ_EINVAL, "%s: the plain relative histogram takes no sink", fn);
  SQ_REQUIRE(p->softmax_scale > 0.f, SQ_EINVAL, "%s: softmax_scale must be positive", fn);
  SQ_REQUIRE(on_gpu(hist) && hist->device.device_id == dev, SQ_EDEVICE, "%s: hist must live on q's device", fn);
  SQ_REQUIRE(hist->dtype.code == kDLFloat && hist->dtype.bits == 64 && hist->dtype.lanes == 1, SQ_EDTYPE, "%s: hist must be float64", fn);
  SQ_REQUIRE(hist->ndim == 3 && hist->shape[0] == B && hist->shape[1] == Hq && hist->shape[2] == p->bins && is_compact(hist), SQ_ESHAPE,
             "%s: hist must be contiguous [%lld, %lld, %d]", fn, (long long)B, (long long)Hq, (int)p->bins);
  int cur = -1;
  SQ_HIP(hipGetDevice(&cur));
  SQ_REQUIRE(cur == dev, SQ_EDEVICE, "%s: tensors live on device %d but the current device is %d", fn, dev, cur);
  HistArgs a;
  a.q = data_of(q);
  a.k = data_of(k);
  a.hist = (double*)data_of(hist);
  a.q_sb = stride_of(q, 0) * 2;
  a.q_sh = stride_of(q, 1) * 2;
  a.q_sn = stride_of(q, 2) * 2;
  a.k_sb = stride_of(k, 0) * 2;
  a.k_sh = stride_of(k, 1) * 2;
  a.k_sn = stride_of(k, 2) * 2;
  SQ_REQUIRE(a.q_sn % 16 == 0 && a.q_sh % 16 == 0 && a.q_sb % 16 == 0 && a.k_sn % 16 == 0 && a.k_sh % 16 == 0 && a.k_sb % 16 == 0, SQ_ESHAPE,
             "%s: rows of q and k must be 16-byte aligned", fn);
  a.N = (int)N;
  a.Hq = (int)Hq;
  a.groups = (int)(Hq / Hkv);
  a.bins = p->bins;
  a.sink = p->sink;
  a.scale2 = p->softmax_scale * 1.44269504088896340736f;
  const dim3 grid((unsigned)((N + kBM - 1) / kBM), (unsigned)Hq, (unsigned)B);
  if (dt == DType::BF16) launch_histogram<true>(p->kind, grid, (hipStream_t)stream, a);
  else launch_histogram<false>(p->kind, grid, (hipStream_t)stream, a);
  SQ_HIP(hipGetLastError());
  return SQ_OK;
}
