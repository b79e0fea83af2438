// The projections of a decode step for gfx950 (MI355X): y = x . W^T (+ bias) (+ residual) for at most eight rows of
// x.  In the reference's runtime these are the tensor-library matmuls of wqkv, wo, mlp and lm
// (model_hub/qwen.py:302-326, 293-300) on a [batch, 1, hidden] activation.  With one to eight activation rows the
// product is a pass over the weights: every weight is read once from HBM and used `rows` times, so the kernel is
// HBM-bound (algorithmic bytes = N x K weights x 2) and is laid out for that, not for the matrix cores: one wave
// owns R output features, its 64 lanes walk the K axis in 16-byte steps (1 KB per wave and load, several loads in
// flight), the activation rows sit in LDS, products go through the packed 16-bit dot instruction
// (v_dot2c_f32_bf16 / v_dot2c_f32_f16: fp32 accumulation), and the R x rows partial sums of the 64 lanes are folded
// by a transposing butterfly.  Rounding points: the fp32 sum plus the bias is rounded once to the tensor dtype (what
// a GEMM with a bias epilogue gives); a residual is then added as a second tensor operator would (rounded again).
// The gated form (sq_linear_rows_silu_and_mul) is the first projection of the MLP together with the activation that
// follows it (model_hub/qwen.py:320-324): a wave owns features f and f + N/2 of the [gate | up] weight, so both
// halves of an output pair end in one wave and out[f] = up * (gate * sigmoid(gate)) leaves with the rounding points
// of the stand-alone pass (the product, sigmoid and gate * sigmoid each rounded to the tensor dtype).
// The rotary form (sq_linear_rows_rope) is the fused q/k/v projection together with the rotary embedding of its q
// and k parts (model_hub/qwen.py:302-312, 352-379): a wave owns features i and i + head_dim/2 of one head, rotates
// the pair by the position's cos/sin (fp32 products and sums without fused multiply-add, one rounding, as sq_rope
// does) and stores both; the waves behind the rotated part produce plain features (v).
// The sq_rmsnorm_linear_rows* forms take the activation before its RMS norm (model_hub/qwen.py:345-350 in front of wqkv and
// of mlp, and in front of lm): while the first weights are on their way, the workgroup's waves normalise the rows
// into LDS with the operator sequence of the stand-alone pass (rmsnorm_kernel: the same association of the sum of
// squares, the same roundings), so the result has the same bits and the norm's launch, its output tensor and its round
// trip through memory go away.  Every workgroup repeats the norm of the few rows; that is 14 KB of L2 reads each.
#include "common.hpp"

namespace sq {
namespace {

constexpr int kLinThreads = 256;   // four waves: the workgroup of a large matrix
constexpr int kLinMaxWaves = 16;   // a matrix of at most 256 x 16 waves runs as one workgroup per CU
// Activation rows in LDS, K-chunk by K-chunk: up to 20480 elements of one row (a whole row of the widest projection,
// four workgroups per CU), 5120 of each of four; with eight rows 2048 of each, which keeps five workgroups on a CU.
constexpr int kLinLdsBytes = 40960, kLinLdsBytes8 = 32768;
constexpr int kLinMaxRows = 8;

struct LinArgs {
  const char* x;
  const char* w;
  const char* bias;   // nullable
  const char* res;    // nullable
  char* y;
  int64_t x_sr, w_sr, r_sr, y_sr;   // row strides in bytes
  int32_t rows;                     // rows of x actually present (<= M)
  int32_t n, k;
  int32_t chunk;   // elements of every activation row per LDS pass (a multiple of 8)
  // rotary form only
  const void* pos;       // [rows] int32 or int64
  const float* table;    // [max_pos, head_dim]: cos | sin
  int32_t pos_is_i64, max_pos, head_dim, rope_features;
  // rotary form with the KV cache behind it: the k and v features also go to row valid_length[m] of the caches
  char* k_cache;                 // nullable
  char* v_cache;
  int64_t cache_sb;              // bytes per sequence of a cache
  const int32_t* valid_length;   // [rows]
  int32_t* attend_length;        // [rows] or null: receives valid_length + 1
  int32_t max_length, q_features, kv_features;
  // RMS norm of the activation rows in front of the product (null: none); needs chunk == k
  const char* norm_w;   // [k]
  float eps;
};

enum { kModePlain = 0, kModeGated = 1, kModeRope = 2 };

typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2_t;
typedef __attribute__((ext_vector_type(2))) _Float16 f16x2_t;

template <bool BF16>
__device__ __forceinline__ float dot2(uint32_t a, uint32_t b, float c) {
  if constexpr (BF16) return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2_t, a), __builtin_bit_cast(bf16x2_t, b), c, false);
  else return __builtin_amdgcn_fdot2(__builtin_bit_cast(f16x2_t, a), __builtin_bit_cast(f16x2_t, b), c, false);
}
template <bool BF16>
__device__ __forceinline__ float ld16(const char* p) {
  const uint32_t bits = *(const uint16_t*)p;
  if constexpr (BF16) return bf16_bits_to_f32(bits);
  else return (float)__builtin_bit_cast(_Float16, (uint16_t)bits);
}
template <bool BF16>
__device__ __forceinline__ float cv16(uint32_t bits) {   // the low 16 bits as a value
  if constexpr (BF16) return bf16_bits_to_f32(bits & 0xffffu);
  else return (float)__builtin_bit_cast(_Float16, (uint16_t)bits);
}
template <bool BF16>
__device__ __forceinline__ uint16_t st16(float x) {
  if constexpr (BF16) return (uint16_t)f32_to_bf16_bits(x);
  else return __builtin_bit_cast(uint16_t, (_Float16)x);
}
template <bool BF16>
__device__ __forceinline__ float rnd16(float x) {
  if constexpr (BF16) return bf16_bits_to_f32(f32_to_bf16_bits(x));
  else return (float)(_Float16)x;
}

// x2 * (x1 * sigmoid(x1)) with sigmoid and x1 * sigmoid rounded to the tensor dtype: the formula of silu_mul_kernel
// (same instructions, so the same bits; the caller rounds the last product)
template <bool BF16>
__device__ __forceinline__ float silu_mul_elem(float x1, float x2) {
  const float sg = rnd16<BF16>(__builtin_amdgcn_rcpf(1.0f + __expf(-x1)));
  return x2 * rnd16<BF16>(x1 * sg);
}

// M = activation rows the registers are sized for (1, 2, 4, 8), R = output features per wave (1, 2, 4),
// U = 16-byte weight loads per feature a lane keeps in flight (eight loads per lane in all).
// kModeGated: the wave's R features are R/2 pairs (f, f + n/2) and the output has n/2 columns.
// kModeRope (R = 2): wave w < rope_features / 2 owns the pair (i, i + head_dim / 2) of a head, later waves two plain features.
template <bool BF16, int M, int R, int MODE = kModePlain>
__global__ __launch_bounds__(kLinMaxWaves * 64) void linear_rows_kernel(LinArgs a) {
  constexpr bool GATED = MODE == kModeGated, ROPE = MODE == kModeRope;
  static_assert(!GATED || R % 2 == 0, "a gated wave owns whole pairs");
  static_assert(!ROPE || R == 2, "a rotary wave owns one pair");
  constexpr int RO = GATED ? R / 2 : R;   // output columns per wave
  const int n_out = GATED ? a.n / 2 : a.n;
  constexpr int U = 8 / R;
  extern __shared__ u32x4_t xs[];   // [M][chunk / 8]
  const int kLinChunk = a.chunk, row16 = a.chunk / 8;
  const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
  int64_t feat0 = ((int64_t)blockIdx.x * (blockDim.x >> 6) + wave) * RO;
  const char* wrow[R];
  [[maybe_unused]] int64_t rope_f[2] = {0, 0};   // the two features of a rotary wave
  [[maybe_unused]] bool paired = false;
  [[maybe_unused]] int rope_i = 0;               // index of the pair inside its head
  if constexpr (ROPE) {
    const int64_t w = (int64_t)blockIdx.x * (blockDim.x >> 6) + wave;
    const int half = a.head_dim / 2;
    paired = w < a.rope_features / 2;
    if (paired) {
      rope_i = (int)(w % half);
      rope_f[0] = w / half * a.head_dim + rope_i;
      rope_f[1] = rope_f[0] + half;
    } else {
      rope_f[0] = a.rope_features + (w - a.rope_features / 2) * 2;
      rope_f[1] = rope_f[0] + 1;
    }
    feat0 = rope_f[0];
#pragma unroll
    for (int r = 0; r < R; ++r) wrow[r] = a.w + (rope_f[r] < a.n ? rope_f[r] : (int64_t)a.n - 1) * a.w_sr;
  } else {
#pragma unroll
    for (int r = 0; r < R; ++r) {
      const int64_t col = (feat0 + r % RO < n_out) ? feat0 + r % RO : (int64_t)n_out - 1;   // columns past the end re-read the last one
      wrow[r] = a.w + (col + (r >= RO ? n_out : 0)) * a.w_sr;                               // second half of a pair: feature col + n/2
    }
  }
  const bool live = feat0 < n_out;
  float acc[R * M];
#pragma unroll
  for (int i = 0; i < R * M; ++i) acc[i] = 0.f;

  // What the epilogue adds to or multiplies with the result does not depend on the result: the bias, the residual, the
  // row's position with its cos / sin pair, the cache row's number.  Requested here, they arrive during the main loop;
  // requested in the epilogue they were two dependent round trips at the end of a kernel that is a few microseconds long.
  constexpr int V = R * M;
  const int idx = lane & (V - 1);
  const int r = idx / M, m = idx % M;
  const int64_t col = feat0 + r % RO;
  const bool row_ok = live && lane < V && m < a.rows;
  float pf_bias = 0.f, pf_res = 0.f, pf_cs = 0.f, pf_sn = 0.f;
  int pf_row = -1;
  if constexpr (GATED) {
    const int64_t f = (col < n_out ? col : (int64_t)n_out - 1) + (r >= RO ? n_out : 0);
    if (a.bias && live) pf_bias = ld16<BF16>(a.bias + f * 2);
  } else if constexpr (ROPE) {
    const int64_t f = rope_f[r] < a.n ? rope_f[r] : (int64_t)a.n - 1;
    if (a.bias && live) pf_bias = ld16<BF16>(a.bias + f * 2);
    if (row_ok) {
      if (paired && lane < M) {
        int64_t p = a.pos_is_i64 ? ((const int64_t*)a.pos)[m] : (int64_t)((const int32_t*)a.pos)[m];
        p = p < 0 ? 0 : (p >= a.max_pos ? a.max_pos - 1 : p);
        const float* trow = a.table + p * a.head_dim;
        pf_cs = trow[rope_i];
        pf_sn = trow[a.head_dim / 2 + rope_i];
      }
      if (a.k_cache) pf_row = a.valid_length[m];
    }
  } else {
    if (row_ok && col < a.n) {
      if (a.bias) pf_bias = ld16<BF16>(a.bias + col * 2);
      if (a.res) pf_res = ld16<BF16>(a.res + m * a.r_sr + col * 2);
    }
  }

  for (int k0 = 0; k0 < a.k; k0 += kLinChunk) {
    const int chunks = ((a.k - k0 < kLinChunk) ? (a.k - k0) : kLinChunk) / 8;
    u32x4_t wv[R][U];
    auto request = [&](int base) {   // base: the batch's first 16-byte step (wave-uniform)
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int cc = base + lane + 64 * u;
        const int64_t off = ((int64_t)k0 + (int64_t)(cc < chunks ? cc : chunks - 1) * 8) * 2;   // past the end: re-read the last step
#pragma unroll
        for (int r = 0; r < R; ++r) wv[r][u] = __builtin_nontemporal_load((const u32x4_t*)(wrow[r] + off));
      }
    };
    auto consume = [&](int base) {
#pragma unroll
      for (int u = 0; u < U; ++u) {
        const int cc = base + lane + 64 * u;
        if (cc < chunks) {
#pragma unroll
          for (int m = 0; m < M; ++m) {
            const u32x4_t xv = xs[m * row16 + cc];
#pragma unroll
            for (int r = 0; r < R; ++r)
#pragma unroll
              for (int j = 0; j < 4; ++j) acc[r * M + m] = dot2<BF16>(wv[r][u][j], xv[j], acc[r * M + m]);
          }
        }
      }
    };
    if (live) request(0);   // the first weights are on their way while the activations are staged
    if (k0) __syncthreads();
    if (a.norm_w) {
      // The sum of squares in the association of rmsnorm_kernel -- lane l owns the 16-byte chunks l, l + 64, ...; each
      // chunk's eight rounded squares are summed on their own, the chunk sums are added in ascending order, the lanes
      // fold by a fixed butterfly -- but spread over the waves: (row, chunk index) pairs go round the waves, the chunk
      // sums meet in LDS, and every wave folds them for itself.  Then x * r (rounded) * weight (rounded by the pack).
      const int nw = (int)(blockDim.x >> 6);
      const int per_lane = (chunks + 63) >> 6;
      const int tasks = M * per_lane;
      float* part = (float*)(xs + M * row16);   // [M][per_lane][64]
      // task t = (row t / per_lane, chunk index t % per_lane); with one row the division by a kernel argument (a software
      // routine of some thirty instructions, on the path between the staging and the main loop) drops out
      auto row_of = [&](int t) { return M == 1 ? 0 : t / per_lane; };
      auto idx_of = [&](int t) { return M == 1 ? t : t % per_lane; };
      auto x_chunk = [&](int t) {
        const int m = row_of(t), c = lane + 64 * idx_of(t);
        return *(const u32x4_t*)(a.x + (int64_t)(m < a.rows ? m : a.rows - 1) * a.x_sr + (c < chunks ? c : chunks - 1) * 16);
      };
      auto w_chunk = [&](int t) {
        const int c = lane + 64 * idx_of(t);
        return *(const u32x4_t*)(a.norm_w + (c < chunks ? c : chunks - 1) * 16);
      };
      auto squares = [&](int t, const u32x4_t& v) {
        float p = 0.f;
        if (lane + 64 * idx_of(t) < chunks) {
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const float lo = cv16<BF16>(v[j]), hi = cv16<BF16>(v[j] >> 16);
            p += rnd16<BF16>(lo * lo);
            p += rnd16<BF16>(hi * hi);
          }
        }
        part[t * 64 + lane] = p;
      };
      // a wave's first two chunks and their weights stay in registers across the barrier; further ones are read again
      constexpr int KEEP = 2;
      u32x4_t xk[KEEP], gk[KEEP];
#pragma unroll
      for (int i = 0; i < KEEP; ++i) {
        const int t = wave + i * nw;
        if (t < tasks) {
          xk[i] = x_chunk(t);
          gk[i] = w_chunk(t);
        }
      }
#pragma unroll
      for (int i = 0; i < KEEP; ++i) {
        const int t = wave + i * nw;
        if (t < tasks) squares(t, xk[i]);
      }
      for (int t = wave + KEEP * nw; t < tasks; t += nw) squares(t, x_chunk(t));
      __syncthreads();
      float r[M];
#pragma unroll
      for (int m = 0; m < M; ++m) {
        float sum = 0.f;
        for (int c = 0; c < per_lane; ++c) sum += part[(m * per_lane + c) * 64 + lane];
#pragma unroll
        for (int sft = 32; sft > 0; sft >>= 1) sum += __shfl_xor(sum, sft);
        const float var = rnd16<BF16>(sum / (float)a.k);
        const float ve = rnd16<BF16>(var + a.eps);
        r[m] = rnd16<BF16>(1.0f / sqrtf(ve));
      }
      auto scale = [&](int t, const u32x4_t& v, const u32x4_t& g) {
        const int m = row_of(t), c = lane + 64 * idx_of(t);
        float rr = r[0];
#pragma unroll
        for (int i = 1; i < M; ++i) rr = (m == i) ? r[i] : rr;
        if (c < chunks) {
          u32x4_t o;
#pragma unroll
          for (int j = 0; j < 4; ++j) {
            const float lo = cv16<BF16>(v[j]), hi = cv16<BF16>(v[j] >> 16);
            const float glo = cv16<BF16>(g[j]), ghi = cv16<BF16>(g[j] >> 16);
            o[j] = (uint32_t)st16<BF16>(rnd16<BF16>(lo * rr) * glo) | ((uint32_t)st16<BF16>(rnd16<BF16>(hi * rr) * ghi) << 16);
          }
          xs[m * row16 + c] = o;
        }
      };
#pragma unroll
      for (int i = 0; i < KEEP; ++i) {
        const int t = wave + i * nw;
        if (t < tasks) scale(t, xk[i], gk[i]);
      }
      for (int t = wave + KEEP * nw; t < tasks; t += nw) scale(t, x_chunk(t), w_chunk(t));
    } else {
#pragma unroll
      for (int m = 0; m < M; ++m) {
        const char* xr = a.x + (int64_t)(m < a.rows ? m : a.rows - 1) * a.x_sr + (int64_t)k0 * 2;
#pragma unroll 4
        for (int c = threadIdx.x; c < chunks; c += blockDim.x) xs[m * row16 + c] = *(const u32x4_t*)(xr + c * 16);
      }
    }
    __syncthreads();
    if (live) {
      for (int base = 0; base < chunks; base += 64 * U) {
        if (base) request(base);
        consume(base);
      }
    }
  }
  if (!live) return;

  // Fold the 64 lanes.  While more than one value is left, a step over lane bit s halves the list: a lane keeps the
  // even or the odd entry of each pair (by its bit s) and receives the partner's partial sum of that entry.  After
  // log2(V) steps lane l holds entry (l mod V), summed over the low lane bits; plain butterflies finish the rest.
  int width = V, s = 0;
#pragma unroll
  for (; (1 << s) < V; ++s) {
    const bool odd = (lane >> s) & 1;
#pragma unroll
    for (int i = 0; i < width / 2; ++i) {
      const float keep = odd ? acc[2 * i + 1] : acc[2 * i];
      const float send = odd ? acc[2 * i] : acc[2 * i + 1];
      acc[i] = keep + __shfl_xor(send, 1 << s);
    }
    width /= 2;
  }
#pragma unroll
  for (; s < 6; ++s) acc[0] += __shfl_xor(acc[0], 1 << s);

  float v = acc[0];
  if constexpr (GATED) {
    if (a.bias) v += pf_bias;
    v = rnd16<BF16>(v);                                    // the projection's own rounding
    const float up = __shfl(v, (lane + RO * M) & 63);      // lane idx + (R/2) M holds the pair's second half for the same row
    if (lane < RO * M && col < n_out && m < a.rows) *(uint16_t*)(a.y + m * a.y_sr + col * 2) = st16<BF16>(silu_mul_elem<BF16>(v, up));
  } else if constexpr (ROPE) {
    if (a.bias) v += pf_bias;
    v = rnd16<BF16>(v);                                   // the projection's own rounding
    const float second = __shfl(v, (lane + M) & 63);      // lane idx + M holds feature rope_f[1] of the same row
    if (paired) {
      if (lane < M && m < a.rows) {
        const float cs = pf_cs, sn = pf_sn;
        float o1, o2;
        {
          // separate fp32 products and sums, as the stand-alone rotary pass forms them
#pragma clang fp contract(off)
          const float a1 = v * cs, b1 = second * sn;
          const float a2 = v * sn, b2 = second * cs;
          o1 = a1 - b1;
          o2 = a2 + b2;
        }
        *(uint16_t*)(a.y + m * a.y_sr + rope_f[0] * 2) = st16<BF16>(o1);
        *(uint16_t*)(a.y + m * a.y_sr + rope_f[1] * 2) = st16<BF16>(o2);
        if (a.k_cache && rope_f[0] >= a.q_features) {   // a pair of a k head: its place in the new cache row
          const int row = pf_row;
          if (row >= 0 && row < a.max_length) {          // (a full sequence stays as it is, as in the append pass)
            char* dst = a.k_cache + m * a.cache_sb + ((int64_t)row * a.kv_features - a.q_features) * 2;
            *(uint16_t*)(dst + rope_f[0] * 2) = st16<BF16>(o1);
            *(uint16_t*)(dst + rope_f[1] * 2) = st16<BF16>(o2);
          }
        }
      }
    } else if (lane < V && rope_f[r] < a.n && m < a.rows) {
      *(uint16_t*)(a.y + m * a.y_sr + rope_f[r] * 2) = st16<BF16>(v);
      if (a.k_cache) {                                   // behind the rotated part: v
        const int row = pf_row;
        if (row >= 0 && row < a.max_length)
          *(uint16_t*)(a.v_cache + m * a.cache_sb + ((int64_t)row * a.kv_features + rope_f[r] - a.rope_features) * 2) = st16<BF16>(v);
      }
    }
    if (a.k_cache && a.attend_length && blockIdx.x == 0 && wave == 0 && lane < a.rows) {
      const int row = a.valid_length[lane];
      a.attend_length[lane] = row < a.max_length ? row + 1 : row;
    }
  } else {
    if (lane < V && col < a.n && m < a.rows) {
      if (a.bias) v += pf_bias;
      if (a.res) v = rnd16<BF16>(v) + pf_res;
      *(uint16_t*)(a.y + m * a.y_sr + col * 2) = st16<BF16>(v);
    }
  }
}

// elements of one activation row the LDS staging buffer holds when the registers are sized for m rows (1, 2, 4, 8)
constexpr int chunk_cap(int m) { return (m == 8 ? kLinLdsBytes8 : kLinLdsBytes) / (2 * m) / 8 * 8; }
int max_chunk(int rows) { return chunk_cap(rows <= 1 ? 1 : rows <= 2 ? 2 : rows <= 4 ? 4 : 8); }

template <bool BF16, int M>
void launch_rows(LinArgs a, int R, int mode, hipStream_t stream) {
  const bool gated = mode == kModeGated;
  if (mode == kModeRope) R = 2;
  const int64_t waves = mode == kModeRope ? a.rope_features / 2 + (a.n - a.rope_features + 1) / 2
                                          : gated ? (a.n / 2 + R / 2 - 1) / (R / 2) : (a.n + R - 1) / R;
  // Waves per workgroup: a matrix that fits 256 workgroups of at most 16 waves runs as exactly one workgroup per
  // CU (every CU gets the same number of waves and stages the activation rows once); larger ones as workgroups of
  // four waves, which the dispatcher hands out as CUs free up.
  const int64_t per_cu = (waves + 255) / 256;
  const int wpw = per_cu <= kLinMaxWaves ? (int)(per_cu < 1 ? 1 : per_cu) : kLinThreads / 64;
  const dim3 grid((unsigned)((waves + wpw - 1) / wpw)), block(wpw * 64);
  constexpr int cap = chunk_cap(M);
  a.chunk = a.k < cap ? a.k : cap;
  // (with the norm in front: the chunk sums of the rows behind the rows themselves)
  const size_t lds = (size_t)M * a.chunk * 2 + (a.norm_w ? (size_t)M * ((a.k / 8 + 63) / 64) * 256 : 0);
  if (mode == kModeRope) hipLaunchKernelGGL((linear_rows_kernel<BF16, M, 2, kModeRope>), grid, block, lds, stream, a);
  else if (gated) {
    if (R == 4) hipLaunchKernelGGL((linear_rows_kernel<BF16, M, 4, kModeGated>), grid, block, lds, stream, a);
    else hipLaunchKernelGGL((linear_rows_kernel<BF16, M, 2, kModeGated>), grid, block, lds, stream, a);
  } else if (R == 4) hipLaunchKernelGGL((linear_rows_kernel<BF16, M, 4>), grid, block, lds, stream, a);
  else if (R == 2) hipLaunchKernelGGL((linear_rows_kernel<BF16, M, 2>), grid, block, lds, stream, a);
  else hipLaunchKernelGGL((linear_rows_kernel<BF16, M, 1>), grid, block, lds, stream, a);
}

template <bool BF16>
void launch(const LinArgs& a, int mode, hipStream_t stream) {
  const bool gated = mode == kModeGated;
  // Features per wave: more of them re-use each activation chunk read from LDS (and shrink the share of the
  // LDS staging, which every workgroup repeats), fewer of them give more waves to a small matrix.
  const int m = a.rows <= 1 ? 1 : a.rows <= 2 ? 2 : a.rows <= 4 ? 4 : 8;
  int R = (a.n >= 32768) ? 4 : (a.n >= 12288) ? 2 : 1;
  if ((m >= 4 || gated) && R < 2) R = 2;
  if (m == 8) R = 4;
  switch (m) {
    case 1: launch_rows<BF16, 1>(a, R, mode, stream); break;
    case 2: launch_rows<BF16, 2>(a, R, mode, stream); break;
    case 4: launch_rows<BF16, 4>(a, R, mode, stream); break;
    default: launch_rows<BF16, 8>(a, R, mode, stream); break;
  }
}

}  // namespace
}  // namespace sq

using namespace sq;

namespace {
struct RopeSpec {
  const DLTensor* position_ids;
  const DLTensor* cos_sin_cache;
  int32_t head_dim, rope_features;
  DLTensor* key_cache;       // all four null, or the cache behind the projection
  DLTensor* value_cache;
  const DLTensor* valid_length;
  DLTensor* attend_length;   // may be null
};

struct NormSpec {
  const DLTensor* weight;
  float epsilon;
};

int linear_rows(const char* fn, int mode, const DLTensor* x, const DLTensor* weight, const DLTensor* bias, const DLTensor* residual,
                DLTensor* out, void* stream, const RopeSpec* rope = nullptr, const NormSpec* norm = nullptr) {
  const bool gated = mode == kModeGated;
  SQ_REQUIRE(x && weight && out, SQ_EINVAL, "%s: null tensor argument", fn);
  int rc;
  if ((rc = check_tensor(x, "x", 2, x->device.device_id))) return rc;
  const int dev = x->device.device_id;
  const DType dt = dtype_of(x);
  SQ_REQUIRE(dt == DType::BF16 || dt == DType::F16, SQ_EDTYPE, "%s: x must be bf16 or fp16", fn);
  const int64_t M = x->shape[0], K = x->shape[1];
  SQ_REQUIRE(M >= 1 && M <= kLinMaxRows, SQ_EUNSUPPORTED, "%s: x must have 1 to %d rows (got %lld); larger products belong to a GEMM", fn,
             kLinMaxRows, (long long)M);
  SQ_REQUIRE(K > 0 && K % 8 == 0, SQ_EUNSUPPORTED, "%s: the inner dimension must be a positive multiple of 8 (got %lld)", fn, (long long)K);
  if ((rc = check_tensor(weight, "weight", 2, dev))) return rc;
  const int64_t N = weight->shape[0];
  SQ_REQUIRE(dtype_of(weight) == dt, SQ_EDTYPE, "%s: weight must have x's dtype", fn);
  SQ_REQUIRE(N > 0 && N < (1ll << 31) && weight->shape[1] == K, SQ_ESHAPE, "%s: weight must be [N, %lld] (got [%lld, %lld])", fn, (long long)K,
             (long long)N, (long long)weight->shape[1]);
  if ((rc = check_tensor(out, "out", 2, dev))) return rc;
  SQ_REQUIRE(!gated || N % 2 == 0, SQ_ESHAPE, "%s: the weight must hold two halves of equal size (got %lld rows)", fn, (long long)N);
  const int64_t NO = gated ? N / 2 : N;
  SQ_REQUIRE(dtype_of(out) == dt && out->shape[0] == M && out->shape[1] == NO, SQ_ESHAPE, "%s: out must be [%lld, %lld] of x's dtype", fn,
             (long long)M, (long long)NO);
  SQ_REQUIRE(stride_of(x, 1) == 1 && stride_of(weight, 1) == 1 && stride_of(out, 1) == 1, SQ_ESHAPE, "%s: the last dimension must be contiguous", fn);
  SQ_REQUIRE((stride_of(x, 0) % 8 == 0 || M == 1) && (stride_of(weight, 0) % 8 == 0 || N == 1), SQ_ESHAPE, "%s: rows of x and weight must be 16-byte aligned",
             fn);
  SQ_REQUIRE(((uintptr_t)data_of(x) % 16 == 0) && ((uintptr_t)data_of(weight) % 16 == 0), SQ_ESHAPE, "%s: x and weight must be 16-byte aligned", fn);
  if (bias) {
    if ((rc = check_tensor(bias, "bias", 1, dev))) return rc;
    SQ_REQUIRE(dtype_of(bias) == dt && bias->shape[0] == N && stride_of(bias, 0) == 1, SQ_ESHAPE, "%s: bias must be a contiguous [%lld] of x's dtype", fn,
               (long long)N);
  }
  if (residual) {
    if ((rc = check_tensor(residual, "residual", 2, dev))) return rc;
    SQ_REQUIRE(dtype_of(residual) == dt && residual->shape[0] == M && residual->shape[1] == N && stride_of(residual, 1) == 1, SQ_ESHAPE,
               "%s: residual must be [%lld, %lld] of x's dtype with a contiguous last dimension", fn, (long long)M, (long long)N);
  }
  LinArgs a;
  a.norm_w = nullptr;
  a.eps = 0.f;
  if (norm) {
    const DLTensor* nw = norm->weight;
    SQ_REQUIRE(nw, SQ_EINVAL, "%s: null tensor argument", fn);
    if ((rc = check_tensor(nw, "norm_weight", 1, dev))) return rc;
    SQ_REQUIRE(dtype_of(nw) == dt && nw->shape[0] == K && stride_of(nw, 0) == 1 && (uintptr_t)data_of(nw) % 16 == 0, SQ_ESHAPE,
               "%s: norm_weight must be a contiguous, 16-byte aligned [%lld] of x's dtype", fn, (long long)K);
    const int64_t cap = max_chunk((int)M) < 8192 ? max_chunk((int)M) : 8192;   // (8192: the longest row of sq_rmsnorm)
    SQ_REQUIRE(K <= cap, SQ_EUNSUPPORTED, "%s: with %lld activation rows the normalised row can have at most %lld elements (got %lld)",
               fn, (long long)M, (long long)cap, (long long)K);
    a.norm_w = data_of(nw);
    a.eps = norm->epsilon;
  }
  a.pos = nullptr;
  a.table = nullptr;
  a.pos_is_i64 = a.max_pos = a.head_dim = a.rope_features = 0;
  a.k_cache = a.v_cache = nullptr;
  a.cache_sb = 0;
  a.valid_length = nullptr;
  a.attend_length = nullptr;
  a.max_length = a.q_features = a.kv_features = 0;
  if (mode == kModeRope) {
    const DLTensor* pos = rope->position_ids;
    const DLTensor* tab = rope->cos_sin_cache;
    SQ_REQUIRE(pos && tab, SQ_EINVAL, "%s: null tensor argument", fn);
    SQ_REQUIRE(rope->head_dim > 0 && rope->head_dim % 2 == 0, SQ_EUNSUPPORTED, "%s: head_dim must be even (got %d)", fn, (int)rope->head_dim);
    SQ_REQUIRE(rope->rope_features >= 0 && rope->rope_features <= N && rope->rope_features % rope->head_dim == 0, SQ_ESHAPE,
               "%s: rope_features must be whole heads of %d within the %lld output features (got %d)", fn, (int)rope->head_dim, (long long)N,
               (int)rope->rope_features);
    SQ_REQUIRE(on_gpu(pos) && pos->device.device_id == dev && on_gpu(tab) && tab->device.device_id == dev, SQ_EDEVICE,
               "%s: position_ids and cos_sin_cache must live on the tensors' device", fn);
    const bool i64 = pos->dtype.code == kDLInt && pos->dtype.bits == 64 && pos->dtype.lanes == 1;
    SQ_REQUIRE((i64 || dtype_of(pos) == DType::I32) && numel_of(pos) == M && is_compact(pos), SQ_ESHAPE,
               "%s: position_ids must be a contiguous int32 or int64 tensor of %lld entries", fn, (long long)M);
    SQ_REQUIRE(dtype_of(tab) == DType::F32 && tab->ndim == 2 && tab->shape[1] == rope->head_dim && is_compact(tab) && tab->shape[0] > 0 &&
                   tab->shape[0] < ((int64_t)1 << 31),
               SQ_ESHAPE, "%s: cos_sin_cache must be a contiguous fp32 [max_position, %d] table (cos | sin)", fn, (int)rope->head_dim);
    a.pos = data_of(pos);
    a.table = (const float*)data_of(tab);
    a.pos_is_i64 = i64 ? 1 : 0;
    a.max_pos = (int)tab->shape[0];
    a.head_dim = rope->head_dim;
    a.rope_features = rope->rope_features;
    if (rope->key_cache || rope->value_cache || rope->valid_length || rope->attend_length) {
      const DLTensor* kc = rope->key_cache;
      const DLTensor* vc = rope->value_cache;
      const DLTensor* vl = rope->valid_length;
      SQ_REQUIRE(kc && vc && vl, SQ_EINVAL, "%s: key_cache, value_cache and valid_length go together", fn);
      const int64_t kvf = N - rope->rope_features;   // width of v = width of k
      SQ_REQUIRE(kvf > 0 && kvf % rope->head_dim == 0 && rope->rope_features >= kvf, SQ_ESHAPE,
                 "%s: the output must be [q | k | v] with k and v of equal width (rope_features %d of %lld)", fn, (int)rope->rope_features, (long long)N);
      const DLTensor* both[2] = {kc, vc};
      for (const DLTensor* t : both) {
        int rc2;
        if ((rc2 = check_tensor(t, "cache", 4, dev))) return rc2;
        SQ_REQUIRE(dtype_of(t) == dt && is_compact(t) && t->shape[0] == M && t->shape[2] * t->shape[3] == kvf && t->shape[3] == rope->head_dim &&
                       t->shape[1] == kc->shape[1] && t->shape[1] < ((int64_t)1 << 31),
                   SQ_ESHAPE, "%s: the caches must be contiguous [%lld, L, Hkv, %d] of x's dtype with Hkv * %d = %lld", fn, (long long)M,
                   (int)rope->head_dim, (int)rope->head_dim, (long long)kvf);
      }
      const DLTensor* lens[2] = {vl, rope->attend_length};
      for (const DLTensor* t : lens) {
        if (!t) continue;
        SQ_REQUIRE(on_gpu(t) && t->device.device_id == dev, SQ_EDEVICE, "%s: length tensors must live on the cache's device", fn);
        SQ_REQUIRE(dtype_of(t) == DType::I32 && t->ndim == 1 && t->shape[0] == M && is_compact(t), SQ_ESHAPE,
                   "%s: length tensors must be contiguous int32 [%lld]", fn, (long long)M);
      }
      a.k_cache = data_of(kc);
      a.v_cache = data_of(vc);
      a.cache_sb = kc->shape[1] * kvf * 2;
      a.valid_length = (const int32_t*)data_of(vl);
      a.attend_length = rope->attend_length ? (int32_t*)data_of(rope->attend_length) : nullptr;
      a.max_length = (int)kc->shape[1];
      a.q_features = (int)(rope->rope_features - kvf);
      a.kv_features = (int)kvf;
    }
  }
  int cur = -1;
  SQ_HIP(hipGetDevice(&cur));
  SQ_REQUIRE(cur == dev, SQ_EDEVICE, "%s: tensors live on device %d but the current device is %d", fn, dev, cur);
  a.x = data_of(x);
  a.w = data_of(weight);
  a.bias = bias ? data_of(bias) : nullptr;
  a.res = residual ? data_of(residual) : nullptr;
  a.y = data_of(out);
  a.x_sr = stride_of(x, 0) * 2;
  a.w_sr = stride_of(weight, 0) * 2;
  a.r_sr = residual ? stride_of(residual, 0) * 2 : 0;
  a.y_sr = stride_of(out, 0) * 2;
  a.rows = (int)M;
  a.n = (int)N;
  a.k = (int)K;
  if (dt == DType::BF16) launch<true>(a, mode, (hipStream_t)stream);
  else launch<false>(a, mode, (hipStream_t)stream);
  SQ_HIP(hipGetLastError());
  return SQ_OK;
}
}  // namespace

extern "C" int sq_linear_rows(const DLTensor* x, const DLTensor* weight, const DLTensor* bias, const DLTensor* residual,
                              DLTensor* out, void* stream) {
  return linear_rows("sq_linear_rows", kModePlain, x, weight, bias, residual, out, stream);
}

extern "C" int sq_linear_rows_silu_and_mul(const DLTensor* x, const DLTensor* weight, const DLTensor* bias, DLTensor* out, void* stream) {
  return linear_rows("sq_linear_rows_silu_and_mul", kModeGated, x, weight, bias, nullptr, out, stream);
}

extern "C" int sq_linear_rows_rope(const DLTensor* x, const DLTensor* weight, const DLTensor* bias, const DLTensor* position_ids,
                                   const DLTensor* cos_sin_cache, int32_t head_dim, int32_t rope_features, DLTensor* out,
                                   DLTensor* key_cache, DLTensor* value_cache, const DLTensor* valid_length, DLTensor* attend_length,
                                   void* stream) {
  const RopeSpec rope{position_ids, cos_sin_cache, head_dim, rope_features, key_cache, value_cache, valid_length, attend_length};
  return linear_rows("sq_linear_rows_rope", kModeRope, x, weight, bias, nullptr, out, stream, &rope);
}

extern "C" int sq_rmsnorm_linear_rows(const DLTensor* x, const DLTensor* norm_weight, float epsilon, const DLTensor* weight, const DLTensor* bias,
                                      const DLTensor* residual, DLTensor* out, void* stream) {
  const NormSpec norm{norm_weight, epsilon};
  return linear_rows("sq_rmsnorm_linear_rows", kModePlain, x, weight, bias, residual, out, stream, nullptr, &norm);
}

extern "C" int sq_rmsnorm_linear_rows_silu_and_mul(const DLTensor* x, const DLTensor* norm_weight, float epsilon, const DLTensor* weight,
                                                   const DLTensor* bias, DLTensor* out, void* stream) {
  const NormSpec norm{norm_weight, epsilon};
  return linear_rows("sq_rmsnorm_linear_rows_silu_and_mul", kModeGated, x, weight, bias, nullptr, out, stream, nullptr, &norm);
}

extern "C" int sq_rmsnorm_linear_rows_rope(const DLTensor* x, const DLTensor* norm_weight, float epsilon, const DLTensor* weight,
                                           const DLTensor* bias, const DLTensor* position_ids, const DLTensor* cos_sin_cache, int32_t head_dim,
                                           int32_t rope_features, DLTensor* out, DLTensor* key_cache, DLTensor* value_cache,
                                           const DLTensor* valid_length, DLTensor* attend_length, void* stream) {
  const RopeSpec rope{position_ids, cos_sin_cache, head_dim, rope_features, key_cache, value_cache, valid_length, attend_length};
  const NormSpec norm{norm_weight, epsilon};
  return linear_rows("sq_rmsnorm_linear_rows_rope", kModeRope, x, weight, bias, nullptr, out, stream, &rope, &norm);
}
