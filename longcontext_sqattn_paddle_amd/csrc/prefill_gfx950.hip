// Causal / sink+window prefill attention for gfx950 (MI355X).
//
// Replaces the reference's Triton prefill kernels and their wrappers:
//   full causal      sqattn/attn_triton.py:10-87 (_attn_fwd_inner), :90-213 (_attn_fwd), :216-315 (attn_causal)
//   relative window  sqattn/attn_triton_mix_relative.py:8-99, :102-306, :309-483
//   absolute window  sqattn/attn_triton_mix_bad.py:9-98, :101-282, :285-426
// All three run the same KV-block step (S = q~.k, running max, p = exp2(S-m), l += sum p, optional e4m3
// round trip of p, acc += fp16(p).fp16(v)); they differ only in which 64-key blocks a query block visits.
//
// Design (CDNA4, 64-wide waves, 2 waves per SIMD, at most 256 registers per lane):
//   * workgroup = WAVES (8) waves x 32 query rows of one q-head; K and V^T tiles of 64 keys are copied once per
//     workgroup into rings of 4 LDS buffers by global_load_lds (unpadded, XOR-swizzled) and shared by all its rows;
//     one workgroup barrier per two tiles;
//   * S^T = K . Q~^T on v_mfma_f32_32x32x16 (bf16 or f16): K rows are the A operand straight out of LDS, Q~
//     stays in registers as the B operand for the whole kernel.  The accumulator then holds, per lane,
//     one query row and 32 of the 64 keys, so the row max needs one cross-lane exchange and the row sum none;
//   * P^T in that accumulator layout *is* the B-operand layout of O^T += V^T . P^T (f16 MFMA, or the K=64 fp8 MFMA
//     when P and V are e4m3), provided V^T is stored with the matching key permutation -- a one-off pre-pass
//     writes V as transposed, permuted tiles into the workspace (O(N) work against the O(N^2) main loop);
//   * the tile step is laid out by hand in slots of one MFMA plus the vector and LDS work that runs beside it;
//   * blockIdx -> (kv head, q head, q block) mapping keeps the q-heads of one KV head on the same XCD(s) so
//     their K/V tiles are shared in that XCD's L2, and issues the longest (last) query blocks first.
#include <type_traits>

#include "common.hpp"

namespace sq {
namespace {

constexpr int kD = 128;
constexpr int kBN = 64;                  // keys per tile (BLOCK_N of every reference kernel)
// LDS tiles are unpadded and XOR-swizzled at 16-byte granularity (they are filled by global_load_lds, which
// writes 64 consecutive 16-byte slots per wave instruction): chunk c of K row n sits in slot c ^ (n & 15),
// chunk c of V^T row d in slot c ^ ((d >> 1) & 7).  The 16 rows a quarter-wave reads at one chunk index then
// fall into 16 different 16-byte bank groups.
constexpr int kKStride = 256;            // bytes per K row in LDS
constexpr int kVStride = 128;            // bytes per V^T row in LDS
constexpr int kKTileBytes = kBN * kKStride;
constexpr int kVTileBytes = kD * kVStride;
constexpr int kStageBytes = kKTileBytes + kVTileBytes;
constexpr int kMaxHeads = 128;

struct PrefillArgs {
  const void* q;
  const void* k;
  const void* q4;   // operands of the 4-bit window range (null: same as q/k)
  const void* k4;
  const _Float16* vt;  // [B, Hkv, nT, 128, 64] fp16 transposed, permuted V tiles (MODE 0..3)
  const uint8_t* vt8;  // [B, Hkv, nT, 128, 64] e4m3 transposed, permuted V tiles (MODE 4)
  const float* v_inv_scale;  // [B, Hkv, 128] absmax/448 per channel (MODE 4)
  void* out;
  float* lse;
  int64_t q_sb, q_sh, q_sn;
  int64_t k_sb, k_sh, k_sn;
  int64_t o_sb, o_sh, o_sn;
  int32_t B, Hq, Hkv, group, Nq, Nk, nT, nQB;
  int32_t q_offset, p_quant, window_mode, block_m, sink, out_dtype;
  int32_t sched_mode, sched_xpp, sched_items, sched_pairs;
  const float* k_scale;   // MODE 6: per-token scales of the int8 key codes in `k`, fp32 [B, Hkv, nT * 64]
  int32_t q_quant;   // 8: the rows of q (not of q4) are fake-quantised to 8 bits per token as they are loaded
  float sm;
  int32_t w8[kMaxHeads];
  int32_t w4[kMaxHeads];
};

struct PrepArgs {
  const void* v;
  _Float16* vt;
  uint8_t* vt8;          // e4m3 tiles (MODE 4)
  uint32_t* vmax_bits;   // [B, Hkv, 128] running |v| maximum as fp32 bit patterns (MODE 4)
  float* v_inv_scale;    // [B, Hkv, 128]
  int64_t v_sb, v_sh, v_sn;
  int32_t Nk, nT, Hkv, is_bf16;
};

// position of key u (0..15) inside its group of 16 in the V^T tile: bits 2 and 3 swapped, so that the 8
// keys a lane owns in one half of the S^T accumulator are 8 consecutive halfs.
__device__ __forceinline__ int perm16(int u) { return (u & 3) | ((u & 4) << 1) | ((u & 8) >> 1); }

__global__ __launch_bounds__(256) void prefill_prep_v_kernel(PrepArgs a) {
  const int j = blockIdx.x, kvh = blockIdx.y, b = blockIdx.z;
  const int o = threadIdx.x & 15;    // channel octet
  const int tq = threadIdx.x >> 4;   // key quad
  const uint16_t* vb = (const uint16_t*)a.v + (int64_t)b * a.v_sb + (int64_t)kvh * a.v_sh;
  _Float16 h[4][8];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int n = j * kBN + 4 * tq + i;
    uint4 raw = make_uint4(0, 0, 0, 0);
    if (n < a.Nk) raw = *(const uint4*)(vb + (int64_t)n * a.v_sn + 8 * o);
    const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const uint32_t bits = (e & 1) ? (w[e >> 1] >> 16) : (w[e >> 1] & 0xffffu);
      h[i][e] = a.is_bf16 ? (_Float16)bf16_bits_to_f32(bits) : __builtin_bit_cast(_Float16, (uint16_t)bits);
    }
  }
  _Float16* tile = a.vt + (((int64_t)b * a.Hkv + kvh) * a.nT + j) * (int64_t)(kD * kBN);
  const int pos = (4 * tq & ~15) | perm16(4 * tq & 15);
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    f16x4_t val = {h[0][e], h[1][e], h[2][e], h[3][e]};
    *(f16x4_t*)(tile + (8 * o + e) * kBN + pos) = val;
  }
}

// ---- fp8 P.V path (MODE 4): V is quantised to e4m3 with one scale per (batch, kv head, channel).
// (1) per-channel |v| maximum over all keys: every workgroup reduces one 64-key tile and merges with an integer
// atomic max (non-negative floats order like their bit patterns).
__global__ void prefill_fill_u32_kernel(uint32_t* p, int n) {
  for (int i = threadIdx.x; i < n; i += blockDim.x) p[i] = 0u;
}

__global__ __launch_bounds__(256) void prefill_vabsmax_kernel(PrepArgs a) {
  __shared__ float red[16][kD];
  const int j = blockIdx.x, kvh = blockIdx.y, b = blockIdx.z;
  const int o = threadIdx.x & 15, tq = threadIdx.x >> 4;
  const uint16_t* vb = (const uint16_t*)a.v + (int64_t)b * a.v_sb + (int64_t)kvh * a.v_sh;
  float mx[8] = {0, 0, 0, 0, 0, 0, 0, 0};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int n = j * kBN + 4 * tq + i;
    if (n < a.Nk) {
      const uint4 raw = *(const uint4*)(vb + (int64_t)n * a.v_sn + 8 * o);
      const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
      for (int e = 0; e < 8; ++e) {
        const uint32_t bits = (e & 1) ? (w[e >> 1] >> 16) : (w[e >> 1] & 0xffffu);
        const float x = a.is_bf16 ? bf16_bits_to_f32(bits) : (float)__builtin_bit_cast(_Float16, (uint16_t)bits);
        mx[e] = fmaxf(mx[e], fabsf(x));
      }
    }
  }
#pragma unroll
  for (int e = 0; e < 8; ++e) red[tq][8 * o + e] = mx[e];
  __syncthreads();
  if (threadIdx.x < kD) {
    float m = 0.f;
#pragma unroll
    for (int r = 0; r < 16; ++r) m = fmaxf(m, red[r][threadIdx.x]);
    atomicMax(a.vmax_bits + ((int64_t)b * a.Hkv + kvh) * kD + threadIdx.x, __float_as_uint(m));
  }
}

// (2) e4m3 tiles, transposed and permuted for v_mfma_f32_32x32x64_f8f6f4: key u of a tile sits at byte
// 32 g + 16 bn + 4 (w >> 3) + (w & 3) of its channel row, with bn = u >> 5, w = u & 31, g = (w >> 2) & 1 -- the order
// in which a lane of the S^T accumulator holds its 32 keys.
__global__ __launch_bounds__(256) void prefill_prep_v8_kernel(PrepArgs a) {
  const int j = blockIdx.x, kvh = blockIdx.y, b = blockIdx.z;
  const int o = threadIdx.x & 15;    // channel octet
  const int tq = threadIdx.x >> 4;   // key quad
  const uint16_t* vb = (const uint16_t*)a.v + (int64_t)b * a.v_sb + (int64_t)kvh * a.v_sh;
  const int64_t ch0 = ((int64_t)b * a.Hkv + kvh) * kD + 8 * o;
  float sc[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    // power-of-two scale 2^floor(log2(448/amax)): bf16/fp16 values times it are exact in fp32, so the e4m3
    // conversion only ever sees exact values (v_cvt_pk_fp8_f32 mis-rounds inputs that lie within an fp32 ulp or
    // two of a tie, which arbitrary scales hit systematically for 8-bit-mantissa inputs); fp8 is a floating
    // format, so a power-of-two scale costs no precision
    const float amax = __uint_as_float(a.vmax_bits[ch0 + e]);
    int ex = 1;
    if (amax > 0.f) (void)frexpf(448.f / amax, &ex);   // 448/amax = f * 2^ex, f in [0.5, 1)
    sc[e] = ldexpf(1.f, ex - 1);
    if (j == 0 && tq == 0) a.v_inv_scale[ch0 + e] = ldexpf(1.f, 1 - ex);
  }
  float x[4][8];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    const int n = j * kBN + 4 * tq + i;
    uint4 raw = make_uint4(0, 0, 0, 0);
    if (n < a.Nk) raw = *(const uint4*)(vb + (int64_t)n * a.v_sn + 8 * o);
    const uint32_t w[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      const uint32_t bits = (e & 1) ? (w[e >> 1] >> 16) : (w[e >> 1] & 0xffffu);
      const float v = a.is_bf16 ? bf16_bits_to_f32(bits) : (float)__builtin_bit_cast(_Float16, (uint16_t)bits);
      x[i][e] = fminf(fmaxf(v * sc[e], -448.f), 448.f);
    }
  }
  uint8_t* tile = a.vt8 + (((int64_t)b * a.Hkv + kvh) * a.nT + j) * (int64_t)(kD * kBN);
  const int pos = 32 * (tq & 1) + 16 * (tq >> 3) + 4 * ((tq >> 1) & 3);
#pragma unroll
  for (int e = 0; e < 8; ++e) {
    int pk = __builtin_amdgcn_cvt_pk_fp8_f32(x[0][e], x[1][e], 0, false);
    pk = __builtin_amdgcn_cvt_pk_fp8_f32(x[2][e], x[3][e], pk, true);
    *(int*)(tile + (8 * o + e) * kBN + pos) = pk;
  }
}

template <bool BF16>
__device__ __forceinline__ f32x16_t mfma_qk32(const uint4& a, const uint4& b, f32x16_t c) {
  if constexpr (BF16) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b),
                                                   c, 0, 0, 0);
  } else {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c,
                                                  0, 0, 0);
  }
}

__device__ __forceinline__ f32x16_t mfma_pv32(const uint4& a, const uint4& b, f32x16_t c) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c, 0,
                                                0, 0);
}

__device__ __forceinline__ uint32_t pack_f16(float lo, float hi) {
  typedef __attribute__((ext_vector_type(2))) float f32x2_t;
  typedef __attribute__((ext_vector_type(2))) _Float16 f16x2_t;
  f32x2_t v = {lo, hi};
  return __builtin_bit_cast(uint32_t, __builtin_convertvector(v, f16x2_t));
}

// one 16-bit element of the tensor dtype as a value, and back (round to nearest even)
template <bool BF16>
__device__ __forceinline__ float elem16(uint32_t bits) {
  if constexpr (BF16) return bf16_bits_to_f32(bits & 0xffffu);
  else return (float)__builtin_bit_cast(_Float16, (uint16_t)bits);
}
template <bool BF16>
__device__ __forceinline__ uint32_t bits16(float x) {
  if constexpr (BF16) return f32_to_bf16_bits(x);
  else return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)x);
}

template <bool BF16>
__device__ __forceinline__ uint32_t scale_pair(uint32_t w, float sm) {
  if constexpr (BF16) {
    const float lo = bf16_bits_to_f32(w & 0xffffu) * sm;
    const float hi = bf16_bits_to_f32(w >> 16) * sm;
    return pack_bf16x2(lo, hi);
  } else {
    const float lo = (float)__builtin_bit_cast(_Float16, (uint16_t)(w & 0xffffu)) * sm;
    const float hi = (float)__builtin_bit_cast(_Float16, (uint16_t)(w >> 16)) * sm;
    return pack_f16(lo, hi);
  }
}

// The KV tiles one 64-row wave visits, in tile units (multiples of 64 keys).
struct WaveRanges {
  int sink_hi;    // [0, sink_hi)
  int win_lo;     // [win_lo, win_hi): window tiles strictly before the query block
  int win_hi;
  int r4_lo;      // [r4_lo, r4_hi): tiles of the 4-bit window range (subset of the window tiles)
  int r4_hi;
  int diag_lo;    // [diag_lo, diag_hi]: tiles of the query block itself up to this wave's own diagonal tile
  int diag_hi;
  __device__ __forceinline__ bool visits(int j) const {
    return j < sink_hi || (j >= win_lo && j < win_hi) || (j >= diag_lo && j <= diag_hi);
  }
};

__device__ __forceinline__ WaveRanges wave_ranges(const PrefillArgs& a, int pos0, int head) {
  WaveRanges r;
  if (a.window_mode == SQ_WINDOW_NONE) {  // attn_triton.py:57-63
    r.sink_hi = 0;
    r.win_lo = 0;
    r.win_hi = pos0 / kBN;
    r.r4_lo = r.r4_hi = 0;
    r.diag_lo = r.diag_hi = pos0 / kBN;
    return r;
  }
  // attn_triton_mix_relative.py:36-75 / attn_triton_mix_bad.py:37-74
  const int qs = pos0 / a.block_m * a.block_m;
  const int qe = qs + a.block_m;
  const int w8 = a.w8[head], w4 = a.w4[head];
  const int left4 = max(a.sink, qe - w4);
  const int left8 = max(a.sink, qe - w8);
  r.sink_hi = min(a.sink, qs) / kBN;
  int lo = qs, hi = qs;
  r.r4_lo = r.r4_hi = 0;
  if (left8 < qs) lo = left8;
  if (left4 < left8) {  // range 2 non-empty; the host guarantees left8 <= qs here
    r.r4_lo = left4 / kBN;
    r.r4_hi = left8 / kBN;
    lo = left4;
  }
  r.win_lo = lo / kBN;
  r.win_hi = hi / kBN;
  r.diag_lo = qs / kBN;
  r.diag_hi = pos0 / kBN;
  return r;
}

// v_max3_f32 without the canonicalising self-max the compiler adds around fmaxf of MFMA results
__device__ __forceinline__ float max3(float a, float b, float c) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3" : "=v"(r) : "v"(a), "v"(b), "v"(c));
  return r;
}

// Chains of max3 as single asm statements: the compiler puts a wait-state nop behind every asm statement that a
// vector instruction follows, so a chain written as separate statements carries one nop per link.
__device__ __forceinline__ float max3_of8(float a0, float a1, float a2, float a3, float a4, float a5, float a6, float a7) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3\n\tv_max3_f32 %0, %0, %4, %5\n\tv_max3_f32 %0, %0, %6, %7\n\tv_max3_f32 %0, %0, %8, %8"
      : "=&v"(r)
      : "v"(a0), "v"(a1), "v"(a2), "v"(a3), "v"(a4), "v"(a5), "v"(a6), "v"(a7));
  return r;
}
__device__ __forceinline__ float max3_of5(float a0, float a1, float a2, float a3, float a4) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3\n\tv_max3_f32 %0, %0, %4, %5" : "=&v"(r) : "v"(a0), "v"(a1), "v"(a2), "v"(a3), "v"(a4));
  return r;
}
__device__ __forceinline__ float max3_of4(float a0, float a1, float a2, float a3) {
  float r;
  asm("v_max3_f32 %0, %1, %2, %3\n\tv_max3_f32 %0, %0, %4, %4" : "=&v"(r) : "v"(a0), "v"(a1), "v"(a2), "v"(a3));
  return r;
}

// max3 above is opaque to the compiler's hazard logic, which therefore does not separate it from a matrix
// instruction that has just written its inputs.  Where a max3 chain directly follows such instructions, this
// supplies the wait states by hand (the longest requirement, after a 16-pass MFMA, is below 32).
__device__ __forceinline__ void mfma_settle(f32x16_t& x, f32x16_t& y) {
  asm volatile("s_nop 15\n\ts_nop 15" : "+v"(x), "+v"(y));
}

// exchange with the lane 32 away (the other half of the keys of the same query row)
__device__ __forceinline__ float xor32_max(float v) {
  const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return fmaxf(__uint_as_float(sw[0]), __uint_as_float(sw[1]));
}
__device__ __forceinline__ float xor32_sum(float v) {
  const auto sw = __builtin_amdgcn_permlane32_swap(__float_as_uint(v), __float_as_uint(v), false, false);
  return __uint_as_float(sw[0]) + __uint_as_float(sw[1]);
}

constexpr float kLog2_448 = 8.807354922057604f;  // log2(448)

// Quantise 8 probabilities (one k-step of the P.V MFMA) and pack them as fp16 B-operand registers.
//   MODE 0  p.to(fp16)
//   MODE 1  fp16(e4m3(p*448)/448)   reference static scale (attn_triton.py:81-82): sc = 448, inv = 1/448
//   MODE 2  fp16(e4m3(p*sc)*inv)    block absmax scale a: sc = 448/a, inv = a/448
//   MODE 3  fp16(e4m3(p448))        p448 = 448*p, the factor folded into the exponent; the 1/448 cancels in
//                                   acc/l because l is accumulated from p448 as well
template <int MODE>
__device__ __forceinline__ uint4 quant_pack8(const f32x16_t& s, int t, float sc, float inv) {
  uint32_t w[4];
#pragma unroll
  for (int h = 0; h < 2; ++h) {
    const float p0 = s[8 * t + 4 * h + 0], p1 = s[8 * t + 4 * h + 1], p2 = s[8 * t + 4 * h + 2], p3 = s[8 * t + 4 * h + 3];
    if constexpr (MODE == 0) {
      w[2 * h] = pack_f16(p0, p1);
      w[2 * h + 1] = pack_f16(p2, p3);
    } else if constexpr (MODE == 3) {
      int pk = __builtin_amdgcn_cvt_pk_fp8_f32(p0, p1, 0, false);
      pk = __builtin_amdgcn_cvt_pk_fp8_f32(p2, p3, pk, true);
      w[2 * h] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(pk, 1.0f, false));
      w[2 * h + 1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(pk, 1.0f, true));
    } else {
      float q0 = p0 * sc, q1 = p1 * sc, q2 = p2 * sc, q3 = p3 * sc;
      if constexpr (MODE == 2) {
        q0 = fminf(q0, 448.f);
        q1 = fminf(q1, 448.f);
        q2 = fminf(q2, 448.f);
        q3 = fminf(q3, 448.f);
      }
      int pk = __builtin_amdgcn_cvt_pk_fp8_f32(q0, q1, 0, false);
      pk = __builtin_amdgcn_cvt_pk_fp8_f32(q2, q3, pk, true);
      typedef __attribute__((ext_vector_type(2))) float f32x2_t;
      const f32x2_t lo = __builtin_amdgcn_cvt_scalef32_pk_f32_fp8(pk, 1.0f, false);
      const f32x2_t hi = __builtin_amdgcn_cvt_scalef32_pk_f32_fp8(pk, 1.0f, true);
      w[2 * h] = pack_f16(lo[0] * inv, lo[1] * inv);
      w[2 * h + 1] = pack_f16(hi[0] * inv, hi[1] * inv);
    }
  }
  return make_uint4(w[0], w[1], w[2], w[3]);
}

// Four probabilities -> two fp16 B-operand words, MODE as in quant_pack8 (0, 1 or 3)
template <int MODE>
__device__ __forceinline__ void quant_pack4(float p0, float p1, float p2, float p3, uint32_t& w0, uint32_t& w1) {
  if constexpr (MODE == 0) {
    w0 = pack_f16(p0, p1);
    w1 = pack_f16(p2, p3);
  } else if constexpr (MODE == 3) {
    int pk = __builtin_amdgcn_cvt_pk_fp8_f32(p0, p1, 0, false);
    pk = __builtin_amdgcn_cvt_pk_fp8_f32(p2, p3, pk, true);
    w0 = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(pk, 1.0f, false));
    w1 = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_f16_fp8(pk, 1.0f, true));
  } else {
    int pk = __builtin_amdgcn_cvt_pk_fp8_f32(p0 * 448.f, p1 * 448.f, 0, false);
    pk = __builtin_amdgcn_cvt_pk_fp8_f32(p2 * 448.f, p3 * 448.f, pk, true);
    typedef __attribute__((ext_vector_type(2))) float f32x2_t;
    const f32x2_t lo = __builtin_amdgcn_cvt_scalef32_pk_f32_fp8(pk, 1.0f, false);
    const f32x2_t hi = __builtin_amdgcn_cvt_scalef32_pk_f32_fp8(pk, 1.0f, true);
    constexpr float inv = 1.0f / 448.0f;
    w0 = pack_f16(lo[0] * inv, lo[1] * inv);
    w1 = pack_f16(hi[0] * inv, hi[1] * inv);
  }
}

// One workgroup = WAVES waves x 32 query rows of one q-head (2 waves per SIMD when WAVES == 8, so that one
// wave's MFMA phase overlaps the other's softmax phase).  MODE as in quant_pack8.
// DUAL (WAVES == 8, absolute windows with their own 4-bit operands, block_m == 128): the workgroup holds two query blocks,
// A = waves 0..3 and B = waves 4..7, whose 4-bit ranges end 128 keys apart.  On the up to two tiles in between -- 8-bit
// for A, 4-bit for B -- the blocks want different K tiles, so those tiles are walked twice: once as they are (B skips
// them), once as 4-bit copies right behind (A skips those).  Everywhere else the blocks agree, or only one of them visits.
template <bool BF16, int WAVES, int MODE, bool DUAL = false>
__global__ __launch_bounds__(WAVES * 64) void prefill_kernel(PrefillArgs a) {
  constexpr int NT = WAVES * 64;
  constexpr int CH = (kBN * kD * 2 / 16) / NT;  // 16-byte chunks per thread and tile operand
  constexpr int ROWS = 32;                      // query rows per wave
  // MODE 6: Q.K^T on the int8 matrix instruction -- `k` holds the 8-bit codes of the (centred) key, one byte per element,
  // `k_scale` their per-token scales; the query rows' codes and scale are formed here as the rows are loaded.  The scores
  // are sum(code products) x scale_k x (scale_q log2e / sqrt(D)); from there on the step is MODE 0's (fp16 P, fp16 V), on
  // the plain schedule MODE 2 also uses (no hand-placed slots).
  constexpr bool kQK8 = MODE == 6;
  constexpr bool kPlain = MODE == 2 || MODE == 6;   // tile step left to the compiler's scheduling
  constexpr bool kPV8 = MODE == 4 || MODE == 5;     // e4m3 V tiles, fp8 P.V
  extern __shared__ __attribute__((aligned(16))) char smem[];
  // MODE 2: tile maxima of the two waves of a 64-row group, behind the tile rings (which start at LDS address 0)
  float (*s_amax)[WAVES] = (float (*)[WAVES])(smem + 4 * kStageBytes);

  // ---- schedule: blockIdx -> (pair = (b, kvh), item = (q block descending, head in group))
  int pair, item;
  {
    const int id = blockIdx.x;
    if (a.sched_mode == 0) {  // pairs share the 8 XCDs evenly: sched_xpp XCDs per pair
      const int xcd = id & 7, s = id >> 3;
      pair = xcd / a.sched_xpp;
      item = s * a.sched_xpp + xcd % a.sched_xpp;
    } else if (a.sched_mode == 1) {  // one XCD works through pairs xcd, xcd+8, ...
      const int xcd = id & 7, s = id >> 3;
      pair = (s / a.sched_items) * 8 + xcd;
      item = s % a.sched_items;
    } else {
      pair = id % a.sched_pairs;
      item = id / a.sched_pairs;
    }
    if (item >= a.sched_items || pair >= a.sched_pairs) return;
  }
  const int b = pair / a.Hkv, kvh = pair % a.Hkv;
  const int hg = item % a.group;
  const int qb = a.nQB - 1 - item / a.group;
  const int head = kvh * a.group + hg;

  const int tid = threadIdx.x;
  const int lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);   // wave-uniform: keep it (and all it feeds) in SGPRs
  const int c32 = lane & 31, g = lane >> 5;

  const int row_wg0 = qb * (WAVES * ROWS);          // first query row of the workgroup
  const int row_w0 = row_wg0 + wave * ROWS;         // first query row of this wave
  const int pos0 = a.q_offset + row_w0;             // its absolute position
  const bool wave_active = row_w0 < a.Nq;
  const WaveRanges wr = wave_ranges(a, pos0, head);

  // ---- workgroup-level tile schedule: segment A = sink tiles, segment B = window .. last diagonal
  int segA_hi = 0, segB_lo = 1 << 30, segB_hi = 0;
#pragma unroll
  for (int w = 0; w < WAVES; ++w) {
    const int rw = row_wg0 + w * ROWS;
    if (rw < a.Nq) {
      const WaveRanges o = wave_ranges(a, a.q_offset + rw, head);
      segA_hi = max(segA_hi, o.sink_hi);
      segB_lo = min(segB_lo, min(o.win_lo, o.diag_lo));
      segB_hi = max(segB_hi, o.diag_hi + 1);
    }
  }
  segB_hi = min(segB_hi, a.nT);
  if (segB_lo <= segA_hi) {  // contiguous: one segment
    segA_hi = 0;
    segB_lo = 0;
  }
  // separate 4-bit operands run with WAVES*32 == block_m (all waves agree on a tile's operand set), or as DUAL
  const bool distinct4 = (WAVES < 8 || DUAL) && a.q4 != nullptr;
  // The tiles that are copied from the 4-bit key, [t4_lo, t4_hi): the 4-bit range of the workgroup's first query block.
  // DUAL: tiles [c_lo, c_lo + n_dup), from where block A's 4-bit range ends to where block B's ends (128 keys later, unless
  // the sink cuts both), are walked twice -- first as 4-bit copies for B, then as they are for A.
  int t4_lo = wr.r4_lo, t4_hi = wr.r4_hi, c_lo = 0, n_dup = 0;
  if constexpr (DUAL) {
    const WaveRanges wa = wave_ranges(a, a.q_offset + row_wg0, head);
    t4_lo = wa.r4_lo;
    t4_hi = wa.r4_hi;
    if (row_wg0 + 4 * ROWS < a.Nq) {
      const int qeA = (a.q_offset + row_wg0) / a.block_m * a.block_m + a.block_m, qeB = qeA + a.block_m;
      const int left8A = max(a.sink, qeA - a.w8[head]), left8B = max(a.sink, qeB - a.w8[head]), left4B = max(a.sink, qeB - a.w4[head]);
      if (left4B < left8B && left8A < left8B) {
        c_lo = left8A / kBN;
        n_dup = (left8B - left8A) / kBN;
        if (t4_hi <= t4_lo) t4_lo = c_lo;   // block A has no 4-bit range of its own (the sink cuts it): the copies are all there is
        t4_hi = c_lo;                        // (where A has one, it ends at c_lo anyway)
      }
    }
  }
  // ---- Q~ fragments (B operand of S^T = K.Q~^T): lane (column = query row c32, k-group g)
  uint4 qf[8];
  auto load_q = [&](const void* qbase) __attribute__((always_inline)) {
    const uint16_t* qp = (const uint16_t*)qbase + (int64_t)b * a.q_sb + (int64_t)head * a.q_sh;
    const int row = max(min(row_w0 + c32, a.Nq - 1), 0);
    const uint16_t* rp = qp + (int64_t)row * a.q_sn + 8 * g;
    uint4 raw[8];
#pragma unroll
    for (int kk = 0; kk < 8; ++kk) raw[kk] = *(const uint4*)(rp + 16 * kk);
    if (a.q_quant == 8 && qbase == a.q) {
      // IntegerQuantizer(8, True, "per_token").fake_quant_tensor of the row (fake_quant.py:33-35, 47-52, 114-125) with the
      // operations of the stand-alone pre-pass (prepass_rows_kernel: the same maximum, the same correctly rounded
      // division, round half away, clamp, product, rounding to the tensor dtype), so the operand has the same bits as a
      // row that went through that pass and memory.  The row's 128 elements sit in this lane and the lane 32 away.
      float amax = 0.f;
#pragma unroll
      for (int kk = 0; kk < 8; ++kk) {
        const uint32_t w[4] = {raw[kk].x, raw[kk].y, raw[kk].z, raw[kk].w};
#pragma unroll
        for (int j = 0; j < 4; ++j) amax = fmaxf(amax, fmaxf(fabsf(elem16<BF16>(w[j] & 0xffffu)), fabsf(elem16<BF16>(w[j] >> 16))));
      }
      amax = fmaxf(xor32_max(amax), 1e-5f);
      const Divisor scale = make_divisor(amax / 127.f);
      auto qdq_elem = [&](float x) {   // clamp(round(x / scale) + zero, -128, 127) * scale with zero = 0.0 (turns -0.0 into +0.0)
        const float t = divide(x, scale);
        return fminf(fmaxf(copysignf(floorf(fabsf(t) + 0.5f), t) + 0.0f, -128.f), 127.f) * scale.d;
      };
      auto qdq_word = [&](uint32_t w) {
        return bits16<BF16>(qdq_elem(elem16<BF16>(w & 0xffffu))) | (bits16<BF16>(qdq_elem(elem16<BF16>(w >> 16))) << 16);
      };
#pragma unroll
      for (int kk = 0; kk < 8; ++kk) raw[kk] = make_uint4(qdq_word(raw[kk].x), qdq_word(raw[kk].y), qdq_word(raw[kk].z), qdq_word(raw[kk].w));
    }
#pragma unroll
    for (int kk = 0; kk < 8; ++kk)
      qf[kk] = make_uint4(scale_pair<BF16>(raw[kk].x, a.sm), scale_pair<BF16>(raw[kk].y, a.sm), scale_pair<BF16>(raw[kk].z, a.sm),
                          scale_pair<BF16>(raw[kk].w, a.sm));
  };
  // MODE 6: the row's 8-bit codes as the B operand of v_mfma_i32_32x32x32_i8 -- k-step kk covers dimensions 32 kk .. +31,
  // of which this lane holds 16 g .. +15 (the lane 32 away the rest; the K fragments are cut the same way, so the pairing
  // of the products does not depend on how the instruction numbers its k index) -- and the row's scale times log2e / sqrt(D).
  typedef __attribute__((ext_vector_type(4))) int i32x4_t;
  typedef __attribute__((ext_vector_type(16))) int i32x16_t;
  i32x4_t qc[4] = {};
  float q_scale = 0.f;
  // (the query rows are loaded further down, behind the first tile copies, so that both travel at the same time)
  bool q_is4 = false;

  f32x16_t O[4];
#pragma unroll
  for (int bd = 0; bd < 4; ++bd)
#pragma unroll
    for (int i = 0; i < 16; ++i) O[bd][i] = 0.f;
  // Online-softmax state of this lane's query row.  The score accumulators are *initialised* with
  // cinit = kC - m_run (kC = log2(448) in MODE 3, else 0), so the MFMA chain delivers S - m_run + kC and, as
  // long as the running maximum does not move, p (or 448 p) is a bare exp2 of the accumulator.
  constexpr float kC = (MODE >= 3 && MODE <= 5) ? kLog2_448 : 0.f;
  // Lazy re-centring (the modes whose P is a plain fp16 number: MODE 0, and MODE 6, which differs from it in the Q.K^T
  // product only): a row maximum may rise up to kLazy (in log2 units) above the reference before the accumulators are
  // rescaled.  p is rounded to fp16, which has the same ten mantissa bits at 2^8 as at 1, so p = 2^(s - reference) up to
  // 2^8 is the same probability with the same relative rounding error (2^-11) as the reference's
  // 2^(s - running maximum) <= 1 -- not the same bits, and small probabilities keep more of their bits than there; the
  // fp32 accumulators and the denominator carry the common factor until the division at the end.  A row is shifted only
  // when its own maximum passes the limit, so its arithmetic does not depend on the other rows of the wave.  With
  // re-centring at once, one row of the wave's 32 finding a new maximum sends the whole wave through the rescale path
  // (some 110 vector instructions): about 32 (1 + ln(tiles / 32)) times per wave, which is 8 % of the tiles of a
  // 131072-key causal row and 40 % of the 214 tiles of a sink + 10 % window.  The e4m3 modes with the static scale (1, 3,
  // 4) need p <= 1 for their grid and re-centre at once; MODE 5 has a rule of its own (kDefer below).
  constexpr float kLazy = (MODE == 0 || MODE == 6) ? 8.f : 0.f;
  constexpr float kMove = kC + kLazy;
  // MODE 5 takes neither the block scale nor the decision to move the reference from the row's maximum of the tile but
  // from the row's SUM of the tile's probabilities, which the denominator needs anyway: the maximum tree (26 vector
  // instructions per tile) goes.  The probabilities of a tile are formed against the standing reference without looking
  // at the scores first; a row whose sum then exceeds 2^16 moves its reference up by a whole number of binades
  // (exact rescaling, also of the tile just packed, through the scale operand of its MFMA), and a row whose sum is not
  // finite -- a score more than 2^100 above everything the row has seen -- has the tile recomputed from the key rows in
  // memory against the tile's own maximum (redo_tile).  The scale needs the whole tile's sum, so the tile's P.V product
  // is deferred by one visited step: the conversions to e4m3 run under the P.V MFMAs of the tile before.
  constexpr bool kDefer = MODE == 5;
  constexpr float kSumLimit = 448.f * 65536.f;   // 2^16 in units of the probabilities as formed (times 448)
  constexpr float kRedoLimit = 1.329227995784916e36f;   // 2^120: beyond it (or not a number) the tile is formed again
  float m_run = 0.f;       // reference point of the exponent; the first visited tile replaces it by the row maximum
  float l_run = 0.f;       // this lane's share of the denominator (times 448 in MODE 3)
  bool first = true;       // wave-uniform: no tile visited yet
  f32x16_t Cinit;
#pragma unroll
  for (int i = 0; i < 16; ++i) Cinit[i] = kC;

  const _Float16* vt_base = a.vt + ((int64_t)b * a.Hkv + kvh) * (int64_t)a.nT * (kD * kBN);

  // ---- tile staging: global -> LDS directly (no registers), CH wave instructions of 64 x 16 bytes per operand.
  // K and V^T have their own double buffers because the K tile runs one step ahead of the V^T tile (below).
  typedef __attribute__((address_space(3))) void* lds_ptr_t;
  const int64_t k_head_off = (int64_t)b * a.k_sb + (int64_t)kvh * a.k_sh;
  char* const kbase_lds = smem;                     // 4 x 16 KB
  char* const vbase_lds = smem + 4 * kKTileBytes;   // 4 x 16 KB (8 KB used per buffer in the fp8 mode)
  auto stage_k16 = [&](int j, int stage, bool use4) {
    char* kbuf = kbase_lds + stage * kKTileBytes;
    const uint16_t* kb = (const uint16_t*)(use4 ? a.k4 : a.k) + k_head_off;
    // DUAL runs this form for the first and the last few tiles only (stage_k_full in between): its per-lane addresses, for
    // two key tensors, are formed here and not hoisted into registers the tile loop has no room for
    int ln = lane;
    if constexpr (DUAL) asm volatile("; clamped tile copy" : "+v"(ln));
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const int q = wave * CH + c;                       // wave instruction index 0..15 -> 1 KB of the tile
      const int kr = 4 * q + (ln >> 4);                  // K row in the tile
      const int kc = (ln & 15) ^ (kr & 15);              // global chunk that lands in this lane's slot
      const int n = min(j * kBN + kr, a.Nk - 1);
      __builtin_amdgcn_global_load_lds((const void*)(kb + (int64_t)n * a.k_sn + 8 * kc), (lds_ptr_t)(kbuf + q * 1024), 16, 0, 0);
    }
  };
  // MODE 6: a tile of key codes is 64 rows x 128 bytes = 8 KB (one wave instruction of 8 rows per 1 KB; 16-byte chunk c
  // of row r lands in slot c ^ (r & 7)), followed by the tile's 64 scales (one 4-byte copy per lane of wave 0)
  auto stage_k8 = [&](int j, int stage) {
    char* kbuf = kbase_lds + stage * kKTileBytes;
    const char* kb = (const char*)a.k + k_head_off;
    constexpr int CH8 = CH / 2;
#pragma unroll
    for (int c = 0; c < CH8; ++c) {
      const int q = wave * CH8 + c;
      const int kr = 8 * q + (lane >> 3);
      const int kc = (lane & 7) ^ (kr & 7);
      const int n = min(j * kBN + kr, a.Nk - 1);
      __builtin_amdgcn_global_load_lds((const void*)(kb + (int64_t)n * a.k_sn + 16 * kc), (lds_ptr_t)(kbuf + q * 1024), 16, 0, 0);
    }
    if (wave == 0)
      __builtin_amdgcn_global_load_lds((const void*)(a.k_scale + (((int64_t)b * a.Hkv + kvh) * a.nT + j) * kBN + lane),
                                       (lds_ptr_t)(kbuf + kBN * kD), 4, 0, 0);
  };
  auto stage_k = [&](int j, int stage, bool use4) {
    if constexpr (kQK8) stage_k8(j, stage);
    else stage_k16(j, stage, use4);
  };
  auto stage_v = [&](int j, int stage) {
    char* vbuf = vbase_lds + stage * kVTileBytes;
    if constexpr (kPV8) {
      // e4m3 tile: 128 rows x 64 bytes = 8 KB, one wave instruction per wave; 16-byte chunk c of row d -> slot
      // c ^ ((d >> 2) & 3), which spreads the 16 rows a quarter-wave reads over all 16 bank groups
      const uint8_t* vsrc8 = a.vt8 + (((int64_t)b * a.Hkv + kvh) * a.nT + j) * (int64_t)(kD * kBN);
      const int vr = 16 * wave + (lane >> 2);
      const int vc = (lane & 3) ^ ((vr >> 2) & 3);
      uint32_t off = (uint32_t)(vr * kBN + 16 * vc);
      asm volatile("" : "+v"(off));   // 32-bit per-lane offset next to the uniform 64-bit tile base
      __builtin_amdgcn_global_load_lds((const void*)(vsrc8 + off), (lds_ptr_t)(vbuf + wave * 1024), 16, 0, 0);
      return;
    }
    const _Float16* vsrc = vt_base + (int64_t)j * (kD * kBN);
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      const int q = wave * CH + c;
      const int vr = 8 * q + (lane >> 3);                // V^T row (channel)
      const int vc = (lane & 7) ^ ((vr >> 1) & 7);
      __builtin_amdgcn_global_load_lds((const void*)(vsrc + vr * kBN + 8 * vc), (lds_ptr_t)(vbuf + q * 1024), 16, 0, 0);
    }
  };
  // staging of full K tiles of the unquantised operand: uniform tile base + per-lane 32-bit offset, no per-lane
  // 64-bit arithmetic in the loop
  uint32_t kvoff[CH];
#pragma unroll
  for (int c = 0; c < CH; ++c) {
    const int q = wave * CH + c;
    const int kr = 4 * q + (lane >> 4);
    const int kc = (lane & 15) ^ (kr & 15);
    kvoff[c] = (uint32_t)(kr * (int)a.k_sn + 8 * kc) * 2u;
  }
  const char* const k_bytes = (const char*)a.k + k_head_off * 2;
  // (the 4-bit key as a byte distance from the 8-bit one: a choice between two integers, where a choice between the two
  // captured pointers made the compiler keep this lambda's captures in memory)
  const int64_t k4_delta = DUAL ? (int64_t)((const char*)a.k4 - (const char*)a.k) : 0;
  const uint32_t k_tile_bytes = (uint32_t)(kBN * a.k_sn * 2);
  auto stage_k_full = [&](int j, int stage, bool use4) {
    const char* base = k_bytes + ((DUAL && use4) ? k4_delta : (int64_t)0) + (uint64_t)(uint32_t)j * k_tile_bytes;
    char* kbuf = kbase_lds + stage * kKTileBytes;
#pragma unroll
    for (int c = 0; c < CH; ++c) {
      uint32_t off = kvoff[c];
      asm volatile("" : "+v"(off));   // stays a 32-bit per-lane offset next to the uniform 64-bit tile base
      __builtin_amdgcn_global_load_lds((const void*)(base + off), (lds_ptr_t)(kbuf + (wave * CH + c) * 1024), 16, 0, 0);
    }
  };

  const int ksw = c32 & 15;          // swizzle of this lane's K rows (c32 and c32 + 32 share it)
  const uint32_t smem_addr = (uint32_t)(uintptr_t)(lds_ptr_t)smem;
  // byte offset of k-step kk's chunk inside this lane's K rows: c32 * 256 + (((2 kk + g) ^ ksw) << 4) =
  // kx0 ^ (kk << 5), and the same holds after adding a ring buffer's base (a multiple of 256; the rings start at
  // LDS address 0)
  const uint32_t kx0 = c32 * kKStride + ((g ^ ksw) << 4);
  // MODE 4 with the main loop unrolled over the four ring buffers: the LDS address of every fragment is a
  // per-lane constant plus an immediate offset, so the tile step spends no vector instruction on addresses
  constexpr bool kStaticRing = !kPlain;
  uint32_t kxr[8];
#pragma unroll
  for (int kk = 0; kk < 8; ++kk) kxr[kk] = smem_addr + (kx0 ^ (kk << 5));
  const uint32_t v8lo_base = smem_addr + 4 * kKTileBytes + c32 * 64 + (((2 * g) ^ ((c32 >> 2) & 3)) << 4);
  const uint32_t v8hi_base = v8lo_base ^ 16;
  uint32_t vxr[4];   // fp16 V^T fragments: key group m of this lane's rows
#pragma unroll
  for (int m = 0; m < 4; ++m)
    vxr[m] = smem_addr + 4 * kKTileBytes + ((c32 * kVStride + ((g ^ ((c32 >> 1) & 7)) << 4)) ^ (m << 5));
  typedef __attribute__((ext_vector_type(8))) int i32x8_t;
  i32x8_t P8 = {0, 0, 0, 0, 0, 0, 0, 0};   // MODE 4: e4m3 probabilities of the current tile (registers reused tile after tile)
  // MODE 5 multiplies a tile's probabilities with V one visited step later (kDefer): P8w holds the pending tile, which the
  // step's four P.V MFMAs consume while the current tile is packed, underneath them, into registers its probabilities
  // leave; it takes the current tile over at the end of the step.  It is zero while nothing is pending, so those MFMAs
  // then add nothing.  (Eight scalars, not a vector: the pack builtin takes the word it half-overwrites as two shorts,
  // and with the words kept as elements of a vector every element's old value came out as element 0's -- a wrong fold of
  // the element extraction with the cast.)
  int P8w[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  int e_pend = 127;    // E8M0 exponent of the pending tile's block scale
  int pend_t = -1;     // step of the pending tile (wave-uniform), -1: none
  const int vsw = (c32 >> 1) & 7;    // swizzle of this lane's V^T rows (32 bd + c32)

  // S^T = K . Q~^T + Cinit for one tile: 16 MFMAs that nothing below depends on until the next step
  auto qk_tile = [&](const char* kbuf, f32x16_t (&S)[2]) {
    if constexpr (kQK8) {
      i32x16_t acc0 = {}, acc1 = {};
#pragma unroll
      for (int kk = 0; kk < 4; ++kk) {
        const i32x4_t a0 = *(const i32x4_t*)(kbuf + c32 * kD + (((2 * kk + g) ^ (c32 & 7)) << 4));
        const i32x4_t a1 = *(const i32x4_t*)(kbuf + (32 + c32) * kD + (((2 * kk + g) ^ (c32 & 7)) << 4));
        acc0 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a0, qc[kk], acc0, 0, 0, 0);
        acc1 = __builtin_amdgcn_mfma_i32_32x32x32_i8(a1, qc[kk], acc1, 0, 0, 0);
      }
      // accumulator element i of block bn is key 32 bn + 8 (i >> 2) + 4 g + (i & 3): four neighbouring scales per read
      const float* sk = (const float*)(kbuf + kBN * kD);
#pragma unroll
      for (int q4i = 0; q4i < 4; ++q4i) {
        const float4 s0 = *(const float4*)(sk + 8 * q4i + 4 * g);
        const float4 s1 = *(const float4*)(sk + 32 + 8 * q4i + 4 * g);
        const float f0[4] = {s0.x, s0.y, s0.z, s0.w}, f1[4] = {s1.x, s1.y, s1.z, s1.w};
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          S[0][4 * q4i + e] = __builtin_fmaf((float)acc0[4 * q4i + e] * f0[e], q_scale, Cinit[4 * q4i + e]);
          S[1][4 * q4i + e] = __builtin_fmaf((float)acc1[4 * q4i + e] * f1[e], q_scale, Cinit[4 * q4i + e]);
        }
      }
      return;
    }
    {
      const uint4 a0 = *(const uint4*)(kbuf + c32 * kKStride + ((g ^ ksw) << 4));
      const uint4 a1 = *(const uint4*)(kbuf + (32 + c32) * kKStride + ((g ^ ksw) << 4));
      S[0] = mfma_qk32<BF16>(a0, qf[0], Cinit);
      S[1] = mfma_qk32<BF16>(a1, qf[0], Cinit);
    }
#pragma unroll
    for (int kk = 1; kk < 8; ++kk) {
      const uint4 a0 = *(const uint4*)(kbuf + c32 * kKStride + (((2 * kk + g) ^ ksw) << 4));
      const uint4 a1 = *(const uint4*)(kbuf + (32 + c32) * kKStride + (((2 * kk + g) ^ ksw) << 4));
      S[0] = mfma_qk32<BF16>(a0, qf[kk], S[0]);
      S[1] = mfma_qk32<BF16>(a1, qf[kk], S[1]);
    }
  };

  // MODE 4: maximum over this lane's 32 scores of a tile, as four independent chains
  auto lane_max = [&](const f32x16_t (&S)[2]) {
    float c[4];
#pragma unroll
    for (int h = 0; h < 4; ++h) {
      const f32x16_t& s = S[h >> 1];
      const int o = 8 * (h & 1);
      c[h] = max3(s[o], s[o + 1], s[o + 2]);
      c[h] = max3(c[h], s[o + 3], s[o + 4]);
      c[h] = max3(c[h], s[o + 5], s[o + 6]);
      c[h] = max3(c[h], s[o + 7], s[o + 7]);
    }
    return max3(max3(c[0], c[1], c[2]), c[3], c[3]);
  };
  // MODE 4: row maximum (relative to the running reference) of the tile whose scores the next step consumes, and
  // whether any row's maximum moved; both computed one step ahead, under the P.V MFMAs
  float tmax_row = 0.f;
  bool moved = false;

  // Q~ fragments of the other operand set, one 16-byte piece at a time (a handful of switches per wave: no need for all
  // eight loads in flight, and the registers they would take are the tile step's).  The 8-bit quantiser of load_q does
  // not apply: a launch with its own 4-bit operands gets both sets quantised by the caller (q_quant == 0, checked on the host).
  auto reload_q = [&](const void* qbase) __attribute__((always_inline)) {
    // (the lane index is laundered so that the row addresses are formed here, at one of a wave's two or three switches,
    // and not hoisted out of the tile loop into registers that loop has no room for)
    int ln = lane;
    asm volatile("; operand set switch" : "+v"(ln));
    const uint16_t* qp = (const uint16_t*)qbase + (int64_t)b * a.q_sb + (int64_t)head * a.q_sh;
    const int row = max(min(row_w0 + (ln & 31), a.Nq - 1), 0);
    const uint16_t* rp = qp + (int64_t)row * a.q_sn + 8 * (ln >> 5);
#pragma unroll
    for (int kk = 0; kk < 8; ++kk) {
      const uint4 raw = *(const uint4*)(rp + 16 * kk);
      qf[kk] = make_uint4(scale_pair<BF16>(raw.x, a.sm), scale_pair<BF16>(raw.y, a.sm), scale_pair<BF16>(raw.z, a.sm), scale_pair<BF16>(raw.w, a.sm));
    }
  };
  // kDefer, rare: the scores of tile j (step t) once more, from the key rows in memory instead of the LDS ring -- the same
  // MFMAs in the same order, so the same bits.  One fragment at a time: this path may not raise the kernel's register count.
  auto redo_tile = [&](int j, bool use4, bool masked, f32x16_t (&S)[2]) __attribute__((always_inline)) {
    const char* kb = (const char*)a.k + (use4 ? (int64_t)((const char*)a.k4 - (const char*)a.k) : (int64_t)0) + k_head_off * 2;
    int ln = lane;
    asm volatile("; tile from memory" : "+v"(ln));
    // (with separate 4-bit operands the fragments in qf may already belong to the next step's operand set)
    bool other_q = false;
    if constexpr (WAVES < 8 || DUAL) {
      other_q = distinct4 && use4 != q_is4;
      if (other_q) reload_q(use4 ? a.q4 : a.q);
    }
#pragma unroll
    for (int bn = 0; bn < 2; ++bn) {
      const int n = min(j * kBN + 32 * bn + (ln & 31), a.Nk - 1);
      const char* rp = kb + ((int64_t)n * a.k_sn + 8 * (ln >> 5)) * 2;
#pragma unroll
      for (int kk = 0; kk < 8; ++kk) {
        const uint4 ka = *(const uint4*)(rp + 32 * kk);
        asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
        S[bn] = mfma_qk32<BF16>(ka, qf[kk], kk == 0 ? Cinit : S[bn]);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
    if constexpr (WAVES < 8 || DUAL) {
      if (other_q) reload_q(q_is4 ? a.q4 : a.q);
    }
    if (masked) {
      const int rel = pos0 + (ln & 31) - j * kBN - 4 * (ln >> 5);
#pragma unroll
      for (int bn = 0; bn < 2; ++bn)
#pragma unroll
        for (int i = 0; i < 16; ++i)
          if (32 * bn + 8 * (i >> 2) + (i & 3) > rel) S[bn][i] = -INFINITY;
    }
    mfma_settle(S[0], S[1]);
  };
  // kDefer: the P.V product of the pending tile on its own, for a wave that does not visit the step after it (or has
  // reached the end): V^T fragments from the tile's ring buffer, four MFMAs, and the words back to zero.
  auto flush_pv = [&](auto rg) __attribute__((always_inline)) {   // rg: ring position of the pending tile's step
    constexpr int R = decltype(rg)::value;
    // one fragment pair at a time: this path may not raise the kernel's register count
    static_for<0, 4>([&](auto I) {
      constexpr int bd = decltype(I)::value;
      u32x4_t vlo = lds_read128<R * kVTileBytes + bd * 2048>(v8lo_base), vhi = lds_read128<R * kVTileBytes + bd * 2048>(v8hi_base);
      lds_wait<0>(vlo, vhi);
      const i32x8_t av = {(int)vlo[0], (int)vlo[1], (int)vlo[2], (int)vlo[3], (int)vhi[0], (int)vhi[1], (int)vhi[2], (int)vhi[3]};
      const i32x8_t pb = {P8w[0], P8w[1], P8w[2], P8w[3], P8w[4], P8w[5], P8w[6], P8w[7]};
      O[bd] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(av, pb, O[bd], 0, 0, 0, 0x7f7f7f7f, 0, e_pend);
      __builtin_amdgcn_sched_barrier(0);
    });
#pragma unroll
    for (int r = 0; r < 8; ++r) P8w[r] = 0;
    pend_t = -1;
  };

  // softmax update + P.V for the tile whose scores are in S.  Once the running maximum of this tile is settled,
  // the Q.K^T MFMAs of the following tile (K in knext, result in Snext) are issued in the same straight-line
  // block as the exponentials, conversions and P.V MFMAs, so that the matrix pipe and the vector ALU of this
  // wave work side by side.
  auto softmax_pv = [&](auto rg, int j, int it, bool use4, const char* vbuf, bool masked, f32x16_t (&S)[2], const char* knext, f32x16_t (&Snext)[2]) {
    constexpr int R = decltype(rg)::value;   // it & 3, known at compile time
    // MODE 4: the first K fragments of the next tile are requested before anything else, so that their LDS
    // latency passes under the row-maximum bookkeeping
    const uint32_t klane = smem_addr + (((it + 1) & 3) * kKTileBytes) + kx0;
    u32x4_t kf[16];
    // K fragments are requested this many MFMA slots ahead (even, 2..8); the fp16 P.V modes have fewer registers to spare
    constexpr int kDepth = kPV8 ? 4 : 2;
    auto kread = [&](auto I) {
      constexpr int i = decltype(I)::value;
      if constexpr (kStaticRing) kf[i] = lds_read128<((R + 1) & 3) * kKTileBytes + (i & 1) * 32 * kKStride>(kxr[i >> 1]);
      else kf[i] = lds_read128<(i & 1) * 32 * kKStride>(klane ^ ((i >> 1) << 5));
    };
    if constexpr (!kPlain) static_for<0, kDepth>(kread);
    if (masked) {  // causal mask inside the query block's own tiles (attn_triton.py:69-71)
      // One tile in thousands takes this branch.  The laundered copy of g keeps the branch a branch and stops
      // the compiler from hoisting 32 per-lane column constants out of the loop into precious registers.
      int gm = g;
      asm volatile("; causal mask" : "+v"(gm));
      const int rel = pos0 + c32 - j * kBN - 4 * gm;   // key index (within the tile, minus 4g) of the diagonal
#pragma unroll
      for (int bn = 0; bn < 2; ++bn)
#pragma unroll
        for (int i = 0; i < 16; ++i)
          if (32 * bn + 8 * (i >> 2) + (i & 3) > rel) S[bn][i] = -INFINITY;
    }
    // row maximum of S - m_run + kC; the row's other 32 keys live in lane^32
    float tmax;
    bool slow;
    if constexpr (kDefer) {
      // only a wave's first tile looks at its scores before exponentiating them: it sets the reference
      slow = first;
      tmax = 0.f;
      if (__builtin_expect(first, 0)) {
        mfma_settle(S[0], S[1]);
        tmax = xor32_max(lane_max(S));
      }
    } else if constexpr (!kPlain) {
      if (masked) {
        tmax_row = xor32_max(lane_max(S));
        moved = __any(tmax_row > kMove);
      }
      tmax = tmax_row;   // came out of the previous step's P.V phase
      slow = first || moved;
    } else {
      tmax = max3(S[0][0], S[1][0], S[0][1]);
#pragma unroll
      for (int i = 1; i < 15; ++i) tmax = max3(tmax, S[1][i], S[0][i + 1]);
      tmax = max3(tmax, S[1][15], S[1][15]);
      tmax = xor32_max(tmax);
      slow = first || __any(tmax > kMove);
    }
    if (slow) {
      // some row's maximum moved by d (on the first tile: from the arbitrary reference 0 to the row maximum):
      // shift the scores, rescale the accumulators, re-centre the accumulator initialiser
      asm volatile("; new row maximum" ::: "memory");
      const float d = first ? (tmax - kC) : ((tmax > kMove) ? tmax - kC : 0.f);
      const float alpha = first ? 0.f : __builtin_amdgcn_exp2f(-d);
      m_run += d;
      l_run *= alpha;
#pragma unroll
      for (int bn = 0; bn < 2; ++bn)
#pragma unroll
        for (int i = 0; i < 16; ++i) S[bn][i] -= d;
#pragma unroll
      for (int bd = 0; bd < 4; ++bd) O[bd] *= alpha;
      const float c = kC - m_run;
#pragma unroll
      for (int i = 0; i < 16; ++i) Cinit[i] = c;
      first = false;
    }
    if constexpr (kDefer) {
      __builtin_amdgcn_s_setprio(0);
      // Hand-scheduled tile step.  16 slots of {Q.K^T MFMA of the next tile, one LDS prefetch, two exponentials of the
      // current tile and their addition to the row sum}; the row sum's exchange with the lane that holds the row's other
      // 32 keys and the block exponent; then 4 slots of {fp8 P.V MFMA of the PENDING tile (the one visited before this
      // one; its V^T tile is in ring buffer R - 1), two LDS prefetches, four packs of the current tile to e4m3}.
      // LDS requests, in order: K fragments 0 .. 15 (kDepth ahead of their MFMA), then V^T fragments 0 .. 7 (lo and hi
      // half of the rows of P.V slot r / 2): four in the last four Q.K^T slots, which request no K fragment any more, two
      // more behind each of the first two P.V MFMAs -- two slots ahead of their use.
      static_assert(kDepth == 4, "the wait counts below are those of K fragments requested four slots ahead");
      constexpr int kVoff = ((R + 3) & 3) * kVTileBytes;
      u32x4_t vlo[4], vhi[4];
      auto vread = [&](auto RR) __attribute__((always_inline)) {
        constexpr int rr = decltype(RR)::value;
        if constexpr (rr & 1) vhi[rr >> 1] = lds_read128<kVoff + (rr >> 1) * 2048>(v8hi_base);
        else vlo[rr >> 1] = lds_read128<kVoff + (rr >> 1) * 2048>(v8lo_base);
      };
      float ps[2] = {0.f, 0.f};
      static_for<0, 16>([&](auto I) {
        constexpr int i = decltype(I)::value;
        constexpr int bn = i & 1, kk = i >> 1;
        lds_wait<3>(kf[i]);     // behind it: K fragments i + 1 .. i + 3, or in the last slots V^T fragments in their place
        __builtin_amdgcn_sched_barrier(0);
        constexpr int sb = i >> 3, e = 2 * (i & 7);
        const float p0 = __builtin_amdgcn_exp2f(S[sb][e]), p1 = __builtin_amdgcn_exp2f(S[sb][e + 1]);
        S[sb][e] = p0;
        S[sb][e + 1] = p1;
        ps[i & 1] += p0;
        ps[i & 1] += p1;
        __builtin_amdgcn_sched_barrier(0);
        const uint4 ka = make_uint4(kf[i][0], kf[i][1], kf[i][2], kf[i][3]);
        if constexpr (kk == 0) Snext[bn] = mfma_qk32<BF16>(ka, qf[0], Cinit);
        else Snext[bn] = mfma_qk32<BF16>(ka, qf[kk], Snext[bn]);
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (i + kDepth < 16) kread(std::integral_constant<int, i + kDepth>{});
        else vread(std::integral_constant<int, i + kDepth - 16>{});
        __builtin_amdgcn_sched_barrier(0);
      });
      // The row's sum of the tile, rs = 448 sum 2^(s - reference).  Block scale 2^-k with rs 2^-k in [128, 256): every
      // scaled probability is below 256 (e4m3 reaches 448), the row's largest one at least 2.  The E8M0 exponent of 2^k is
      // eb = frexp exponent + 119, kept in [67, 245]: the pack divides by 2^(eb - 127), the MFMA multiplies by it.
      // (only rs_lane and eb stay live through the P.V slots: the rare paths below form the row sum again)
      // (this chain of dependent instructions sits behind the first P.V MFMA, not in front of it)
      float rs_lane = ps[0] + ps[1];
      int eb = 127;
      float pack_scale = 1.f;
      typedef __attribute__((ext_vector_type(2))) short i16x2_t;
      int P8n[8];
      auto pack_words = [&](auto BD, float sc) __attribute__((always_inline)) {   // words 2 bd, 2 bd + 1: S[bd >> 1][8 (bd & 1) .. + 7]
        constexpr int bd = decltype(BD)::value;
        constexpr int sb = bd >> 1, o = 8 * (bd & 1);
        // (each pack writes one half of the word and keeps the other: the halves start out as whatever the register held)
        int u0, u1;
        asm volatile("" : "=v"(u0), "=v"(u1));
        i16x2_t w0 = __builtin_bit_cast(i16x2_t, u0), w1 = __builtin_bit_cast(i16x2_t, u1);
        w0 = __builtin_amdgcn_cvt_scalef32_pk_fp8_f32(w0, S[sb][o], S[sb][o + 1], sc, false);
        w0 = __builtin_amdgcn_cvt_scalef32_pk_fp8_f32(w0, S[sb][o + 2], S[sb][o + 3], sc, true);
        w1 = __builtin_amdgcn_cvt_scalef32_pk_fp8_f32(w1, S[sb][o + 4], S[sb][o + 5], sc, false);
        w1 = __builtin_amdgcn_cvt_scalef32_pk_fp8_f32(w1, S[sb][o + 6], S[sb][o + 7], sc, true);
        P8n[2 * bd] = __builtin_bit_cast(int, w0);
        P8n[2 * bd + 1] = __builtin_bit_cast(int, w1);
      };
      static_for<0, 4>([&](auto I) {
        constexpr int bd = decltype(I)::value;
        lds_wait<(bd < 3) ? 2 : 0>(vlo[bd], vhi[bd]);   // the next pair is behind it, except for the last
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (bd > 0) {
          pack_words(std::integral_constant<int, bd - 1>{}, pack_scale);
          __builtin_amdgcn_sched_barrier(0);
        }
        const i32x8_t av = {(int)vlo[bd][0], (int)vlo[bd][1], (int)vlo[bd][2], (int)vlo[bd][3],
                            (int)vhi[bd][0], (int)vhi[bd][1], (int)vhi[bd][2], (int)vhi[bd][3]};
        const i32x8_t pb = {P8w[0], P8w[1], P8w[2], P8w[3], P8w[4], P8w[5], P8w[6], P8w[7]};
        O[bd] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(av, pb, O[bd], 0, 0, 0, 0x7f7f7f7f, 0, e_pend);
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (bd < 2) {
          vread(std::integral_constant<int, 2 * bd + 4>{});
          vread(std::integral_constant<int, 2 * bd + 5>{});
        }
        if constexpr (bd == 0) {
          const float rs_row = xor32_sum(rs_lane);
          eb = min(max(__builtin_amdgcn_frexp_expf(rs_row) + 119, 67), 245);
          moved = __any(!(rs_row <= kSumLimit));
          pack_scale = __int_as_float(eb << 23);
        }
        if constexpr (bd == 3) pack_words(I, pack_scale);
        __builtin_amdgcn_sched_barrier(0);
      });
#pragma unroll
      for (int r = 0; r < 8; ++r) P8w[r] = P8n[r];
      __builtin_amdgcn_s_setprio(3);
      if (__builtin_expect(moved, 0)) {   // one tile in thousands
        asm volatile("; reference moves" ::: "memory");
        float rs_row = xor32_sum(rs_lane);
        int fe = __builtin_amdgcn_frexp_expf(rs_row);
        if (__builtin_expect(__any(!(rs_row < kRedoLimit)), 0)) {
          // A row's sum overflowed: its probabilities are lost.  The tile's scores are formed again from the key rows in
          // memory (the K tile may have left the ring), such a row takes the tile's maximum as its new reference, and the
          // tile is exponentiated, summed and packed once more for all rows (rows that were fine get the bits they had).
          const bool redo = !(rs_row < kRedoLimit);
          redo_tile(j, use4, masked, S);
          const float tm = xor32_max(lane_max(S));
          const float d = redo ? tm - kC : 0.f;
          const float alpha = __builtin_amdgcn_exp2f(-d);
          m_run += d;
          l_run *= alpha;
#pragma unroll
          for (int bd = 0; bd < 4; ++bd) O[bd] *= alpha;
          float q0 = 0.f, q1 = 0.f;
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            S[0][i] = __builtin_amdgcn_exp2f(S[0][i] - d);
            S[1][i] = __builtin_amdgcn_exp2f(S[1][i] - d);
          }
          // the additions in the order of the slots above: slot i takes S[i >> 3][2 (i & 7)] and its neighbour
#pragma unroll
          for (int i = 0; i < 16; i += 2) {
            q0 += S[i >> 3][2 * (i & 7)];
            q0 += S[i >> 3][2 * (i & 7) + 1];
            q1 += S[(i + 1) >> 3][2 * ((i + 1) & 7)];
            q1 += S[(i + 1) >> 3][2 * ((i + 1) & 7) + 1];
          }
          rs_lane = q0 + q1;
          rs_row = xor32_sum(rs_lane);
          fe = __builtin_amdgcn_frexp_expf(rs_row);
          eb = min(max(fe + 119, 67), 245);
          const float sc = __int_as_float(eb << 23);
          static_for<0, 4>([&](auto I) { pack_words(I, sc); });
#pragma unroll
          for (int r = 0; r < 8; ++r) P8w[r] = P8n[r];
#pragma unroll
          for (int i = 0; i < 16; ++i) {
            Snext[0][i] -= d;
            Snext[1][i] -= d;
          }
        }
        // rows whose sum passed the limit: the reference goes up by n binades, rs 2^-n in [256, 512)
        const int n = (rs_row > kSumLimit) ? fe - 9 : 0;
        const float down = __int_as_float((127 - n) << 23);
        const float nf = (float)n;
        m_run += nf;
        l_run *= down;
        rs_lane *= down;
#pragma unroll
        for (int bd = 0; bd < 4; ++bd) O[bd] *= down;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
          Snext[0][i] -= nf;
          Snext[1][i] -= nf;
        }
        eb = max(eb - n, 1);
        const float c = kC - m_run;
#pragma unroll
        for (int i = 0; i < 16; ++i) Cinit[i] = c;
      }
      l_run += rs_lane;
      e_pend = eb;
      pend_t = it;
      return;
    }
    if constexpr (kPV8) {   // MODE 4 (MODE 5 has returned above)
      __builtin_amdgcn_s_setprio(0);
      // Hand-scheduled tile step.  16 slots of {Q.K^T MFMA of the next tile, one LDS prefetch, two exponentials
      // and one e4m3 pack of the current tile}, then 4 slots of {fp8 P.V MFMA, two LDS prefetches, 8 additions of
      // the row sum}.  K fragments are read 4 slots ahead of the MFMA that consumes them.
      // P^T is the e4m3 B operand of one K=64 MFMA per 32 output channels: byte 16 bn + i of this lane's
      // 32 bytes is the probability in S[bn][i]; the V^T tiles were permuted to the same key order.
      constexpr int kVoff = kStaticRing ? R * kVTileBytes : 0;
      const uint32_t vlo_addr = kStaticRing ? v8lo_base : v8lo_base + (it & 3) * kVTileBytes;
      const uint32_t vhi_addr = kStaticRing ? v8hi_base : v8hi_base + (it & 3) * kVTileBytes;
      u32x4_t vlo[4], vhi[4];
      // Order inside a slot: the wait for the K fragment, the two exponentials and the pack, then the MFMA, then the
      // next LDS request (vector work in front of the MFMA measured 1 % faster than behind it).  An MFMA placed directly
      // behind an inline-asm statement (the wait or the request) would get a hazard s_nop from the compiler, 20 per tile.
      static_for<0, 16>([&](auto I) {
        constexpr int i = decltype(I)::value;
        constexpr int bn = i & 1, kk = i >> 1;
        lds_wait<kDepth - 1>(kf[i]);
        __builtin_amdgcn_sched_barrier(0);
        constexpr int sb = i >> 3, e = 2 * (i & 7), r = 4 * sb + ((i & 7) >> 1);
        const float p0 = __builtin_amdgcn_exp2f(S[sb][e]), p1 = __builtin_amdgcn_exp2f(S[sb][e + 1]);
        S[sb][e] = p0;
        S[sb][e + 1] = p1;
        P8[r] = __builtin_amdgcn_cvt_pk_fp8_f32(p0, p1, P8[r], (i & 1) != 0);
        __builtin_amdgcn_sched_barrier(0);
        const uint4 ka = make_uint4(kf[i][0], kf[i][1], kf[i][2], kf[i][3]);
        if constexpr (kk == 0) Snext[bn] = mfma_qk32<BF16>(ka, qf[0], Cinit);
        else Snext[bn] = mfma_qk32<BF16>(ka, qf[kk], Snext[bn]);
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (i + kDepth < 16) {
          kread(std::integral_constant<int, i + kDepth>{});
        } else {  // the K fragments are all requested: start on the V^T fragments, in the order the P.V slots use them
          constexpr int rr = i + kDepth - 16;
          if constexpr (rr & 1) vhi[rr >> 1] = lds_read128<kVoff + (rr >> 1) * 2048>(vhi_addr);
          else vlo[rr >> 1] = lds_read128<kVoff + (rr >> 1) * 2048>(vlo_addr);
        }
        __builtin_amdgcn_sched_barrier(0);
      });
      // P.V slots: the vector ALU is nearly idle under the four K=64 MFMAs, so the row sum of this tile and the
      // lane maximum of the next tile's scores are computed here (additions before the MFMA, max3 behind it)
      float ps[2] = {0.f, 0.f}, cm[4];
      static_for<0, 4>([&](auto I) {
        constexpr int bd = decltype(I)::value;
        // requests issued so far: kDepth in the Q.K slots, two more per earlier P.V slot
        constexpr int issued = (kDepth + 2 * bd < 8) ? kDepth + 2 * bd : 8;
        lds_wait<issued - 2 * bd - 2>(vlo[bd], vhi[bd]);
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
          ps[0] += S[bd >> 1][8 * (bd & 1) + e];
          ps[1] += S[bd >> 1][8 * (bd & 1) + 4 + e];
        }
        __builtin_amdgcn_sched_barrier(0);
        const i32x8_t av = {(int)vlo[bd][0], (int)vlo[bd][1], (int)vlo[bd][2], (int)vlo[bd][3],
                            (int)vhi[bd][0], (int)vhi[bd][1], (int)vhi[bd][2], (int)vhi[bd][3]};
        O[bd] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(av, P8, O[bd], 0, 0, 0, 0x7f7f7f7f, 0, 0x7f7f7f7f);
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (issued < 8) {
          vlo[issued / 2] = lds_read128<kVoff + (issued / 2) * 2048>(vlo_addr);
          vhi[issued / 2] = lds_read128<kVoff + (issued / 2) * 2048>(vhi_addr);
        }
        if constexpr (bd < 3) {
          // a quarter of the next tile's scores: Snext[bd >> 1][8 (bd & 1) .. +7]; both halves are complete by now.
          // The fourth quarter is spread over the first three slots, so that only the final reduction is left
          // behind the last MFMA.
          const f32x16_t& sn = Snext[bd >> 1];
          constexpr int o = 8 * (bd & 1);
          cm[bd] = max3_of8(sn[o], sn[o + 1], sn[o + 2], sn[o + 3], sn[o + 4], sn[o + 5], sn[o + 6], sn[o + 7]);
          const f32x16_t& s3 = Snext[1];
          if constexpr (bd == 0) cm[3] = max3(s3[8], s3[9], s3[10]);
          if constexpr (bd == 1) cm[3] = max3(cm[3], s3[11], s3[12]);
          if constexpr (bd == 2) cm[3] = max3_of4(cm[3], s3[13], s3[14], s3[15]);
        }
        __builtin_amdgcn_sched_barrier(0);
      });
      // (placing this reduction in the third slot as well, ahead of the last MFMA, measured 0.8 % slower)
      tmax_row = xor32_max(max3_of4(cm[0], cm[1], cm[2], cm[3]));
      l_run += ps[0] + ps[1];
      moved = __any(tmax_row > kMove);
      __builtin_amdgcn_s_setprio(3);
      return;
    }
    if constexpr (MODE == 0 || MODE == 1 || MODE == 3) {
      // Hand-scheduled tile step, fp16 P.V: 16 slots of {Q.K^T MFMA of the next tile, one LDS prefetch, two
      // exponentials, and every other slot the conversion of four finished probabilities}, then 16 slots of
      // {P.V MFMA, one LDS prefetch, two additions of the row sum, later two steps of the next tile's row maximum}.
      // P.V slot s multiplies V^T rows 32 (s & 3) .. +31 with the keys of group m = s >> 2 (8 keys per lane), whose
      // probabilities are the B operand words Pw[m][0..3].
      // Order inside a slot, held by scheduling barriers: the wait, the MFMA, the LDS request, then the vector work (1.2 %
      // faster than the order the compiler chose, and 3 % faster than the vector work in front of the MFMA -- the other
      // way round than in the fp8 steps, whose slots carry more vector work per MFMA).
      __builtin_amdgcn_s_setprio(0);
      const uint32_t vlane = smem_addr + 4 * kKTileBytes + (it & 3) * kVTileBytes + c32 * kVStride + ((g ^ vsw) << 4);
      u32x4_t vf[16];
      uint32_t Pw[4][4];
      auto vread = [&](auto I) {
        constexpr int sl = decltype(I)::value;
        if constexpr (kStaticRing) vf[sl] = lds_read128<R * kVTileBytes + (sl & 3) * 32 * kVStride>(vxr[sl >> 2]);
        else vf[sl] = lds_read128<(sl & 3) * 32 * kVStride>(vlane ^ ((sl >> 2) << 5));
      };
      auto pack_unit = [&](auto U) {   // probabilities 4u .. 4u+3 of the tile (in S order)
        constexpr int u = decltype(U)::value;
        const f32x16_t& sv = S[u >> 2];
        constexpr int o = 4 * (u & 3);
        quant_pack4<MODE>(sv[o], sv[o + 1], sv[o + 2], sv[o + 3], Pw[u >> 1][2 * (u & 1)], Pw[u >> 1][2 * (u & 1) + 1]);
      };
      static_for<0, 16>([&](auto I) {
        constexpr int i = decltype(I)::value;
        constexpr int bn = i & 1, kk = i >> 1;
        lds_wait<kDepth - 1>(kf[i]);
        __builtin_amdgcn_sched_barrier(0);
        const uint4 ka = make_uint4(kf[i][0], kf[i][1], kf[i][2], kf[i][3]);
        if constexpr (kk == 0) Snext[bn] = mfma_qk32<BF16>(ka, qf[0], Cinit);
        else Snext[bn] = mfma_qk32<BF16>(ka, qf[kk], Snext[bn]);
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (i + kDepth < 16) kread(std::integral_constant<int, i + kDepth>{});
        else vread(std::integral_constant<int, i + kDepth - 16>{});
        __builtin_amdgcn_sched_barrier(0);
        constexpr int sb = i >> 3, e = 2 * (i & 7);
        S[sb][e] = __builtin_amdgcn_exp2f(S[sb][e]);
        S[sb][e + 1] = __builtin_amdgcn_exp2f(S[sb][e + 1]);
        if constexpr (i >= 2 && (i & 1) == 0) pack_unit(std::integral_constant<int, (i - 2) / 2>{});
        __builtin_amdgcn_sched_barrier(0);
      });
      float ps[2] = {0.f, 0.f}, cm[4], tm = 0.f;
      auto max_pair = [&](auto K) {   // two links of the lane maximum over the next tile's scores (9 pairs), one asm each
        constexpr int k = decltype(K)::value;
        if constexpr (k < 8) {
          constexpr int h = k >> 1, o = 8 * (h & 1);
          const f32x16_t& sn = Snext[h >> 1];
          if constexpr ((k & 1) == 0) cm[h] = max3_of5(sn[o], sn[o + 1], sn[o + 2], sn[o + 3], sn[o + 4]);
          else cm[h] = max3_of4(cm[h], sn[o + 5], sn[o + 6], sn[o + 7]);
        } else {
          tm = max3_of4(cm[0], cm[1], cm[2], cm[3]);
        }
      };
      static_for<0, 16>([&](auto I) {
        constexpr int sl = decltype(I)::value;
        constexpr int m = sl >> 2, bd = sl & 3;
        constexpr int issued = (kDepth + sl < 16) ? kDepth + sl : 16;   // V^T requests issued before this slot
        lds_wait<issued - sl - 1>(vf[sl]);
        __builtin_amdgcn_sched_barrier(0);
        const uint4 av = make_uint4(vf[sl][0], vf[sl][1], vf[sl][2], vf[sl][3]);
        O[bd] = mfma_pv32(av, make_uint4(Pw[m][0], Pw[m][1], Pw[m][2], Pw[m][3]), O[bd]);
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (issued < 16) vread(std::integral_constant<int, issued>{});
        __builtin_amdgcn_sched_barrier(0);
        if constexpr (sl == 0) pack_unit(std::integral_constant<int, 7>{});
        ps[0] += S[sl >> 3][2 * (sl & 7)];
        ps[1] += S[sl >> 3][2 * (sl & 7) + 1];
        if constexpr (sl >= 7) max_pair(std::integral_constant<int, sl - 7>{});
        __builtin_amdgcn_sched_barrier(0);
      });
      tmax_row = xor32_max(tm);
      moved = __any(tmax_row > kMove);
      l_run += ps[0] + ps[1];
      __builtin_amdgcn_s_setprio(3);
      return;
    }
    qk_tile(knext, Snext);   // scores of the next tile, relative to the maximum just settled
    float psum = 0.f;
#pragma unroll
    for (int bn = 0; bn < 2; ++bn)
#pragma unroll
      for (int i = 0; i < 16; ++i) {
        const float p = __builtin_amdgcn_exp2f(S[bn][i]);
        S[bn][i] = p;
        psum += p;
      }
    l_run += psum;

    float sc = 448.f, inv = 1.0f / 448.0f;
    if constexpr (MODE == 2) {  // block absmax over the 64-row group: this wave and its neighbour (wave ^ 1)
      float amax = fmaxf(S[0][0], S[1][0]);
#pragma unroll
      for (int i = 1; i < 16; ++i) amax = fmaxf(amax, fmaxf(S[0][i], S[1][i]));
      if (row_w0 + c32 >= a.Nq) amax = 0.f;   // rows past the end are clamped copies, not part of the block
#pragma unroll
      for (int sh = 1; sh < 32; sh <<= 1) amax = wave_xor_max(amax, sh);
      amax = xor32_max(amax);
      if (lane == 0) s_amax[it & 1][wave] = amax;
      __syncthreads();  // see the matching barrier for waves that skip this tile
      if constexpr (WAVES > 1) amax = fmaxf(amax, s_amax[it & 1][wave ^ 1]);
      sc = 448.f / amax;   // amax > 0: every visited tile has an unmasked key in every row
      inv = amax / 448.f;
    }
    uint4 P[2][2];  // [bn][t]
#pragma unroll
    for (int bn = 0; bn < 2; ++bn)
#pragma unroll
      for (int t = 0; t < 2; ++t) P[bn][t] = quant_pack8<(kPV8 ? 3 : (kQK8 ? 0 : MODE))>(S[bn], t, sc, inv);
    // O^T[d, row] += V^T[d, key] . P^T[key, row]
#pragma unroll
    for (int bd = 0; bd < 4; ++bd)
#pragma unroll
      for (int bn = 0; bn < 2; ++bn)
#pragma unroll
        for (int t = 0; t < 2; ++t) {
          const uint4 av = *(const uint4*)(vbuf + (32 * bd + c32) * kVStride + (((4 * bn + 2 * t + g) ^ vsw) << 4));
          O[bd] = mfma_pv32(av, P[bn][t], O[bd]);
        }
  };

  // ---- main loop, software pipelined inside each wave: in step `it` the wave issues the Q.K^T MFMAs of tile
  // t[it+1] and, while the matrix pipe works on them, runs the softmax of tile t[it] on the vector ALU, then the
  // P.V MFMAs of tile t[it].  K and V^T live in rings of 4 LDS buffers and the workgroup synchronises once per
  // TWO tiles: at the start of a pair (it even) every wave starts the copies of K(t[it+3]), K(t[it+4]),
  // V^T(t[it+2]), V^T(t[it+3]) into the buffers the previous pair finished with, and between the barriers the
  // waves drift apart by up to a tile, which lets one wave's matrix phase overlap another's vector phase.
  // The schedule is addressed by a flat step index t = 0 .. nTot-1: the sink tiles [0, nA) first, then the tiles
  // [segB_lo, segB_hi).  The ring buffer of step t is t & 3.
  // DUAL: the 4-bit copies of tiles [c_lo, c_lo + n_dup) sit at steps [d1 - n_dup, d1), where those tiles would sit
  // anyway; the tiles themselves and everything behind them move up by n_dup steps.  The steps whose K tile comes from
  // the 4-bit key then form one interval [u4_lo, u4_hi): block A's 4-bit range and, right behind it, the copies.
  const int nA = segA_hi, shiftB = segB_lo - segA_hi;
  const int d1 = (DUAL && n_dup > 0) ? c_lo - shiftB + n_dup : (1 << 30);
  const int nTot = max(nA + segB_hi - segB_lo, 0) + n_dup;
  auto tile_of = [&](int t) {
    if (t < nA) return t;
    if constexpr (DUAL) return t + shiftB - (t >= d1 ? n_dup : 0);
    return t + shiftB;
  };
  const int u4_lo = t4_lo - shiftB, u4_hi = t4_hi - shiftB + n_dup;
  // (a wave only ever visits steps whose operand set is the one it wants, so this also tells it which Q~ set a step takes)
  auto step_uses4 = [&](int t) { return distinct4 && t >= u4_lo && t < u4_hi; };
  // steps whose K tile is complete (only the very last tile of the sequence can be partial)
  const int nFull = (nTot > 0 && (tile_of(nTot - 1) + 1) * kBN > a.Nk) ? nTot - 1 : nTot;
  // this wave's tiles in step space: [0, fa) (sink) and [fb, fe] (window up to its diagonal tile); from step fm
  // on the causal mask applies.  A wave without rows visits nothing.
  // DUAL: for block A's waves every tile from c_lo on is its moved-up original, and they skip the copies; for block B's
  // waves the tiles below c_lo + n_dup are the copies, and they skip the originals.
  const int thr = wave < 4 ? c_lo : c_lo + n_dup;
  auto step_of = [&](int j) { return j - shiftB + ((DUAL && j >= thr) ? n_dup : 0); };   // a tile of segment B
  const int fa = wave_active ? wr.sink_hi : 0;
  const int fb = wave_active ? step_of(wr.win_lo) : (1 << 30);
  const int fe = step_of(wr.diag_hi), fm = step_of(wr.diag_lo);
  const int sk_lo = (DUAL && n_dup > 0) ? (wave < 4 ? d1 - n_dup : d1) : 0;
  auto visits_step = [&](int t) {
    const bool in = t < fa || (t >= fb && t <= fe);
    if constexpr (DUAL) return in && (unsigned)(t - sk_lo) >= (unsigned)n_dup;
    return in;
  };

  // kDefer: a tile's V^T is needed one step after its K (the P.V product runs a visited step late), so its copy starts
  // a step later as well and the buffer is refilled a step later: V^T(t) is read in step t + 1, or in a flush before the
  // workgroup has left step t + 1
  if (0 < nTot) {
    stage_k(tile_of(0), 0, step_uses4(0));
    stage_v(tile_of(0), 0);
  }
  if (1 < nTot) {
    stage_k(tile_of(1), 1, step_uses4(1));
    if constexpr (!kDefer) stage_v(tile_of(1), 1);
  }
  if (2 < nTot) stage_k(tile_of(2), 2, step_uses4(2));
  if constexpr (kDefer) {
    // ring buffer 3 is read by step 0's P.V MFMAs, which have zeros for probabilities: it must hold finite numbers
    for (int i = tid; i < kVTileBytes / 16; i += NT) *(uint4*)(vbase_lds + 3 * kVTileBytes + 16 * i) = make_uint4(0, 0, 0, 0);
  }
  // the wave's query rows, requested while the first tiles are on their way
  if constexpr (kQK8) {
    const uint16_t* qp = (const uint16_t*)a.q + (int64_t)b * a.q_sb + (int64_t)head * a.q_sh;
    const int row = max(min(row_w0 + c32, a.Nq - 1), 0);
    const uint16_t* rp = qp + (int64_t)row * a.q_sn + 16 * g;
    uint4 raw[4][2];
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      raw[kk][0] = *(const uint4*)(rp + 32 * kk);
      raw[kk][1] = *(const uint4*)(rp + 32 * kk + 8);
    }
    float amax = 0.f;
#pragma unroll
    for (int kk = 0; kk < 4; ++kk)
#pragma unroll
      for (int hf = 0; hf < 2; ++hf) {
        const uint32_t w[4] = {raw[kk][hf].x, raw[kk][hf].y, raw[kk][hf].z, raw[kk][hf].w};
#pragma unroll
        for (int j = 0; j < 4; ++j) amax = fmaxf(amax, fmaxf(fabsf(elem16<BF16>(w[j] & 0xffffu)), fabsf(elem16<BF16>(w[j] >> 16))));
      }
    amax = fmaxf(xor32_max(amax), 1e-5f);
    const Divisor scale = make_divisor(amax / 127.f);
    auto code = [&](float x) {   // clamp(round(x / scale), -128, 127), fake_quant.py:114-116
      const float t = divide(x, scale);
      return (uint32_t)((int)fminf(fmaxf(copysignf(floorf(fabsf(t) + 0.5f), t) + 0.0f, -128.f), 127.f) & 0xff);
    };
#pragma unroll
    for (int kk = 0; kk < 4; ++kk)
#pragma unroll
      for (int hf = 0; hf < 2; ++hf) {
        const uint32_t w[4] = {raw[kk][hf].x, raw[kk][hf].y, raw[kk][hf].z, raw[kk][hf].w};
#pragma unroll
        for (int j = 0; j < 2; ++j)   // four elements (two words) per code word
          qc[kk][2 * hf + j] = (int)(code(elem16<BF16>(w[2 * j] & 0xffffu)) | (code(elem16<BF16>(w[2 * j] >> 16)) << 8) |
                                     (code(elem16<BF16>(w[2 * j + 1] & 0xffffu)) << 16) | (code(elem16<BF16>(w[2 * j + 1] >> 16)) << 24));
      }
    q_scale = scale.d * a.sm;
  } else {
    load_q(a.q);
  }
  __builtin_amdgcn_s_waitcnt(0);
  __syncthreads();
  auto switch_q = [&](int t) __attribute__((always_inline)) {   // t: a step this wave visits
    if constexpr (WAVES < 8 || DUAL) {
      if (distinct4) {  // switch the Q~ operand set when entering/leaving the 4-bit window range
        const bool want4 = step_uses4(t);
        if (want4 != q_is4) {
          reload_q(want4 ? a.q4 : a.q);
          q_is4 = want4;
        }
      }
    }
  };
  f32x16_t Sa[2], Sb[2];
  bool vis_cur = nTot > 0 && visits_step(0);
  if (vis_cur) {
    switch_q(0);
    qk_tile(kbase_lds, Sa);
    if constexpr (!kPlain && !kDefer) {
      mfma_settle(Sa[0], Sa[1]);
      tmax_row = xor32_max(lane_max(Sa));
      moved = __any(tmax_row > kMove);
    }
  }
  __syncthreads();   // ring buffer 0 is about to be refilled: every wave has read K(step 0) out of it
  auto step = [&](auto rg, int t, f32x16_t (&Scur)[2], f32x16_t (&Snxt)[2]) {   // rg = t & 3
    if ((t & 1) == 0) {   // start of a pair: refill the four buffers the previous pair released
      if (t + 4 < nFull) {
        const int j2 = tile_of(t + 2), j3 = tile_of(t + 3), j4 = tile_of(t + 4);
        if constexpr (WAVES == 8 && !kQK8) {
          stage_k_full(j3, (t + 3) & 3, DUAL && step_uses4(t + 3));
          stage_k_full(j4, t & 3, DUAL && step_uses4(t + 4));
        } else {
          stage_k(j3, (t + 3) & 3, step_uses4(t + 3));
          stage_k(j4, t & 3, step_uses4(t + 4));
        }
        if constexpr (kDefer) {
          stage_v(tile_of(t + 1), (t + 1) & 3);
          stage_v(j2, (t + 2) & 3);
        } else {
          stage_v(j2, (t + 2) & 3);
          stage_v(j3, (t + 3) & 3);
        }
      } else {
        if (t + 3 < nTot) stage_k(tile_of(t + 3), (t + 3) & 3, step_uses4(t + 3));
        if (t + 4 < nTot) stage_k(tile_of(t + 4), t & 3, step_uses4(t + 4));
        if constexpr (kDefer) {
          if (t + 1 < nTot) stage_v(tile_of(t + 1), (t + 1) & 3);
          if (t + 2 < nTot) stage_v(tile_of(t + 2), (t + 2) & 3);
        } else {
          if (t + 2 < nTot) stage_v(tile_of(t + 2), (t + 2) & 3);
          if (t + 3 < nTot) stage_v(tile_of(t + 3), (t + 3) & 3);
        }
      }
    }
    const bool vis_nxt = visits_step(t + 1);
    const char* knext = kbase_lds + ((t + 1) & 3) * kKTileBytes;
    if constexpr (WAVES < 8 || DUAL) {
      if (vis_nxt) switch_q(t + 1);
    }
    if (vis_cur) {
      // Q.K^T of the next tile is computed even if this wave will not use it (the buffer then holds an older
      // tile or nothing meaningful; the result is dropped): the common path stays free of branches
      softmax_pv(rg, tile_of(t), t, step_uses4(t), vbase_lds + (t & 3) * kVTileBytes, t >= fm, Scur, knext, Snxt);
    } else {
      if (vis_nxt) {
        qk_tile(knext, Snxt);
        if constexpr (!kPlain && !kDefer) {
          mfma_settle(Snxt[0], Snxt[1]);
          tmax_row = xor32_max(lane_max(Snxt));
          moved = __any(tmax_row > kMove);
        }
      }
      if constexpr (MODE == 2) {
        if (lane == 0) s_amax[t & 1][wave] = 0.f;  // a wave that skips the tile contributes nothing to the block maximum
        __syncthreads();                            // every wave passes one such barrier per tile
      }
    }
    if (t & 1) {          // end of a pair
      __builtin_amdgcn_s_waitcnt(0);   // this wave's share of the tiles staged at the start of the pair has landed
      __syncthreads();
    }
    if constexpr (kDefer) {
      // the wave leaves its range: the last tile's P.V product now (its V^T tile has landed -- it was staged for the next
      // step -- and the buffer is not refilled before the end of that step)
      if (__builtin_expect(pend_t >= 0 && !vis_nxt, 0)) flush_pv(rg);
    }
    vis_cur = vis_nxt;
  };
  // both steps of a pair always run (the second one idles when the number of steps is odd), so that every wave
  // passes the same barriers
  for (int t = 0; t < nTot; t += 4) {   // unrolled over the four ring buffers (steps past the end idle)
    step(std::integral_constant<int, 0>{}, t, Sa, Sb);
    step(std::integral_constant<int, 1>{}, t + 1, Sb, Sa);
    step(std::integral_constant<int, 2>{}, t + 2, Sa, Sb);
    step(std::integral_constant<int, 3>{}, t + 3, Sb, Sa);
  }

  // ---- epilogue: out = acc / l (attn_triton.py:208-209), lse2 = log2(l) + m (:210-213)
  if (!wave_active) return;
  // (kDefer: nothing is pending here -- the step after a wave's last visited step is never visited, so that step flushed)
  const float l = xor32_sum(l_run);
  const int row = row_w0 + c32;
  if (row >= a.Nq) return;
  const int64_t obase = (int64_t)b * a.o_sb + (int64_t)head * a.o_sh + (int64_t)row * a.o_sn;
  const float inv_l = 1.0f / l;   // one division per row instead of 64 per lane: within 1 ulp of acc / l, before the rounding to the output type
#pragma unroll
  for (int bd = 0; bd < 4; ++bd)
#pragma unroll
    for (int i4 = 0; i4 < 4; ++i4) {
      const int d = 32 * bd + 8 * i4 + 4 * g;
      float v[4];
#pragma unroll
      for (int e = 0; e < 4; ++e) v[e] = O[bd][4 * i4 + e] * inv_l;
      if constexpr (kPV8) {  // undo the per-channel V scale
        const float4 isc = *(const float4*)(a.v_inv_scale + ((int64_t)b * a.Hkv + kvh) * kD + d);
        v[0] *= isc.x;
        v[1] *= isc.y;
        v[2] *= isc.z;
        v[3] *= isc.w;
      }
      if (a.out_dtype == 0) {
        uint2 w = make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
        *(uint2*)((uint16_t*)a.out + obase + d) = w;
      } else if (a.out_dtype == 1) {
        uint2 w = make_uint2(pack_f16(v[0], v[1]), pack_f16(v[2], v[3]));
        *(uint2*)((uint16_t*)a.out + obase + d) = w;
      } else {
        *(float4*)((float*)a.out + obase + d) = make_float4(v[0], v[1], v[2], v[3]);
      }
    }
  if (a.lse && g == 0) {
    const float lt = (MODE >= 3 && MODE <= 5) ? l * (1.0f / 448.0f) : l;
    a.lse[((int64_t)b * a.Hq + head) * a.Nq + row] = log2f(lt) + m_run;
  }
}

}  // namespace
}  // namespace sq

using namespace sq;

extern "C" size_t sq_prefill_workspace_bytes(int64_t batch, int64_t num_kv_heads, int64_t kv_len, int64_t head_dim) {
  (void)head_dim;
  if (batch <= 0 || num_kv_heads <= 0 || kv_len <= 0) return 0;
  const int64_t nT = (kv_len + kBN - 1) / kBN;
  return (size_t)(batch * num_kv_heads * nT) * (size_t)(kD * kBN) * sizeof(_Float16);
}

namespace {
int prefill_impl(const DLTensor* q, const DLTensor* k, const DLTensor* v, const DLTensor* q4, const DLTensor* k4, DLTensor* out,
                 DLTensor* lse, DLTensor* workspace, const sq_prefill_params* p, void* stream, const DLTensor* k_scale);
}

extern "C" int sq_prefill_fwd(const DLTensor* q, const DLTensor* k, const DLTensor* v, const DLTensor* q4,
                              const DLTensor* k4, DLTensor* out, DLTensor* lse, DLTensor* workspace,
                              const sq_prefill_params* p, void* stream) {
  return prefill_impl(q, k, v, q4, k4, out, lse, workspace, p, stream, nullptr);
}

extern "C" int sq_prefill_int8qk_fwd(const DLTensor* q, const DLTensor* k_codes, const DLTensor* k_scale, const DLTensor* v,
                                     DLTensor* out, DLTensor* lse, DLTensor* workspace, const sq_prefill_params* p, void* stream) {
  SQ_REQUIRE(k_scale, SQ_EINVAL, "sq_prefill_int8qk_fwd: k_scale is null");
  return prefill_impl(q, k_codes, v, nullptr, nullptr, out, lse, workspace, p, stream, k_scale);
}

namespace {
// k_scale != null: `k` holds int8 codes and the scores come from the int8 matrix instruction (sq_prefill_int8qk_fwd)
int prefill_impl(const DLTensor* q, const DLTensor* k, const DLTensor* v, const DLTensor* q4, const DLTensor* k4, DLTensor* out,
                 DLTensor* lse, DLTensor* workspace, const sq_prefill_params* p, void* stream, const DLTensor* k_scale) {
  SQ_REQUIRE(p, SQ_EINVAL, "sq_prefill_fwd: params is null");
  SQ_REQUIRE(q && k && v && out, SQ_EINVAL, "sq_prefill_fwd: q, k, v and out must be non-null");
  SQ_REQUIRE(p->layout == SQ_LAYOUT_HND || p->layout == SQ_LAYOUT_NHD, SQ_EINVAL, "tensor_layout %d not supported", p->layout);
  SQ_REQUIRE(p->p_quant >= SQ_P_NONE && p->p_quant <= SQ_P_E4M3_MX_FP8_PV, SQ_EINVAL, "sq_prefill_fwd: p_quant %d not supported", p->p_quant);
  SQ_REQUIRE((q4 == nullptr) == (k4 == nullptr), SQ_EINVAL, "sq_prefill_fwd: q4 and k4 must be given together");
  int rc;
  const int dev = q->device.device_id;
  if ((rc = check_tensor(q, "q", 4, dev)) || (rc = check_tensor(k, "k", 4, dev)) || (rc = check_tensor(v, "v", 4, dev)) ||
      (rc = check_tensor(out, "out", 4, dev)))
    return rc;
  if (q4 && ((rc = check_tensor(q4, "q4", 4, dev)) || (rc = check_tensor(k4, "k4", 4, dev)))) return rc;
  const DType dt = dtype_of(q);
  SQ_REQUIRE(dt == DType::BF16 || dt == DType::F16, SQ_EDTYPE, "sq_prefill_fwd: q must be bf16 or fp16");
  if (k_scale) {
    SQ_REQUIRE(k->dtype.code == kDLInt && k->dtype.bits == 8 && k->dtype.lanes == 1 && dtype_of(v) == dt, SQ_EDTYPE,
               "sq_prefill_int8qk_fwd: k_codes must be int8 and v of q's dtype");
    SQ_REQUIRE(p->p_quant == SQ_P_NONE && p->q_quant == 0, SQ_EINVAL,
               "sq_prefill_int8qk_fwd: p_quant and q_quant must be 0 (the query's codes are formed by the kernel, P stays fp16)");
  } else {
    SQ_REQUIRE(dtype_of(k) == dt && dtype_of(v) == dt, SQ_EDTYPE, "sq_prefill_fwd: q, k, v dtypes differ");
  }
  if (q4) SQ_REQUIRE(dtype_of(q4) == dt && dtype_of(k4) == dt, SQ_EDTYPE, "sq_prefill_fwd: q4/k4 dtype differs from q");
  const DType odt = dtype_of(out);
  SQ_REQUIRE(odt == DType::BF16 || odt == DType::F16 || odt == DType::F32, SQ_EDTYPE, "sq_prefill_fwd: out must be bf16, fp16 or fp32");
  const bool hnd = p->layout == SQ_LAYOUT_HND;
  const int hdim = hnd ? 1 : 2, ndim = hnd ? 2 : 1;
  const int64_t B = q->shape[0], Hq = q->shape[hdim], Nq = q->shape[ndim], D = q->shape[3];
  const int64_t Hkv = k->shape[hdim], Nk = k->shape[ndim];
  SQ_REQUIRE(D == kD, SQ_EINVAL, "Unsupported head_dim: %lld (the kernels take 128; pad smaller heads with zeros)", (long long)D);
  SQ_REQUIRE(B > 0 && Hq > 0 && Hkv > 0 && Nq > 0 && Nk > 0, SQ_ESHAPE, "sq_prefill_fwd: empty tensor");
  SQ_REQUIRE(Hq % Hkv == 0, SQ_ESHAPE, "sq_prefill_fwd: Hq=%lld not a multiple of Hkv=%lld", (long long)Hq, (long long)Hkv);
  SQ_REQUIRE(Hq <= kMaxHeads, SQ_EUNSUPPORTED, "sq_prefill_fwd: more than %d q heads", kMaxHeads);
  SQ_REQUIRE(k->shape[0] == B && k->shape[3] == D, SQ_ESHAPE, "sq_prefill_fwd: k shape mismatch");
  for (int i = 0; i < 4; ++i) {
    SQ_REQUIRE(v->shape[i] == k->shape[i], SQ_ESHAPE, "sq_prefill_fwd: v shape differs from k");
    SQ_REQUIRE(out->shape[i] == q->shape[i], SQ_ESHAPE, "sq_prefill_fwd: out shape differs from q");
    if (q4) {
      SQ_REQUIRE(q4->shape[i] == q->shape[i] && k4->shape[i] == k->shape[i], SQ_ESHAPE, "sq_prefill_fwd: q4/k4 shapes differ from q/k");
      SQ_REQUIRE(stride_of(q4, i) == stride_of(q, i) && stride_of(k4, i) == stride_of(k, i), SQ_ESHAPE,
                 "sq_prefill_fwd: q4/k4 strides differ from q/k");
    }
  }
  SQ_REQUIRE(p->q_offset >= 0 && p->q_offset % kBN == 0, SQ_EINVAL, "sq_prefill_fwd: q_offset must be a non-negative multiple of 64");
  SQ_REQUIRE(p->q_offset + Nq == Nk, SQ_ESHAPE,
             "qo_len and kv_len must be equal for causal attention (q_offset + qo_len = %lld, kv_len = %lld)",
             (long long)(p->q_offset + Nq), (long long)Nk);
  SQ_REQUIRE(Nk < (1ll << 31) - 65536, SQ_EUNSUPPORTED, "sq_prefill_fwd: more than 2^31 keys");
  // a 64-key tile is copied with one 64-bit tile base and 32-bit per-lane byte offsets: a tile must span less than 4 GiB
  SQ_REQUIRE(stride_of(k, ndim) > 0 && stride_of(k, ndim) < (1ll << 24) && stride_of(v, ndim) > 0 && stride_of(v, ndim) < (1ll << 31), SQ_EUNSUPPORTED,
             "sq_prefill_fwd: token stride of k must be below 2^24 elements (got %lld)", (long long)stride_of(k, ndim));
  const DLTensor* ts[5] = {q, k, v, out, nullptr};
  for (int t = 0; t < 4; ++t)
    for (int i = 0; i < 3; ++i)
      SQ_REQUIRE(stride_of(ts[t], i) % (t == 3 && odt == DType::F32 ? 4 : 8) == 0 || ts[t]->shape[i] == 1, SQ_ESHAPE,
                 "sq_prefill_fwd: strides must keep rows 16-byte aligned");
  if (lse) {
    SQ_REQUIRE(on_gpu(lse) && lse->device.device_id == dev, SQ_EDEVICE, "sq_prefill_fwd: lse not on the same device");
    SQ_REQUIRE(dtype_of(lse) == DType::F32 && numel_of(lse) == B * Hq * Nq && is_compact(lse), SQ_ESHAPE,
               "sq_prefill_fwd: lse must be a compact fp32 [B,Hq,Nq]");
  }
  int waves = 8;
  if (p->window_mode == SQ_WINDOW_SIZES) {
    SQ_REQUIRE(p->block_m == 64 || p->block_m == 128, SQ_EINVAL, "sq_prefill_fwd: block_m must be 64 or 128");
    SQ_REQUIRE(p->sink >= 0, SQ_EINVAL, "sink_size must be a non-negative integer, got %d", p->sink);
    SQ_REQUIRE(p->sink % kBN == 0, SQ_EUNSUPPORTED, "sq_prefill_fwd: sink_size %d is not a multiple of 64", p->sink);
    SQ_REQUIRE(p->w8 && p->w4 && p->num_heads_w == Hq, SQ_EINVAL, "sq_prefill_fwd: w8/w4 must hold one window per q head");
    SQ_REQUIRE(p->q_offset % p->block_m == 0, SQ_EINVAL, "sq_prefill_fwd: q_offset must be a multiple of block_m");
    for (int h = 0; h < Hq; ++h) {
      SQ_REQUIRE(p->w8[h] >= 0 && p->w4[h] >= 0, SQ_EINVAL, "sq_prefill_fwd: negative window size for head %d", h);
      SQ_REQUIRE(p->w8[h] % kBN == 0 && p->w4[h] % kBN == 0, SQ_EUNSUPPORTED,
                 "sq_prefill_fwd: window sizes must be multiples of 64 (head %d: %d / %d)", h, p->w8[h], p->w4[h]);
      // with w4 > w8 and w8 < block_m the reference's 4-bit range overlaps the diagonal block unmasked
      SQ_REQUIRE(!(p->w4[h] > p->w8[h] && p->w8[h] < p->block_m), SQ_EUNSUPPORTED,
                 "sq_prefill_fwd: head %d: a 4-bit window wider than an 8-bit window smaller than block_m reads future keys "
                 "in the reference and is not supported", h);
    }
    // separate 4-bit operands: a workgroup of one 64-row query block (two waves), or, for 128-row blocks, of two blocks
    // that walk the few tiles on which they disagree twice (DUAL)
    if (q4 && p->block_m == 64) waves = 2;
  } else {
    SQ_REQUIRE(p->window_mode == SQ_WINDOW_NONE, SQ_EINVAL, "sq_prefill_fwd: window_mode %d not supported", p->window_mode);
    SQ_REQUIRE(!q4, SQ_EINVAL, "sq_prefill_fwd: q4/k4 only apply to window mode");
  }
  SQ_REQUIRE(!(p->p_quant >= SQ_P_E4M3_FP8_PV && q4), SQ_EUNSUPPORTED,
             "sq_prefill_fwd: the fp8 P.V mode does not take separate 4-bit operands");
  const size_t need = sq_prefill_workspace_bytes(B, Hkv, Nk, D);
  SQ_REQUIRE(workspace && on_gpu(workspace) && workspace->device.device_id == dev, SQ_EWORKSPACE,
             "sq_prefill_fwd: workspace missing or not on the device");
  SQ_REQUIRE((size_t)numel_of(workspace) * (workspace->dtype.bits / 8) >= need && is_compact(workspace), SQ_EWORKSPACE,
             "sq_prefill_fwd: workspace too small: need %zu bytes", need);
  SQ_REQUIRE(((uintptr_t)data_of(workspace) & 15) == 0, SQ_EWORKSPACE, "sq_prefill_fwd: workspace not 16-byte aligned");

  hipStream_t st = (hipStream_t)stream;
  int cur = -1;
  SQ_HIP(hipGetDevice(&cur));
  SQ_REQUIRE(cur == dev, SQ_EDEVICE, "sq_prefill_fwd: tensors live on device %d but the current device is %d", dev, cur);

  const int nT = (int)((Nk + kBN - 1) / kBN);
  const bool pv8 = p->p_quant >= SQ_P_E4M3_FP8_PV;
  char* wsp = data_of(workspace);
  // workspace: fp16 tiles (modes 0-3), or e4m3 tiles (half the size) followed by the per-channel scale tables
  const size_t tiles8 = ((size_t)B * Hkv * nT * (kD * kBN) + 255) / 256 * 256;
  PrepArgs pa;
  pa.v = data_of(v);
  pa.vt = (_Float16*)wsp;
  pa.vt8 = (uint8_t*)wsp;
  pa.vmax_bits = (uint32_t*)(wsp + tiles8);
  pa.v_inv_scale = (float*)(wsp + tiles8 + (size_t)B * Hkv * kD * 4);
  pa.v_sb = stride_of(v, 0);
  pa.v_sh = stride_of(v, hdim);
  pa.v_sn = stride_of(v, ndim);
  pa.Nk = (int)Nk;
  pa.nT = nT;
  pa.Hkv = (int)Hkv;
  pa.is_bf16 = dt == DType::BF16;
  const dim3 pgrid(nT, (unsigned)Hkv, (unsigned)B);
  if (pv8) {
    SQ_REQUIRE(tiles8 + (size_t)B * Hkv * kD * 8 <= need, SQ_EWORKSPACE, "sq_prefill_fwd: workspace too small for the fp8 tiles");
    hipLaunchKernelGGL(prefill_fill_u32_kernel, dim3(1), dim3(256), 0, st, pa.vmax_bits, (int)(B * Hkv * kD));
    hipLaunchKernelGGL(prefill_vabsmax_kernel, pgrid, dim3(256), 0, st, pa);
    hipLaunchKernelGGL(prefill_prep_v8_kernel, pgrid, dim3(256), 0, st, pa);
  } else {
    hipLaunchKernelGGL(prefill_prep_v_kernel, pgrid, dim3(256), 0, st, pa);
  }
  SQ_HIP(hipGetLastError());

  PrefillArgs local;  // passed to the kernel by value (about 1.2 KB with the per-head windows)
  memset(&local, 0, sizeof(local));
  local.q = data_of(q);
  local.k = data_of(k);
  local.q4 = q4 ? data_of(q4) : nullptr;
  local.k4 = k4 ? data_of(k4) : nullptr;
  local.k_scale = nullptr;
  if (k_scale) {
    int rc2;
    if ((rc2 = check_tensor(k_scale, "k_scale", 3, dev))) return rc2;
    SQ_REQUIRE(dtype_of(k_scale) == DType::F32 && k_scale->shape[0] == B && k_scale->shape[1] == Hkv && k_scale->shape[2] == (int64_t)nT * kBN &&
                   is_compact(k_scale),
               SQ_ESHAPE, "sq_prefill_int8qk_fwd: k_scale must be a contiguous fp32 [B, Hkv, %lld] (tokens rounded up to whole tiles)",
               (long long)nT * kBN);
    SQ_REQUIRE(stride_of(k, ndim) % 16 == 0 && stride_of(k, hdim) % 16 == 0 && stride_of(k, 0) % 16 == 0, SQ_ESHAPE,
               "sq_prefill_int8qk_fwd: rows of k_codes must start on 16-byte boundaries");
    local.k_scale = (const float*)data_of(k_scale);
  }
  local.vt = pa.vt;
  local.vt8 = pa.vt8;
  local.v_inv_scale = pa.v_inv_scale;
  local.out = data_of(out);
  local.lse = lse ? (float*)data_of(lse) : nullptr;
  local.q_sb = stride_of(q, 0);
  local.q_sh = stride_of(q, hdim);
  local.q_sn = stride_of(q, ndim);
  local.k_sb = stride_of(k, 0);
  local.k_sh = stride_of(k, hdim);
  local.k_sn = stride_of(k, ndim);
  local.o_sb = stride_of(out, 0);
  local.o_sh = stride_of(out, hdim);
  local.o_sn = stride_of(out, ndim);
  local.B = (int)B;
  local.Hq = (int)Hq;
  local.Hkv = (int)Hkv;
  local.group = (int)(Hq / Hkv);
  local.Nq = (int)Nq;
  local.Nk = (int)Nk;
  local.nT = nT;
  const int rows_wg = waves * 32;
  local.nQB = (int)((Nq + rows_wg - 1) / rows_wg);
  SQ_REQUIRE(p->q_quant == 0 || p->q_quant == 8, SQ_EINVAL, "sq_prefill_fwd: q_quant must be 0 or 8 (got %d)", (int)p->q_quant);
  SQ_REQUIRE(!(p->q_quant && q4), SQ_EINVAL, "sq_prefill_fwd: q_quant applies to launches without a separate 4-bit operand set");
  local.q_quant = p->q_quant;
  local.q_offset = (int)p->q_offset;
  local.p_quant = p->p_quant;
  local.window_mode = p->window_mode;
  local.block_m = p->window_mode == SQ_WINDOW_SIZES ? p->block_m : 128;
  local.sink = p->sink;
  local.out_dtype = odt == DType::BF16 ? 0 : (odt == DType::F16 ? 1 : 2);
  const int64_t d_og = p->head_dim_og > 0 ? p->head_dim_og : D;
  SQ_REQUIRE(d_og <= kD, SQ_EINVAL, "Unsupported head_dim: %lld", (long long)d_og);
  local.sm = (float)(1.0 / sqrt((double)d_og) * 1.44269504);
  if (p->window_mode == SQ_WINDOW_SIZES)
    for (int h = 0; h < Hq; ++h) {
      local.w8[h] = p->w8[h];
      local.w4[h] = p->w4[h];
    }
  const int pairs = (int)(B * Hkv);
  const int items = local.group * local.nQB;
  local.sched_pairs = pairs;
  local.sched_items = items;
  unsigned blocks;
  if (pairs <= 8 && 8 % pairs == 0) {
    local.sched_mode = 0;
    local.sched_xpp = 8 / pairs;
    blocks = 8u * (unsigned)((items + local.sched_xpp - 1) / local.sched_xpp);
  } else if (pairs % 8 == 0) {
    local.sched_mode = 1;
    local.sched_xpp = 1;
    blocks = (unsigned)pairs * (unsigned)items;
  } else {
    local.sched_mode = 2;
    local.sched_xpp = 1;
    blocks = (unsigned)pairs * (unsigned)items;
  }
  const size_t smem = 4 * (size_t)kStageBytes + 64;   // rings of 4 K tiles and 4 V^T tiles, MODE 2's block maxima
  const bool bf = dt == DType::BF16;
#define SQ_LAUNCH_PREFILL(BF, W, M)                                                                              \
  do {                                                                                                           \
    SQ_HIP(hipFuncSetAttribute((const void*)prefill_kernel<BF, W, M>, hipFuncAttributeMaxDynamicSharedMemorySize, \
                               (int)smem));                                                                      \
    hipLaunchKernelGGL((prefill_kernel<BF, W, M>), dim3(blocks), dim3(W * 64), smem, st, local);                 \
  } while (0)
#define SQ_LAUNCH_PREFILL_DUAL(BF, M)                                                                                  \
  do {                                                                                                                \
    SQ_HIP(hipFuncSetAttribute((const void*)prefill_kernel<BF, 8, M, true>, hipFuncAttributeMaxDynamicSharedMemorySize, \
                               (int)smem));                                                                           \
    hipLaunchKernelGGL((prefill_kernel<BF, 8, M, true>), dim3(blocks), dim3(8 * 64), smem, st, local);                \
  } while (0)
#define SQ_LAUNCH_DUAL(BF)                                          \
  do {                                                              \
    switch (p->p_quant) {                                           \
      case SQ_P_NONE: SQ_LAUNCH_PREFILL_DUAL(BF, 0); break;          \
      case SQ_P_E4M3_STATIC: SQ_LAUNCH_PREFILL_DUAL(BF, 1); break;   \
      case SQ_P_E4M3_BLOCK: SQ_LAUNCH_PREFILL_DUAL(BF, 2); break;    \
      default: SQ_LAUNCH_PREFILL_DUAL(BF, 3); break;                 \
    }                                                               \
  } while (0)
#define SQ_LAUNCH_MODE(BF, W)                                   \
  do {                                                          \
    if (k_scale) {                                              \
      SQ_LAUNCH_PREFILL(BF, W, 6);                              \
      break;                                                    \
    }                                                           \
    switch (p->p_quant) {                                       \
      case SQ_P_NONE: SQ_LAUNCH_PREFILL(BF, W, 0); break;        \
      case SQ_P_E4M3_STATIC: SQ_LAUNCH_PREFILL(BF, W, 1); break; \
      case SQ_P_E4M3_BLOCK: SQ_LAUNCH_PREFILL(BF, W, 2); break;  \
      case SQ_P_E4M3_FP8_PV: SQ_LAUNCH_PREFILL(BF, 8, 4); break; \
      case SQ_P_E4M3_MX_FP8_PV: SQ_LAUNCH_PREFILL(BF, 8, 5); break; \
      default: SQ_LAUNCH_PREFILL(BF, W, 3); break;               \
    }                                                           \
  } while (0)
  if (waves == 8 && q4) {
    if (bf) SQ_LAUNCH_DUAL(true); else SQ_LAUNCH_DUAL(false);
  } else if (waves == 8) {
    if (bf) SQ_LAUNCH_MODE(true, 8); else SQ_LAUNCH_MODE(false, 8);
  } else {
    if (bf) SQ_LAUNCH_MODE(true, 2); else SQ_LAUNCH_MODE(false, 2);
  }
#undef SQ_LAUNCH_DUAL
#undef SQ_LAUNCH_PREFILL_DUAL
#undef SQ_LAUNCH_MODE
#undef SQ_LAUNCH_PREFILL
  SQ_HIP(hipGetLastError());
  return SQ_OK;
}
}  // namespace
