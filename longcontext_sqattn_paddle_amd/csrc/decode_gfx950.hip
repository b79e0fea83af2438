// Split-KV decode attention for gfx950 (MI355X): one query token per sequence against a GQA KV cache.
//
// Replaces the reference's `_attn_decode_fwd` + `attn_unified` decode branch
// (sqattn/attn_triton_decode.py:175-241, 244-324).  The reference runs one program per (batch, q-head)
// and streams the whole cache serially, re-reading each KV head once per q-head of its group.  Here a
// workgroup owns one (batch, kv-head, token range): it streams that range ONCE for all q-heads of the
// group, writes a normalised partial output with its base-2 log-sum-exp, and a second tiny kernel merges
// the partials (lse = log2 sum_s 2^lse_s, o = sum_s 2^(lse_s-lse) o_s).
//
// Data path per wave and 16-token tile (HBM-bound; everything else is sized to stay out of the way):
//   K : 4 x 16-byte loads per lane, lane (r=lane%16, g=lane/16) reads K[n0+r][32kk+8g .. +7]  -> A operand
//   S^T[token, head] = K . Q~^T  on v_mfma_f32_16x16x32 (bf16/f16 in, fp32 acc); Q~ (16 padded heads) lives
//        in registers as the B operand; lane (r,g) ends up with head r, tokens n0+4g+i, i<4.
//   V : 4 x 16-byte loads per lane, load i reads V[n0+4g+i][8r .. 8r+7] (full 256-byte rows per 16 lanes)
//   O^T[d, head] += V^T . P^T  on v_mfma_f32_16x16x16 of the tensor dtype with k = the tile's 16 tokens: the A operand is
//        eight channels of the lane's four V rows (two v_perm_b32 per channel offset), the B operand the lane's own p as
//        hi + lo (p rounded to the tensor dtype plus the rounded remainder, relative error 2^-16 for bf16) -- no
//        transposition, no LDS, V exact, standing in for the reference's fp32 `p * v.to(float32)` (:234).
#include <mutex>

#include "common.hpp"

// Scratch of sq_decode_fwd_noalloc: the split-KV partials of one call, in place of the caller's workspace.  One copy
// per GPU the library is loaded on, held until the process ends; its contents are the last call's partials.  In host
// code this name is only a handle for hipGetSymbolAddress; the device address is looked up once per device.
constexpr size_t kNoAllocScratchBytes = 8u << 20;
static __device__ __align__(256) unsigned char scratch[kNoAllocScratchBytes];
constexpr int kMaxDevices = 64;
static void* g_scratch_ptr[kMaxDevices] = {};
static std::mutex g_scratch_mutex;

namespace sq {
namespace {


constexpr int kD = 128;          // head_dim handled by the kernels (the host pads smaller heads with zeros)
constexpr int kWaves = 4;
constexpr int kTile = 16;        // tokens per MFMA tile
constexpr int kOStride = 132;    // padded row of the cross-wave merge buffer (floats)

struct DecodeArgs {
  const void* q;
  const void* k;
  const void* v;
  const int32_t* seqlens;
  const int32_t* ids;   // gather mode: [B * Hkv, L] cache rows to attend to per (sequence, kv head); negative = none
  int64_t ids_sg;       // its row stride
  float* part_o;    // [B, Hq, S, D] normalised partial outputs
  float* part_lse;  // [B, Hq, S]    base-2 LSE of each partial (-inf = empty)
  int64_t q_sb, q_sh;
  int64_t k_sb, k_sh, k_sn;
  int64_t v_sb, v_sh, v_sn;
  int32_t B, Hq, Hkv, L, group, head_chunks, num_splits, chunk, p_quant;
  int32_t cache_len;  // gather mode: rows per sequence in the cache (L is then the length of the id lists)
  int32_t hpw;  // kv heads per workgroup (1, 2 or 4): 4/hpw waves share one kv head and interleave its tiles
  int32_t by_length;  // 1: the B * num_splits workgroups of a head group are dealt to the sequences in proportion to their lengths
  float sm;  // log2e / sqrt(D_original), rounded to fp32
};

constexpr int kMaxShareBatch = 32;

// Ragged batches: with the same number of splits for every sequence the longest sequence decides when the call ends
// (lengths uniform in [96K, 128K]: 12 % of the time nothing but that tail).  Dealing the W = B * num_splits workgroups in
// proportion to the lengths evens that out: every sequence gets one workgroup, the other W - B go by cumulative rounding
// of (W - B) * (tokens up to and including the sequence) / (all tokens), so the shares add up to W exactly.  Sequence i
// then owns workgroups [base, base + n) and the same slots of the partial results, which are laid out [Hq, W] in this
// mode.  The split kernel (want_b < 0: finds the owner of workgroup w) and the combine kernel (want_b = its sequence)
// both call this, so they agree by construction.
// Every wave computes the whole table at once, one sequence per lane (B <= 32): one load, an integer prefix sum by
// shuffles (lengths in units of 32 tokens, so that 32 sequences of 2^31 tokens fit 32 bits), one 32-bit integer division
// per lane -- exact arithmetic, so the two kernels cannot disagree whatever flags they are compiled with.  For the
// division the prefix and the total are shifted right until the total is below 2^20 (the product with W - B < 2^12 then
// fits 32 bits; a 64-bit division is a software routine that cost the combine kernel 3 us at batch 8): the shares stay
// monotone and add up to W exactly, and proportional to 2^-20.  A loop over the sequences with a load and a division
// in every round took longer than the rest of the combine kernel.
__device__ __forceinline__ void share_of(const int32_t* seqlens, int B, int Lmax, int W, int want_b, int w, int& b, int& base, int& n) {
  const int lane = threadIdx.x & 63;
  const uint32_t len = lane < B ? ((uint32_t)min(max(seqlens[lane], 0), Lmax) + 31u) >> 5 : 0u;
  uint32_t cum = len;   // inclusive prefix
#pragma unroll
  for (int d = 1; d < kMaxShareBatch; d <<= 1) {
    const uint32_t v = __shfl_up(cum, d);
    if (lane >= d) cum += v;
  }
  const uint32_t total = __shfl(cum, B - 1);
  const int sh = max(0, 12 - (int)__builtin_clz(total | 1u));       // total >> sh < 2^20
  const uint32_t ts = total >> sh;
  const int e1 = ts > 0u ? (int)((uint32_t)(W - B) * (cum >> sh) / ts) : 0;   // W - B exactly for the last sequence
  int e0 = __shfl_up(e1, 1);
  if (lane == 0) e0 = 0;
  const int bs = lane + e0, ni = 1 + e1 - e0;
  const bool mine = lane < B && (want_b >= 0 ? lane == want_b : (w >= bs && w < bs + ni));
  const unsigned long long mask = __ballot(mine);
  b = 0;
  base = 0;
  n = 1;
  if (mask) {
    const int src = __ffsll((long long)mask) - 1;
    b = src;
    base = __shfl(bs, src);
    n = __shfl(ni, src);
  }
}

// 16-byte load of cache data that is read exactly once: non-temporal, so it does not displace useful lines
__device__ __forceinline__ uint4 stream_load(const uint16_t* p) {
  typedef __attribute__((ext_vector_type(4))) unsigned u32x4_t;
  const u32x4_t v = __builtin_nontemporal_load((const u32x4_t*)p);
  return make_uint4(v[0], v[1], v[2], v[3]);
}

template <bool BF16>
__device__ __forceinline__ float elem_to_f32(uint32_t bits16) {
  if constexpr (BF16) {
    return bf16_bits_to_f32(bits16);
  } else {
    return (float)__builtin_bit_cast(_Float16, (uint16_t)bits16);
  }
}

template <bool BF16>
__device__ __forceinline__ uint32_t f32_to_elem(float x) {
  if constexpr (BF16) {
    return f32_to_bf16_bits(x);
  } else {
    return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)x);
  }
}

template <bool BF16>
__device__ __forceinline__ f32x4_t mfma_qk(const uint4& a, const uint4& b, f32x4_t c) {
  if constexpr (BF16) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8_t, a), __builtin_bit_cast(bf16x8_t, b),
                                                   c, 0, 0, 0);
  } else {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8_t, a), __builtin_bit_cast(f16x8_t, b), c,
                                                  0, 0, 0);
  }
}

template <bool BF16>
__device__ __forceinline__ f32x4_t mfma_pv16(const i32x2_t& a, const i32x2_t& b, f32x4_t c) {
  typedef __attribute__((ext_vector_type(4))) short i16x4_t;
  if constexpr (BF16) {
    return __builtin_amdgcn_mfma_f32_16x16x16bf16_1k(__builtin_bit_cast(i16x4_t, a), __builtin_bit_cast(i16x4_t, b), c, 0, 0, 0);
  } else {
    return __builtin_amdgcn_mfma_f32_16x16x16f16(__builtin_bit_cast(f16x4_t, a), __builtin_bit_cast(f16x4_t, b), c, 0, 0, 0);
  }
}

// GATHER: token t of the stream is cache row ids[b * Hkv + kvh][t] instead of row t (attention over a selection of
// the cache, e.g. the tokens of the best-scoring k-means clusters); entries that are negative or beyond the cache
// are skipped.
// BYLEN: the workgroups of a ragged batch dealt by length (share_of); a template parameter so that the code of the other launches
// is the code without it.
template <bool BF16, bool GATHER, bool BYLEN>
__global__ __launch_bounds__(kWaves * 64) void decode_splitkv_kernel(DecodeArgs a) {
  __shared__ float s_o[kWaves][16][kOStride];
  __shared__ float s_m[kWaves][16];
  __shared__ float s_l[kWaves][16];

  // Workgroup = (token range, hpw kv heads, batch).  With hpw = 4 each wave streams one kv head over the same
  // token range, so the workgroup as a whole reads whole cache rows of an NHD cache ([B, L, Hkv, D]).
  int split = blockIdx.x, b = blockIdx.z, nsp = a.num_splits;
  int64_t slot_stride = a.num_splits;     // partial rows: (b * Hq + hq) * num_splits + split, or hq * W + workgroup
  int64_t slot0 = (int64_t)b * a.Hq * a.num_splits + split;
  if constexpr (BYLEN) {
    const int W = a.B * a.num_splits, w = (int)blockIdx.z * a.num_splits + (int)blockIdx.x;
    int base;
    share_of(a.seqlens, a.B, a.L, W, -1, w, b, base, nsp);
    split = w - base;
    slot_stride = W;
    slot0 = w;
  }
  const int hy = blockIdx.y / a.head_chunks;
  const int hc = blockIdx.y % a.head_chunks;
  const int lane = threadIdx.x & 63;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
  const int r = lane & 15;
  const int g = lane >> 4;
  const int wpg = kWaves / a.hpw;            // waves per kv head
  const int hsub = wave / wpg;               // which kv head of the workgroup this wave serves
  const int wsub = wave % wpg;               // its position among the waves of that head
  const int kvh = hy * a.hpw + hsub;

  int Lb = a.seqlens ? a.seqlens[b] : a.L;
  Lb = min(max(Lb, 0), a.L);
  // Tokens are dealt to the workgroups tile by tile (tile = 16 tokens): workgroup `split` takes tiles split,
  // split + S, split + 2S, ...  At any moment all resident workgroups then read neighbouring tiles, i.e. the chip
  // sweeps the cache front to back, which HBM serves much better than hundreds of separate streams.
  const int t1 = Lb;
  const int ntiles_all = (Lb + kTile - 1) / kTile;
  const int ntiles = (ntiles_all - split + nsp - 1) / nsp;   // tiles of this workgroup (<= 0: none)
  const int h0 = hc * 16;                    // first head of this chunk inside the kv group
  const int nh = min(16, a.group - h0);      // heads handled here
  const int hq0 = kvh * a.group + h0;        // absolute first q head of this wave

  if (ntiles <= 0) {  // empty split: weight 0 in the merge
    for (int i = threadIdx.x; i < a.hpw * nh * kD; i += blockDim.x) {
      const int hs = i / (nh * kD), h = (i / kD) % nh, d = i % kD;
      const int hq = (hy * a.hpw + hs) * a.group + h0 + h;
      a.part_o[((int64_t)hq * slot_stride + slot0) * kD + d] = 0.f;
      if (d == 0) a.part_lse[(int64_t)hq * slot_stride + slot0] = -INFINITY;
    }
    return;
  }

  const uint16_t* kbase = (const uint16_t*)a.k + (int64_t)b * a.k_sb + (int64_t)kvh * a.k_sh;
  const uint16_t* vbase = (const uint16_t*)a.v + (int64_t)b * a.v_sb + (int64_t)kvh * a.v_sh;

  float m = -INFINITY;   // running max of head r (identical in the 4 lanes that share r)
  float l = 0.f;         // this lane's share of the running denominator
  f32x4_t acc[8];        // acc[e][i] = O^T[d = 32g + 8i + e][head r]
#pragma unroll
  for (int e = 0; e < 8; ++e) acc[e] = f32x4_t{0.f, 0.f, 0.f, 0.f};

  // loads are clamped to the last valid token so that nothing past the valid prefix is touched; bit i of `valid`
  // says whether token n0 + 4g + i (the one whose score this lane holds in s[i]) takes part
  const int32_t* idp = GATHER ? a.ids + ((int64_t)b * a.Hkv + kvh) * a.ids_sg : nullptr;
  auto load_tile = [&](int tile, uint4 (&kf)[4], uint4 (&vf)[4], int& valid) {
    const int n0 = (split + tile * nsp) * kTile;
    int tk = min(n0 + r, t1 - 1);
    if constexpr (GATHER) tk = min(max(idp[tk], 0), a.cache_len - 1);
    const uint16_t* kp = kbase + (int64_t)tk * a.k_sn + 8 * g;
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) kf[kk] = stream_load(kp + 32 * kk);
    valid = 0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      const int pos = n0 + 4 * g + i;
      int tv = min(pos, t1 - 1);
      bool ok = pos < t1;
      if constexpr (GATHER) {
        const int id = idp[tv];
        ok = ok && id >= 0 && id < a.cache_len;
        tv = min(max(id, 0), a.cache_len - 1);
      }
      valid |= (int)ok << i;
      vf[i] = stream_load(vbase + (int64_t)tv * a.v_sn + 8 * r);
    }
  };
  // four register sets: the loads of the wave's next three tiles are in flight while it works on the current one
  // (a workgroup of a 128K-token cache only has 16 tiles).  The first loads are issued before the query is
  // fetched and scaled, so that the two latencies overlap.
  constexpr int kSets = 4;
  uint4 kR[kSets][4], vR[kSets][4];
  int mR[kSets];
  int tile = wsub;
#pragma unroll
  for (int u = 0; u < kSets - 1; ++u)
    if (tile + u * wpg < ntiles) load_tile(tile + u * wpg, kR[u], vR[u], mR[u]);

  // Q~ fragments (B operand): lane (col head r, k-group g) holds q~[r][32kk+8g .. +7]
  uint4 qf[4];
  {
    const uint16_t* qp = (const uint16_t*)a.q + (int64_t)b * a.q_sb + (int64_t)(hq0 + r) * a.q_sh;
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) {
      uint32_t w[4] = {0, 0, 0, 0};
      if (r < nh) {
        const uint4 raw = *(const uint4*)(qp + 32 * kk + 8 * g);
        const uint32_t in[4] = {raw.x, raw.y, raw.z, raw.w};
#pragma unroll
        for (int j = 0; j < 4; ++j) {
          const float lo = elem_to_f32<BF16>(in[j] & 0xffffu) * a.sm;
          const float hi = elem_to_f32<BF16>(in[j] >> 16) * a.sm;
          w[j] = f32_to_elem<BF16>(lo) | (f32_to_elem<BF16>(hi) << 16);
        }
      }
      qf[kk] = make_uint4(w[0], w[1], w[2], w[3]);
    }
  }

  auto compute_tile = [&](const uint4 (&kf)[4], const uint4 (&vf)[4], int valid) {
    f32x4_t s = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int kk = 0; kk < 4; ++kk) s = mfma_qk<BF16>(kf[kk], qf[kk], s);

    float p[4];
    float tmax = -INFINITY;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      p[i] = ((valid >> i) & 1) ? s[i] : -INFINITY;
      tmax = fmaxf(tmax, p[i]);
    }
    tmax = wave_xor_max(tmax, 16);
    tmax = wave_xor_max(tmax, 32);
    const float m_new = fmaxf(m, tmax);
    // nothing valid so far (only a selection can produce such a tile): any finite reference keeps exp2 off inf - inf
    const float m_ref = (m_new == -INFINITY) ? 0.f : m_new;
    // the bare v_exp_f32: arguments are <= 0, and results below the normal range may flush to zero
    const float alpha = __builtin_amdgcn_exp2f(m - m_ref);    // exp2(-inf) = 0 on the first tile
    float psum = 0.f;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      p[i] = __builtin_amdgcn_exp2f(p[i] - m_ref);
      psum += p[i];
    }
    l = l * alpha + psum;
    if (a.p_quant == SQ_P_E4M3_STATIC) {
#pragma unroll
      for (int i = 0; i < 4; ++i) p[i] = (float)(_Float16)(e4m3_roundtrip(p[i] * 448.f) / 448.f);
    }
    if (__any(alpha != 1.f)) {
#pragma unroll
      for (int e = 0; e < 8; ++e) acc[e] *= alpha;
    }
    // P.V on the 16-bit matrix instruction with K = 16 tokens: V stays exact, and p goes in as the sum of two 16-bit
    // numbers, p = hi + lo with hi = p rounded to the tensor dtype and lo = the rounded remainder (relative error
    // 2^-16 for bf16, 2^-22 for fp16), both accumulated in fp32.  Operand layouts need no transposition: lane
    // (r, g) holds V[token 4g + j][channel 8r + e] in vf[j] and p[token 4g + j][head r] in p[j], which is the A
    // (16 channels 8m + e x 16 tokens) and the B (16 tokens x 16 heads) operand of one MFMA per e.  16 MFMAs of four
    // passes per tile, where the fp32 instruction (one token quartet and one e at a time) took 32 of eight.
    i32x2_t p_hi, p_lo;
    {
      float rem[4];
      uint32_t hb[4], lb[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        hb[i] = f32_to_elem<BF16>(p[i]);
        rem[i] = p[i] - elem_to_f32<BF16>(hb[i]);
        lb[i] = f32_to_elem<BF16>(rem[i]);
      }
      p_hi = i32x2_t{(int)(hb[0] | (hb[1] << 16)), (int)(hb[2] | (hb[3] << 16))};
      p_lo = i32x2_t{(int)(lb[0] | (lb[1] << 16)), (int)(lb[2] | (lb[3] << 16))};
    }
    const uint32_t vw[4][4] = {{vf[0].x, vf[0].y, vf[0].z, vf[0].w}, {vf[1].x, vf[1].y, vf[1].z, vf[1].w},
                               {vf[2].x, vf[2].y, vf[2].z, vf[2].w}, {vf[3].x, vf[3].y, vf[3].z, vf[3].w}};
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      // element e of the four tokens' rows: the low or the high halves of word e >> 1
      const uint32_t sel = (e & 1) ? 0x07060302u : 0x05040100u;
      const i32x2_t av = {(int)__builtin_amdgcn_perm(vw[1][e >> 1], vw[0][e >> 1], sel), (int)__builtin_amdgcn_perm(vw[3][e >> 1], vw[2][e >> 1], sel)};
      acc[e] = mfma_pv16<BF16>(av, p_hi, acc[e]);
      acc[e] = mfma_pv16<BF16>(av, p_lo, acc[e]);
    }
    m = m_new;
  };
  while (tile < ntiles) {
#pragma unroll
    for (int u = 0; u < kSets; ++u) {
      const int tn = tile + (kSets - 1) * wpg;
      if (tn < ntiles) load_tile(tn, kR[(u + kSets - 1) % kSets], vR[(u + kSets - 1) % kSets], mR[(u + kSets - 1) % kSets]);
      compute_tile(kR[u], vR[u], mR[u]);
      tile += wpg;
      if (tile >= ntiles) break;
    }
  }

  // fold the 4 lane groups' shares of l, then merge the waves that share a kv head through LDS
  l += __shfl_xor(l, 16);
  l += __shfl_xor(l, 32);
  if (wpg == 1) {
    // one wave per kv head (the usual case): the wave's registers are the whole partial, no merge through LDS, and
    // one division per lane (the general path below divides every element, which a wave alone on its SIMD feels:
    // the two together took 4 us off every call).  The normalised partial differs from o / l by at most 1 ulp.
    if (r < nh) {
      const int64_t row = (int64_t)(hq0 + r) * slot_stride + slot0;
      float* po = a.part_o + row * kD + 32 * g;
      const bool any = l > 0.f;
      const float inv = any ? 1.f / l : 0.f;
#pragma unroll
      for (int i = 0; i < 4; ++i) {
        *(float4*)(po + 8 * i) = make_float4(acc[0][i] * inv, acc[1][i] * inv, acc[2][i] * inv, acc[3][i] * inv);
        *(float4*)(po + 8 * i + 4) = make_float4(acc[4][i] * inv, acc[5][i] * inv, acc[6][i] * inv, acc[7][i] * inv);
      }
      if (g == 0) a.part_lse[row] = any ? m + log2f(l) : -INFINITY;
    }
    return;
  }
#pragma unroll
  for (int e = 0; e < 8; ++e)
#pragma unroll
    for (int i = 0; i < 4; ++i) s_o[wave][r][32 * g + 8 * i + e] = acc[e][i];
  if (g == 0) {
    s_m[wave][r] = m;
    s_l[wave][r] = l;
  }
  __syncthreads();
  for (int hs = 0; hs < a.hpw; ++hs)
  for (int idx = threadIdx.x; idx < nh * kD; idx += blockDim.x) {
    const int h = idx >> 7, d = idx & (kD - 1);
    const int w0 = hs * wpg;
    float mm = -INFINITY;
    for (int w = 0; w < wpg; ++w) mm = fmaxf(mm, s_m[w0 + w][h]);
    float lt = 0.f, o = 0.f;
    for (int w = 0; w < wpg; ++w) {
      // 0 for a wave that saw no valid token (m = -inf); when no wave did, the partial is empty
      const float sc = (mm > -INFINITY) ? exp2f(s_m[w0 + w][h] - mm) : 0.f;
      lt += s_l[w0 + w][h] * sc;
      o += s_o[w0 + w][h][d] * sc;
    }
    const int hq = (hy * a.hpw + hs) * a.group + h0 + h;
    const int64_t row = (int64_t)hq * slot_stride + slot0;
    a.part_o[row * kD + d] = (lt > 0.f) ? o / lt : 0.f;
    if (d == 0) a.part_lse[row] = (lt > 0.f) ? mm + log2f(lt) : -INFINITY;
  }
}

struct CombineArgs {
  const float* part_o;
  const float* part_lse;
  void* out;
  float* lse;  // may be null
  int64_t o_sb, o_sh;
  int32_t Hq, num_splits, out_dtype;  // 0 bf16, 1 f16, 2 f32
  const int32_t* seqlens;             // by_length: the lengths the split kernel dealt its workgroups by
  int32_t B, L, by_length;
};

constexpr int kCombineThreads = 1024;
constexpr int kCombineChunk = 32;                       // output channels per workgroup
constexpr int kCombineGroups = kCombineThreads / kCombineChunk;   // 32 groups of 32 threads, each sums every 32nd split

// One workgroup per (q head, batch, 32 output channels): 32 groups of 32 threads (one thread per channel), each sums
// every 32nd split.  A thread's first eight partial outputs are requested before anything else, so that they travel while
// the weights of the splits are formed (maximum and sum of 2^(lse - max): one shuffle reduction per wave, the 16 wave
// results through LDS, three barriers in all).
__global__ __launch_bounds__(kCombineThreads) void decode_combine_kernel(CombineArgs a) {
  extern __shared__ float s_w[];          // [num_splits] weights, then [32][32] partial outputs
  __shared__ float s_red[2][kCombineThreads / 64];
  const int h = blockIdx.x, b = blockIdx.y, tid = threadIdx.x;
  int S = a.num_splits;
  int64_t row0 = ((int64_t)b * a.Hq + h) * S;
  if (a.by_length) {   // this sequence's slots among the W of the head
    const int W = a.B * a.num_splits;
    int bb, base;
    share_of(a.seqlens, a.B, a.L, W, b, 0, bb, base, S);
    row0 = (int64_t)h * W + base;
  }
  const int dl = tid & (kCombineChunk - 1), grp = tid / kCombineChunk;
  const int d = blockIdx.z * kCombineChunk + dl;
  const float* po = a.part_o + row0 * kD + d;
  constexpr int G = kCombineGroups;
  constexpr int kPre = 8;
  float x[kPre];
#pragma unroll
  for (int i = 0; i < kPre; ++i) x[i] = (grp + i * G < S) ? po[(int64_t)(grp + i * G) * kD] : 0.f;
  float mx = -INFINITY;
  for (int s = tid; s < S; s += kCombineThreads) mx = fmaxf(mx, a.part_lse[row0 + s]);
#pragma unroll
  for (int m = 32; m > 0; m >>= 1) mx = fmaxf(mx, __shfl_xor(mx, m));
  if ((tid & 63) == 0) s_red[0][tid >> 6] = mx;
  __syncthreads();
#pragma unroll
  for (int w = 0; w < kCombineThreads / 64; ++w) mx = fmaxf(mx, s_red[0][w]);
  float tot = 0.f;
  for (int s = tid; s < S; s += kCombineThreads) {
    const float w = (mx > -INFINITY) ? exp2f(a.part_lse[row0 + s] - mx) : 0.f;
    s_w[s] = w;
    tot += w;
  }
#pragma unroll
  for (int m = 32; m > 0; m >>= 1) tot += __shfl_xor(tot, m);
  if ((tid & 63) == 0) s_red[1][tid >> 6] = tot;
  __syncthreads();
  tot = 0.f;
#pragma unroll
  for (int w = 0; w < kCombineThreads / 64; ++w) tot += s_red[1][w];   // the same order in every thread
  float o = 0.f;
#pragma unroll
  for (int i = 0; i < kPre; ++i)
    if (grp + i * G < S) o += s_w[grp + i * G] * x[i];                  // an empty split has weight 0 and a zero partial
  int s = grp + kPre * G;
  for (; s + 3 * G < S; s += 4 * G) {   // 4 independent loads in flight
    const float w0 = s_w[s], w1 = s_w[s + G], w2 = s_w[s + 2 * G], w3 = s_w[s + 3 * G];
    const float x0 = po[(int64_t)s * kD], x1 = po[(int64_t)(s + G) * kD], x2 = po[(int64_t)(s + 2 * G) * kD],
                x3 = po[(int64_t)(s + 3 * G) * kD];
    o += w0 * x0 + w1 * x1 + w2 * x2 + w3 * x3;
  }
  for (; s < S; s += G) o += s_w[s] * po[(int64_t)s * kD];
  float* s_part = s_w + S;
  s_part[grp * kCombineChunk + dl] = o;
  __syncthreads();
  if (grp == 0) {
    o = 0.f;
#pragma unroll
    for (int q = 0; q < G; ++q) o += s_part[q * kCombineChunk + dl];
    o = (tot > 0.f) ? o / tot : 0.f;
    const int64_t off = (int64_t)b * a.o_sb + (int64_t)h * a.o_sh + d;
    if (a.out_dtype == 0) {
      ((uint16_t*)a.out)[off] = (uint16_t)f32_to_bf16_bits(o);
    } else if (a.out_dtype == 1) {
      ((_Float16*)a.out)[off] = (_Float16)o;
    } else {
      ((float*)a.out)[off] = o;
    }
    if (a.lse && d == 0) a.lse[(int64_t)b * a.Hq + h] = (tot > 0.f) ? mx + log2f(tot) : -INFINITY;
  }
}

}  // namespace
}  // namespace sq

using namespace sq;

extern "C" int32_t sq_decode_num_splits(int64_t batch, int64_t num_kv_heads, int64_t max_len) {
  if (batch <= 0 || num_kv_heads <= 0 || max_len <= 0) return 1;
  // One workgroup per CU and never more workgroups than the 256 CUs: measured at batch 1, 256 workgroups stream a
  // 1M-token cache in 306 us, 512 in 324 us, and any count that is not a multiple of 256 leaves some CUs with twice
  // the work of the others (320 workgroups: 425 us).  At least 64 tokens (4 waves x 1 tile) per workgroup.
  const int64_t target_blocks = 256;
  const int64_t hpw = (num_kv_heads % 4 == 0) ? 4 : ((num_kv_heads % 2 == 0) ? 2 : 1);
  const int64_t groups = batch * (num_kv_heads / hpw);
  int64_t s = target_blocks / groups;   // rounded down: 255 workgroups are fine, 257 are not
  const int64_t max_s = (max_len * hpw + 63) / 64;   // at least one tile of 16 tokens per wave (4096 tokens: 256 workgroups 16.2 us, 64 workgroups 18.2 us)
  if (s > max_s) s = max_s;
  if (s < 1) s = 1;
  if (s > 4096) s = 4096;
  return (int32_t)s;
}

extern "C" size_t sq_decode_workspace_bytes(int64_t batch, int64_t num_q_heads, int64_t head_dim, int32_t num_splits) {
  (void)head_dim;
  if (batch <= 0 || num_q_heads <= 0 || num_splits <= 0) return 0;
  return (size_t)batch * num_q_heads * num_splits * (kD + 1) * sizeof(float);
}

// Shared body of sq_decode_fwd (token_ids == null) and sq_decode_selected_fwd.  The messages keep the name of the
// dense entry point for both.
// Partials go to `workspace`, or, when `own_scratch` is given, to that device buffer of `own_scratch_bytes` bytes.
static int decode_impl(const DLTensor* q, const DLTensor* kcache, const DLTensor* vcache, const DLTensor* seqlens,
                       const DLTensor* token_ids, DLTensor* out, DLTensor* lse, DLTensor* workspace,
                       const sq_decode_params* params, void* stream, void* own_scratch = nullptr,
                       size_t own_scratch_bytes = 0) {
  SQ_REQUIRE(params, SQ_EINVAL, "sq_decode_fwd: params is null");
  SQ_REQUIRE(q && kcache && vcache && out, SQ_EINVAL, "sq_decode_fwd: q, kcache, vcache and out must be non-null");
  SQ_REQUIRE(params->layout == SQ_LAYOUT_HND || params->layout == SQ_LAYOUT_NHD, SQ_EINVAL,
             "tensor_layout %d not supported", params->layout);
  SQ_REQUIRE(params->p_quant == SQ_P_NONE || params->p_quant == SQ_P_E4M3_STATIC, SQ_EINVAL,
             "sq_decode_fwd: p_quant %d not supported", params->p_quant);
  int rc;
  const int dev = q->device.device_id;
  if ((rc = check_tensor(q, "q", 4, dev)) || (rc = check_tensor(kcache, "kcache", 4, dev)) ||
      (rc = check_tensor(vcache, "vcache", 4, dev)) || (rc = check_tensor(out, "out", 4, dev)))
    return rc;
  const DType dt = dtype_of(q);
  SQ_REQUIRE(dt == DType::BF16 || dt == DType::F16, SQ_EDTYPE, "sq_decode_fwd: q must be bf16 or fp16");
  SQ_REQUIRE(dtype_of(kcache) == dt && dtype_of(vcache) == dt, SQ_EDTYPE, "sq_decode_fwd: q, kcache, vcache dtypes differ");
  const DType odt = dtype_of(out);
  SQ_REQUIRE(odt == DType::BF16 || odt == DType::F16 || odt == DType::F32, SQ_EDTYPE,
             "sq_decode_fwd: out must be bf16, fp16 or fp32");
  const bool hnd = params->layout == SQ_LAYOUT_HND;
  const int hdim = hnd ? 1 : 2, ndim = hnd ? 2 : 1;
  const int64_t B = q->shape[0], Hq = q->shape[hdim], Nq = q->shape[ndim], D = q->shape[3];
  const int64_t Hkv = kcache->shape[hdim], Lcache = kcache->shape[ndim];
  int64_t L = Lcache;   // length of the token stream: the cache, or the id lists of a selection
  if (token_ids) {
    SQ_REQUIRE(on_gpu(token_ids) && token_ids->device.device_id == dev, SQ_EDEVICE, "sq_decode_selected_fwd: token_ids not on the same device");
    SQ_REQUIRE(dtype_of(token_ids) == DType::I32 && token_ids->ndim == 2 && token_ids->shape[0] == B * Hkv && token_ids->shape[1] > 0 &&
                   stride_of(token_ids, 1) == 1,
               SQ_ESHAPE, "sq_decode_selected_fwd: token_ids must be int32 [B * Hkv = %lld, k] with contiguous rows", (long long)(B * Hkv));
    L = token_ids->shape[1];
  }
  SQ_REQUIRE(D == kD, SQ_EINVAL, "Unsupported head_dim: %lld (the kernels take 128; pad smaller heads with zeros)", (long long)D);
  SQ_REQUIRE(Nq == 1, SQ_ESHAPE, "sq_decode_fwd: query length must be 1, got %lld", (long long)Nq);
  SQ_REQUIRE(B > 0 && Hq > 0 && Hkv > 0 && L > 0 && Lcache > 0, SQ_ESHAPE, "sq_decode_fwd: empty tensor");
  SQ_REQUIRE(Hq % Hkv == 0, SQ_ESHAPE, "sq_decode_fwd: Hq=%lld not a multiple of Hkv=%lld", (long long)Hq, (long long)Hkv);
  SQ_REQUIRE(kcache->shape[0] == B && kcache->shape[3] == D, SQ_ESHAPE, "sq_decode_fwd: kcache shape mismatch");
  for (int i = 0; i < 4; ++i)
    SQ_REQUIRE(vcache->shape[i] == kcache->shape[i], SQ_ESHAPE, "sq_decode_fwd: vcache shape differs from kcache");
  for (int i = 0; i < 4; ++i) SQ_REQUIRE(out->shape[i] == q->shape[i], SQ_ESHAPE, "sq_decode_fwd: out shape differs from q");
  SQ_REQUIRE(L < (1ll << 31) - 65536 && Lcache < (1ll << 31) - 65536, SQ_EUNSUPPORTED, "sq_decode_fwd: cache longer than 2^31 tokens");
  SQ_REQUIRE(stride_of(kcache, ndim) % 8 == 0 && stride_of(vcache, ndim) % 8 == 0 && stride_of(kcache, hdim) % 8 == 0 &&
                 stride_of(vcache, hdim) % 8 == 0 && stride_of(kcache, 0) % 8 == 0 && stride_of(vcache, 0) % 8 == 0 &&
                 stride_of(q, hdim) % 8 == 0 && stride_of(q, 0) % 8 == 0,
             SQ_ESHAPE, "sq_decode_fwd: strides must be multiples of 8 elements (16-byte vector loads)");
  if (seqlens) {
    SQ_REQUIRE(on_gpu(seqlens) && seqlens->device.device_id == dev, SQ_EDEVICE, "sq_decode_fwd: seqlens not on the same device");
    SQ_REQUIRE(dtype_of(seqlens) == DType::I32 && seqlens->ndim == 1 && seqlens->shape[0] == B && stride_of(seqlens, 0) == 1,
               SQ_ESHAPE, "sq_decode_fwd: seqlens must be a contiguous int32 [B]");
  }
  if (lse) {
    SQ_REQUIRE(on_gpu(lse) && lse->device.device_id == dev, SQ_EDEVICE, "sq_decode_fwd: lse not on the same device");
    SQ_REQUIRE(dtype_of(lse) == DType::F32 && numel_of(lse) == B * Hq && is_compact(lse), SQ_ESHAPE,
               "sq_decode_fwd: lse must be a compact fp32 tensor of B*Hq elements");
  }
  int32_t S = params->num_splits > 0 ? params->num_splits : sq_decode_num_splits(B, Hkv, L);
  if (S > L) S = (int32_t)L;
  int64_t chunk = (L + S - 1) / S;
  chunk = (chunk + kTile * kWaves - 1) / (kTile * kWaves) * (kTile * kWaves);
  const size_t need = sq_decode_workspace_bytes(B, Hq, D, S);
  SQ_REQUIRE(S <= 4096, SQ_EINVAL, "sq_decode_fwd: num_splits %d above 4096", S);
  float* ws_data;
  if (own_scratch) {
    SQ_REQUIRE(need <= own_scratch_bytes, SQ_EWORKSPACE,
               "sq_decode_fwd_noalloc: batch %lld x %lld q heads x %d splits needs %zu bytes of partial results, the library's "
               "scratch holds %zu; use sq_decode_fwd with a workspace (or fewer splits)",
               (long long)B, (long long)Hq, S, need, own_scratch_bytes);
    ws_data = (float*)own_scratch;
  } else {
    SQ_REQUIRE(workspace && on_gpu(workspace) && workspace->device.device_id == dev, SQ_EWORKSPACE,
               "sq_decode_fwd: workspace missing or not on the device");
    SQ_REQUIRE((size_t)numel_of(workspace) * (workspace->dtype.bits / 8) >= need && is_compact(workspace), SQ_EWORKSPACE,
               "sq_decode_fwd: workspace too small: need %zu bytes", need);
    SQ_REQUIRE(((uintptr_t)data_of(workspace) & 15) == 0, SQ_EWORKSPACE, "sq_decode_fwd: workspace not 16-byte aligned");
    ws_data = (float*)data_of(workspace);
  }

  const int64_t group = Hq / Hkv;
  DecodeArgs a;
  a.q = data_of(q);
  a.k = data_of(kcache);
  a.v = data_of(vcache);
  a.seqlens = seqlens ? (const int32_t*)data_of(seqlens) : nullptr;
  a.ids = token_ids ? (const int32_t*)data_of(token_ids) : nullptr;
  a.ids_sg = token_ids ? stride_of(token_ids, 0) : 0;
  a.cache_len = (int32_t)Lcache;
  a.part_o = ws_data;
  a.part_lse = a.part_o + (size_t)B * Hq * S * kD;
  a.q_sb = stride_of(q, 0);
  a.q_sh = stride_of(q, hdim);
  a.k_sb = stride_of(kcache, 0);
  a.k_sh = stride_of(kcache, hdim);
  a.k_sn = stride_of(kcache, ndim);
  a.v_sb = stride_of(vcache, 0);
  a.v_sh = stride_of(vcache, hdim);
  a.v_sn = stride_of(vcache, ndim);
  a.B = (int32_t)B;
  a.Hq = (int32_t)Hq;
  a.Hkv = (int32_t)Hkv;
  a.L = (int32_t)L;
  a.group = (int32_t)group;
  a.head_chunks = (int32_t)((group + 15) / 16);
  a.hpw = (Hkv % 4 == 0) ? 4 : ((Hkv % 2 == 0) ? 2 : 1);
  a.num_splits = S;
  // the library's own choice of splits on a ragged batch: workgroups in proportion to the lengths.  A caller that names
  // num_splits gets exactly that many for every sequence (a sequence's partition then does not depend on its batch mates).
  a.by_length = (seqlens && params->num_splits <= 0 && B > 1 && B <= kMaxShareBatch && S > 1 && B * (int64_t)S <= 4096) ? 1 : 0;
  a.chunk = (int32_t)chunk;
  a.p_quant = params->p_quant;
  const int64_t d_og = params->head_dim_og > 0 ? params->head_dim_og : D;
  SQ_REQUIRE(d_og <= kD, SQ_EINVAL, "Unsupported head_dim: %lld", (long long)d_og);
  a.sm = (float)(1.0 / sqrt((double)d_og) * 1.44269504);

  hipStream_t st = (hipStream_t)stream;
  int cur = -1;
  SQ_HIP(hipGetDevice(&cur));
  SQ_REQUIRE(cur == dev, SQ_EDEVICE, "sq_decode_fwd: tensors live on device %d but the current device is %d", dev, cur);
  const dim3 grid((unsigned)S, (unsigned)(Hkv / a.hpw * a.head_chunks), (unsigned)B);
#define SQ_LAUNCH_DECODE(BF, GA)                                                                                        \
  do {                                                                                                                 \
    if (a.by_length) hipLaunchKernelGGL((decode_splitkv_kernel<BF, GA, true>), grid, dim3(kWaves * 64), 0, st, a);     \
    else hipLaunchKernelGGL((decode_splitkv_kernel<BF, GA, false>), grid, dim3(kWaves * 64), 0, st, a);                \
  } while (0)
  if (token_ids) {
    if (dt == DType::BF16) SQ_LAUNCH_DECODE(true, true);
    else SQ_LAUNCH_DECODE(false, true);
  } else {
    if (dt == DType::BF16) SQ_LAUNCH_DECODE(true, false);
    else SQ_LAUNCH_DECODE(false, false);
  }
#undef SQ_LAUNCH_DECODE
  SQ_HIP(hipGetLastError());
  CombineArgs c;
  c.part_o = a.part_o;
  c.part_lse = a.part_lse;
  c.out = data_of(out);
  c.lse = lse ? (float*)data_of(lse) : nullptr;
  c.o_sb = stride_of(out, 0);
  c.o_sh = stride_of(out, hdim);
  c.Hq = (int32_t)Hq;
  c.num_splits = S;
  c.out_dtype = odt == DType::BF16 ? 0 : (odt == DType::F16 ? 1 : 2);
  c.seqlens = a.seqlens;
  c.B = (int32_t)B;
  c.L = (int32_t)L;
  c.by_length = a.by_length;
  const size_t max_slots = a.by_length ? (size_t)B * S : (size_t)S;   // a sequence may own up to all of a head's workgroups
  hipLaunchKernelGGL(decode_combine_kernel, dim3((unsigned)Hq, (unsigned)B, kD / kCombineChunk), dim3(kCombineThreads),
                     (max_slots + kCombineGroups * kCombineChunk) * sizeof(float), st, c);
  SQ_HIP(hipGetLastError());
  return SQ_OK;
}

extern "C" int sq_decode_fwd(const DLTensor* q, const DLTensor* kcache, const DLTensor* vcache, const DLTensor* seqlens,
                             DLTensor* out, DLTensor* lse, DLTensor* workspace, const sq_decode_params* params,
                             void* stream) {
  return decode_impl(q, kcache, vcache, seqlens, nullptr, out, lse, workspace, params, stream);
}

extern "C" int sq_decode_selected_fwd(const DLTensor* q, const DLTensor* kcache, const DLTensor* vcache,
                                      const DLTensor* token_ids, const DLTensor* seqlens, DLTensor* out, DLTensor* lse,
                                      DLTensor* workspace, const sq_decode_params* params, void* stream) {
  SQ_REQUIRE(token_ids, SQ_EINVAL, "sq_decode_selected_fwd: token_ids is null");
  return decode_impl(q, kcache, vcache, seqlens, token_ids, out, lse, workspace, params, stream);
}

extern "C" size_t sq_decode_noalloc_scratch_bytes(void) { return kNoAllocScratchBytes; }

// The device address of `scratch` on the current device, looked up once per device (every GPU holds its own copy of the
// array at its own address).  The look-up may load the library's code object on first use, so a caller that records
// HIP graphs runs it beforehand (sq_decode_noalloc_init); afterwards it is a table read.
static int noalloc_scratch(int dev, void** out) {
  SQ_REQUIRE(dev >= 0 && dev < kMaxDevices, SQ_EDEVICE, "sq_decode_fwd_noalloc: device id %d out of range", dev);
  std::lock_guard<std::mutex> guard(g_scratch_mutex);
  if (!g_scratch_ptr[dev]) {
    void* p = nullptr;
    SQ_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
    SQ_REQUIRE(p, SQ_EHIP, "sq_decode_fwd_noalloc: hipGetSymbolAddress returned a null address");
    g_scratch_ptr[dev] = p;
  }
  *out = g_scratch_ptr[dev];
  return SQ_OK;
}

extern "C" int sq_decode_noalloc_init(void) {
  int cur = -1;
  SQ_HIP(hipGetDevice(&cur));
  void* ptr;
  return noalloc_scratch(cur, &ptr);
}

extern "C" int sq_decode_fwd_noalloc(const DLTensor* q, const DLTensor* kcache, const DLTensor* vcache, const DLTensor* seqlens,
                                     DLTensor* out, DLTensor* lse, const sq_decode_params* params, void* stream) {
  SQ_REQUIRE(q, SQ_EINVAL, "sq_decode_fwd_noalloc: q is null");
  SQ_REQUIRE(on_gpu(q), SQ_EDEVICE, "sq_decode_fwd_noalloc: q is not on a ROCm device");
  const int dev = q->device.device_id;
  int cur = -1;
  SQ_HIP(hipGetDevice(&cur));
  SQ_REQUIRE(cur == dev, SQ_EDEVICE, "sq_decode_fwd_noalloc: tensors live on device %d but the current device is %d", dev, cur);
  void* ptr;
  int rc = noalloc_scratch(dev, &ptr);
  if (rc) return rc;
  return decode_impl(q, kcache, vcache, seqlens, nullptr, out, lse, nullptr, params, stream, ptr, kNoAllocScratchBytes);
}
