// Fused operand pre-pass of the SQAttn plugin closure for gfx950 (MI355X).
//
// Replaces the tensor passes of the reference's `mp_triton_wrapper(...).attention_fn`
// (sqattn/attn_replacer.py:334-365) for the integer quantiser types:
//   :334-337  repeat_kv + permute           -> not materialised: the attention kernel reads the kv heads in place
//   :338-339  key -= key.mean(token axis)   -> column sums (two deterministic stages, fp64) + subtraction in the
//                                              tensor dtype
//   :361-365  five fake-quant passes        -> IntegerQuantizer(8|4, True, "per_token") on query and centred key
//                                              (sqattn/fake_quant.py:33-35, 47-52, 114-125), and
//                                              IntegerQuantizer(8, True, "per_channel") on value, whose range is
//                                              taken over dims (0, 1) of the [B, H, N, D] tensor (:30-32), i.e. one
//                                              scale per (token, channel) shared by batch and heads
// Every output element is computed with the same fp32 operations as the reference's formula (division by the
// scale, round half away from zero as sign(x) * floor(|x| + 0.5), clamp, multiplication by the scale, cast to
// the tensor dtype), so the results are bit-identical to a CPU restatement.
//
// HBM-bound streaming work: every input element is read once (K twice: sums, then quantisation) and every
// output element written once; rows of 128 channels are handled by 16 lanes x 16 bytes.
#include "common.hpp"

namespace sq {
namespace {

constexpr int kPD = 128;          // channels per row (head_dim)
constexpr int kSumBlocks = 512;   // partial-sum workgroups of the key mean (upper bound)

struct View {   // [B, N, H, 128] addressed by element strides (either memory layout)
  char* p;
  int64_t sb, sn, sh;
};

// The row kernels split a row number into (batch, token, head) with FastDiv (common.hpp): the 64-bit divisions they
// used before were a few hundred vector instructions per row, more than the quantisation itself.
struct PrepassArgs {
  View q, k, v, q8, q4, k8, k4, v8;
  FastDiv div_hq, div_hkv, div_n;
  int32_t small;    // every row number is below 2^31: the splits use fastdiv
  double* part;     // [nblk, B*Hkv*128]
  uint16_t* mean;   // [B*Hkv*128] bits of the key mean in the tensor dtype
  int32_t B, N, Hq, Hkv, is_bf16, nblk, tok_per_blk, want4;
  // integer operands of a real int8 Q.K^T (null: not wanted): the 8-bit codes of the centred key, laid out like key with
  // one byte per element, and the per-token scales, fp32 [B, Hkv, scale_stride] (token index last)
  View kcodes;
  float* kscale;
  int64_t scale_stride;
};


template <bool BF16>
__device__ __forceinline__ float ld(uint32_t bits16) {
  if constexpr (BF16) return bf16_bits_to_f32(bits16);
  return (float)__builtin_bit_cast(_Float16, (uint16_t)bits16);
}
template <bool BF16>
__device__ __forceinline__ uint32_t st(float x) {
  if constexpr (BF16) return f32_to_bf16_bits(x);
  return (uint32_t)__builtin_bit_cast(uint16_t, (_Float16)x);
}
template <bool BF16>
__device__ __forceinline__ void unpack8(const uint4& r, float (&x)[8]) {
  const uint32_t w[4] = {r.x, r.y, r.z, r.w};
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    x[2 * i] = ld<BF16>(w[i] & 0xffffu);
    x[2 * i + 1] = ld<BF16>(w[i] >> 16);
  }
}
template <bool BF16>
__device__ __forceinline__ uint4 pack8(const float (&x)[8]) {
  uint32_t w[4];
#pragma unroll
  for (int i = 0; i < 4; ++i) {
    if constexpr (BF16) w[i] = pack_bf16x2(x[2 * i], x[2 * i + 1]);
    else w[i] = st<BF16>(x[2 * i]) | (st<BF16>(x[2 * i + 1]) << 16);
  }
  return make_uint4(w[0], w[1], w[2], w[3]);
}

// paddle.round / the reference's rounding: half away from zero, evaluated in fp32 exactly like
// sign(x) * floor(abs(x) + 0.5)
__device__ __forceinline__ float round_half_away(float t) { return copysignf(floorf(fabsf(t) + 0.5f), t); }

// quant-dequant of one value: clamp(round(x / scale) + zero, qmin, qmax) * scale   (fake_quant.py:114-125, zero point 0),
// with the shared-divisor division of common.hpp (bit-identical to x / scale for these operand ranges: the
// divisor lies in [1e-5 / 127, 65504 / 7] and |x / scale| <= 128).
// `round(x / scale) + zero` with the symmetric quantiser's zero point 0.0 (fake_quant.py:114-116): the addition is
// kept because it turns a rounded -0.0 into +0.0, so a small negative x comes out as +0.0 like in the reference
__device__ __forceinline__ float qdq(float x, const Divisor& s, float qmin, float qmax) {
  const float q = fminf(fmaxf(round_half_away(divide(x, s)) + 0.0f, qmin), qmax);
  return q * s.d;
}

// FloatQuantizer(e4m3 | e5m2, True, ...).fake_quant_tensor of one value (fake_quant.py:151-204, 231-248):
// t = clamp(x / scale, +-fmax); E = floor(log2(|t| + 1e-30)); f = |t| / 2^E - 1; E' = clip(E, 1 - bias, bias);
// f' = clip(round(f * 2^MB) / 2^MB, 0, 1 - 2^-MB); y = (1 + f') * 2^E' * sign(t), clipped to +-(2 - 2^-MB) * 2^bias, zero
// kept; result y * scale.  Every step is the reference's fp32 operation (the divisions and multiplications by powers of
// two are exact), except that E is read from the exponent field of |t| + 1e-30 instead of floor(log2(.)): the two agree
// unless a library's fp32 log2 rounds a value a few units in the last place below a power of two up to the integer,
// where the reference's own result depends on that library.
template <int EB, int MB>
__device__ __forceinline__ float qdq_float(float x, const Divisor& s) {
  constexpr float fmax = EB == 4 ? 448.f : 57344.f;
  constexpr int bias = (1 << (EB - 1)) - 1;
  constexpr float eps = 1.0f / (1 << MB);
  constexpr float max_val = (2.0f - eps) * (float)(1u << bias);
  const float t = fminf(fmaxf(divide(x, s) + 0.0f, -fmax), fmax);
  const float av = fabsf(t);
  const int E = (int)((__float_as_uint(av + 1e-30f) >> 23) & 255u) - 127;
  const float f = av * ldexpf(1.0f, -E) - 1.0f;
  const int Ec = min(max(E, 1 - bias), bias);
  const float fq = fminf(fmaxf(round_half_away(f * (float)(1 << MB)) * eps, 0.0f), 1.0f - eps);
  float y = (1.0f + fq) * ldexpf(1.0f, Ec);
  y = fminf(y, max_val);
  y = (av == 0.0f) ? 0.0f : copysignf(y, t);
  return y * s.d;
}
// the 8-bit quantiser of a call: 0 integer (symmetric, +-127 range), 1 e4m3, 2 e5m2
template <int QT>
__device__ __forceinline__ float qdq8(float x, const Divisor& s) {
  if constexpr (QT == 1) return qdq_float<4, 3>(x, s);
  else if constexpr (QT == 2) return qdq_float<5, 2>(x, s);
  else return qdq(x, s, -128.f, 127.f);
}
template <int QT>
__device__ __forceinline__ float scale_of(float amax) {
  return amax / (QT == 1 ? 448.f : (QT == 2 ? 57344.f : 127.f));
}

// ---- key mean, stage 1: workgroup b sums tokens [b*tok_per_blk, ...) of every (batch, kv head, channel) in fp64.
// With few columns (Qwen2.5-7B: 4 kv heads x 16 groups of 8 channels = 64) the 256 threads split the tokens of the
// workgroup between them and combine through LDS in a fixed order.
template <bool BF16>
__global__ __launch_bounds__(256) void prepass_ksum_kernel(PrepassArgs a) {
  __shared__ double red[256][8];
  const int ncol8 = a.B * a.Hkv * (kPD / 8);   // column groups of 8 channels
  const int n0 = blockIdx.x * a.tok_per_blk, n1 = min(n0 + a.tok_per_blk, a.N);
  const int TL = ncol8 < 256 ? 256 / ncol8 : 1;   // token lanes per column group
  for (int cg0 = 0; cg0 < ncol8; cg0 += 256) {
    const int cg = cg0 + (TL > 1 ? (int)threadIdx.x % ncol8 : (int)threadIdx.x);
    const int tl = TL > 1 ? (int)threadIdx.x / ncol8 : 0;
    const bool live = cg < ncol8 && tl < TL;
    double s[8] = {0, 0, 0, 0, 0, 0, 0, 0};
    if (live) {
      const int c8 = cg % (kPD / 8), h = (cg / (kPD / 8)) % a.Hkv, b = cg / ((kPD / 8) * a.Hkv);
      const uint16_t* base = (const uint16_t*)a.k.p + b * a.k.sb + h * a.k.sh + 8 * c8;
      // eight rows requested before the first is used: with one row in flight per lane the workgroups of this small
      // grid keep too few bytes on the wire
      int n = n0 + tl;
      for (; n + 7 * TL < n1; n += 8 * TL) {
        uint4 raw[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) raw[u] = *(const uint4*)(base + (int64_t)(n + u * TL) * a.k.sn);
#pragma unroll
        for (int u = 0; u < 8; ++u) {
          float x[8];
          unpack8<BF16>(raw[u], x);
#pragma unroll
          for (int e = 0; e < 8; ++e) s[e] += (double)x[e];
        }
      }
      for (; n < n1; n += TL) {
        float x[8];
        unpack8<BF16>(*(const uint4*)(base + (int64_t)n * a.k.sn), x);
#pragma unroll
        for (int e = 0; e < 8; ++e) s[e] += (double)x[e];
      }
    }
    if (TL > 1) {
#pragma unroll
      for (int e = 0; e < 8; ++e) red[threadIdx.x][e] = s[e];
      __syncthreads();
      if (live && tl == 0) {
        for (int u = 1; u < TL; ++u)
#pragma unroll
          for (int e = 0; e < 8; ++e) s[e] += red[u * ncol8 + cg][e];
      }
      __syncthreads();
    }
    if (live && tl == 0) {
      double* dst = a.part + (int64_t)blockIdx.x * (ncol8 * 8) + cg * 8;
#pragma unroll
      for (int e = 0; e < 8; ++e) dst[e] = s[e];
    }
  }
}

// ---- key mean, stage 2: 16 lanes per column add the partial sums l, l+16, ... and combine in a fixed tree;
// mean = dtype(float(sum / N))
template <bool BF16>
__global__ __launch_bounds__(256) void prepass_kmean_kernel(PrepassArgs a) {
  const int ncol = a.B * a.Hkv * kPD;
  const int c = (blockIdx.x * blockDim.x + threadIdx.x) >> 4, l = threadIdx.x & 15;
  double s = 0;
  if (c < ncol) {   // four partial sums requested at a time (one after the other they were 32 dependent round trips)
    double s4[4] = {0, 0, 0, 0};
    int b = l;
    for (; b + 48 < a.nblk; b += 64) {
      double v[4];
#pragma unroll
      for (int u = 0; u < 4; ++u) v[u] = a.part[(int64_t)(b + 16 * u) * ncol + c];
#pragma unroll
      for (int u = 0; u < 4; ++u) s4[u] += v[u];
    }
    for (; b < a.nblk; b += 16) s4[0] += a.part[(int64_t)b * ncol + c];
    s = (s4[0] + s4[1]) + (s4[2] + s4[3]);
  }
#pragma unroll
  for (int sh = 8; sh >= 1; sh >>= 1) s += __shfl_xor(s, sh);
  if (c >= ncol || l != 0) return;
  // two roundings on purpose (fp64 -> fp32 -> tensor dtype), like a mean accumulated in fp32 and cast to the
  // tensor dtype; the empty asm keeps the compiler from merging them into one fp64 -> fp16 conversion
  float mf = (float)(s / (double)a.N);
  asm volatile("" : "+v"(mf));
  a.mean[c] = (uint16_t)st<BF16>(mf);
}

// ---- per-token 8-bit (and 4-bit) fake quantisation of the rows of q (CENTRE = false) or of k minus its mean
template <bool BF16, bool CENTRE, int QT>
__global__ __launch_bounds__(256) void prepass_rows_kernel(PrepassArgs a) {
  const View& src = CENTRE ? a.k : a.q;
  const View& d8 = CENTRE ? a.k8 : a.q8;
  const View& d4 = CENTRE ? a.k4 : a.q4;
  const int H = CENTRE ? a.Hkv : a.Hq;
  const int64_t rows = (int64_t)a.B * a.N * H;
  const int l16 = threadIdx.x & 15;
  // two consecutive rows per 16-lane group, both loads issued before any arithmetic
  constexpr int R = 2;
  const int64_t row0 = ((int64_t)blockIdx.x * (blockDim.x / 16) + (threadIdx.x >> 4)) * R;
  if (row0 >= rows) return;   // whole 16-lane groups leave together; the shuffles below stay inside a group
  uint4 raw[R], mraw[R];
  int64_t off8[R], off4[R], nn[R], bbv[R];
  int hh[R];
  bool live[R];
#pragma unroll
  for (int u = 0; u < R; ++u) {
    const int64_t row = row0 + u;
    live[u] = row < rows;
    const int64_t rr = live[u] ? row : row0;
    int h;
    int64_t n, b;
    if (a.small) {
      const uint32_t t = fastdiv((uint32_t)rr, CENTRE ? a.div_hkv : a.div_hq);
      h = (int)((uint32_t)rr - t * (uint32_t)H);
      const uint32_t bb = fastdiv(t, a.div_n);
      n = t - bb * (uint32_t)a.N;
      b = bb;
    } else {
      h = (int)(rr % H);
      n = (rr / H) % a.N;
      b = rr / ((int64_t)H * a.N);
    }
    hh[u] = h;
    nn[u] = n;
    bbv[u] = b;
    {   // rows are read once and written once: non-temporal accesses keep them from displacing each other in L2
      const u32x4_t w = __builtin_nontemporal_load((const u32x4_t*)((const uint16_t*)src.p + b * src.sb + n * src.sn + h * src.sh + 8 * l16));
      raw[u] = make_uint4(w[0], w[1], w[2], w[3]);
    }
    if constexpr (CENTRE) mraw[u] = *(const uint4*)(a.mean + ((int)b * H + h) * kPD + 8 * l16);
    off8[u] = b * d8.sb + n * d8.sn + h * d8.sh + 8 * l16;
    off4[u] = a.want4 ? b * d4.sb + n * d4.sn + h * d4.sh + 8 * l16 : 0;
  }
#pragma unroll
  for (int u = 0; u < R; ++u) {
    float x[8];
    unpack8<BF16>(raw[u], x);
    if constexpr (CENTRE) {
      float m[8];
      unpack8<BF16>(mraw[u], m);
#pragma unroll
      for (int e = 0; e < 8; ++e) x[e] = ld<BF16>(st<BF16>(x[e] - m[e]));   // the subtraction rounds to the tensor dtype
    }
    float amax = 0.f;
#pragma unroll
    for (int e = 0; e < 8; ++e) amax = fmaxf(amax, fabsf(x[e]));
#pragma unroll
    for (int sh = 1; sh < 16; sh <<= 1) amax = fmaxf(amax, __shfl_xor(amax, sh));
    amax = fmaxf(amax, 1e-5f);
    if (!live[u]) continue;
    if (d8.p) {
      const Divisor scale = make_divisor(scale_of<QT>(amax));
      float y[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) y[e] = qdq8<QT>(x[e], scale);
      const uint4 o = pack8<BF16>(y);
      __builtin_nontemporal_store(u32x4_t{o.x, o.y, o.z, o.w}, (u32x4_t*)((uint16_t*)d8.p + off8[u]));
    }
    if constexpr (CENTRE && QT == 0) {
      if (a.kcodes.p) {   // the codes themselves (what qdq multiplies by the scale) and the scale
        const Divisor scale = make_divisor(amax / 127.f);
        uint32_t w[2] = {0, 0};
#pragma unroll
        for (int e = 0; e < 8; ++e) {
          const int c = (int)fminf(fmaxf(round_half_away(divide(x[e], scale)) + 0.0f, -128.f), 127.f);
          w[e >> 2] |= (uint32_t)(c & 0xff) << (8 * (e & 3));
        }
        const int h = hh[u];
        const int64_t n = nn[u], b = bbv[u];
        *(uint2*)((char*)a.kcodes.p + b * a.kcodes.sb + n * a.kcodes.sn + h * a.kcodes.sh + 8 * l16) = make_uint2(w[0], w[1]);
        if (l16 == 0) a.kscale[(b * H + h) * a.scale_stride + n] = scale.d;
      }
    }
    if (a.want4) {
      const Divisor scale = make_divisor(amax / 7.f);
      float y[8];
#pragma unroll
      for (int e = 0; e < 8; ++e) y[e] = qdq(x[e], scale, -8.f, 7.f);
      const uint4 o = pack8<BF16>(y);
      __builtin_nontemporal_store(u32x4_t{o.x, o.y, o.z, o.w}, (u32x4_t*)((uint16_t*)d4.p + off4[u]));
    }
  }
}

// ---- value: one 8-bit scale per (token, channel) over batch and heads
template <bool BF16, int QT>
__global__ __launch_bounds__(256) void prepass_v_kernel(PrepassArgs a) {
  const int64_t t = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;   // (token, group of 8 channels)
  if (t >= (int64_t)a.N * (kPD / 8)) return;
  const int c8 = (int)(t % (kPD / 8));
  const int64_t n = t / (kPD / 8);
  const uint16_t* base = (const uint16_t*)a.v.p + n * a.v.sn + 8 * c8;
  float amax[8] = {0, 0, 0, 0, 0, 0, 0, 0};
  const int nrow = a.B * a.Hkv;
  if (nrow <= 8) {
    // few (batch, head) rows per token (Qwen2.5-7B: 4): all of them requested at once and kept in registers, so that V
    // is read once and no load waits for the one before it
    uint4 raw[8];
    int64_t oo[8];
    int b = 0, h = 0;
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      raw[r] = make_uint4(0, 0, 0, 0);
      oo[r] = 0;
      if (r < nrow) {
        raw[r] = *(const uint4*)(base + b * a.v.sb + h * a.v.sh);
        oo[r] = b * a.v8.sb + h * a.v8.sh;
        if (++h == a.Hkv) {
          h = 0;
          ++b;
        }
      }
    }
#pragma unroll
    for (int r = 0; r < 8; ++r) {
      float x[8];
      unpack8<BF16>(raw[r], x);   // rows past nrow are zeros: no effect on the maximum
#pragma unroll
      for (int e = 0; e < 8; ++e) amax[e] = fmaxf(amax[e], fabsf(x[e]));
    }
    Divisor sc[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) sc[e] = make_divisor(scale_of<QT>(fmaxf(amax[e], 1e-5f)));
    uint16_t* ob = (uint16_t*)a.v8.p + n * a.v8.sn + 8 * c8;
#pragma unroll
    for (int r = 0; r < 8; ++r)
      if (r < nrow) {
        float x[8], y[8];
        unpack8<BF16>(raw[r], x);
#pragma unroll
        for (int e = 0; e < 8; ++e) y[e] = qdq8<QT>(x[e], sc[e]);
        *(uint4*)(ob + oo[r]) = pack8<BF16>(y);
      }
    return;
  }
  for (int b = 0; b < a.B; ++b)
    for (int h = 0; h < a.Hkv; ++h) {
      float x[8];
      unpack8<BF16>(*(const uint4*)(base + b * a.v.sb + h * a.v.sh), x);
#pragma unroll
      for (int e = 0; e < 8; ++e) amax[e] = fmaxf(amax[e], fabsf(x[e]));
    }
  Divisor scale[8];
#pragma unroll
  for (int e = 0; e < 8; ++e) scale[e] = make_divisor(scale_of<QT>(fmaxf(amax[e], 1e-5f)));
  uint16_t* obase = (uint16_t*)a.v8.p + n * a.v8.sn + 8 * c8;
  for (int b = 0; b < a.B; ++b)
    for (int h = 0; h < a.Hkv; ++h) {
      float x[8], y[8];
      unpack8<BF16>(*(const uint4*)(base + b * a.v.sb + h * a.v.sh), x);
#pragma unroll
      for (int e = 0; e < 8; ++e) y[e] = qdq8<QT>(x[e], scale[e]);
      *(uint4*)(obase + b * a.v8.sb + h * a.v8.sh) = pack8<BF16>(y);
    }
}

int make_view(const DLTensor* t, const char* name, int layout, int dev, DType dt, int64_t B, int64_t N, int64_t H, View* out) {
  int rc;
  if ((rc = check_tensor(t, name, 4, dev))) return rc;
  SQ_REQUIRE(dtype_of(t) == dt, SQ_EDTYPE, "sq_fake_quant_prepass: %s must have the dtype of query", name);
  const int nd = layout == SQ_LAYOUT_HND ? 2 : 1, hd = layout == SQ_LAYOUT_HND ? 1 : 2;
  SQ_REQUIRE(t->shape[0] == B && t->shape[nd] == N && t->shape[hd] == H && t->shape[3] == kPD, SQ_ESHAPE,
             "sq_fake_quant_prepass: %s has the wrong shape", name);
  for (int d = 0; d < 3; ++d)
    SQ_REQUIRE(stride_of(t, d) % 8 == 0 || t->shape[d] == 1, SQ_ESHAPE, "sq_fake_quant_prepass: rows of %s are not 16-byte aligned", name);
  out->p = data_of(t);
  out->sb = stride_of(t, 0);
  out->sn = stride_of(t, nd);
  out->sh = stride_of(t, hd);
  return SQ_OK;
}

int tokens_per_block(int64_t N) { return (int)((N + kSumBlocks - 1) / kSumBlocks); }

}  // namespace
}  // namespace sq

using namespace sq;

extern "C" size_t sq_fake_quant_prepass_workspace_bytes(int64_t batch, int64_t num_kv_heads, int64_t num_tokens) {
  if (batch <= 0 || num_kv_heads <= 0 || num_tokens <= 0) return 0;
  const int tpb = tokens_per_block(num_tokens);
  const int64_t nblk = (num_tokens + tpb - 1) / tpb;
  const size_t cols = (size_t)batch * num_kv_heads * kPD;
  return (size_t)nblk * cols * sizeof(double) + ((cols * 2 + 255) & ~(size_t)255);
}

namespace {
int prepass_impl(const DLTensor* query, const DLTensor* key, const DLTensor* value, DLTensor* q8, DLTensor* q4, DLTensor* k8, DLTensor* k4,
                 DLTensor* v8, DLTensor* workspace, int32_t layout, int32_t qk_qtype, int32_t v_qtype, void* stream, DLTensor* k_codes,
                 DLTensor* k_scale);
}

extern "C" int sq_fake_quant_prepass_typed(const DLTensor* query, const DLTensor* key, const DLTensor* value, DLTensor* q8,
                                           DLTensor* q4, DLTensor* k8, DLTensor* k4, DLTensor* v8, DLTensor* workspace,
                                           int32_t layout, int32_t qk_qtype, int32_t v_qtype, void* stream) {
  return prepass_impl(query, key, value, q8, q4, k8, k4, v8, workspace, layout, qk_qtype, v_qtype, stream, nullptr, nullptr);
}

extern "C" int sq_fake_quant_prepass_int8qk(const DLTensor* query, const DLTensor* key, const DLTensor* value, DLTensor* k_codes,
                                            DLTensor* k_scale, DLTensor* v8, DLTensor* workspace, int32_t layout, void* stream) {
  SQ_REQUIRE(k_codes && k_scale, SQ_EINVAL, "sq_fake_quant_prepass_int8qk: null tensor argument");
  return prepass_impl(query, key, value, nullptr, nullptr, nullptr, nullptr, v8, workspace, layout, SQ_QTYPE_INT, SQ_QTYPE_INT, stream, k_codes,
                      k_scale);
}

namespace {
int prepass_impl(const DLTensor* query, const DLTensor* key, const DLTensor* value, DLTensor* q8, DLTensor* q4, DLTensor* k8, DLTensor* k4,
                 DLTensor* v8, DLTensor* workspace, int32_t layout, int32_t qk_qtype, int32_t v_qtype, void* stream, DLTensor* k_codes,
                 DLTensor* k_scale) {
  SQ_REQUIRE(qk_qtype >= SQ_QTYPE_INT && qk_qtype <= SQ_QTYPE_E5M2 && v_qtype >= SQ_QTYPE_INT && v_qtype <= SQ_QTYPE_E5M2, SQ_EINVAL,
             "Invalid quantization type: %d / %d", (int)qk_qtype, (int)v_qtype);
  SQ_REQUIRE(query && key && value && (k8 || k_codes) && v8, SQ_EINVAL, "sq_fake_quant_prepass: null tensor argument");
  SQ_REQUIRE((q4 == nullptr) == (k4 == nullptr), SQ_EINVAL, "sq_fake_quant_prepass: q4 and k4 must be given together");
  // q8 == NULL: the query rows are left alone (the attention kernel can quantise them as it loads them, q_quant = 8)
  SQ_REQUIRE(q8 || !q4, SQ_EINVAL, "sq_fake_quant_prepass: without q8 there are no 4-bit operands either");
  const bool skip_q = q8 == nullptr;
  SQ_REQUIRE(layout == SQ_LAYOUT_HND || layout == SQ_LAYOUT_NHD, SQ_EINVAL, "Unknown tensor layout: %d", (int)layout);
  int rc;
  if ((rc = check_tensor(query, "query", 4, query->device.device_id))) return rc;
  const int dev = query->device.device_id;
  const DType dt = dtype_of(query);
  SQ_REQUIRE(dt == DType::BF16 || dt == DType::F16, SQ_EDTYPE, "sq_fake_quant_prepass: query must be bf16 or fp16");
  const int nd = layout == SQ_LAYOUT_HND ? 2 : 1, hd = layout == SQ_LAYOUT_HND ? 1 : 2;
  SQ_REQUIRE(query->shape[3] == kPD, SQ_EUNSUPPORTED, "sq_fake_quant_prepass: head_dim must be %d (pad smaller heads with zeros)", kPD);
  if ((rc = check_tensor(key, "key", 4, dev))) return rc;
  const int64_t B = query->shape[0], N = query->shape[nd], Hq = query->shape[hd], Hkv = key->shape[hd];
  SQ_REQUIRE(B > 0 && N > 0 && Hq > 0 && Hkv > 0, SQ_ESHAPE, "sq_fake_quant_prepass: empty tensor");
  SQ_REQUIRE(B * N * Hq < (int64_t)1 << 40 && B * Hkv * kPD < (int64_t)1 << 24, SQ_EUNSUPPORTED, "sq_fake_quant_prepass: tensor too large");
  // the kernels index tokens with 32-bit integers and the launches take 32-bit grid sizes (32 rows per workgroup)
  SQ_REQUIRE(N < ((int64_t)1 << 31) - 65536 && B < ((int64_t)1 << 20) && B * N * Hq / 32 < ((int64_t)1 << 31) - 1, SQ_EUNSUPPORTED,
             "sq_fake_quant_prepass: more than 2^31 tokens per sequence or 2^36 query rows");
  PrepassArgs a;
  memset(&a, 0, sizeof(a));
  if ((rc = make_view(query, "query", layout, dev, dt, B, N, Hq, &a.q)) || (rc = make_view(key, "key", layout, dev, dt, B, N, Hkv, &a.k)) ||
      (rc = make_view(value, "value", layout, dev, dt, B, N, Hkv, &a.v)) || (!skip_q && (rc = make_view(q8, "q8", layout, dev, dt, B, N, Hq, &a.q8))) ||
      (k8 && (rc = make_view(k8, "k8", layout, dev, dt, B, N, Hkv, &a.k8))) || (rc = make_view(v8, "v8", layout, dev, dt, B, N, Hkv, &a.v8)))
    return rc;
  if (k_codes) {
    // int8 [like key]; rows of 128 bytes on 16-byte boundaries.  k_scale: fp32 [B, Hkv, >= N], contiguous
    if ((rc = check_tensor(k_codes, "k_codes", 4, dev)) || (rc = check_tensor(k_scale, "k_scale", 3, dev))) return rc;
    SQ_REQUIRE(k_codes->dtype.code == kDLInt && k_codes->dtype.bits == 8 && k_codes->dtype.lanes == 1, SQ_EDTYPE,
               "sq_fake_quant_prepass_int8qk: k_codes must be int8");
    SQ_REQUIRE(k_codes->shape[0] == B && k_codes->shape[nd] == N && k_codes->shape[hd] == Hkv && k_codes->shape[3] == kPD, SQ_ESHAPE,
               "sq_fake_quant_prepass_int8qk: k_codes has the wrong shape");
    for (int d = 0; d < 3; ++d)
      SQ_REQUIRE(stride_of(k_codes, d) % 16 == 0 || k_codes->shape[d] == 1, SQ_ESHAPE, "sq_fake_quant_prepass_int8qk: rows of k_codes are not 16-byte aligned");
    SQ_REQUIRE(dtype_of(k_scale) == DType::F32 && k_scale->shape[0] == B && k_scale->shape[1] == Hkv && k_scale->shape[2] >= N && is_compact(k_scale),
               SQ_ESHAPE, "sq_fake_quant_prepass_int8qk: k_scale must be a contiguous fp32 [B, Hkv, >= N]");
    a.kcodes.p = data_of(k_codes);
    a.kcodes.sb = stride_of(k_codes, 0);
    a.kcodes.sn = stride_of(k_codes, nd);
    a.kcodes.sh = stride_of(k_codes, hd);
    a.kscale = (float*)data_of(k_scale);
    a.scale_stride = k_scale->shape[2];
  }
  if (q4 && ((rc = make_view(q4, "q4", layout, dev, dt, B, N, Hq, &a.q4)) || (rc = make_view(k4, "k4", layout, dev, dt, B, N, Hkv, &a.k4))))
    return rc;
  const size_t need = sq_fake_quant_prepass_workspace_bytes(B, Hkv, N);
  SQ_REQUIRE(workspace && on_gpu(workspace) && workspace->device.device_id == dev, SQ_EWORKSPACE,
             "sq_fake_quant_prepass: workspace missing or not on the device");
  SQ_REQUIRE((size_t)numel_of(workspace) * (workspace->dtype.bits / 8) >= need && is_compact(workspace), SQ_EWORKSPACE,
             "sq_fake_quant_prepass: workspace too small: need %zu bytes", need);
  SQ_REQUIRE(((uintptr_t)data_of(workspace) & 255) == 0, SQ_EWORKSPACE, "sq_fake_quant_prepass: workspace not 256-byte aligned");
  int cur = -1;
  SQ_HIP(hipGetDevice(&cur));
  SQ_REQUIRE(cur == dev, SQ_EDEVICE, "sq_fake_quant_prepass: tensors live on device %d but the current device is %d", dev, cur);

  a.B = (int)B;
  a.N = (int)N;
  a.Hq = (int)Hq;
  a.Hkv = (int)Hkv;
  a.is_bf16 = dt == DType::BF16;
  a.div_hq = make_fastdiv((uint32_t)Hq);
  a.div_hkv = make_fastdiv((uint32_t)Hkv);
  a.div_n = make_fastdiv((uint32_t)N);
  a.small = (B * N * (Hq > Hkv ? Hq : Hkv) < (1ll << 31)) ? 1 : 0;
  a.tok_per_blk = tokens_per_block(N);
  a.nblk = (int)((N + a.tok_per_blk - 1) / a.tok_per_blk);
  a.want4 = q4 != nullptr;
  const size_t cols = (size_t)B * Hkv * kPD;
  a.part = (double*)data_of(workspace);
  a.mean = (uint16_t*)(data_of(workspace) + (size_t)a.nblk * cols * sizeof(double));
  hipStream_t s = (hipStream_t)stream;
  const int64_t qrows = B * N * Hq, krows = B * N * Hkv, vthreads = N * (kPD / 8);
#define SQ_PREPASS_ROWS(BF, QT)                                                                                        \
  do {                                                                                                                 \
    if (!skip_q)                                                                                                       \
      hipLaunchKernelGGL((prepass_rows_kernel<BF, false, QT>), dim3((unsigned)((qrows + 31) / 32)), dim3(256), 0, s, a); \
    hipLaunchKernelGGL((prepass_rows_kernel<BF, true, QT>), dim3((unsigned)((krows + 31) / 32)), dim3(256), 0, s, a);  \
  } while (0)
#define SQ_PREPASS_LAUNCH(BF)                                                                                       \
  do {                                                                                                              \
    hipLaunchKernelGGL(prepass_ksum_kernel<BF>, dim3(a.nblk), dim3(256), 0, s, a);                                  \
    hipLaunchKernelGGL(prepass_kmean_kernel<BF>, dim3((unsigned)((cols * 16 + 255) / 256)), dim3(256), 0, s, a);    \
    if (qk_qtype == SQ_QTYPE_E4M3) SQ_PREPASS_ROWS(BF, 1);                                                          \
    else if (qk_qtype == SQ_QTYPE_E5M2) SQ_PREPASS_ROWS(BF, 2);                                                     \
    else SQ_PREPASS_ROWS(BF, 0);                                                                                    \
    const dim3 vgrid((unsigned)((vthreads + 255) / 256));                                                           \
    if (v_qtype == SQ_QTYPE_E4M3) hipLaunchKernelGGL((prepass_v_kernel<BF, 1>), vgrid, dim3(256), 0, s, a);         \
    else if (v_qtype == SQ_QTYPE_E5M2) hipLaunchKernelGGL((prepass_v_kernel<BF, 2>), vgrid, dim3(256), 0, s, a);    \
    else hipLaunchKernelGGL((prepass_v_kernel<BF, 0>), vgrid, dim3(256), 0, s, a);                                  \
  } while (0)
  if (a.is_bf16) SQ_PREPASS_LAUNCH(true);
  else SQ_PREPASS_LAUNCH(false);
#undef SQ_PREPASS_LAUNCH
#undef SQ_PREPASS_ROWS
  SQ_HIP(hipGetLastError());
  return SQ_OK;
}
}  // namespace

extern "C" int sq_fake_quant_prepass(const DLTensor* query, const DLTensor* key, const DLTensor* value, DLTensor* q8,
                                     DLTensor* q4, DLTensor* k8, DLTensor* k4, DLTensor* v8, DLTensor* workspace,
                                     int32_t layout, void* stream) {
  return sq_fake_quant_prepass_typed(query, key, value, q8, q4, k8, k4, v8, workspace, layout, SQ_QTYPE_INT, SQ_QTYPE_INT, stream);
}
