/*
 * libsqattn_hip.so -- C ABI of the MI355X (gfx950) implementation of SQAttn's attention hot path.
 *
 * Every entry point takes borrowed DLPack tensors (device pointers, shapes, strides in elements), plain
 * scalars and a HIP stream handle (`hipStream_t` passed as `void*`, NULL = the null stream); it enqueues
 * work on that stream and returns without synchronising unless stated otherwise.  Nothing is retained
 * after the call returns; outputs and workspaces are allocated by the caller.  (One piece of device memory lives
 * inside the library and says so where it is declared: the partials array of sq_decode_fwd_noalloc.)  Return value: SQ_OK or a
 * negative SQ_E* code; `sq_last_error()` then holds a message (thread-local).  No entry point throws or
 * aborts.  Tensors must live on one ROCm device (DLPack device type kDLROCM, or kDLCUDA as some
 * PyTorch-ROCm builds report), have a contiguous last dimension and a 16-byte aligned base address.
 *
 * Reference interfaces replaced (paths relative to the reference repository):
 *   sq_prefill_fwd            sqattn/attn_triton.py:216-315 (attn_causal -> _attn_fwd launch :279-310),
 *                             sqattn/attn_triton_mix_relative.py:309-483 (launch :439-475),
 *                             sqattn/attn_triton_mix_bad.py:285-426 (launch :388-424)
 *   sq_prefill_int8qk_fwd     the same launches with the query/key product on the int8 matrix instruction
 *   sq_fake_quant_prepass_int8qk  sqattn/attn_replacer.py:338-339, 361-365 for that path (key codes and scales, v8)
 *   sq_decode_fwd             sqattn/attn_triton_decode.py:244-361 (decode launch :293-324)
 *   sq_decode_fwd_noalloc     no reference counterpart: sq_decode_fwd for callers that cannot allocate device memory
 *   sq_decode_noalloc_init    no reference counterpart: its one-off set-up, for callers that record HIP graphs
 *   sq_decode_selected_fwd    no reference counterpart: the same decode over the tokens sq_topk_select picked
 *   sq_kmeans_train           cache_hub/kmeans.py:127-196 (assign launch :147-173, update launch :175-193)
 *   sq_kmeans_train_stateful  the same step inside the iteration loop of segment_k_means (cache_hub/kmeans.py:356-368)
 *   sq_reverse_index          cache_hub/kmeans.py:233-262
 *   sq_index_add              cache_hub/kmeans.py:307-329
 *   sq_topk_select            no reference counterpart (defined by this build's benchmark configuration)
 *   sq_kv_cache_store         cache_hub/flash_attn_cache.py:153-232 (prefill_update_kv_cache: the two slice copies)
 *   sq_kv_cache_append        cache_hub/flash_attn_cache.py:239-256 (decode_update_kv_cache)
 *   sq_kv_cache_reorder       no reference counterpart: a copy of a layer's cache in k-means cluster order
 *   sq_attention_histogram    sqattn/attn_replacer.py:253-278 (cal_attn_weight) + sqattn/window_search.py:20-87, 244-321
 *                             (the four histogram reductions over the dense map; capture slot model_hub/qwen.py:38-41)
 *   sq_rmsnorm                model_hub/utils.py:15-19 (rmsnorm; caller model_hub/qwen.py:345-350)
 *   sq_silu_and_mul           model_hub/utils.py:4-13 (silu_and_mul; caller model_hub/qwen.py:319-326)
 *   sq_rope                   model_hub/utils.py:21-106 (apply_rope_with_cos_sin_cache_inplace; caller qwen.py:352-367)
 *   sq_linear_rows            the matmuls of a decode step: model_hub/qwen.py:293-300 (lm), :302-312 (wqkv), :314-317 (wo),
 *                             :319-326 (mlp), called from model_hub/LLM.py:88-116 (layer_decode)
 *   sq_linear_rows_silu_and_mul  model_hub/qwen.py:320-324 (gate_up_proj and silu_and_mul of mlp) on a decode step
 *   sq_linear_rows_rope       model_hub/qwen.py:302-312 (wqkv) + :352-379 (rotary embedding of q and k) on a decode step
 *   sq_rmsnorm_linear_rows, sq_rmsnorm_linear_rows_silu_and_mul, sq_rmsnorm_linear_rows_rope
 *                             the three forms above together with the RMS norm in front of them: model_hub/LLM.py:92-93 + :95
 *                             (input_layernorm, wqkv), :110-114 (post_attention_layernorm, mlp), :161-163 (norm, lm)
 *   sq_fake_quant_prepass_typed  the same with the float quantiser types of sqattn/attn_replacer.py:340-358
 *   sq_fake_quant_prepass     sqattn/attn_replacer.py:334-365 (GQA expand, key centring and the five fake-quant
 *                             passes of mp_triton_wrapper's closure), sqattn/fake_quant.py:24-58, 98-125
 */
#ifndef SQATTN_H_
#define SQATTN_H_

#include <stddef.h>
#include <stdint.h>

#include "sq_dlpack.h"

#ifdef __cplusplus
extern "C" {
#endif

#define SQ_ABI_VERSION 3

enum {
  SQ_OK = 0,
  SQ_EINVAL = -1,       /* bad argument value (layout, head_dim > 128, sink, mode, null pointer)  */
  SQ_ESHAPE = -2,       /* shapes/strides inconsistent with each other                            */
  SQ_EDEVICE = -3,      /* tensor not on a ROCm device, or tensors on different devices           */
  SQ_EDTYPE = -4,       /* unsupported element type                                               */
  SQ_EUNSUPPORTED = -5, /* valid in the reference but outside what the kernels implement          */
  SQ_EHIP = -6,         /* a HIP runtime call failed (message carries hipGetErrorString)          */
  SQ_EWORKSPACE = -7    /* workspace missing or too small                                         */
};

enum { SQ_LAYOUT_HND = 0, SQ_LAYOUT_NHD = 1 };

/* Quantisation of the softmax probabilities before P.V */
enum {
  SQ_P_NONE = 0,         /* p.to(fp16)                               attn_triton.py:83           */
  SQ_P_E4M3_STATIC = 1,  /* fp16(fp16(e4m3(p*448))/448)              attn_triton.py:81-82        */
  SQ_P_E4M3_BLOCK = 2,   /* per (64 rows x 64 keys) absmax scale a: e4m3(p*448/a)*a/448 (no ref.) */
  SQ_P_E4M3_STATIC_FAST = 3, /* same e4m3 grid as STATIC with the factor 448 folded into the exponent  */
                         /* of p and the 1/448 cancelled against the denominator: skips the       */
                         /* reference's fp16 rounding of p/448 (relative 2^-11), prefill only      */
  SQ_P_E4M3_FP8_PV = 4,  /* e4m3 P as in STATIC_FAST *and* e4m3 V (one scale per batch, kv head and   */
                         /* channel, from a pre-pass): P.V runs on the fp8 matrix pipe.  No reference */
                         /* counterpart (it keeps V in fp16, attn_triton.py:83); prefill only         */
  SQ_P_E4M3_MX_FP8_PV = 5 /* as FP8_PV with a block scale on P: one power of two per query row and     */
                         /* 64-key tile, taken from the row's sum of the tile's probabilities (scaled */
                         /* sum in [128, 256), every scaled probability below 256), carried in the    */
                         /* scale operand of the block-scaled fp8 MFMA; the row's reference point is  */
                         /* set by its first tile and moves, by whole binades, when a tile's sum      */
                         /* exceeds 2^16; prefill only                                                */
};

enum { SQ_WINDOW_NONE = 0, SQ_WINDOW_SIZES = 1 };

int sq_abi_version(void);
const char* sq_last_error(void);

/* ---------------------------------------------------------------------------------------- prefill */
typedef struct sq_prefill_params {
  int32_t layout;        /* SQ_LAYOUT_*: q/out [B,Hq,Nq,D] + k/v [B,Hkv,Nk,D], or [B,N,H,D]               */
  int32_t p_quant;       /* SQ_P_*                                                                        */
  int32_t head_dim_og;   /* head_dim before zero-padding to 128: softmax scale = log2e/sqrt(head_dim_og); */
                         /* 0 = the tensors' D (attn_triton.py:236-250)                                   */
  int64_t q_offset;      /* absolute position of query row 0 (0 in the reference, which needs Nq == Nk)   */
  int32_t window_mode;   /* SQ_WINDOW_NONE: full causal (attn_triton.py). SQ_WINDOW_SIZES: sink + windows */
  int32_t block_m;       /* query-block size that defines the window ranges: 64 (relative wrapper,        */
                         /* attn_triton_mix_relative.py:423) or 128 (absolute, attn_triton_mix_bad.py:386) */
  int32_t sink;          /* sink size in tokens, multiple of 64                                           */
  int32_t num_heads_w;   /* number of entries of w8/w4 (== Hq)                                            */
  const int32_t* w8;     /* HOST arrays: per-head 8-bit / 4-bit window sizes in tokens (multiples of 64). */
  const int32_t* w4;     /* The relative wrapper converts ratios with ceil128(int(f32(ratio)*kv_len)).    */
  int32_t q_quant;       /* 0: q as given.  8: every row of q (not of q4) goes through the symmetric 8-bit  */
                         /* per-token fake quantiser as it is loaded -- IntegerQuantizer(8, True,          */
                         /* "per_token"), sqattn/fake_quant.py:33-35, 47-52, 114-125, the pass             */
                         /* sqattn/attn_replacer.py:361 runs on the query -- with the bits the pass        */
                         /* sq_fake_quant_prepass writes, so the closure need not write and re-read q8     */
} sq_prefill_params;

/* Bytes of device workspace sq_prefill_fwd needs (fp16 transposed V tiles). */
size_t sq_prefill_workspace_bytes(int64_t batch, int64_t num_kv_heads, int64_t kv_len, int64_t head_dim);

/*
 * out = softmax2(q~ k^T) v per the reference's blockwise algorithm, q~ = q * log2e/sqrt(D) rounded to q's
 * dtype.  q, k, v: bf16 or fp16 (same type), D == 128 (the host zero-pads smaller heads).  q4/k4 (may be NULL = alias of q/k) are the
 * operands used inside the 4-bit window range.  out: bf16/fp16/fp32, same shape as q.
 * lse (may be NULL): fp32 [B,Hq,Nq], base-2 log-sum-exp (attn_triton.py:210-213).
 */
int sq_prefill_fwd(const DLTensor* q, const DLTensor* k, const DLTensor* v, const DLTensor* q4,
                   const DLTensor* k4, DLTensor* out, DLTensor* lse, DLTensor* workspace,
                   const sq_prefill_params* params, void* stream);

/*
 * The same attention with Q.K^T as a real integer product (the second half of what sqattn/attn_replacer.py:334-365 and
 * the launch sqattn/attn_triton_mix_relative.py:439-475 only simulate: they fake-quantise query and key to 8 bits and
 * then multiply them as bf16).  k_codes: int8, laid out like k above, the per-token symmetric 8-bit codes of the
 * (centred) key; k_scale: fp32 [B, Hkv, ceil64(Nk)], their scales (sq_fake_quant_prepass_int8qk writes both).  q is the
 * raw query: the kernel forms each row's codes and scale as it loads the row (the quantiser of :361).  A score is
 * (sum of code products, exact in int32) * scale_k * (scale_q * log2e / sqrt(D)) in fp32; the reference's path differs
 * from it by the bf16 rounding of code * scale (fake_quant.py:85) and of the scaled query (attn_triton.py:251).
 * Everything else -- ranges, masking, fp16 P, v, out, lse, workspace, params (p_quant and q_quant must be 0, no 4-bit
 * operand set) -- as for sq_prefill_fwd.
 */
int sq_prefill_int8qk_fwd(const DLTensor* q, const DLTensor* k_codes, const DLTensor* k_scale, const DLTensor* v,
                          DLTensor* out, DLTensor* lse, DLTensor* workspace, const sq_prefill_params* p, void* stream);

/* ----------------------------------------------------------------------------------------- decode */
typedef struct sq_decode_params {
  int32_t layout;      /* SQ_LAYOUT_HND: q [B,Hq,1,D], caches [B,Hkv,L,D]; SQ_LAYOUT_NHD: [B,1,Hq,D], [B,L,Hkv,D] */
  int32_t p_quant;     /* SQ_P_NONE or SQ_P_E4M3_STATIC (attn_triton_decode.py:232-233)                        */
  int32_t num_splits;  /* KV splits per (batch, kv head); 0 = let the library choose.  With 0, seqlens and a batch of
                          2 .. 32 sequences the library deals its batch * splits workgroups to the sequences in
                          proportion to their lengths (a ragged batch then ends when its data ends, not when its
                          longest sequence does); a positive value gives every sequence exactly that many splits, and a
                          sequence's result then does not depend on its batch mates.  The workspace is the same.        */
  int32_t head_dim_og; /* head_dim before zero-padding to 128 (0 = the tensors' D)                             */
} sq_decode_params;

/* Number of splits the library would choose, and the workspace needed for a given number of splits. */
int32_t sq_decode_num_splits(int64_t batch, int64_t num_kv_heads, int64_t max_len);
size_t sq_decode_workspace_bytes(int64_t batch, int64_t num_q_heads, int64_t head_dim, int32_t num_splits);

/*
 * One query token per sequence against a KV cache; seqlens (int32 [B], may be NULL = L) gives the valid
 * prefix of each sequence.  The K-mean subtraction of attn_unified (attn_triton_decode.py:268-269) is
 * omitted: it cannot change a softmax.  out same shape as q; lse (may be NULL) fp32 [B,Hq,1].
 */
int sq_decode_fwd(const DLTensor* q, const DLTensor* kcache, const DLTensor* vcache, const DLTensor* seqlens,
                  DLTensor* out, DLTensor* lse, DLTensor* workspace, const sq_decode_params* params,
                  void* stream);

/*
 * sq_decode_fwd without a workspace argument and without any allocation.  No counterpart in the reference: it is for
 * callers that cannot allocate device memory -- code under HIP graph capture, tight serving loops, harnesses that
 * forbid hipMalloc.  The split-KV partial results go to a device array inside the library
 * (sq_decode_noalloc_scratch_bytes() = 8 MiB per GPU, held until the process ends) instead of a caller workspace; the
 * kernels and the results are those of sq_decode_fwd with the same num_splits, bit for bit.  A call whose partials
 * (batch * q heads * splits * 516 bytes) exceed the array returns SQ_EWORKSPACE.  q's device must be the current
 * device.  The call allocates and frees nothing.  The first use on a device looks the array's address up, which may
 * load the library's code object: call sq_decode_noalloc_init() once per device (with that device current) before
 * recording a HIP graph that contains sq_decode_fwd_noalloc; without it the first sq_decode_fwd_noalloc call does the
 * look-up itself.  All calls on one GPU share that GPU's array: calls that overlap in time on one GPU (different
 * streams, or threads) race; order them on one stream or with events.
 */
size_t sq_decode_noalloc_scratch_bytes(void);
int sq_decode_noalloc_init(void);
int sq_decode_fwd_noalloc(const DLTensor* q, const DLTensor* kcache, const DLTensor* vcache, const DLTensor* seqlens,
                          DLTensor* out, DLTensor* lse, const sq_decode_params* params, void* stream);

/*
 * The same decode over a selection of the cache (no reference counterpart; it consumes what sq_topk_select
 * emits): token_ids int32 [B * Hkv, k], row b * Hkv + kvh lists the cache rows the q heads of kv head kvh of
 * sequence b attend to, in any order; entries that are negative (the missing tail of a selection) or not below
 * the cache length are skipped.  seqlens (int32 [B], may be NULL = k) limits each sequence to a prefix of its
 * lists.  A head with no valid entry gets a zero output and lse = -inf.  Workspace as for sq_decode_fwd with
 * max_len = k.
 */
int sq_decode_selected_fwd(const DLTensor* q, const DLTensor* kcache, const DLTensor* vcache,
                           const DLTensor* token_ids, const DLTensor* seqlens, DLTensor* out, DLTensor* lse,
                           DLTensor* workspace, const sq_decode_params* params, void* stream);

/* ---------------------------------------------------------------------------------------- k-means */
size_t sq_kmeans_workspace_bytes(int64_t groups, int64_t num_tokens, int64_t num_centroids, int64_t dim);

/*
 * One Lloyd step: idx[g,n] = argmax_c <data[g,n], centroids[g,c]> (lowest index on ties); cnt = cluster
 * sizes; centroids[g,c] <- mean of its tokens (L2-normalised if `normalize`), stored only where cnt > 0.
 * data, centroids: bf16 [G,N,D] / [G,C,D], D == 128, C % 32 == 0 (kmeans.py:146); idx int32 [G,N];
 * cnt int32 [G,C].  Cluster sums are exact (fp64 accumulation), hence independent of summation order.
 */
int sq_kmeans_train(const DLTensor* data, DLTensor* centroids, DLTensor* idx, DLTensor* cnt,
                    DLTensor* workspace, int32_t normalize, void* stream);

/*
 * The same Lloyd step for a run of iterations over the same data (the loop of segment_k_means, cache_hub/kmeans.py:356-368),
 * with the exact cluster sums carried in the workspace from one call to the next.  After the first few iterations hardly
 * any token changes its cluster, and re-summing every row in every iteration reads the keys a second time for nothing.
 *   SQ_KMEANS_STATELESS      what sq_kmeans_train does; nothing is kept;
 *   SQ_KMEANS_KEEP_SUMS      the same step, and the clusters' exact fp64 sums and sizes stay in the workspace;
 *   SQ_KMEANS_APPLY_CHANGES  idx must hold the previous call's assignment and the workspace the sums that call left
 *                            (KEEP_SUMS or APPLY_CHANGES, same data, same shapes, nothing else run on the workspace's
 *                            tail in between -- sq_reverse_index, sq_index_add and sq_topk_select leave it alone):
 *                            the tokens whose cluster changes are subtracted from their old cluster's sum and added to
 *                            their new one's, and the centroids are formed from the sums.
 * The sums are exact, so every mode gives the same centroids, idx and cnt, bit for bit; APPLY_CHANGES costs the assign
 * pass plus work in proportion to the tokens that moved (slower than a re-sum only when most of them move).
 */
enum { SQ_KMEANS_STATELESS = 0, SQ_KMEANS_KEEP_SUMS = 1, SQ_KMEANS_APPLY_CHANGES = 2 };
int sq_kmeans_train_stateful(const DLTensor* data, DLTensor* centroids, DLTensor* idx, DLTensor* cnt,
                             DLTensor* workspace, int32_t normalize, int32_t state, void* stream);

/* clusters[g,c,0:cnt] = token ids with idx == c in ascending order (rest 0); cluster_size = counts. */
int sq_reverse_index(const DLTensor* idx, DLTensor* clusters, DLTensor* cluster_size, DLTensor* workspace,
                     void* stream);

/* out[g,c,:] = sum of value[g,n,:] over idx[g,n] == c, cast to value's dtype; out [G,C,D]. */
int sq_index_add(const DLTensor* value, const DLTensor* idx, DLTensor* out, DLTensor* workspace, void* stream);

/*
 * Centroid-scored token selection: per group g = b*Hkv + kvh, clusters ranked by
 * max_{h in group} <query[b,h], centroids[g,c]> (ties -> lower c); whole clusters taken in rank order
 * until k tokens are emitted; missing tail = -1.  query bf16 [B,Hq,D]; out int32 [G,k], rows contiguous and at least
 * k apart (it may be the leading columns of a wider list that sq_decode_selected_fwd reads).
 * With 1024 clusters the workgroups of a group share its score phase and hand over through one arrival word per
 * group in the workspace.  The workspace needs no initialisation (any contents are fine) and may be shared with the
 * other k-means entry points; calls that overlap in time must use different workspaces, as for every entry point
 * that takes one.
 */
int sq_topk_select(const DLTensor* query, const DLTensor* centroids, const DLTensor* clusters,
                   const DLTensor* cluster_size, DLTensor* out, DLTensor* workspace, int32_t num_kv_groups,
                   void* stream);

/* Bytes of scratch sq_fake_quant_prepass needs (partial column sums of the key, its mean). */
size_t sq_fake_quant_prepass_workspace_bytes(int64_t batch, int64_t num_kv_heads, int64_t num_tokens);

/*
 * Operand pre-pass of the plugin closure for the integer quantiser types, fused and without expanding the kv
 * heads: key_c = key - mean over tokens (mean = dtype(float(exact sum / N)), subtraction rounded to the tensor
 * dtype); q8/q4 = IntegerQuantizer(8|4, True, "per_token").fake_quant_tensor(query); k8/k4 the same of key_c;
 * v8 = IntegerQuantizer(8, True, "per_channel").fake_quant_tensor(value), whose scale is per (token, channel)
 * over batch and heads as in the reference (range over dims 0 and 1 of [B,H,N,D]).  q4 and k4 may both be null; q8 may
 * be null as well (with q4 and k4): the query is then left alone, for a caller that sets sq_prefill_params.q_quant = 8.
 * query/q8/q4 [B,N,Hq,128] and key/value/k8/k4/v8 [B,N,Hkv,128] for SQ_LAYOUT_NHD ([B,H,N,128] for
 * SQ_LAYOUT_HND), bf16 or fp16, all of one dtype; any strides with a contiguous last dimension and 16-byte
 * aligned rows.  Outputs are bit-identical to the formulas evaluated in fp32 on the host.
 */
int sq_fake_quant_prepass(const DLTensor* query, const DLTensor* key, const DLTensor* value, DLTensor* q8,
                          DLTensor* q4, DLTensor* k8, DLTensor* k4, DLTensor* v8, DLTensor* workspace,
                          int32_t layout, void* stream);

/*
 * The same pre-pass with the closure's other quantiser types (sqattn/attn_replacer.py:340-358): qk_qtype selects the
 * 8-bit quantiser of query and centred key (SQ_QTYPE_INT: IntegerQuantizer(8, True, "per_token"); SQ_QTYPE_E4M3 /
 * SQ_QTYPE_E5M2: FloatQuantizer(..., True, "per_token"), the float simulation of sqattn/fake_quant.py:151-204 with the
 * scale absmax / 448 resp. / 57344), v_qtype the one of value ("per_channel").  The 4-bit outputs are always the
 * integer quantiser's, as in the reference.  Outputs equal the formulas evaluated in fp32 on the host, except that the
 * float simulation's exponent is read from the exponent field instead of floor(log2(.)): the two differ only where a
 * library's fp32 log2 rounds a value just below a power of two up to the integer.
 */
enum { SQ_QTYPE_INT = 0, SQ_QTYPE_E4M3 = 1, SQ_QTYPE_E5M2 = 2 };
/*
 * The pre-pass for a real integer Q.K^T (sq_prefill_int8qk_fwd): key centring as above, then instead of the fake-
 * quantised key its two factors -- k_codes int8 [like key] = clamp(round(key_c / scale), -128, 127), the codes
 * IntegerQuantizer(8, True, "per_token") multiplies by its scale (sqattn/fake_quant.py:114-125), and k_scale fp32
 * [B, Hkv, S >= N] = that scale per token (entries past N are left alone) -- and v8 as above.  The query is not touched:
 * the attention kernel forms its codes and scale from the rows it loads.
 */
int sq_fake_quant_prepass_int8qk(const DLTensor* query, const DLTensor* key, const DLTensor* value, DLTensor* k_codes,
                                 DLTensor* k_scale, DLTensor* v8, DLTensor* workspace, int32_t layout, void* stream);

int sq_fake_quant_prepass_typed(const DLTensor* query, const DLTensor* key, const DLTensor* value, DLTensor* q8,
                                DLTensor* q4, DLTensor* k8, DLTensor* k4, DLTensor* v8, DLTensor* workspace,
                                int32_t layout, int32_t qk_qtype, int32_t v_qtype, void* stream);

/*
 * Prefill side of the KV cache (cache_hub/flash_attn_cache.py:153-232): rows [valid_start, T) of one sequence's
 * key_states / value_states [1, T, Hkv, D] go to rows [0, T - valid_start) of sequence `batch_index` of
 * key_cache / value_cache [B, max_length, Hkv, D] (the per-layer buffers of :60-81, contiguous).  bf16 or fp16,
 * states and caches of one dtype; the states may be strided views with contiguous D and 16-byte aligned heads.
 * T > max_length is an error as in the reference (:170-172), so is a batch of more than one sequence (:166-169).
 */
int sq_kv_cache_store(const DLTensor* key_states, const DLTensor* value_states, DLTensor* key_cache,
                      DLTensor* value_cache, int32_t batch_index, int64_t valid_start, void* stream);

/*
 * Decode side of the KV cache (cache_hub/flash_attn_cache.py:239-256): for every sequence b the new token's
 * key_states[b, 0] / value_states[b, 0] ([B, 1, Hkv, D]) are written to row valid_length[b] of the caches.
 * valid_length is int32 [B] on the device and is read there, so the call needs no host synchronisation.
 * attend_length (int32 [B], may be null) receives valid_length[b] + 1, the number of cached tokens the attention
 * of this decode step covers (what sq_decode_fwd takes as seqlens).  advance != 0 also stores that value to
 * valid_length: the reference advances the length once per step, after the last layer (:253-255).  A sequence
 * whose cache is full (valid_length[b] == max_length) is left unchanged.
 */
int sq_kv_cache_append(const DLTensor* key_states, const DLTensor* value_states, DLTensor* key_cache,
                       DLTensor* value_cache, DLTensor* valid_length, DLTensor* attend_length, int32_t advance,
                       void* stream);

/*
 * A copy of a layer's KV cache with each kv head's rows permuted (no counterpart in the reference, whose k-means code
 * in cache_hub/kmeans.py has no consumer): key_out[b, p, h] = key_cache[b, order[b * Hkv + h][p], h], the same for
 * value.  With `order` = the tokens of every head listed cluster by cluster (the order triton_reverse_index stores
 * them in, cache_hub/kmeans.py:199-262), a selection of whole clusters becomes runs of neighbouring rows of the copy,
 * and sq_decode_selected_fwd on the copy, with positions in place of token ids, reads them as such.
 * key_cache / value_cache [B, L, Hkv, D], key_out / value_out [B, n, Hkv, D], all contiguous, one 16-bit dtype;
 * order int32 [B * Hkv, n]; entries outside [0, L) give zero rows.
 */
int sq_kv_cache_reorder(const DLTensor* key_cache, const DLTensor* value_cache, const DLTensor* order, DLTensor* key_out,
                        DLTensor* value_out, void* stream);

/*
 * RMS normalisation of the rows of x [R, dim] (model_hub/utils.py:15-19): out = (x * rsqrt(mean(x^2) + epsilon))
 * * weight, with the reference's operator sequence on 16-bit tensors -- square, mean (fp32 accumulation), + epsilon,
 * rsqrt, x * r, * weight, each result rounded to the tensor dtype.  x, out [R, dim] (row strides free, 16-byte
 * aligned rows), weight [dim]; bf16 or fp16, all of one dtype; dim a multiple of 8, at most 8192.
 */
int sq_rmsnorm(const DLTensor* x, const DLTensor* weight, DLTensor* out, float epsilon, void* stream);

/*
 * out = x2 * (x1 * sigmoid(x1)) for x = [x1 | x2] [R, 2 I] -> out [R, I] (model_hub/utils.py:4-13), the three tensor
 * operators each rounded to the tensor dtype.  bf16 or fp16; I a multiple of 8.
 */
int sq_silu_and_mul(const DLTensor* x, DLTensor* out, void* stream);

/*
 * out = x . weight^T (+ bias) (+ residual) for 1 to 8 rows of x: the projections of a decode step, which the
 * reference runs as tensor-library matmuls on a [batch, 1, hidden] activation (model_hub/qwen.py:302-326, lm head
 * :293-300).  x [M, K], weight [N, K] (the layout of a Linear layer's weight), bias [N] or NULL, residual [M, N] or
 * NULL, out [M, N]; bf16 or fp16, all of one dtype; K a multiple of 8; rows of x and weight 16-byte aligned (row
 * strides free), last dimensions contiguous.  fp32 accumulation; the sum plus the bias is rounded once to the tensor
 * dtype, and with a residual that rounded value plus the residual is rounded again (the two tensor operators of
 * `residual + linear(x)`).  out may be the residual tensor itself; it must not overlap x.  M > 8 returns
 * SQ_EUNSUPPORTED: such a product is a GEMM and belongs to the BLAS library.
 */
int sq_linear_rows(const DLTensor* x, const DLTensor* weight, const DLTensor* bias, const DLTensor* residual,
                   DLTensor* out, void* stream);

/*
 * out = silu_and_mul(x . weight^T (+ bias)) for 1 to 8 rows of x: the first projection of the MLP and the activation
 * behind it in one pass (model_hub/qwen.py:320-324 on a decode step's activation).  weight [2 I, K] = [gate | up] as
 * the reference stores gate_up_proj, bias [2 I] or NULL, out [M, I] = up * (gate * sigmoid(gate)) with the values
 * sq_linear_rows followed by sq_silu_and_mul give (the projection rounded to the tensor dtype, then the three
 * rounded operators of the activation).  Other requirements as for sq_linear_rows.
 */
int sq_linear_rows_silu_and_mul(const DLTensor* x, const DLTensor* weight, const DLTensor* bias, DLTensor* out, void* stream);

/*
 * out = x . weight^T (+ bias) with the rotary embedding applied to the first rope_features output features, for 1 to 8
 * rows of x: the fused q/k/v projection of a decode step and the rotation of its q and k parts in one pass
 * (model_hub/qwen.py:302-312 wqkv, :352-379 apply_rotary_pos_emb / position_embedd).  The first rope_features
 * features are whole heads of head_dim; feature i < head_dim / 2 of a head is rotated with feature i + head_dim / 2 by
 * row position_ids[m] of cos_sin_cache (fp32 [max_position, head_dim], cos | sin), exactly as sq_rope rotates the
 * rounded output of sq_linear_rows; the remaining features (v) are the plain projection.  position_ids: int32 or
 * int64, one entry per row of x.  Other requirements as for sq_linear_rows.
 *
 * With key_cache / value_cache ([M, L, Hkv, head_dim], contiguous) and valid_length (int32 [M]) the output is
 * [q | k | v] with k and v of Hkv * head_dim features each, and the rotated k and the v of row m are also written to
 * row valid_length[m] of the caches -- the copies of sq_kv_cache_append (cache_hub/flash_attn_cache.py:248-252) --
 * and attend_length (int32 [M], may be NULL) receives valid_length + 1.  valid_length itself is not changed: the
 * reference advances it once per step after the last layer (:253-255), which stays with sq_kv_cache_append
 * (advance != 0).  All four NULL: no cache.
 */
int sq_linear_rows_rope(const DLTensor* x, const DLTensor* weight, const DLTensor* bias, const DLTensor* position_ids,
                        const DLTensor* cos_sin_cache, int32_t head_dim, int32_t rope_features, DLTensor* out,
                        DLTensor* key_cache, DLTensor* value_cache, const DLTensor* valid_length, DLTensor* attend_length,
                        void* stream);

/*
 * The three projections above applied to rmsnorm(x, norm_weight, epsilon) instead of x, in one pass: the layer norm in
 * front of wqkv, of the MLP and of the lm head on a decode step (model_hub/qwen.py:345-350 called from
 * model_hub/LLM.py:92-95, 110-114, 161-163).  norm_weight [K] of x's dtype, contiguous and 16-byte aligned.  The
 * normalised rows have the bits sq_rmsnorm writes (same operator sequence, same summation order), so each call returns
 * what sq_rmsnorm followed by the plain form returns.  K at most 8192 (sq_rmsnorm's limit) for one or two rows of x,
 * 5120 for three or four, 2048 for five to eight: a normalised row has to fit the staging buffer (SQ_EUNSUPPORTED beyond).
 * Other arguments and requirements as for the plain forms.
 */
int sq_rmsnorm_linear_rows(const DLTensor* x, const DLTensor* norm_weight, float epsilon, const DLTensor* weight, const DLTensor* bias,
                           const DLTensor* residual, DLTensor* out, void* stream);
int sq_rmsnorm_linear_rows_silu_and_mul(const DLTensor* x, const DLTensor* norm_weight, float epsilon, const DLTensor* weight,
                                        const DLTensor* bias, DLTensor* out, void* stream);
int sq_rmsnorm_linear_rows_rope(const DLTensor* x, const DLTensor* norm_weight, float epsilon, const DLTensor* weight, const DLTensor* bias,
                                const DLTensor* position_ids, const DLTensor* cos_sin_cache, int32_t head_dim, int32_t rope_features,
                                DLTensor* out, DLTensor* key_cache, DLTensor* value_cache, const DLTensor* valid_length,
                                DLTensor* attend_length, void* stream);

/*
 * Rotary position embedding of query [T, Hq * head_dim] and key [T, Hkv * head_dim] (T = batch * seq_len tokens)
 * with the rows position_ids[t] of cos_sin_cache, fp32 [max_position, head_dim] holding cos in the first half of a
 * row and sin in the second (model_hub/utils.py:21-106): per head, out1 = x1 cos - x2 sin, out2 = x1 sin + x2 cos
 * over the two halves, formed in fp32 and rounded once to the tensor dtype.  The outputs have the inputs' shape
 * and may be the inputs themselves.  position_ids int32 or int64, T entries, each in [0, max_position) (the
 * caller's responsibility; the kernel clamps).
 */
int sq_rope(const DLTensor* query, const DLTensor* key, DLTensor* query_out, DLTensor* key_out,
            const DLTensor* position_ids, const DLTensor* cos_sin_cache, int32_t head_dim, void* stream);

/*
 * Calibration histograms of the window search, straight from Q and K: for every (batch, query head) the causal
 * attention probabilities p[i, j] = softmax_j(softmax_scale * q_i . k_j) are added, weighted, into hist[b, h, bin].
 * Replaces the reference's dense attention map [Hq, N, N] (sqattn/attn_replacer.py:253-278, stored as
 * `current_attention`, model_hub/qwen.py:38-41) and the index-tensor + bincount reductions over it:
 *   SQ_HIST_ABSOLUTE       bin = i - j,                         weight p * (i - j); distances >= bins are dropped,
 *                          keys j < sink excluded   (sqattn/window_search.py:20-48 with sink = 0, :283-321)
 *   SQ_HIST_RELATIVE       bin = floor(bins * (i - j) / max(i, 1)), weight p * (i - j); sink must be 0   (:51-87)
 *   SQ_HIST_RELATIVE_SINK  keys j < sink excluded, rows i <= sink go to bin 0, otherwise
 *                          bin = floor(bins * (i - j) / max(i - sink, 1)); weight p * (bins * rel + 1)   (:244-280)
 * Bins are clamped to [0, bins - 1] and formed with the reference's fp32 operator sequence.  q [B, Hq, N, 128] and
 * k [B, Hkv, N, 128] (views with any strides, contiguous last dimension, 16-byte aligned rows; Hq a multiple of Hkv),
 * bf16 or fp16.  hist float64 [B, Hq, bins], contiguous; the call ADDS to it (clear it before the first sample,
 * keep it across samples as the reference sums its per-sample histograms, window_search.py:158-159).  The relative
 * kinds take at most 8192 bins.  Probabilities are formed in fp32 from the 16-bit inputs (the reference rounds the
 * map itself to the model dtype).
 */
enum { SQ_HIST_ABSOLUTE = 0, SQ_HIST_RELATIVE = 1, SQ_HIST_RELATIVE_SINK = 2 };
typedef struct sq_histogram_params {
  int32_t kind;         /* SQ_HIST_*                                                        */
  int32_t bins;         /* max_len (absolute) or num_bins (relative)                        */
  int32_t sink;         /* sink_len: leading keys left out of the histogram                 */
  float softmax_scale;  /* 1/sqrt(head_dim before padding) (attn_replacer.py:260)            */
} sq_histogram_params;
int sq_attention_histogram(const DLTensor* q, const DLTensor* k, DLTensor* hist, const sq_histogram_params* p, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* SQATTN_H_ */
