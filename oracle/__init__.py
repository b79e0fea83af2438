"""CPU oracle for the SQAttn attention hot path -- TEST INFRASTRUCTURE ONLY.

Everything in this package is a CPU restatement (torch-CPU / numpy) of the
algorithms in the reference's `sqattn/attn_triton.py`, `sqattn/attn_triton_decode.py`,
`sqattn/attn_triton_mix_relative.py`, `sqattn/attn_triton_mix_bad.py`,
`sqattn/fake_quant.py`, `sqattn/attn_replacer.py`, `cache_hub/kmeans.py` and
`cache_hub/flash_attn_cache.py`, `model_hub/utils.py` and `sqattn/window_search.py`.
It exists to check the HIP kernels, never to serve a request: only `tests/`,
`__graft_entry__.smoke()` and the `cpu_baseline` leg of `bench.py` import it.
The product package (`longcontext_sqattn_paddle_amd`) must not import it and
raises when its HIP library is missing.

How each function is pinned (none could be checked against a running copy of
the reference: PaddlePaddle and an NVIDIA GPU are absent, and the reference
ships no golden vectors for this path):

* `attention.exact_attention`      -- closed form softmax(QK^T/sqrt(D))V in fp64; cross-checked
                                      against torch's own CPU `scaled_dot_product_attention`.
* `attention.prefill_blockwise`    -- equals the closed form when P is not quantised; independent of
                                      the row-tile size; brute-force scalar loop on tiny inputs for FP8-P;
                                      window ranges against an explicit [N,N] mask built from the four ranges.
* `attention.decode_*`             -- closed form over the valid prefix; split/combine identity.
* `fake_quant.*`                   -- closed forms, idempotence, absmax -> +-qmax, known answers of the
                                      float simulation worked out by hand from `fake_quant.py:151-204`.
* `kmeans.*`                       -- brute-force argmax, partition invariants, bincount identities.
* `kv_cache.*`                     -- index arithmetic only: element-by-element loops on tiny inputs, untouched-row
                                      and concatenation invariants.
* `layer.*`                        -- torch's own 16-bit CPU operators evaluating the reference's expressions, fp64
                                      closed forms, rotation invariants (parity unpinned: Paddle's rounding points).
* `model.CpuDecoder`               -- assembled from the pieces above and torch's CPU `linear`; no arithmetic of its own.
* `window_search.*`                -- dense float64 restatement of the calibration histograms and the window search:
                                      element-by-element loops on tiny maps, closed forms (uniform rows, one
                                      sub-diagonal, a sink column), conservation sums, known answers of the search
                                      (parity unpinned where the reference rounds the map to 16 bits first).
* `kmeans.topk_select`             -- build-defined (the reference has no top-k code): parity unpinned
                                      by the reference, pinned by brute force only.
"""
