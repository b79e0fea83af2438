"""GPU parity: split-KV decode kernel (through the C ABI) against the CPU oracle."""
import math

import pytest
import torch

from oracle import attention as A
from oracle import inputs

pytestmark = pytest.mark.gpu


def _run(q, kc, vc, lens, layout, **kw):
    from longcontext_sqattn_paddle_amd.sqattn.attn_triton_decode import attn_decode

    dev = torch.device("cuda:0")
    sl = None if lens is None else torch.as_tensor(lens, dtype=torch.int32, device=dev)
    res = attn_decode(q.to(dev), kc.to(dev), vc.to(dev), layout, seqlens=sl, **kw)
    torch.cuda.synchronize()
    return res


def _to_hnd(q, kc, vc):
    return q.permute(0, 2, 1, 3).contiguous(), kc.permute(0, 2, 1, 3).contiguous(), vc.permute(0, 2, 1, 3).contiguous()


@pytest.mark.parametrize("layout", ["NHD", "HND"])
@pytest.mark.parametrize("B,Hq,Hkv,L", [(1, 28, 4, 3000), (3, 28, 4, 1500), (2, 8, 8, 777), (1, 40, 2, 515)])
def test_decode_matches_closed_form(layout, B, Hq, Hkv, L):
    print(f"case decode layout={layout} B={B} Hq={Hq} Hkv={Hkv} L={L}", flush=True)
    q, kc, vc, lens = inputs.decode_inputs(B, Hq, Hkv, L, 128, seed=30 + B)
    lens = [int(x) for x in lens]
    qh, kh, vh = _to_hnd(q, kc, vc)
    ref, lse_ref = A.exact_attention(A.fold_scale(qh, 128), kh, vh, causal=False, kv_lens=lens, score_scale=math.log(2.0))
    args = (q, kc, vc) if layout == "NHD" else (qh, kh, vh)
    out, lse = _run(*args, lens, layout, output_dtype=torch.float32, return_lse=True)
    out = out.cpu()
    out = out[:, 0] if layout == "NHD" else out[:, :, 0]
    rms = float(ref.pow(2).mean().sqrt())
    err = float((out.double() - ref[:, :, 0]).abs().max())
    # stated tolerance: fp32 accumulation + v_exp_f32; inputs are consumed exactly
    assert err < 2e-4 * rms + 1e-6, (err, rms)
    assert torch.allclose(lse.cpu()[:, :, 0].double(), lse_ref[:, :, 0], atol=2e-4)


def test_decode_split_invariance_and_bf16_out():
    q, kc, vc, lens = inputs.decode_inputs(2, 28, 4, 4096, 128, seed=41)
    lens = [4096, 1234]
    outs = [
        _run(q, kc, vc, lens, "NHD", output_dtype=torch.float32, num_splits=s).cpu() for s in (1, 3, 16, 64)
    ]
    for o in outs[1:]:
        assert float((o - outs[0]).abs().max()) < 1e-5   # any partition gives the same result up to fp32 rounding
    ob = _run(q, kc, vc, lens, "NHD", output_dtype=torch.bfloat16).cpu()
    assert torch.equal(ob, outs[0].to(torch.bfloat16)) or float((ob.float() - outs[0]).abs().max()) < 2 ** -8


@pytest.mark.parametrize("lens", [[8192, 17, 3000, 1], [5, 8192], [8192, 0, 4000], [100] * 7 + [8192]])
def test_decode_workgroups_dealt_by_length(lens):
    """With num_splits left to the library a ragged batch's workgroups go to the sequences in proportion to their
    lengths (one each at least): very uneven lengths, a one-token and an empty sequence, against the closed form, and
    against the same call with a named split count (every sequence the same number of splits)."""
    print(f"case decode by length lens={lens}", flush=True)
    B, L = len(lens), 8192
    q, kc, vc, _ = inputs.decode_inputs(B, 28, 4, L, 128, seed=77)
    qh, kh, vh = _to_hnd(q, kc, vc)
    ref, lse_ref = A.exact_attention(A.fold_scale(qh, 128), kh, vh, causal=False, kv_lens=[max(x, 1) for x in lens], score_scale=math.log(2.0))
    out, lse = _run(q, kc, vc, lens, "NHD", output_dtype=torch.float32, return_lse=True)
    named, lse_named = _run(q, kc, vc, lens, "NHD", output_dtype=torch.float32, return_lse=True, num_splits=8)
    out, named, lse, lse_named = out.cpu()[:, 0], named.cpu()[:, 0], lse.cpu()[:, :, 0], lse_named.cpu()[:, :, 0]
    rms = float(ref.pow(2).mean().sqrt())
    for b, n in enumerate(lens):
        if n == 0:   # nothing to attend to: zeros and -inf, from both partitions
            assert float(out[b].abs().max()) == 0.0 and float(named[b].abs().max()) == 0.0
            assert bool(torch.isinf(lse[b]).all()) and bool(torch.isinf(lse_named[b]).all())
            continue
        assert float((out[b].double() - ref[b, :, 0]).abs().max()) < 2e-4 * rms + 1e-6, b
        assert float((out[b] - named[b]).abs().max()) < 1e-5, b
        assert torch.allclose(lse[b].double(), lse_ref[b, :, 0], atol=2e-4)


def test_decode_by_length_replayed_from_a_graph_with_changing_lengths():
    """The length-proportional dealing is computed on the device from `seqlens`, so a captured launch follows the
    lengths it finds at replay time: one graph, four sets of lengths written between the replays (with eager work in
    between), each replay bit-identical to an eager call with those lengths."""
    from longcontext_sqattn_paddle_amd.sqattn.attn_triton_decode import DecodePlan

    dev = torch.device("cuda:0")
    B, L = 3, 6000
    q, kc, vc, _ = inputs.decode_inputs(B, 28, 4, L, 128, seed=91)
    q, kc, vc = q.to(dev), kc.to(dev), vc.to(dev)
    lens = torch.tensor([L, 100, 2500], dtype=torch.int32, device=dev)
    plan = DecodePlan(q, kc, vc, "NHD", torch.float32, seqlens=lens)
    plan.run()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        plan.run()
    for case in ([L, 100, 2500], [1, L, 1], [3000, 3000, 3000], [17, 5999, 0]):
        lens.copy_(torch.tensor(case, dtype=torch.int32))
        graph.replay()
        got = plan.out.clone()
        scratch = torch.randn(1 << 20, device=dev).sum()          # eager work between the replays
        torch.cuda.synchronize()
        eager = _run(q, kc, vc, case, "NHD", output_dtype=torch.float32)
        assert torch.equal(got.view(torch.int32), eager.view(torch.int32)), case
        assert bool(torch.isfinite(scratch))


def test_decode_no_seqlens_fp16_and_small_head_dim():
    g = torch.Generator().manual_seed(5)
    q = torch.randn(2, 8, 1, 64, generator=g).half()
    k = torch.randn(2, 2, 300, 64, generator=g).half()
    v = torch.randn(2, 2, 300, 64, generator=g).half()
    out = _run(q, k, v, None, "HND", output_dtype=torch.float32).cpu()
    ref, _ = A.exact_attention(A.fold_scale(q, 64), k, v, causal=False, score_scale=math.log(2.0))
    assert out.shape == (2, 8, 1, 64)
    assert float((out.double() - ref).abs().max()) < 2e-4


def test_decode_fp8_p_matches_blockwise_oracle():
    q, kc, vc, _ = inputs.decode_inputs(1, 28, 4, 2048, 128, seed=43)
    qh, kh, vh = _to_hnd(q, kc, vc)
    ref, _ = A.decode_blockwise(qh, kh, vh, None, p_quant=A.P_STATIC448)
    exact, _ = A.exact_attention(qh, kh, vh, causal=False)
    out = _run(q, kc, vc, None, "NHD", output_dtype=torch.float32, is_P_fp8_quant=True, num_splits=1).cpu()[:, 0]
    # Both quantise P on an e4m3 grid, but the running max (hence the grid points hit) depends on the
    # order tokens are visited: 16-token tiles over 4 waves here, 64-token blocks in the reference.
    # So the comparison is statistical: same error level against the exact result, high mutual cosine.
    cos = torch.nn.functional.cosine_similarity(out.flatten().double(), ref.flatten().double(), dim=0)
    assert float(cos) > 0.999
    e_k = float((out.double() - exact[:, :, 0]).abs().mean())
    e_o = float((ref.double() - exact[:, :, 0]).abs().mean())
    assert 0.5 < e_k / e_o < 2.0


def test_decode_argument_errors():
    from longcontext_sqattn_paddle_amd.sqattn.attn_triton_decode import attn_decode

    dev = torch.device("cuda:0")
    q = torch.zeros(1, 4, 1, 128, dtype=torch.bfloat16, device=dev)
    k = torch.zeros(1, 2, 64, 128, dtype=torch.bfloat16, device=dev)
    with pytest.raises(ValueError):
        attn_decode(q, k, k, "XYZ")
    with pytest.raises(ValueError):
        attn_decode(torch.zeros(1, 4, 1, 256, dtype=torch.bfloat16, device=dev), k, k)
    with pytest.raises(AssertionError):
        attn_decode(q, k, k[:, :, :32])
    with pytest.raises(ValueError):
        attn_decode(q.float(), k.float(), k.float())


def _selected(q, kc, vc, ids, layout, **kw):
    from longcontext_sqattn_paddle_amd.sqattn.attn_triton_decode import attn_decode_selected

    dev = torch.device("cuda:0")
    res = attn_decode_selected(q.to(dev), kc.to(dev), vc.to(dev), ids.to(dev), layout, **kw)
    torch.cuda.synchronize()
    return res


@pytest.mark.parametrize("layout", ["NHD", "HND"])
@pytest.mark.parametrize("B,Hq,Hkv,L,n", [(1, 28, 4, 5000, 1000), (2, 28, 4, 3000, 333), (1, 8, 8, 777, 16), (2, 6, 2, 900, 2100)])
def test_decode_over_selected_tokens_matches_closed_form(layout, B, Hq, Hkv, L, n):
    """Attention over per-(sequence, kv head) lists of cache rows: random order, duplicates, a tail of -1 and one
    head whose list is empty."""
    print(f"case decode selected layout={layout} B={B} Hq={Hq} Hkv={Hkv} L={L} n={n}", flush=True)
    q, kc, vc, _ = inputs.decode_inputs(B, Hq, Hkv, L, 128, seed=60 + B)
    g = torch.Generator().manual_seed(n)
    ids = torch.randint(0, L, (B * Hkv, n), generator=g, dtype=torch.int32)
    ids[1, n // 2:] = -1                       # missing tail
    ids[B * Hkv - 1, :] = -1                   # a head with nothing selected
    ids[0, 0] = L + 5                          # beyond the cache: skipped as well
    qh, kh, vh = _to_hnd(q, kc, vc)
    ref, lse_ref = A.decode_selected_exact(A.fold_scale(qh, 128), kh, vh, ids, score_scale=math.log(2.0))
    args = (q, kc, vc) if layout == "NHD" else (qh, kh, vh)
    out, lse = _selected(*args, ids, layout, output_dtype=torch.float32, return_lse=True)
    out = out.cpu()
    out = out[:, 0] if layout == "NHD" else out[:, :, 0]
    rms = float(ref.pow(2).mean().sqrt())
    err = float((out.double() - ref[:, :, 0]).abs().max())
    assert err <= 2e-4 * rms, f"max abs err {err} vs rms {rms}"
    empty = lse_ref[:, :, 0] == float("-inf")
    assert bool((lse.cpu()[:, :, 0][empty] == float("-inf")).all()) and bool((out[empty] == 0).all())
    assert torch.allclose(lse.cpu()[:, :, 0][~empty].double(), lse_ref[:, :, 0][~empty], atol=2e-4)


def test_selected_decode_with_all_tokens_equals_dense_decode():
    """The identity list reproduces the dense kernel bit for bit (same tiles, same order)."""
    print("case decode selected identity", flush=True)
    B, Hq, Hkv, L = 2, 28, 4, 2048
    q, kc, vc, _ = inputs.decode_inputs(B, Hq, Hkv, L, 128, seed=71)
    ids = torch.arange(L, dtype=torch.int32).repeat(B * Hkv, 1)
    dense = _run(q, kc, vc, None, "NHD", output_dtype=torch.float32)
    sel = _selected(q, kc, vc, ids, "NHD", output_dtype=torch.float32)
    assert torch.equal(dense, sel)


def test_kmeans_topk_then_selected_decode():
    """The retrieval pipeline end to end: cluster the keys, pick the tokens of the best-scoring clusters for a query,
    attend over them; checked against the closed form over the same ids."""
    from longcontext_sqattn_paddle_amd.cache_hub.kmeans import segment_k_means, topk_select

    print("case kmeans -> topk -> selected decode", flush=True)
    dev = torch.device("cuda:0")
    B, Hq, Hkv, L, C, k = 1, 28, 4, 8192, 128, 1024
    q, kc, vc, _ = inputs.decode_inputs(B, Hq, Hkv, L, 128, seed=72)
    key = kc.permute(0, 2, 1, 3).reshape(B * Hkv, L, 128).contiguous().to(dev)
    val = vc.permute(0, 2, 1, 3).reshape(B * Hkv, L, 128).contiguous().to(dev)
    centroids, _, clusters, cluster_size = segment_k_means(key, val, C, num_iters=3)
    ids = topk_select(q[:, 0].to(dev), centroids, clusters, cluster_size, k, Hq // Hkv)
    torch.cuda.synchronize()
    assert ids.shape == (B * Hkv, k) and int(ids.min()) >= 0 and int(ids.max()) < L
    out = _selected(q, kc, vc, ids.cpu(), "NHD", output_dtype=torch.float32)
    qh, kh, vh = _to_hnd(q, kc, vc)
    ref, _ = A.decode_selected_exact(A.fold_scale(qh, 128), kh, vh, ids.cpu(), score_scale=math.log(2.0))
    err = float((out.cpu()[:, 0].double() - ref[:, :, 0]).abs().max())
    assert err <= 2e-4 * float(ref.pow(2).mean().sqrt())


def test_cluster_ordered_cache_gives_the_same_attention_from_neighbouring_rows():
    """A copy of the cache in cluster order (`sq_kv_cache_reorder`): the copy holds exactly the rows the order names
    (checked row by row on the host), the positions table sends the selection to the same tokens, and the attention
    over positions of the copy equals, bit for bit, the attention over token ids of the original (same rows, same
    order).  The selected positions form runs: one run per selected cluster."""
    from longcontext_sqattn_paddle_amd.cache_hub.kmeans import cluster_order, reorder_cache, segment_k_means, topk_select

    print("case cluster-ordered cache", flush=True)
    dev = torch.device("cuda:0")
    B, Hq, Hkv, L, C, k = 2, 8, 2, 4096, 64, 700
    q, kc, vc, _ = inputs.decode_inputs(B, Hq, Hkv, L, 128, seed=73)
    key = kc.permute(0, 2, 1, 3).reshape(B * Hkv, L, 128).contiguous().to(dev)
    val = vc.permute(0, 2, 1, 3).reshape(B * Hkv, L, 128).contiguous().to(dev)
    centroids, _, clusters, cluster_size = segment_k_means(key, val, C, num_iters=3)
    order, positions = cluster_order(clusters, cluster_size)
    kg, vg = reorder_cache(kc.to(dev), vc.to(dev), order)
    torch.cuda.synchronize()
    G = B * Hkv
    assert order.shape == (G, L) and kg.shape == (B, L, Hkv, 128)
    o = order.cpu().long()
    for g in range(G):
        assert torch.equal(torch.sort(o[g]).values, torch.arange(L))          # a permutation of the head's tokens
        b, h = divmod(g, Hkv)
        assert torch.equal(kg[b, :, h].cpu().view(torch.int16), kc[b, o[g], h].contiguous().view(torch.int16))
        assert torch.equal(vg[b, :, h].cpu().view(torch.int16), vc[b, o[g], h].contiguous().view(torch.int16))
    # positions[g, c, j] is where clusters[g, c, j] went
    cl, sz, pos = clusters.cpu().long(), cluster_size.cpu().long(), positions.cpu().long()
    for g in range(G):
        for c in (0, 17, C - 1):
            n = int(sz[g, c])
            assert torch.equal(o[g, pos[g, c, :n]], cl[g, c, :n])
    qd = q[:, 0].to(dev)
    ids = topk_select(qd, centroids, clusters, cluster_size, k, Hq // Hkv)
    rows = topk_select(qd, centroids, positions, cluster_size, k, Hq // Hkv)
    torch.cuda.synchronize()
    assert torch.equal(torch.gather(o, 1, rows.cpu().long()), ids.cpu().long())
    steps = (rows.cpu()[:, 1:] - rows.cpu()[:, :-1]) != 1
    assert int(steps.sum(dim=1).max()) < C                                    # runs, at most one break per cluster
    a = _selected(q, kc, vc, ids.cpu(), "NHD", output_dtype=torch.float32)
    b_ = _selected(q, kg.cpu(), vg.cpu(), rows.cpu(), "NHD", output_dtype=torch.float32)
    assert torch.equal(a, b_)
    # ids outside the cache give zero rows; shapes are checked
    bad = order.clone()
    bad[0, 5] = -1
    bad[1, 6] = L
    kz, vz = reorder_cache(kc.to(dev), vc.to(dev), bad)
    assert float(kz[0, 5, 0].abs().max()) == 0.0 and float(vz[0, 6, 1].abs().max()) == 0.0
    assert torch.equal(kz[0, 5, 1], kg[0, 5, 1])                              # the other head of that row is untouched
    with pytest.raises(AssertionError):
        reorder_cache(kc.to(dev), vc.to(dev), order[:3])


def test_selected_decode_argument_errors():
    from longcontext_sqattn_paddle_amd.sqattn.attn_triton_decode import attn_decode_selected

    dev = torch.device("cuda:0")
    q = torch.zeros(1, 1, 8, 128, dtype=torch.bfloat16, device=dev)
    kc = torch.zeros(1, 64, 2, 128, dtype=torch.bfloat16, device=dev)
    with pytest.raises(AssertionError, match="token_ids"):
        attn_decode_selected(q, kc, kc, torch.zeros(3, 8, dtype=torch.int32, device=dev), "NHD")
    with pytest.raises(AssertionError, match="token_ids"):
        attn_decode_selected(q, kc, kc, torch.zeros(2, 8, dtype=torch.int64, device=dev), "NHD")


@pytest.mark.parametrize("B,L", [(1, 1048576), (8, 131072)])
def test_full_size_decode_against_closed_form(B, L):
    """The benchmark shapes (1M-token cache at batch 1; 128K-token cache at batch 8 with ragged lengths): every q head
    against the closed form on the CPU."""
    print(f"case decode full size B={B} L={L}", flush=True)
    dev = torch.device("cuda:0")
    Hq, Hkv, D = 28, 4, 128
    g = torch.Generator(device=dev).manual_seed(9)
    q = torch.randn(B, 1, Hq, D, device=dev, generator=g).bfloat16()
    kc = (torch.randn(B, L, Hkv, D, device=dev, generator=g) * 0.5).bfloat16()
    vc = torch.randn(B, L, Hkv, D, device=dev, generator=g).bfloat16()
    lens = [L] if B == 1 else [int(x) for x in torch.randint((3 * L) // 4, L + 1, (B,), generator=torch.Generator().manual_seed(1))]
    from longcontext_sqattn_paddle_amd.sqattn.attn_triton_decode import attn_decode

    out, lse = attn_decode(q, kc, vc, "NHD", torch.float32, return_lse=True,
                           seqlens=torch.tensor(lens, dtype=torch.int32, device=dev))
    torch.cuda.synchronize()
    qf = A.fold_scale(q.cpu().permute(0, 2, 1, 3), D).double()      # [B, Hq, 1, D], carries log2e / sqrt(D)
    for b in range(B):
        kb = kc[b, :lens[b]].cpu().double()
        vb = vc[b, :lens[b]].cpu().double()
        for kvh in range(Hkv):
            s = torch.einsum("nd,hd->hn", kb[:, kvh], qf[b, kvh * 7:(kvh + 1) * 7, 0])
            m = s.max(dim=1, keepdim=True).values
            p = torch.exp2(s - m)
            ref = (p @ vb[:, kvh]) / p.sum(dim=1, keepdim=True)
            ref_lse = (m + torch.log2(p.sum(dim=1, keepdim=True)))[:, 0]
            got = out[b, 0, kvh * 7:(kvh + 1) * 7].cpu().double()
            rms = float(ref.pow(2).mean().sqrt())
            assert float((got - ref).abs().max()) <= 2e-4 * rms + 1e-6
            assert torch.allclose(lse[b, kvh * 7:(kvh + 1) * 7, 0].cpu().double(), ref_lse, atol=2e-4)


@pytest.mark.parametrize("layout", ["NHD", "HND"])
def test_attn_unified_decode_lse_is_in_the_frame_of_the_centred_keys(layout):
    """`attn_unified` subtracts the keys' token mean before its kernel (attn_triton_decode.py:268-269), so the
    log-sum-exp it returns is that of the centred keys' scores; the prefill branch of the same function is in that
    frame too.  The decode kernel here skips the subtraction (the output cannot change) and the wrapper moves the
    log-sum-exp: it must equal the closed form over exactly centred keys (the reference rounds the centred keys to
    the tensor dtype, which moves a score by about 3e-3 here and is not reproduced; tolerance 2e-3 against the
    unrounded closed form, where 1.1 would be the error of not shifting at all)."""
    from longcontext_sqattn_paddle_amd.sqattn.attn_triton_decode import attn_unified

    print(f"case attn_unified decode lse {layout}", flush=True)
    dev = torch.device("cuda:0")
    q, kc, vc, _ = inputs.decode_inputs(2, 28, 4, 2000, 128, seed=77)
    kc = (kc.float() + torch.linspace(-1.0, 1.0, 128)).bfloat16()        # a key mean worth noticing
    qh, kh, vh = _to_hnd(q, kc, vc)
    centred = kh.double() - kh.double().mean(dim=2, keepdim=True)
    ref, lse_ref = A.exact_attention(A.fold_scale(qh, 128).double(), centred, vh.double(), causal=False, score_scale=math.log(2.0))
    _, lse_plain = A.exact_attention(A.fold_scale(qh, 128), kh, vh, causal=False, score_scale=math.log(2.0))
    assert float((lse_plain - lse_ref).abs().max()) > 0.5               # the two frames really differ on this input
    args = (q, kc, vc) if layout == "NHD" else (qh, kh, vh)
    out, lse = attn_unified(*[t.to(dev) for t in args], layout, torch.float32, return_lse=True)
    torch.cuda.synchronize()
    out = out.cpu()
    out = out[:, 0] if layout == "NHD" else out[:, :, 0]
    assert float((out.double() - ref[:, :, 0]).abs().max()) < 2e-4 * float(ref.pow(2).mean().sqrt()) + 1e-6
    assert torch.allclose(lse.cpu().double().view(2, 28), lse_ref[:, :, 0], atol=2e-3)


def test_decode_configurations_drawn_at_random():
    """A seeded sweep over the decode entry point: batch sizes, GQA ratios from 1 to 20 q heads per kv head, cache lengths
    that are not multiples of the 16-token tile, ragged valid lengths down to a single token, both layouts, explicit split
    counts from 1 to more than there are tiles -- each against exact attention over the valid prefix."""
    rng = torch.Generator().manual_seed(77)

    def pick(options):
        return options[int(torch.randint(0, len(options), (1,), generator=rng))]

    for case in range(20):
        B = pick([1, 2, 3, 5])
        Hkv = pick([1, 2, 4])
        Hq = Hkv * pick([1, 2, 7, 20])
        L = int(torch.randint(1, 2600, (1,), generator=rng))
        layout = pick(["NHD", "HND"])
        splits = pick([None, 1, 2, 7, 64, 300])
        q, kc, vc, _ = inputs.decode_inputs(B, Hq, Hkv, L, 128, seed=500 + case)
        lens = [int(torch.randint(1, L + 1, (1,), generator=rng)) for _ in range(B)]
        lens[0] = L if case % 3 else 1
        print(f"case decode #{case}: B={B} Hq={Hq} Hkv={Hkv} L={L} lens={lens} {layout} splits={splits}", flush=True)
        qh, kh, vh = _to_hnd(q, kc, vc)
        ref, lse_ref = A.exact_attention(A.fold_scale(qh, 128), kh, vh, causal=False, kv_lens=lens, score_scale=math.log(2.0))
        args = (q, kc, vc) if layout == "NHD" else (qh, kh, vh)
        kw = {} if splits is None else {"num_splits": splits}
        out, lse = _run(*args, lens, layout, output_dtype=torch.float32, return_lse=True, **kw)
        out = out.cpu()
        out = out[:, 0] if layout == "NHD" else out[:, :, 0]
        rms = float(ref.pow(2).mean().sqrt())
        err = float((out.double() - ref[:, :, 0]).abs().max())
        assert err < 2e-4 * rms + 1e-6, (case, err, rms)
        assert torch.allclose(lse.cpu()[:, :, 0].double(), lse_ref[:, :, 0], atol=2e-4), case
