"""GPU parity: k-means kernels and top-k selection (through the C ABI) against the CPU oracle.

Assignments must equal the oracle's fp64 arg-max except on near-ties: tokens whose best and second-best
scores differ by less than 1e-5 relative, where the fp32 MFMA accumulation may pick the other candidate.
Cluster sums are exact on both sides, so centroids computed from the same assignment must agree bit for
bit (one bf16 ulp is tolerated on at most 0.1 % of the components: the squared norm is reduced in a
different fp64 order before it is rounded to fp32).
"""
import pytest
import torch

from oracle import inputs
from oracle import kmeans as KM

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
NEAR_TIE = 1e-5


def _bf16_ulp_diff(a, b):
    ia = a.view(torch.int16).to(torch.int32)
    ib = b.view(torch.int16).to(torch.int32)
    return (ia - ib).abs()


@pytest.mark.parametrize("normalize", [True, False])
@pytest.mark.parametrize("G,N,C", [(2, 3000, 64), (1, 4096, 160), (1, 9000, 2048), (1, 20000, 8192)])
def test_train_step_teacher_forced(G, N, C, normalize):
    from longcontext_sqattn_paddle_amd.cache_hub.kmeans import _triton_k_means_train

    print(f"case kmeans train G={G} N={N} C={C} normalize={normalize}", flush=True)
    key, _ = inputs.kmeans_inputs(G, N, 128, n_modes=24, seed=50 + C)
    cent0 = key[:, KM.init_centroid_indices(N, C)].clone()
    cent0[:, 7] = cent0[:, 6]                         # duplicate centroid: ties go to the lower index, 7 stays empty
    ref_idx, gap = KM.assign(key, cent0)
    cent_d = cent0.clone().to(DEV)
    _, idx_d, max_cnt = _triton_k_means_train(key.to(DEV), cent_d, normalize_centroids=normalize, return_indices=True)
    torch.cuda.synchronize()
    idx = idx_d.cpu()
    differ = idx != ref_idx
    assert bool((gap[differ] < NEAR_TIE).all()), f"{int(differ.sum())} assignments differ outside near-ties"
    assert int(differ.sum()) <= max(2, N // 2000)
    # centroids from the kernel's own assignment: exact sums -> same bits
    S, cnt = KM.cluster_sums(key, idx, C)
    assert max_cnt == int(cnt.max())
    exp = KM.update(cent0, S, cnt, normalize)
    got = cent_d.cpu()
    ulp = _bf16_ulp_diff(got, exp)
    assert int(ulp.max()) <= 1 and float((ulp > 0).float().mean()) <= 1e-3
    empty = cnt == 0
    assert bool(empty[:, 7].all()) and torch.equal(got[empty], cent0[empty])   # empty clusters keep the old centroid


def test_reverse_index_and_index_add_exact():
    from longcontext_sqattn_paddle_amd.cache_hub.kmeans import triton_index_add, triton_reverse_index

    G, N, C = 3, 5000, 96
    g = torch.Generator().manual_seed(3)
    idx = torch.randint(0, C, (G, N), generator=g, dtype=torch.int32)
    idx[idx == 11] = 12                                   # one empty cluster
    value = torch.randn(G, N, 128, generator=g).bfloat16()
    max_size = int(torch.stack([torch.bincount(idx[i].long(), minlength=C) for i in range(G)]).max())
    clusters, size = triton_reverse_index(idx.to(DEV), C, max_size)
    vsum = triton_index_add(value.to(DEV), idx.to(DEV), C)
    torch.cuda.synchronize()
    rc, rs = KM.reverse_index(idx, C, max_size)
    assert torch.equal(size.cpu(), rs) and torch.equal(clusters.cpu(), rc)
    assert torch.equal(vsum.cpu(), KM.index_add(value, idx, C))


def test_index_add_many_tiles_and_one_huge_cluster():
    """The grouping behind the sums works tile by tile: more tiles than one pass of the sum kernel walks (256), a ragged
    last tile, a cluster far larger than the id list the kernel stages at a time (the tiles sum its rows themselves), one
    with just under 2048 tokens per pass, an empty cluster.  Sums are exact."""
    from longcontext_sqattn_paddle_amd.cache_hub.kmeans import triton_index_add

    G, N, C = 1, 600_001, 32
    g = torch.Generator().manual_seed(17)
    idx = torch.randint(0, C, (G, N), generator=g, dtype=torch.int32)
    u = torch.rand(G, N, generator=g)
    idx[u < 0.5] = 3                                      # about 300 000 tokens in one cluster
    idx[(u >= 0.5) & (u < 0.5156)] = 9                    # about 64 per tile of 2048 tokens: either side of the size from which a tile sums a range itself
    idx[idx == 5] = 6
    value = torch.randn(G, N, 128, generator=g).bfloat16()
    vsum = triton_index_add(value.to(DEV), idx.to(DEV), C)
    torch.cuda.synchronize()
    assert torch.equal(vsum.cpu(), KM.index_add(value, idx, C))


@pytest.mark.parametrize("C", [8192, 5000, 1025])
def test_index_add_many_clusters(C):
    """Cluster counts up to the supported maximum (8192: the grouping kernel's counters, ids and long-range sums then
    take 72 KB of LDS, above the default limit; its prefix over the clusters runs in eight rounds) and counts that are
    not multiples of anything: sums exact, reverse index exact."""
    from longcontext_sqattn_paddle_amd.cache_hub.kmeans import triton_index_add, triton_reverse_index

    G, N = 2, 30_000
    g = torch.Generator().manual_seed(C)
    idx = torch.randint(0, C, (G, N), generator=g, dtype=torch.int32)
    idx[0, :3000] = C - 1                                  # one long range at the last cluster
    value = torch.randn(G, N, 128, generator=g).bfloat16()
    vsum = triton_index_add(value.to(DEV), idx.to(DEV), C)
    msize = int(torch.stack([torch.bincount(idx[i].long(), minlength=C) for i in range(G)]).max())
    clusters, size = triton_reverse_index(idx.to(DEV), C, msize)
    torch.cuda.synchronize()
    assert torch.equal(vsum.cpu(), KM.index_add(value, idx, C))
    rc, rs = KM.reverse_index(idx, C, msize)
    assert torch.equal(size.cpu(), rs) and torch.equal(clusters.cpu(), rc)


@pytest.mark.parametrize("segments", [1, 2])
def test_segment_k_means_end_to_end(segments):
    from longcontext_sqattn_paddle_amd.cache_hub.kmeans import segment_k_means

    G, N, C = 2, 4096, 64
    key, value = inputs.kmeans_inputs(G, N, 128, n_modes=20, seed=61)
    cent, vsum, clusters, size = segment_k_means(key.to(DEV), value.to(DEV), C, num_iters=4, num_segments=segments)
    torch.cuda.synchronize()
    rcent, rvsum, rclusters, rsize = KM.segment_k_means(key, value, C, num_iters=4, num_segments=segments)
    size, clusters = size.cpu(), clusters.cpu()
    assert int(size.sum()) == G * N
    for g in range(G):
        toks = torch.cat([clusters[g, c, : int(size[g, c])] for c in range(C)])
        assert torch.equal(torch.sort(toks).values, torch.arange(N, dtype=torch.int32))
    # free-running iterations: identical unless a near-tie flipped somewhere along the way
    own = torch.empty(G, N, dtype=torch.int64)
    ref = torch.empty(G, N, dtype=torch.int64)
    for g in range(G):
        for c in range(C):
            own[g, clusters[g, c, : int(size[g, c])].long()] = c
            ref[g, rclusters[g, c, : int(rsize[g, c])].long()] = c
    assert float((own == ref).float().mean()) >= 0.999
    ulp = _bf16_ulp_diff(cent.cpu(), rcent)
    assert float((ulp <= 1).float().mean()) >= 0.99
    assert torch.allclose(vsum.cpu().float(), rvsum.float(), atol=0.5, rtol=0.05) or float((own == ref).float().mean()) < 1.0


def test_topk_select_matches_oracle():
    from longcontext_sqattn_paddle_amd.cache_hub.kmeans import topk_select

    B, Hq, groups, N, C, k = 2, 8, 4, 2048, 64, 700
    Hkv = Hq // groups
    key, value = inputs.kmeans_inputs(B * Hkv, N, 128, n_modes=20, seed=71)
    cent, _, clusters, size = KM.segment_k_means(key, value, C, num_iters=3)
    q = torch.randn(B, Hq, 128, generator=torch.Generator().manual_seed(2)).bfloat16()
    sel = topk_select(q.to(DEV), cent.to(DEV), clusters.to(DEV), size.to(DEV), k, groups)
    torch.cuda.synchronize()
    assert torch.equal(sel.cpu(), KM.topk_select(q, cent, clusters, size, k, groups))
    # k larger than the number of tokens: the tail is -1
    sel2 = topk_select(q.to(DEV), cent.to(DEV), clusters.to(DEV), size.to(DEV), N + 50, groups).cpu()
    assert bool((sel2[:, N:] == -1).all()) and bool((sel2[:, :N] >= 0).all())
    for g in range(B * Hkv):
        assert torch.equal(torch.sort(sel2[g, :N]).values, torch.arange(N, dtype=torch.int32))


def test_topk_select_shared_score_phase_repeated():
    """With 1024 clusters several workgroups share a head's score phase and the last to arrive finishes the selection,
    handing the scores over through memory.  Two queries alternate over 1000 calls; every call must reproduce its query's
    oracle result exactly (a score that arrives late, or a counter that is not set back, would show)."""
    from longcontext_sqattn_paddle_amd.cache_hub.kmeans import _workspace, topk_select

    B, Hkv, groups, N, C, k = 2, 4, 7, 8192, 1024, 1000
    G = B * Hkv
    g = torch.Generator().manual_seed(81)
    idx = torch.randint(0, C, (G, N), generator=g, dtype=torch.int32)
    msize = int(torch.stack([torch.bincount(idx[i].long(), minlength=C) for i in range(G)]).max())
    clusters, size = KM.reverse_index(idx, C, msize)
    cent = torch.randn(G, C, 128, generator=g).bfloat16()
    qs = [torch.randn(B, Hkv * groups, 128, generator=g).bfloat16() for _ in range(2)]
    want = [KM.topk_select(q, cent, clusters, size, k, groups) for q in qs]
    dq = [q.to(DEV) for q in qs]
    dc, dcl, dsz = cent.to(DEV), clusters.to(DEV), size.to(DEV)
    ws = _workspace(G, 1, C, DEV)   # one workspace for all calls: a stale score would be the other query's
    outs = [topk_select(dq[i % 2], dc, dcl, dsz, k, groups, workspace=ws) for i in range(1000)]
    torch.cuda.synchronize()
    for i, o in enumerate(outs):
        assert torch.equal(o.cpu(), want[i % 2]), i


def _shared_phase_case(seed):
    B, Hkv, groups, N, C, k = 1, 4, 7, 8192, 1024, 1000
    g = torch.Generator().manual_seed(seed)
    idx = torch.randint(0, C, (B * Hkv, N), generator=g, dtype=torch.int32)
    msize = int(torch.stack([torch.bincount(idx[i].long(), minlength=C) for i in range(B * Hkv)]).max())
    clusters, size = KM.reverse_index(idx, C, msize)
    cent = torch.randn(B * Hkv, C, 128, generator=g).bfloat16()
    q = torch.randn(B, Hkv * groups, 128, generator=g).bfloat16()
    return q, cent, clusters, size, k, groups


@pytest.mark.parametrize("fill", ["ones", "random", "finished", "other_shape"])
def test_topk_select_arrival_words_need_no_initialisation(fill):
    """The arrival words of the shared score phase live in the caller's workspace and are never cleared by the host.
    Whatever the memory holds -- all bits set, random words, the word a finished call leaves, or the words of a call
    with another number of heads -- the first call over it must select what the oracle selects."""
    from longcontext_sqattn_paddle_amd.cache_hub.kmeans import _workspace, topk_select

    q, cent, clusters, size, k, groups = _shared_phase_case(83)
    G, C = cent.shape[0], cent.shape[1]
    want = KM.topk_select(q, cent, clusters, size, k, groups)
    ws = _workspace(G, 1, C, DEV)
    words = ws[: ws.numel() // 4 * 4].view(torch.int32)
    if fill == "ones":
        ws.fill_(0xFF)
    elif fill == "random":
        words.copy_(torch.randint(-2**31, 2**31 - 1, (words.numel(),), generator=torch.Generator().manual_seed(5),
                                  dtype=torch.int64).to(torch.int32).to(DEV))
    elif fill == "finished":
        topk_select(q.to(DEV), cent.to(DEV), clusters.to(DEV), size.to(DEV), k, groups, workspace=ws)
    else:   # a call over 2 of the 4 heads first, then all 4 over the same memory
        topk_select(q[:, : 2 * groups].to(DEV), cent[:2].to(DEV), clusters[:2].to(DEV), size[:2].to(DEV), k, groups,
                    workspace=ws)
    for _ in range(3):
        got = topk_select(q.to(DEV), cent.to(DEV), clusters.to(DEV), size.to(DEV), k, groups, workspace=ws)
        torch.cuda.synchronize()
        assert torch.equal(got.cpu(), want)


def test_topk_select_two_workspaces_on_two_streams():
    """Calls that use different workspaces share nothing: two selections with different queries run on two streams at
    the same time, 200 times, and each must equal its own oracle result."""
    from longcontext_sqattn_paddle_amd.cache_hub.kmeans import _workspace, topk_select

    cases = [_shared_phase_case(s) for s in (85, 86)]
    want = [KM.topk_select(*c) for c in cases]
    dev = [[x.to(DEV) if torch.is_tensor(x) else x for x in c] for c in cases]
    G, C = cases[0][1].shape[0], cases[0][1].shape[1]
    wss = [_workspace(G, 1, C, DEV) for _ in cases]
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    torch.cuda.synchronize()
    outs = [[], []]
    for _ in range(200):
        for i in (0, 1):
            with torch.cuda.stream(streams[i]):
                outs[i].append(topk_select(*dev[i], workspace=wss[i]))
    torch.cuda.synchronize()
    for i in (0, 1):
        for o in outs[i]:
            assert torch.equal(o.cpu(), want[i])


def test_full_size_properties():
    """Benchmark shape (4 heads x 131072 tokens x 128, 1024 centroids): size-independent invariants plus an
    oracle check on a token sample."""
    from longcontext_sqattn_paddle_amd.cache_hub.kmeans import _triton_k_means_train, triton_reverse_index

    G, N, C = 4, 131072, 1024
    key, _ = inputs.kmeans_inputs(G, N, 128, seed=4)
    cent0 = key[:, KM.init_centroid_indices(N, C)].clone()
    kd, cd = key.to(DEV), cent0.clone().to(DEV)
    _, idx_d, max_cnt = _triton_k_means_train(kd, cd, normalize_centroids=True, return_indices=True)
    clusters, size = triton_reverse_index(idx_d, C, max_cnt)
    torch.cuda.synchronize()
    idx, size = idx_d.cpu(), size.cpu()
    assert int(size.sum()) == G * N and int(size.max()) == max_cnt
    for g in range(G):
        assert torch.equal(size[g].long(), torch.bincount(idx[g].long(), minlength=C))
    flat = clusters.cpu()
    for g in range(G):
        mask = torch.arange(flat.shape[2])[None, :] < size[g][:, None]
        assert torch.equal(torch.sort(flat[g][mask]).values, torch.arange(N, dtype=torch.int32))
    sample = slice(5000, 5000 + 4096)
    ref_idx, gap = KM.assign(key[:, sample], cent0)
    differ = idx[:, sample] != ref_idx
    assert bool((gap[differ] < NEAR_TIE).all())
    nrm = cd.cpu()[size > 0].float().norm(dim=-1)
    assert float((nrm - 1).abs().max()) < 1e-2


def test_kmeans_configurations_drawn_at_random():
    """A seeded sweep over the training step and the index helpers: 1 to 5 groups, token counts that are not multiples of the
    256-token tile (down to fewer tokens than centroids), centroid counts from 32 to 1056 (multiples of 32, with and
    without a half block at the end), normalised or not -- each against the oracle under the rules at the top."""
    from longcontext_sqattn_paddle_amd.cache_hub.kmeans import _triton_k_means_train, triton_index_add, triton_reverse_index

    rng = torch.Generator().manual_seed(99)

    def pick(options):
        return options[int(torch.randint(0, len(options), (1,), generator=rng))]

    for case in range(12):
        G = pick([1, 2, 3, 5])
        C = 32 * pick([1, 2, 3, 5, 8, 17, 33])
        N = int(torch.randint(max(40, C // 2), 6000, (1,), generator=rng))
        normalize = bool(case % 2)
        print(f"case kmeans #{case}: G={G} N={N} C={C} normalize={normalize}", flush=True)
        key, value = inputs.kmeans_inputs(G, N, 128, n_modes=min(C, 40), seed=600 + case)
        cent0 = key[:, torch.randint(0, N, (C,), generator=rng)].clone()   # repeated picks give duplicate centroids
        ref_idx, gap = KM.assign(key, cent0)
        cent_d = cent0.clone().to(DEV)
        _, idx_d, max_cnt = _triton_k_means_train(key.to(DEV), cent_d, normalize_centroids=normalize, return_indices=True)
        torch.cuda.synchronize()
        idx = idx_d.cpu()
        differ = idx != ref_idx
        assert bool((gap[differ] < NEAR_TIE).all()), (case, int(differ.sum()))
        S, cnt = KM.cluster_sums(key, idx, C)
        assert max_cnt == int(cnt.max())
        ulp = _bf16_ulp_diff(cent_d.cpu(), KM.update(cent0, S, cnt, normalize))
        assert int(ulp.max()) <= 1 and float((ulp > 0).float().mean()) <= 1e-3, case
        clusters, size = triton_reverse_index(idx_d, C, max_cnt)
        vsum = triton_index_add(value.to(DEV), idx_d, C)
        torch.cuda.synchronize()
        rc, rs = KM.reverse_index(idx, C, max_cnt)
        assert torch.equal(size.cpu(), rs) and torch.equal(clusters.cpu(), rc), case
        assert torch.equal(vsum.cpu(), KM.index_add(value, idx, C)), case


@pytest.mark.parametrize("G,N,C,modes", [(2, 5000, 64, 20), (1, 40000, 1024, 300), (3, 777, 32, 5)])
def test_carried_sums_give_the_bits_of_the_full_resum(G, N, C, modes):
    """`sq_kmeans_train_stateful`: a run of Lloyd steps whose cluster sums are carried in the workspace (one step that
    keeps them, then steps that only apply the tokens that changed cluster) against the same run with every step
    re-summing every row.  The sums are exact, so centroids, assignment and sizes must be equal bit for bit after every
    step -- normalised and un-normalised steps, empty clusters, N not a multiple of the 256-token tile, and a step in
    which nothing moves."""
    from longcontext_sqattn_paddle_amd import _native as NV
    from longcontext_sqattn_paddle_amd.cache_hub.kmeans import _triton_k_means_train, _workspace

    print(f"case k-means carried sums G={G} N={N} C={C}", flush=True)
    key, _ = inputs.kmeans_inputs(G, N, 128, n_modes=modes, seed=70 + C)
    data = key.to(DEV)
    sel = KM.init_centroid_indices(N, C).to(DEV)
    ca, cb = data.index_select(1, sel).contiguous(), data.index_select(1, sel).contiguous()
    ia = torch.empty(G, N, dtype=torch.int32, device=DEV)
    ib = torch.full((G, N), -7, dtype=torch.int32, device=DEV)
    wa, wb = _workspace(G, N, C, DEV), _workspace(G, N, C, DEV)
    wb.fill_(0x5A)      # whatever the workspace held before must not matter
    moved = []
    for step in range(9):
        norm = step != 5                                   # one un-normalised step in the middle of the run
        state = NV.KMEANS_STATELESS if step == 0 else (NV.KMEANS_KEEP_SUMS if step == 1 else NV.KMEANS_APPLY_CHANGES)
        prev = ib.clone()
        _, _, max_a = _triton_k_means_train(data, ca, max_idx=ia, normalize_centroids=norm, return_indices=True, workspace=wa)
        _, _, max_b = _triton_k_means_train(data, cb, max_idx=ib, normalize_centroids=norm, return_indices=True, workspace=wb, state=state)
        torch.cuda.synchronize()
        moved.append(int((prev != ib).sum()))
        assert torch.equal(ia, ib), step
        assert torch.equal(ca.view(torch.int16), cb.view(torch.int16)), step
        assert max_a == max_b, step
    print(f"  tokens that changed cluster per step: {moved}", flush=True)
    # a step in which nothing moves (the same centroids again cannot be had, but the same assignment can: feed the
    # centroids of the stateless run, which are equal, and repeat until the assignment is stable or 20 steps have passed)
    for _ in range(20):
        prev = ib.clone()
        _triton_k_means_train(data, ca, max_idx=ia, normalize_centroids=True, workspace=wa)
        _triton_k_means_train(data, cb, max_idx=ib, normalize_centroids=True, workspace=wb, state=NV.KMEANS_APPLY_CHANGES)
        torch.cuda.synchronize()
        assert torch.equal(ia, ib) and torch.equal(ca.view(torch.int16), cb.view(torch.int16))
        if torch.equal(prev, ib):
            break
    # the sizes the carried state reports are the histogram of the assignment
    cnt = torch.empty(G, C, dtype=torch.int32, device=DEV)
    b = [NV.dl(t) for t in (data, cb, ib, cnt, wb)]
    NV.check(NV.lib().sq_kmeans_train_stateful(*[NV.ptr(x) for x in b], 1, NV.KMEANS_APPLY_CHANGES, NV.current_stream(data.device)))
    torch.cuda.synchronize()
    for g in range(G):
        assert torch.equal(cnt[g].cpu().long(), torch.bincount(ib[g].cpu().long(), minlength=C))


def test_segment_k_means_with_carried_sums_equals_stateless_steps():
    """`segment_k_means` carries the sums from its fourth step on; written out with stateless steps only it must return
    the same centroids, value sums, clusters and sizes (one segment, where the last step continues the carried run, and
    two, where it starts over on the unsegmented data)."""
    from longcontext_sqattn_paddle_amd.cache_hub import kmeans as HK

    key, value = inputs.kmeans_inputs(2, 6000, 128, n_modes=40, seed=81)
    key, value = key.to(DEV), value.to(DEV)
    for segments in (1, 2):
        got = HK.segment_k_means(key, value, 64, num_iters=8, num_segments=segments)
        saved, HK.FULL_RESUM_STEPS = HK.FULL_RESUM_STEPS, 1 << 30       # every step stateless
        try:
            want = HK.segment_k_means(key, value, 64, num_iters=8, num_segments=segments)
        finally:
            HK.FULL_RESUM_STEPS = saved
        torch.cuda.synchronize()
        for a, b in zip(got, want):
            assert a.shape == b.shape and torch.equal(a.view(torch.int16) if a.dtype == torch.bfloat16 else a, b.view(torch.int16) if b.dtype == torch.bfloat16 else b), segments
