"""Pins the k-means restatement with brute force and partition invariants."""
import torch

from oracle import inputs, kmeans as KM


def test_init_indices():
    assert KM.init_centroid_indices(131072, 1024)[:3].tolist() == [64, 192, 320]
    assert KM.init_centroid_indices(1000, 32)[:3].tolist() == [15, 46, 78]   # 31.25*i + 15.625 truncated


def test_assign_is_first_argmax_bruteforce():
    key, _ = inputs.kmeans_inputs(G=2, N=300, D=16, n_modes=8, seed=11)
    cent = key[:, KM.init_centroid_indices(300, 32)]
    cent[:, 5] = cent[:, 3]                      # duplicate centroid: ties must resolve to the lower index
    idx, gap = KM.assign(key, cent)
    for g in range(2):
        for n in range(300):
            best, bi = None, -1
            for c in range(32):
                s = float((key[g, n].double() * cent[g, c].double()).sum())
                if best is None or s > best:
                    best, bi = s, c
            assert int(idx[g, n]) == bi
    assert not (idx == 5).any()
    assert (gap >= 0).all()


def test_train_step_invariants():
    key, _ = inputs.kmeans_inputs(G=2, N=2048, D=32, n_modes=16, seed=12)
    cent0 = key[:, KM.init_centroid_indices(2048, 64)].clone()
    cent1, idx, cnt, _ = KM.train_step(key, cent0, normalize=True)
    assert int(cnt.sum()) == 2 * 2048
    for g in range(2):
        assert torch.equal(cnt[g].long(), torch.bincount(idx[g].long(), minlength=64))
    S, _ = KM.cluster_sums(key, idx, 64)
    assert torch.allclose(S.double().sum(1), key.double().sum(1), atol=1e-3)
    empty = cnt == 0
    assert torch.equal(cent1[empty], cent0[empty])                      # empty clusters keep the old centroid
    nrm = cent1[~empty].float().norm(dim=-1)
    assert torch.allclose(nrm, torch.ones_like(nrm), atol=1e-2)         # unit norm up to bf16 rounding
    cent2, _, _, _ = KM.train_step(key, cent0, normalize=False)
    mean = S / cnt.float()[..., None]
    assert torch.equal(cent2[~empty], mean[~empty].to(cent0.dtype))


def test_segment_k_means_and_reverse_index():
    key, value = inputs.kmeans_inputs(G=2, N=1024, D=32, n_modes=16, seed=13)
    for segs in (1, 2):
        cent, vsum, clusters, size = KM.segment_k_means(key, value, 64, num_iters=4, num_segments=segs)
        assert cent.shape == (2, 64, 32) and vsum.shape == (2, 64, 32)
        assert int(size.sum()) == 2 * 1024 and clusters.shape[2] == int(size.max())
        for g in range(2):
            toks = torch.cat([clusters[g, c, : int(size[g, c])] for c in range(64)])
            assert torch.equal(torch.sort(toks).values, torch.arange(1024, dtype=torch.int32))
        assert torch.allclose(vsum.double().sum(1), value.double().sum(1), atol=0.5)


def test_topk_bruteforce():
    key, value = inputs.kmeans_inputs(G=2, N=512, D=16, n_modes=8, seed=14)
    cent, _, clusters, size = KM.segment_k_means(key, value, 32, num_iters=3)
    q = torch.randn(1, 4, 16, generator=torch.Generator().manual_seed(1)).bfloat16()
    sel = KM.topk_select(q, cent, clusters, size, k=100, num_kv_groups=2)
    for g in range(2):
        sc = (q[0, 2 * g:2 * g + 2].double() @ cent[g].double().T).max(0).values
        order = sorted(range(32), key=lambda c: (-float(sc[c]), c))
        exp = []
        for c in order:
            exp += clusters[g, c, : int(size[g, c])].tolist()
        assert sel[g].tolist() == exp[:100]
