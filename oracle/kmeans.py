"""CPU restatement of the reference's KV k-means (cache_hub/kmeans.py) plus the
build-defined centroid-scored top-k token selection.

TEST INFRASTRUCTURE ONLY (see `oracle/__init__.py`).

Differences from the reference that are part of the contract of this build, not of the oracle alone:
  * cluster sums are the *exact* sums (fp64 accumulation of bf16 values, which is exact for
    ordinary data) rounded once to fp32; the reference adds fp32 atomics in arbitrary order
    (kmeans.py:68-73), so its sums are this value plus order-dependent rounding noise.
  * the squared norm of a centroid is summed in fp64 and rounded to fp32 before the sqrt
    (the reference's `tl.sum` order is unspecified, kmeans.py:123).
  * tokens inside a cluster are listed in ascending order (reference: arbitrary, kmeans.py:224-230).
"""
from __future__ import annotations

import torch


def init_centroid_indices(num_tokens: int, num_centroids: int) -> torch.Tensor:
    """kmeans.py:340-344: `arange(C, fp32) * (N/C) + N/C/2` truncated to int64."""
    idx = torch.arange(num_centroids, dtype=torch.float32) * (num_tokens / num_centroids)
    idx = idx + num_tokens / num_centroids / 2
    return idx.to(torch.int64)


def scores64(data: torch.Tensor, cent: torch.Tensor) -> torch.Tensor:
    """Inner products in fp64 (bf16 x bf16 products are exact; the 128-term sum is exact to ~1e-16)."""
    return data.double() @ cent.double().transpose(-1, -2)


def assign(data: torch.Tensor, cent: torch.Tensor, chunk: int = 16384):
    """argmax_c <data_n, cent_c>, lowest index on ties (kmeans.py:59-67).

    data [G,N,D], cent [G,C,D].  Returns (idx int32 [G,N], rel_gap fp64 [G,N]) where rel_gap is
    (best - second_best) / max(|best|, tiny): tokens with a tiny gap are the documented near-ties
    on which an fp32 accumulation order may legitimately pick the other candidate.
    """
    G, N, _ = data.shape
    idx = torch.empty(G, N, dtype=torch.int32)
    gap = torch.empty(G, N, dtype=torch.float64)
    for g in range(G):
        for n0 in range(0, N, chunk):
            s = scores64(data[g, n0:n0 + chunk], cent[g])
            top2 = torch.topk(s, 2, dim=1).values
            idx[g, n0:n0 + chunk] = torch.argmax(s, dim=1).to(torch.int32)
            gap[g, n0:n0 + chunk] = (top2[:, 0] - top2[:, 1]) / top2[:, 0].abs().clamp(min=1e-30)
    return idx, gap


def cluster_sums(data: torch.Tensor, idx: torch.Tensor, num_centroids: int):
    """Exact per-cluster sums (fp64 -> fp32) and int32 counts (kmeans.py:68-79)."""
    G, N, D = data.shape
    S = torch.zeros(G, num_centroids, D, dtype=torch.float64)
    cnt = torch.zeros(G, num_centroids, dtype=torch.int32)
    for g in range(G):
        S[g].index_add_(0, idx[g].long(), data[g].double())
        cnt[g] = torch.bincount(idx[g].long(), minlength=num_centroids).to(torch.int32)
    return S.float(), cnt


def update(cent: torch.Tensor, S: torch.Tensor, cnt: torch.Tensor, normalize: bool) -> torch.Tensor:
    """`_triton_update_kernel` (kmeans.py:118-124): x = S/cnt, optional L2 normalisation, stored in
    the centroid dtype only where cnt > 0 (empty clusters keep the old centroid)."""
    x = S / cnt.float()[..., None]
    if normalize:
        ss = (x.double() ** 2).sum(dim=-1, keepdim=True).float()
        x = x / torch.sqrt(ss)
    keep = (cnt > 0)[..., None]
    return torch.where(keep, x.to(cent.dtype), cent)


def train_step(data, cent, normalize: bool):
    """`_triton_k_means_train` (kmeans.py:127-196). Returns (new centroids, idx, cnt, rel_gap)."""
    idx, gap = assign(data, cent)
    S, cnt = cluster_sums(data, idx, cent.shape[1])
    return update(cent, S, cnt, normalize), idx, cnt, gap


def reverse_index(idx: torch.Tensor, num_centroids: int, max_cluster_size: int):
    """`triton_reverse_index` (kmeans.py:233-262) with ascending token order inside a cluster."""
    G, N = idx.shape
    clusters = torch.zeros(G, num_centroids, max_cluster_size, dtype=torch.int32)
    size = torch.zeros(G, num_centroids, dtype=torch.int32)
    for g in range(G):
        order = torch.argsort(idx[g].long(), stable=True)
        cnt = torch.bincount(idx[g].long(), minlength=num_centroids)
        size[g] = cnt.to(torch.int32)
        start = torch.cumsum(cnt, 0) - cnt
        for c in range(num_centroids):
            n = int(cnt[c])
            clusters[g, c, :n] = order[int(start[c]):int(start[c]) + n].to(torch.int32)
    return clusters, size


def index_add(value: torch.Tensor, idx: torch.Tensor, num_centroids: int) -> torch.Tensor:
    """`triton_index_add` (kmeans.py:307-329): per-cluster sums of V, cast to V's dtype."""
    S, _ = cluster_sums(value, idx, num_centroids)
    return S.to(value.dtype)


def segment_k_means(key, value, num_centroids: int, num_iters: int = 10, num_segments: int = 1):
    """`segment_k_means` (kmeans.py:332-375). key/value [G,N,D].
    Returns (centroids [G,C,D], value_sum [G,C,D], clusters [G,C,max], cluster_size [G,C])."""
    G, N, D = key.shape
    cidx = init_centroid_indices(N, num_centroids)
    cent = key.index_select(1, cidx)
    assert num_centroids % num_segments == 0
    nps = N // num_segments
    cps = num_centroids // num_segments
    data = key[:, : nps * num_segments].reshape(-1, nps, D)
    cent = cent.reshape(-1, cps, D)
    for _ in range(num_iters - 1):
        cent, _, _, _ = train_step(data, cent, normalize=True)
    data = key.reshape(-1, N, D)
    cent = cent.reshape(-1, num_centroids, D)
    cent, idx, cnt, _ = train_step(data, cent, normalize=False)
    vsum = index_add(value.reshape(-1, N, D), idx, num_centroids)
    clusters, size = reverse_index(idx, num_centroids, int(cnt.max()))
    return cent, vsum, clusters, size


def topk_select(query, cent, clusters, cluster_size, k: int, num_kv_groups: int):
    """Build-defined (no reference code): centroid-scored token selection.

    query [B,Hq,D], cent [B*Hkv? -> G=B*Hkv, C, D] indexed g = b*Hkv + kvh.  Cluster score
    s[g,c] = max over the q-heads of kv-head g of <q_h, cent_{g,c}> (fp64 here), clusters ranked by
    descending score (ties -> lower c), whole clusters taken in rank order, the first k token ids
    emitted (cluster order, then stored order).  If fewer than k tokens exist the tail is -1.
    Returns int32 [G, k].
    """
    G, C, D = cent.shape
    B, Hq, _ = query.shape
    Hkv = Hq // num_kv_groups
    out = torch.full((G, k), -1, dtype=torch.int32)
    for gidx in range(G):
        b, kvh = divmod(gidx, Hkv)
        qh = query[b, kvh * num_kv_groups:(kvh + 1) * num_kv_groups].double()
        s = (qh @ cent[gidx].double().T).max(dim=0).values
        order = torch.argsort(s, descending=True, stable=True)
        pos = 0
        for c in order.tolist():
            n = int(cluster_size[gidx, c])
            take = min(n, k - pos)
            out[gidx, pos:pos + take] = clusters[gidx, c, :take]
            pos += take
            if pos >= k:
                break
    return out
