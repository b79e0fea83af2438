"""KV k-means of the reference's cache_hub/kmeans.py on the gfx950 kernels (same function names).

`segment_k_means(key, value, num_centroids, num_iters=10, num_segments=1)` returns
`(centroids, value_sum, clusters, cluster_size)` exactly like the reference (:332-375).  Differences:
cluster sums are exact (fp64) instead of fp32 atomics in arbitrary order, and tokens inside a cluster are
listed in ascending order instead of arbitrary order.  `topk_select` has no reference counterpart.
"""
from __future__ import annotations

from typing import Optional

import torch

from .. import _native as N


def _require(t, what):
    if not t.is_cuda:
        raise RuntimeError(f"{what} must live on the MI355X (got {t.device}); there is no CPU path")


def _workspace(G: int, num_tokens: int, num_centroids: int, device) -> torch.Tensor:
    need = N.lib().sq_kmeans_workspace_bytes(G, num_tokens, num_centroids, 128)
    return torch.empty(need, dtype=torch.uint8, device=device)


def _triton_k_means_train(data, centroids, max_idx=None, normalize_centroids=True, return_indices=False,
                          workspace: Optional[torch.Tensor] = None, state: int = N.KMEANS_STATELESS):
    """One Lloyd step, centroids updated in place (kmeans.py:127-196).  With `return_indices` also returns
    the assignment and the largest cluster size (a host sync, like the reference's `.item()`, :195).
    `state` (extension, for a run of steps over the same data with the same `max_idx` and `workspace`):
    `N.KMEANS_KEEP_SUMS` leaves the clusters' exact sums in the workspace, `N.KMEANS_APPLY_CHANGES` forms the new
    centroids from those sums and the tokens that changed cluster instead of re-summing every row (same bits)."""
    _require(data, "data")
    batch_size, num_tokens, dim = data.shape
    num_centroids = centroids.shape[1]
    assert num_centroids % 32 == 0
    if max_idx is None:
        max_idx = torch.empty((batch_size, num_tokens), dtype=torch.int32, device=data.device)
    data_cnt = torch.empty((batch_size, num_centroids), dtype=torch.int32, device=data.device)
    if workspace is None:
        workspace = _workspace(batch_size, num_tokens, num_centroids, data.device)
    b = [N.dl(t) for t in (data, centroids, max_idx, data_cnt, workspace)]
    N.check(N.lib().sq_kmeans_train_stateful(*[N.ptr(x) for x in b], 1 if normalize_centroids else 0, int(state),
                                             N.current_stream(data.device)))
    if return_indices:
        return centroids, max_idx, int(data_cnt.max().item())
    return centroids


def triton_reverse_index(max_idx, num_centroids: int, max_cluster_size: int, workspace: Optional[torch.Tensor] = None):
    """clusters[g,c,:size] = token ids of cluster c in ascending order (kmeans.py:233-262)."""
    _require(max_idx, "max_idx")
    batch_size, num_tokens = max_idx.shape
    clusters = torch.empty((batch_size, num_centroids, max(int(max_cluster_size), 1)), dtype=torch.int32, device=max_idx.device)
    cluster_size = torch.empty((batch_size, num_centroids), dtype=torch.int32, device=max_idx.device)
    if workspace is None:
        workspace = _workspace(batch_size, num_tokens, num_centroids, max_idx.device)
    b = [N.dl(t) for t in (max_idx, clusters, cluster_size, workspace)]
    N.check(N.lib().sq_reverse_index(*[N.ptr(x) for x in b], N.current_stream(max_idx.device)))
    return clusters, cluster_size


def triton_index_add(value, max_idx, num_centroids: int, workspace: Optional[torch.Tensor] = None):
    """Per-cluster sums of `value`, in value's dtype (kmeans.py:307-329)."""
    _require(value, "value")
    batch_size, num_tokens, dim = value.shape
    out = torch.empty((batch_size, num_centroids, dim), dtype=value.dtype, device=value.device)
    if workspace is None:
        workspace = _workspace(batch_size, num_tokens, num_centroids, value.device)
    b = [N.dl(t) for t in (value, max_idx, out, workspace)]
    N.check(N.lib().sq_index_add(*[N.ptr(x) for x in b], N.current_stream(value.device)))
    return out


FULL_RESUM_STEPS = 3   # Lloyd steps that re-sum every row before the sums are carried (most tokens still move in them)


def segment_k_means(key, value, num_centroids: int, num_iters: int = 10, num_segments: int = 1):
    """kmeans.py:332-375: strided initial centroids, `num_iters-1` normalised steps on the segmented data,
    one un-normalised step on the whole data, then value sums and the reverse index.

    From the fourth step on the exact cluster sums are carried from step to step and only the tokens that changed
    cluster are re-added (`sq_kmeans_train_stateful`): the same centroids bit for bit, without reading the keys a second
    time per step.  With one segment the final step runs on the same tensors and continues that way."""
    _require(key, "key")
    num_groups, num_tokens, head_dim = key.shape
    centroid_indices = torch.arange(num_centroids, dtype=torch.float32, device=key.device) * (num_tokens / num_centroids)
    centroid_indices += num_tokens / num_centroids / 2
    centroid_indices = centroid_indices.to(torch.int64)
    centroids = torch.index_select(key, dim=1, index=centroid_indices)
    assert num_centroids % num_segments == 0
    num_tokens_per_segment = num_tokens // num_segments
    num_centroids_per_segment = num_centroids // num_segments
    data = key[:, : num_tokens_per_segment * num_segments].reshape((-1, num_tokens_per_segment, head_dim))
    centroids = centroids.reshape((-1, num_centroids_per_segment, head_dim)).contiguous()
    max_idx = torch.empty((data.shape[0], data.shape[1]), dtype=torch.int32, device=data.device)
    ws = _workspace(data.shape[0], data.shape[1], num_centroids_per_segment, key.device)
    carried = False
    for it in range(num_iters - 1):
        state = N.KMEANS_STATELESS if it < FULL_RESUM_STEPS - 1 else (N.KMEANS_APPLY_CHANGES if carried else N.KMEANS_KEEP_SUMS)
        centroids = _triton_k_means_train(data, centroids, max_idx=max_idx, normalize_centroids=True,
                                          return_indices=False, workspace=ws, state=state)
        carried = state != N.KMEANS_STATELESS
    if num_segments == 1 and carried and data.shape[1] == num_tokens:
        # the same tensors, the same workspace: the last (un-normalised) step continues from the carried sums
        centroids, max_idx, max_cluster_size = _triton_k_means_train(data, centroids, max_idx=max_idx, normalize_centroids=False,
                                                                      return_indices=True, workspace=ws, state=N.KMEANS_APPLY_CHANGES)
    else:
        data = key.reshape((-1, num_tokens, head_dim))
        centroids = centroids.reshape((-1, num_centroids, head_dim))
        ws = _workspace(num_groups, num_tokens, num_centroids, key.device)
        centroids, max_idx, max_cluster_size = _triton_k_means_train(data, centroids, normalize_centroids=False,
                                                                      return_indices=True, workspace=ws)
    value_sum = triton_index_add(value.reshape((-1, num_tokens, head_dim)), max_idx, num_centroids, workspace=ws)
    clusters, cluster_size = triton_reverse_index(max_idx, num_centroids, max_cluster_size, workspace=ws)
    return centroids, value_sum, clusters, cluster_size


def topk_select(query, centroids, clusters, cluster_size, k: int, num_kv_groups: int, out=None, workspace=None):
    """Centroid-scored token selection (no reference counterpart): query [B,Hq,D] -> token ids int32 [G,k].
    `out` (int32 [G,k], contiguous) and `workspace` (`_workspace(G, 1, C, device)`) may be passed by a caller that
    selects every step."""
    _require(query, "query")
    G, C, _ = centroids.shape
    if out is None:
        out = torch.empty((G, k), dtype=torch.int32, device=query.device)
    ws = workspace if workspace is not None else _workspace(G, 1, C, query.device)
    b = [N.dl(t) for t in (query, centroids, clusters, cluster_size, out, ws)]
    N.check(N.lib().sq_topk_select(*[N.ptr(x) for x in b], num_kv_groups, N.current_stream(query.device)))
    return out


def cluster_order(clusters: torch.Tensor, cluster_size: torch.Tensor):
    """From the reverse index (`clusters` int32 [G,C,M], `cluster_size` int32 [G,C]) the two tables of a cache kept in
    cluster order (no reference counterpart): `order` int32 [G,n] lists every group's tokens cluster by cluster (n = the
    largest group total; shorter groups are padded with -1), and `positions` int32 [G,C,M] holds, in the layout of
    `clusters`, where each of those tokens sits in that list.  `topk_select(query, centroids, positions, cluster_size,
    ...)` then yields rows of the reordered cache instead of token ids."""
    G, C, M = clusters.shape
    size = cluster_size.to(torch.int64)
    offset = torch.cumsum(size, dim=1) - size                                   # [G,C] exclusive prefix
    slot = torch.arange(M, device=clusters.device).view(1, 1, M)
    used = slot < size.unsqueeze(-1)                                            # [G,C,M]
    positions = torch.where(used, offset.unsqueeze(-1) + slot, torch.zeros_like(slot)).to(torch.int32)
    n = int(size.sum(dim=1).max().item())
    order = torch.full((G, n), -1, dtype=torch.int32, device=clusters.device)
    rows = torch.arange(G, device=clusters.device).view(G, 1, 1).expand(G, C, M)
    order[rows[used], positions[used].long()] = clusters[used]
    return order, positions


def reorder_cache(key_cache: torch.Tensor, value_cache: torch.Tensor, order: torch.Tensor):
    """Copies of a layer's cache [B,L,Hkv,D] with each kv head's rows in the order `order` int32 [B*Hkv,n] gives
    (`sq_kv_cache_reorder`): out[b, p, h] = cache[b, order[b*Hkv + h, p], h]; rows for -1 are zero."""
    _require(key_cache, "key_cache")
    _require(value_cache, "value_cache")
    B, _, H, D = key_cache.shape
    n = order.shape[1]
    key_out = torch.empty((B, n, H, D), dtype=key_cache.dtype, device=key_cache.device)
    value_out = torch.empty_like(key_out)
    b = [N.dl(t) for t in (key_cache, value_cache, order, key_out, value_out)]
    N.check(N.lib().sq_kv_cache_reorder(*[N.ptr(x) for x in b], N.current_stream(key_cache.device)))
    return key_out, value_out

