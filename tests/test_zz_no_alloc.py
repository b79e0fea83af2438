"""`sq_decode_fwd_noalloc` (the entry point for callers that cannot allocate device memory) against `sq_decode_fwd`:
same kernels, partials in the library's own device array instead of a workspace, so the outputs must be equal bit for
bit.  Two calls in a row, the second on a smaller input (the array then still holds the first call's partials), and
the size limit.  "Allocates nothing" is checked against the driver's own count of free device memory
(`hipMemGetInfo`, which also sees a `hipMalloc` made inside the library), not only against torch's allocator; and the
call is recorded into a HIP graph after `sq_decode_noalloc_init` and replayed."""
import ctypes
import gc

import pytest
import torch

from longcontext_sqattn_paddle_amd import _native as N

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


def _call(fn_name, q, k, v, seqlens, out, lse, splits, workspace=None):
    lib = N.lib()
    params = N.DecodeParams(N.LAYOUT["NHD"], 0, splits, 128)
    tensors = [q, k, v, seqlens, out, lse] + ([workspace] if fn_name == "sq_decode_fwd" else [])
    b = [N.dl(t) for t in tensors]
    rc = getattr(lib, fn_name)(*[N.ptr(x) for x in b], params, N.current_stream(q.device))
    return rc, lib.sq_last_error().decode()


def _case(B, Hq, Hkv, L, lens, seed, splits=0):
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, 1, Hq, 128, generator=g).bfloat16().to(DEV)
    k = torch.randn(B, L, Hkv, 128, generator=g).bfloat16().to(DEV)
    v = torch.randn(B, L, Hkv, 128, generator=g).bfloat16().to(DEV)
    sl = torch.tensor(lens, dtype=torch.int32, device=DEV) if lens is not None else None
    lib = N.lib()
    S = splits if splits > 0 else lib.sq_decode_num_splits(B, Hkv, L)
    ws = torch.empty(lib.sq_decode_workspace_bytes(B, Hq, 128, S) // 4, dtype=torch.float32, device=DEV)
    out_a, out_b = (torch.full((B, 1, Hq, 128), float("nan"), dtype=torch.float32, device=DEV) for _ in range(2))
    lse_a, lse_b = (torch.full((B, Hq, 1), float("nan"), dtype=torch.float32, device=DEV) for _ in range(2))
    return (q, k, v, sl), (out_a, lse_a, ws), (out_b, lse_b), S


def test_noalloc_decode_equals_workspace_decode_twice_second_smaller():
    lib = N.lib()
    assert lib.sq_decode_noalloc_scratch_bytes() == 8 << 20
    # first call: 3 ragged sequences x 28/4 heads x 20000 tokens; second: one sequence of 1500 tokens (fewer splits,
    # fewer heads), which must not see anything of the first call's partials
    for B, Hq, Hkv, L, lens, seed in ((3, 28, 4, 20000, [20000, 12345, 777], 1), (1, 8, 2, 1500, [1333], 2)):
        print(f"case noalloc decode B={B} Hq={Hq} Hkv={Hkv} L={L}", flush=True)
        (q, k, v, sl), (out_a, lse_a, ws), (out_b, lse_b), S = _case(B, Hq, Hkv, L, lens, seed)
        rc, msg = _call("sq_decode_fwd", q, k, v, sl, out_a, lse_a, 0, ws)
        assert rc == 0, msg
        assert lib.sq_decode_noalloc_init() == 0, lib.sq_last_error().decode()   # the one-off look-up, outside the measured call
        torch.cuda.synchronize()
        # Tensors of earlier tests that only a collection of reference cycles frees must not be freed between the two
        # readings (after a long run of other tests that was tens of GB): collect now, and keep the collector off
        # for the measured call.  torch's count is its cumulative number of allocations, which a free cannot change.
        gc.collect()
        gc.disable()
        try:
            n_before = torch.cuda.memory_stats()["allocation.all.allocated"]
            before, free_before = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
            rc, msg = _call("sq_decode_fwd_noalloc", q, k, v, sl, out_b, lse_b, 0)
            torch.cuda.synchronize()
            n_after = torch.cuda.memory_stats()["allocation.all.allocated"]
            after, free_after = torch.cuda.memory_allocated(), torch.cuda.mem_get_info()[0]
        finally:
            gc.enable()
        assert rc == 0, msg
        assert n_after == n_before and after == before
        assert free_after == free_before      # the driver's count: no hipMalloc inside the library either
        assert bool(torch.isfinite(out_b).all())
        assert torch.equal(out_a, out_b) and torch.equal(lse_a, lse_b)


def test_noalloc_decode_rejects_sizes_beyond_its_array():
    # 4096 splits x 4 q heads x 516 bytes = 8.45 MB of partials > 8 MiB
    (q, k, v, sl), _, (out_b, lse_b), _ = _case(1, 4, 1, 70000, None, 3, splits=4096)
    rc, msg = _call("sq_decode_fwd_noalloc", q, k, v, sl, out_b, lse_b, 4096)
    assert rc == N.SQ_EWORKSPACE and "scratch" in msg
    # the same call with fewer splits fits and runs
    rc, msg = _call("sq_decode_fwd_noalloc", q, k, v, sl, out_b, lse_b, 64)
    assert rc == 0, msg
    torch.cuda.synchronize()
    assert bool(torch.isfinite(out_b).all())


def test_noalloc_decode_recorded_into_a_graph_and_replayed():
    """What the entry point is for: after `sq_decode_noalloc_init` and one eager call it is recorded into a HIP graph;
    every replay -- with the cache contents changed and eager work in between -- equals the eager `sq_decode_fwd`."""
    lib = N.lib()
    assert lib.sq_decode_noalloc_init() == 0, lib.sq_last_error().decode()
    (q, k, v, sl), (out_a, lse_a, ws), (out_b, lse_b), S = _case(2, 28, 4, 6000, [6000, 4321], 5)
    rc, msg = _call("sq_decode_fwd_noalloc", q, k, v, sl, out_b, lse_b, 0)    # warm-up outside the capture
    assert rc == 0, msg
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        rc, msg = _call("sq_decode_fwd_noalloc", q, k, v, sl, out_b, lse_b, 0)
    assert rc == 0, msg
    g = torch.Generator(device=DEV).manual_seed(9)
    for rep in range(4):
        k.copy_(torch.randn(k.shape, device=DEV, generator=g).bfloat16())
        sl.copy_(torch.tensor([6000 - 100 * rep, 4321 + rep], dtype=torch.int32, device=DEV))
        junk = torch.randn(256, 256, device=DEV) @ torch.randn(256, 256, device=DEV)   # eager work between the replays
        torch.cuda.synchronize()
        out_b.fill_(float("nan"))
        graph.replay()
        rc, msg = _call("sq_decode_fwd", q, k, v, sl, out_a, lse_a, 0, ws)
        assert rc == 0, msg
        torch.cuda.synchronize()
        assert torch.equal(out_a, out_b) and torch.equal(lse_a, lse_b) and bool(torch.isfinite(junk).all()), rep
