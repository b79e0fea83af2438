"""Pins oracle/kv_cache.py (restatement of cache_hub/flash_attn_cache.py:153-256) without a GPU."""
import torch

from oracle import kv_cache as KC


def _states(B, T, H, D, seed, dtype=torch.bfloat16):
    g = torch.Generator().manual_seed(seed)
    return torch.randn(B, T, H, D, generator=g).to(dtype), torch.randn(B, T, H, D, generator=g).to(dtype)


def test_prefill_store_matches_element_loops_and_leaves_other_rows_alone():
    B, L, H, D, T, vs, b0 = 3, 11, 2, 8, 9, 4, 1
    ks, vs_ = _states(1, T, H, D, 1)
    kc = torch.full((B, L, H, D), 7.0, dtype=torch.bfloat16)
    vc = torch.full((B, L, H, D), -7.0, dtype=torch.bfloat16)
    n = KC.prefill_store(kc, vc, ks, vs_, b0, vs)
    assert n == T - vs
    for b in range(B):
        for r in range(L):
            for h in range(H):
                for d in range(D):
                    if b == b0 and r < n:
                        assert kc[b, r, h, d] == ks[0, vs + r, h, d] and vc[b, r, h, d] == vs_[0, vs + r, h, d]
                    else:
                        assert kc[b, r, h, d] == 7.0 and vc[b, r, h, d] == -7.0


def test_decode_append_positions_and_advance():
    B, L, H, D = 3, 6, 2, 8
    kc = torch.zeros(B, L, H, D, dtype=torch.bfloat16)
    vc = torch.zeros(B, L, H, D, dtype=torch.bfloat16)
    lens = torch.tensor([0, 3, 5], dtype=torch.int32)
    kn, vn = _states(B, 1, H, D, 2)
    att = KC.decode_append(kc, vc, kn, vn, lens, advance=False)
    assert att.tolist() == [1, 4, 6] and lens.tolist() == [0, 3, 5]      # not the last layer: lengths stay
    for b, pos in enumerate([0, 3, 5]):
        assert torch.equal(kc[b, pos], kn[b, 0]) and torch.equal(vc[b, pos], vn[b, 0])
        mask = torch.ones(L, dtype=torch.bool)
        mask[pos] = False
        assert float(kc[b, mask].abs().sum()) == 0.0 and float(vc[b, mask].abs().sum()) == 0.0
    att = KC.decode_append(kc, vc, kn, vn, lens, advance=True)           # last layer: same rows, then advance
    assert att.tolist() == [1, 4, 6] and lens.tolist() == [1, 4, 6]


def test_prefill_then_appends_reproduce_the_token_sequence():
    L, H, D, T, steps = 16, 2, 8, 7, 5
    ks, vs_ = _states(1, T + steps, H, D, 3)
    kc = torch.zeros(1, L, H, D, dtype=torch.bfloat16)
    vc = torch.zeros(1, L, H, D, dtype=torch.bfloat16)
    n = KC.prefill_store(kc, vc, ks[:, :T], vs_[:, :T], 0, 2)
    lens = torch.tensor([n], dtype=torch.int32)
    for s in range(steps):
        KC.decode_append(kc, vc, ks[:, T + s:T + s + 1], vs_[:, T + s:T + s + 1], lens, advance=True)
    assert int(lens[0]) == T - 2 + steps
    assert torch.equal(kc[0, :int(lens[0])], ks[0, 2:]) and torch.equal(vc[0, :int(lens[0])], vs_[0, 2:])
