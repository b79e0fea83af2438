"""The committed fixtures of tests/golden are what the oracle produces today: the generator is run again with the file
writes captured and every array is compared with the file (bit patterns and integers exactly, floating-point outputs
to 1e-5, which leaves room for another BLAS summing in another order)."""
import importlib.util
import os

import numpy as np
import pytest

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def _generator():
    spec = importlib.util.spec_from_file_location("make_fixtures", os.path.join(GOLDEN, "make_fixtures.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


@pytest.mark.parametrize("name", ["prefill", "decode", "prepass", "kmeans", "window_search"])
def test_oracle_reproduces_fixture(name, monkeypatch):
    gen = _generator()
    captured = {}
    monkeypatch.setattr(gen.np, "savez_compressed", lambda path, **arrays: captured.update(path=path, arrays=arrays))
    getattr(gen, name)()
    with np.load(captured["path"], allow_pickle=False) as on_disk:
        assert sorted(on_disk.files) == sorted(captured["arrays"])
        for key, fresh in captured["arrays"].items():
            stored = on_disk[key]
            fresh = np.asarray(fresh)
            assert stored.shape == fresh.shape and stored.dtype == fresh.dtype, key
            if np.issubdtype(stored.dtype, np.floating):
                assert np.allclose(stored, fresh, rtol=1e-5, atol=1e-7, equal_nan=True), key
            else:
                assert np.array_equal(stored, fresh), key


def test_fixtures_are_plain_arrays():
    files = sorted(f for f in os.listdir(GOLDEN) if f.endswith(".npz"))
    assert files == ["decode_small.npz", "kmeans_small.npz", "prefill_small.npz", "prepass_small.npz", "window_search_small.npz"]
    for f in files:
        with np.load(os.path.join(GOLDEN, f), allow_pickle=False) as z:
            for key in z.files:
                assert z[key].dtype.kind in "fiu", (f, key)
