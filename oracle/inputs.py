"""Seeded synthetic inputs: the generators live with the product's benchmark workloads; re-exported here
so that tests can say `oracle.inputs`.  TEST INFRASTRUCTURE ONLY (see `oracle/__init__.py`)."""
from longcontext_sqattn_paddle_amd.workloads import (  # noqa: F401
    decode_inputs, kmeans_inputs, plugin_inputs, prefill_inputs)
