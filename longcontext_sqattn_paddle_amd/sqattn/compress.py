"""Layer-by-layer window calibration (`sqattn/compress.py:123-194`, `sqattn/model_utils.py:79-94`).

`compress_model` walks the decoder layers: for every layer but the first and the last it measures the attention-energy
histograms of the calibration samples (`sqattn.window_search`), derives the per-head 8-bit / 4-bit windows, installs the
quantised-window attention closure with them (`sqattn.attn_replacer.mp_triton_wrapper`), and then advances the samples
through the layer so that the next layer is calibrated on what it will actually see.  Returns the reference's
`bits_alloc` dictionary, `{layer: {"bit8": [...], "bit4": [...], "sink": 256}}`, which `process_model` accepts as
`window_sizes`.

The reference fetches its calibration text with `datasets` (`sqattn/calibration.py`); there is no network here, so
the token samples are an argument.
"""
from __future__ import annotations

import types
from typing import Dict, List, Optional

import torch

from .attn_replacer import mp_triton_wrapper
from .window_search import calibrate_layer_windows

SINK_TOKENS = 256       # compress.py:173, 181
MAX_SAMPLE_TOKENS = 5000  # compress.py:145: samples are cut to this length


def get_layer_inputs(model, sample: torch.Tensor, args):
    """compress.py:34-60: the hidden states that enter the first decoder layer for one token sample [1, T], caught
    by the runtime's `capture_layer_inps` hook during a prefill-only `generate`."""
    caught: List[torch.Tensor] = []
    model.capture_layer_inps = caught
    try:
        model.generate(attention_type=args.attn_type, inputs_ids=sample, attention_masks=None, max_new_length=0, verbose=False)
    finally:
        model.capture_layer_inps = None
    torch.cuda.synchronize()
    return caught[0], {}


def batch_layer_infer(layer, batch_inps, batch_layer_kwargs, args, model=None, layer_idx=None):
    """model_utils.py:79-94: every sample through one layer.  (The reference returns from inside its loop, i.e. only
    the first sample's output as a bare tensor; here every sample advances and a list comes back.)"""
    outs = []
    for i, inps in enumerate(batch_inps):
        if inps.ndim == 2:
            inps = inps[None, :, :]
        if model is not None:
            outs.append(model.layer_prefill(layer_idx, 0, inps))
        else:
            outs.append(layer(inps, **(batch_layer_kwargs[i] if len(batch_layer_kwargs) > i else {})))
    return outs


def compress_model(model, tokenizer, device, args, raw_samples: Optional[List[torch.Tensor]] = None) -> Dict[int, dict]:
    """compress.py:123-194.  `raw_samples`: token id tensors [1, T] on the device (the reference builds them from
    `args.calib_dataset`).  `args` carries `attn_type`, `bit8_thres`, `bit4_thres`, optionally `use_relative_distance`,
    `relative_bins`, `sink_window_size`, plus what `mp_triton_wrapper` reads (`quant`, `qk_qtype`, `v_qtype`)."""
    if raw_samples is None:
        raise ValueError("compress_model needs raw_samples: loading a calibration dataset requires network access")
    if not isinstance(raw_samples, (list, tuple)):
        raw_samples = [raw_samples]
    layers = model.layers
    max_len = max(int(s.shape[1]) for s in raw_samples)
    samples_inps, samples_layer_kwargs = [], []
    for sample in raw_samples:
        inps, layer_kwargs = get_layer_inputs(model, sample[:, :MAX_SAMPLE_TOKENS], args)
        samples_inps.append(inps)
        samples_layer_kwargs.append(layer_kwargs)
    # one cache that holds the longest sample (each `generate` above sized it for its own sample)
    model.batch_size, model.max_new_length = 1, 0
    model.init_kv_cache(min(max_len, MAX_SAMPLE_TOKENS), [0])
    bits_alloc: Dict[int, dict] = {}
    for layer_idx, layer in enumerate(layers):
        if layer_idx not in (0, len(layers) - 1):
            _, _, head_windows = calibrate_layer_windows(layer, layer_idx, samples_inps, samples_layer_kwargs, max_len, args, model)
            bit8 = [hw["bit8_relative"] if "bit8_relative" in hw else hw["bit8"] for hw in head_windows]
            bit4 = [hw["bit4_relative"] if "bit4_relative" in hw else hw["bit4"] for hw in head_windows]
            bits_alloc[layer_idx] = {"bit8": bit8, "bit4": bit4, "sink": SINK_TOKENS}
            layer.prefill_attention = types.MethodType(
                mp_triton_wrapper(layer_idx, args=args, bit8_window_sizes=bit8, bit4_window_sizes=bit4, sink_window_size=SINK_TOKENS), layer)
        if layer_idx < len(layers) - 1:   # nothing reads the last layer's outputs (and its prefill would advance the cache's context)
            samples_inps = batch_layer_infer(layer, samples_inps, samples_layer_kwargs, args, model, layer_idx)
    return bits_alloc
