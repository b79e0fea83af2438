"""GPU parity of the drop-in boundary: `process_model` / `mp_triton_wrapper` closures against the oracle's
restatement of the reference closure (sqattn/attn_replacer.py:296-454), plus the fake quantisers."""
import types

import numpy as np

import pytest
import torch

from oracle import attention as A
from oracle import fake_quant as FQ
from oracle import inputs, plugin

pytestmark = pytest.mark.gpu
DEV = "cuda:0"


class _Layer:
    def __init__(self, groups):
        self.num_key_value_groups = groups

    def prefill_attention(self, q, k, v, layer_idx=None):
        raise AssertionError("not patched")


class _Model:
    def __init__(self, n, groups):
        self.layers = [_Layer(groups) for _ in range(n)]


def _args(relative, qk="int", v="int"):
    return types.SimpleNamespace(qk_qtype=qk, v_qtype=v, use_relative_distance=relative)


def _cos(a, b):
    a, b = a.double().flatten(), b.double().flatten()
    return float(a @ b / (a.norm() * b.norm()))


@pytest.mark.parametrize("qtype", ["int", "e4m3"])
def test_fake_quantisers_match_oracle(qtype):
    from longcontext_sqattn_paddle_amd.sqattn.fake_quant import FloatQuantizer, IntegerQuantizer

    x = torch.randn(2, 3, 50, 128, generator=torch.Generator().manual_seed(0)).bfloat16()
    xd = x.to(DEV)
    if qtype == "int":
        for bit, sym, gran in ((8, True, "per_token"), (4, True, "per_token"), (8, True, "per_channel"), (8, False, "per_channel")):
            got = IntegerQuantizer(bit, sym, gran).fake_quant_tensor(xd).cpu()
            assert torch.equal(got, FQ.int_fake_quant(x, bit, sym, gran)), (bit, sym, gran)
    else:
        for fmt, gran in (("e4m3", "per_token"), ("e5m2", "per_channel")):
            got = FloatQuantizer(fmt, True, gran).fake_quant_tensor(xd).cpu()
            ref = FQ.float_fake_quant(x, fmt, gran)
            # log2/exp2 on the device may differ by an ulp from the host's: allow rare one-step differences
            assert float((got.float() - ref.float()).abs().max()) <= float(ref.float().abs().max()) * 0.13
            assert float((got != ref).float().mean()) < 1e-3


def test_process_model_binds_and_skips_like_the_reference():
    from longcontext_sqattn_paddle_amd.sqattn.attn_replacer import process_model

    m = _Model(4, 4)
    ws = {1: {"bit8": 0.1, "bit4": 0.1, "sink": 64}, 2: {"bit8": [0.1] * 4, "bit4": [0.2] * 4, "sink": 64}}
    process_model(m, "SQAttn", ws, _args(True))
    assert "prefill_attention" not in vars(m.layers[0]) and "prefill_attention" in vars(m.layers[1])
    assert process_model(m, "SDPA") is m and process_model(m, "FlashAttn") is m
    with pytest.raises(ValueError):
        process_model(m, "Other")


@pytest.mark.parametrize("relative,bit8,bit4", [(True, 0.1, 0.1), (True, [0.05, 0.1, 0.2, 0.3], [0.4, 0.1, 0.2, 0.5]),
                                                (False, 256, 512), (False, [128, 256, 384, 2048], [256, 256, 640, 2048])])
def test_plugin_closure_matches_oracle(relative, bit8, bit4):
    from longcontext_sqattn_paddle_amd.sqattn.attn_replacer import process_model

    q, k, v = inputs.plugin_inputs(1, 4, 1, 2048, 128, seed=1)
    m = _Model(2, 4)
    process_model(m, "SQAttn", {1: {"bit8": bit8, "bit4": bit4, "sink": 0}}, _args(relative))
    out = m.layers[1].prefill_attention(q.to(DEV), k.to(DEV), v.to(DEV), None)
    torch.cuda.synchronize()
    assert out.shape == (1, 2048, 512) and out.dtype == torch.bfloat16
    ref = plugin.plugin_attention(q, k, v, num_kv_groups=4, bit8=bit8, bit4=bit4, sink=256, relative=relative)
    o, r = out.float().cpu(), ref.float()
    rms = float(r.pow(2).mean().sqrt())
    assert _cos(o, r) >= 0.99999
    # both sides round the same fp32 result to bf16: one bf16 ulp of the largest output plus kernel noise
    assert float((o - r).abs().max()) <= 2 ** -7 * float(r.abs().max()) + 2e-3 * rms


def test_plugin_closure_with_float_quantiser_types():
    """qk_qtype / v_qtype e4m3 (sqattn/attn_replacer.py:340-358) through the fused pre-pass and the windowed kernel."""
    from longcontext_sqattn_paddle_amd.sqattn.attn_replacer import process_model

    q, k, v = inputs.plugin_inputs(1, 4, 1, 1024, 128, seed=4)
    m = _Model(2, 4)
    process_model(m, "SQAttn", {1: {"bit8": 0.25, "bit4": 0.25, "sink": 0}}, _args(True, "e4m3", "e4m3"))
    out = m.layers[1].prefill_attention(q.to(DEV), k.to(DEV), v.to(DEV), None)
    torch.cuda.synchronize()
    ref = plugin.plugin_attention(q, k, v, num_kv_groups=4, bit8=0.25, bit4=0.25, sink=256, relative=True, qk_qtype="e4m3", v_qtype="e4m3")
    o, r = out.float().cpu(), ref.float()
    assert _cos(o, r) >= 0.9999
    assert float((o - r).abs().max()) <= 2 ** -7 * float(r.abs().max()) + 5e-3 * float(r.pow(2).mean().sqrt())
    with pytest.raises(ValueError):
        process_model(m, "SQAttn", {1: {"bit8": 0.25, "bit4": 0.25, "sink": 0}}, _args(True, "fp4", "int"))
        m.layers[1].prefill_attention(q.to(DEV), k.to(DEV), v.to(DEV), None)


def test_process_model_takes_the_window_sizes_the_reference_calibration_writes():
    """The reference's window search returns 1 token when a head's histogram is empty and the histogram's length when the
    threshold is never reached (sqattn/window_search.py:90-128), and its configuration keeps a 256-token sink: a
    configuration like that must run (sizes rounded as documented: 1 -> 128, 1000 -> 1024), not raise."""
    from longcontext_sqattn_paddle_amd.sqattn.attn_replacer import process_model

    q, k, v = inputs.plugin_inputs(1, 4, 1, 1536, 128, seed=3)
    m = _Model(2, 4)
    process_model(m, "SQAttn", {1: {"bit8": [1, 1, 1000, 5000], "bit4": [1, 1000, 1000, 5000], "sink": 256}}, _args(False))
    out = m.layers[1].prefill_attention(q.to(DEV), k.to(DEV), v.to(DEV), None)
    torch.cuda.synchronize()
    ref = plugin.plugin_attention(q, k, v, num_kv_groups=4, bit8=[128, 128, 1024, 5120], bit4=[128, 1024, 1024, 5120], sink=256, relative=False)
    o, r = out.float().cpu(), ref.float()
    assert _cos(o, r) >= 0.99999
    assert float((o - r).abs().max()) <= 2 ** -7 * float(r.abs().max()) + 2e-3 * float(r.pow(2).mean().sqrt())


def test_config1_full_causal_with_block_fp8_p():
    """Benchmark configuration 1: seq 4096, 4 q-heads on 1 kv head, int8 fake-quant, windows >= N (full causal),
    P quantised to e4m3 with per-64x64-block absmax scales (a mode the reference closure itself never enables)."""
    from longcontext_sqattn_paddle_amd import _native as N
    from longcontext_sqattn_paddle_amd.sqattn.attn_replacer import mp_triton_wrapper

    q, k, v = inputs.plugin_inputs(1, 4, 1, 4096, 128, seed=1)
    fn = mp_triton_wrapper(0, bit8_window_sizes=2.0, bit4_window_sizes=2.0, sink_window_size=256, args=_args(True))
    out = fn(_Layer(4), q.to(DEV), k.to(DEV), v.to(DEV), None, p_quant=N.P_E4M3_BLOCK)
    torch.cuda.synchronize()
    ref = plugin.plugin_attention(q, k, v, num_kv_groups=4, bit8=2.0, bit4=2.0, sink=256, relative=True, p_quant=A.P_BLOCK_ABSMAX)
    o, r = out.float().cpu(), ref.float()
    assert _cos(o, r) >= 0.99995
    exact, _ = A.exact_attention(q.permute(0, 2, 1, 3), k.permute(0, 2, 1, 3), v.permute(0, 2, 1, 3))
    e = exact.permute(0, 2, 1, 3).reshape(1, 4096, 512)
    assert _cos(o, e) >= 0.999   # int8 Q/K/V + e4m3 P against exact attention: the benchmark's stated bar


def test_decode_slot():
    from longcontext_sqattn_paddle_amd.sqattn.attn_replacer import decode_attention_fn

    q, kc, vc, lens = inputs.decode_inputs(2, 8, 2, 1024, 128, seed=9)
    lens_d = lens.to(DEV)
    out = decode_attention_fn(_Layer(4), q.to(DEV), kc.to(DEV), vc.to(DEV), None, seqlens=lens_d)[0]
    torch.cuda.synchronize()
    ref, _ = A.exact_attention(q.permute(0, 2, 1, 3), kc.permute(0, 2, 1, 3), vc.permute(0, 2, 1, 3), causal=False,
                               kv_lens=[int(x) for x in lens])
    assert out.shape == (2, 1, 8 * 128)
    assert _cos(out.float().cpu(), ref.permute(0, 2, 1, 3).reshape(2, 1, 1024)) >= 0.9999


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("layout", ["NHD", "HND"])
def test_query_quantised_while_loaded_equals_the_separate_pass(dtype, layout):
    """sq_prefill_params.q_quant = 8: the 8-bit per-token fake quantisation of the query rows inside the attention kernel
    gives the output bits of the same kernel on a query that went through sq_fake_quant_prepass -- for rows with large and
    tiny ranges, an all-zero row, GQA, a length that is not a multiple of the tile."""
    from longcontext_sqattn_paddle_amd.sqattn.attn_triton_mix_relative import attn_hierarchical_relative_window
    from longcontext_sqattn_paddle_amd.sqattn.fake_quant import fused_int_prepass

    B, N, Hq, Hkv, D = 2, 1100, 14, 2, 128
    g = torch.Generator().manual_seed(321)
    q = torch.randn(B, N, Hq, D, generator=g) * torch.logspace(-6, 2, N)[None, :, None, None]   # row ranges from 1e-6 to 100
    q[0, 5] = 0.0
    q[1, 7, 3] = 1e-7
    k = torch.randn(B, N, Hkv, D, generator=g)
    v = torch.randn(B, N, Hkv, D, generator=g)
    q, k, v = (t.to(dtype).to(DEV) for t in (q, k, v))
    if layout == "HND":
        q, k, v = (t.permute(0, 2, 1, 3).contiguous() for t in (q, k, v))
    q8, _, k8, _, v8 = fused_int_prepass(q, k, v, want_4bit=False, tensor_layout=layout)
    none, _, k8b, _, v8b = fused_int_prepass(q, k, v, want_4bit=False, tensor_layout=layout, skip_query=True)
    assert none is None and torch.equal(k8, k8b) and torch.equal(v8, v8b)
    two, lse2 = attn_hierarchical_relative_window(q8, k8, q8, k8, v8, 0.25, 0.5, 128, layout, torch.float32, return_lse=True)
    one, lse1 = attn_hierarchical_relative_window(q, k8, q, k8, v8, 0.25, 0.5, 128, layout, torch.float32, return_lse=True, q_quant=8)
    torch.cuda.synchronize()
    assert torch.equal(one.view(torch.int32), two.view(torch.int32)) and torch.equal(lse1.view(torch.int32), lse2.view(torch.int32))
    with pytest.raises(ValueError):
        attn_hierarchical_relative_window(q, k8, q, k8, v8, 0.25, 0.5, 128, layout, torch.float32, q_quant=4)
    with pytest.raises(ValueError):
        fused_int_prepass(q, k, v, want_4bit=True, tensor_layout=layout, skip_query=True)


@pytest.mark.parametrize("bit8,bit4,N,Hq,Hkv", [(0.1, 0.1, 2048, 4, 1), ([0.05, 0.1, 0.2, 0.3], [0.4, 0.1, 0.2, 0.5], 2048, 4, 2),
                                                 (2.0, 2.0, 700, 14, 2), (0.25, 0.5, 4096, 4, 1)])
def test_integer_qk_closure_matches_its_oracle(bit8, bit4, N, Hq, Hkv):
    """args.int8_qk: Q.K^T on the int8 matrix instruction (codes of the query formed in the kernel, codes and scales of
    the centred key from sq_fake_quant_prepass_int8qk) against the oracle's integer-product restatement: both round the
    same fp32 result to bf16, so one bf16 step of the largest output plus kernel noise; and against the reference's
    fake-quantised bf16 product it stays within the two bf16 roundings that path applies to its operands (cosine, 1 % band).
    The last case is benchmark configuration 1's shape (4 q heads / 1 kv head, 4096 tokens) with windows."""
    from longcontext_sqattn_paddle_amd.sqattn.attn_replacer import process_model

    print(f"case int8 qk closure N={N} Hq={Hq} Hkv={Hkv} bit8={bit8} bit4={bit4}", flush=True)
    q, k, v = inputs.plugin_inputs(1, Hq, Hkv, N, 128, seed=3)
    args = _args(True)
    args.int8_qk = True
    m = _Model(2, Hq // Hkv)
    process_model(m, "SQAttn", {1: {"bit8": bit8, "bit4": bit4, "sink": 0}}, args)
    out = m.layers[1].prefill_attention(q.to(DEV), k.to(DEV), v.to(DEV), None)
    torch.cuda.synchronize()
    assert out.shape == (1, N, Hq * 128) and out.dtype == torch.bfloat16
    ref = plugin.plugin_attention(q, k, v, num_kv_groups=Hq // Hkv, bit8=bit8, bit4=bit4, sink=256, relative=True, int8_qk=True)
    o, r = out.float().cpu(), ref.float()
    rms = float(r.pow(2).mean().sqrt())
    assert _cos(o, r) >= 0.99999
    assert float((o - r).abs().max()) <= 2 ** -7 * float(r.abs().max()) + 2e-3 * rms
    fake = plugin.plugin_attention(q, k, v, num_kv_groups=Hq // Hkv, bit8=bit8, bit4=bit4, sink=256, relative=True).float()
    assert _cos(o, fake) >= 0.9999 and float((o - fake).abs().max()) <= 0.01 * float(fake.abs().max()) + 0.02 * rms
    with pytest.raises(ValueError):
        bad = _args(False)
        bad.int8_qk = True
        process_model(m, "SQAttn", {1: {"bit8": 256, "bit4": 256, "sink": 0}}, bad)
        m.layers[1].prefill_attention(q.to(DEV), k.to(DEV), v.to(DEV), None)


def test_integer_qk_closure_configurations_drawn_at_random():
    """Eight closure configurations with args.int8_qk drawn from a seeded generator: batch, GQA ratio, ragged lengths,
    per-head window ratios (4-bit wider or narrower than 8-bit), bf16 / fp16, query rows whose ranges span eight decades,
    an all-zero query row and an all-zero key row; each against the integer-product oracle."""
    from longcontext_sqattn_paddle_amd.sqattn.attn_replacer import process_model

    rng = np.random.default_rng(20240611)
    for case in range(8):
        B = int(rng.choice([1, 2]))
        Hkv = int(rng.choice([1, 2, 4]))
        group = int(rng.choice([1, 2, 4, 7]))
        Hq = Hkv * group
        N = int(rng.integers(130, 1500))
        dtype = torch.bfloat16 if rng.random() < 0.6 else torch.float16
        bit8 = [float(rng.choice([0.05, 0.1, 0.25, 0.5, 1.0])) for _ in range(Hq)]
        bit4 = [float(rng.choice([0.05, 0.1, 0.3, 0.6, 1.0])) for _ in range(Hq)]
        print(f"case {case}: B={B} Hq={Hq} Hkv={Hkv} N={N} {dtype} bit8={bit8} bit4={bit4}", flush=True)
        g = torch.Generator().manual_seed(1000 + case)
        q = torch.randn(B, N, Hq, 128, generator=g) * torch.logspace(-4, 1.5, N)[torch.randperm(N, generator=g)][None, :, None, None]
        k = torch.randn(B, N, Hkv, 128, generator=g) + 0.5 * torch.randn(1, 1, Hkv, 128, generator=g)
        v = torch.randn(B, N, Hkv, 128, generator=g)
        q[0, N // 3, 0] = 0.0
        k[0, N // 2, 0] = 0.0
        q, k, v = q.to(dtype), k.to(dtype), v.to(dtype)
        args = _args(True)
        args.int8_qk = True
        m = _Model(2, group)
        process_model(m, "SQAttn", {1: {"bit8": bit8, "bit4": bit4, "sink": 0}}, args)
        out = m.layers[1].prefill_attention(q.to(DEV), k.to(DEV), v.to(DEV), None)
        torch.cuda.synchronize()
        assert out.shape == (B, N, Hq * 128) and out.dtype == torch.bfloat16   # attn_replacer.py:434: bf16 whatever the inputs
        ref = plugin.plugin_attention(q, k, v, num_kv_groups=group, bit8=bit8, bit4=bit4, sink=256, relative=True, int8_qk=True)
        o, r = out.float().cpu(), ref.to(torch.bfloat16).float()
        assert torch.isfinite(o).all()
        rms = float(r.pow(2).mean().sqrt())
        assert _cos(o, r) >= 0.99999, case
        assert float((o - r).abs().max()) <= 2 ** -7 * float(r.abs().max()) + 2e-3 * rms, case



@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
def test_delayed_sdpa_wrapper_quantised_branch_on_the_device(dtype):
    """The masked-SDPA emulation of the mixed-precision windows (attn_replacer.py:36-190) with its operands on the GPU:
    key centring, the five fake-quantisers, the [L, 2L] mask (scalar and per-head windows) and SDPA over
    [8-bit keys ; 4-bit keys], against the oracle's float64 restatement.  Tolerance: fp32 operands 1e-3 absolute (the
    library's SDPA accumulates in fp32, and the key mean's summation order may move an element across a rounding boundary
    of its quantiser; a wrong mask or operand shows at 1e-2 and more); bf16 operands cosine >= 0.9995 and 3e-2 of the largest output (bf16 scores)."""
    from longcontext_sqattn_paddle_amd.sqattn.attn_replacer import construct_mix_bit_mask, delayed_sdpa_wrapper
    from oracle import plugin

    print(f"case delayed_sdpa_wrapper on the device, {dtype}", flush=True)
    g = torch.Generator().manual_seed(5)
    q, k, v = (torch.randn(2, 3, 80, 64, generator=g).to(dtype) for _ in range(3))
    k = (k.float() + 0.7).to(dtype)
    args = types.SimpleNamespace(quant=True, qk_qtype="int", v_qtype="int", vis_attn=False)
    for w8, w4, sink in ((6, 10, 4), ([4, 9, 80], [8, 0, 5], 2), (1, 0, 0)):
        out = delayed_sdpa_wrapper(0, w8, w4, sink, args)(None, q.to(DEV), k.to(DEV), v.to(DEV), None, scaling=1.0)
        torch.cuda.synchronize()
        assert out.is_cuda and out.shape == (2, 80, 3 * 64)
        ref = plugin.masked_sdpa_emulation(q, k, v, bit8_window=w8, bit4_window=w4, sink=sink)
        got = out.cpu().view(2, 80, 3, 64).permute(0, 2, 1, 3).double()
        if dtype == torch.float32:
            assert float((got - ref).abs().max()) < 1e-3, (w8, w4)
        else:
            assert _cos(got, ref) >= 0.9995 and float((got - ref).abs().max()) <= 3e-2 * float(ref.abs().max()), (w8, w4)
        assert torch.equal(construct_mix_bit_mask(80, w8, w4, sink, DEV).cpu(), plugin.mix_bit_mask(80, w8, w4, sink))
    # the plain branch on the device: SDPA with the caller's mask
    plain = delayed_sdpa_wrapper(0, 0, 0, 0, types.SimpleNamespace(quant=False))(None, q.to(DEV), k.to(DEV), v.to(DEV), None, tensor_layout="HND")
    want = torch.nn.functional.scaled_dot_product_attention(q.double(), k.double(), v.double(), is_causal=True).transpose(1, 2).reshape(2, 80, 192)
    assert float((plain.cpu().double() - want).abs().max()) <= (1e-4 if dtype == torch.float32 else 3e-2 * float(want.abs().max()))
