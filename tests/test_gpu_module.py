"""GPU tests of the module layer: DynamicLinear / SwitchLinear forward through every lane against
the oracle's switched_forward, LUT-driven dispatch, temp-cache behaviour and the profiler loop."""
import json
import os

import numpy as np
import pytest

torch = pytest.importorskip("torch")
from oracle import kairos_oracle as O

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def gpu():
    if not torch.cuda.is_available():
        pytest.skip("no GPU")
    return torch.device("cuda")


def make_linear(N, K, bias, seed=10):
    w = O.synth_weights(N, K, seed)
    lin = torch.nn.Linear(K, N, bias=bias, dtype=torch.float16)
    with torch.no_grad():
        lin.weight.copy_(torch.from_numpy(w))
        if bias:
            lin.bias.copy_(torch.from_numpy(np.random.default_rng(seed).standard_normal(N).astype(np.float16)))
    return lin, w


@pytest.mark.parametrize("cls_name", ["DynamicLinear", "SwitchLinear"])
@pytest.mark.parametrize("bias", [False, True])
def test_every_lane_matches_oracle(gpu, cls_name, bias):
    from kairos.dynamic_linear_v2 import COMP_TYPE_NAME, DynamicLinear      # ids 0..7: version 2 adds 6 and 7
    from kairos.switch_linear import SwitchLinear
    cls = {"DynamicLinear": DynamicLinear, "SwitchLinear": SwitchLinear}[cls_name]
    N, K = 256, 1024
    lin, w = make_linear(N, K, bias)
    dl = cls.from_module(lin.cuda(), 'cuda')
    prep = O.prepare_weights(w)
    for key in ("qweight", "scales", "scaled_zeros", "scales_to8", "scaled_zeros_to8", "scales_1"):
        got = getattr(dl, key).cpu().numpy()
        assert np.array_equal(got.view(np.uint16), prep[key].view(np.uint16)), key   # GPU-side prep == oracle
    b = lin.bias.detach().cpu().numpy() if bias else None
    for M in (1, 9, 40, 200):
        x = O.synth_acts(M, K, seed=M)
        xd = torch.from_numpy(x).cuda()[None]
        for name, cid in COMP_TYPE_NAME.items():
            out = dl._forward(xd, M, cid)
            assert out.shape == (1, M, N) and out.dtype == torch.float16
            ref = O.switched_forward(x, prep, cid, bias=b)
            err = O.max_abs_rel(out[0].cpu().numpy(), ref)
            assert err < 1e-2, (name, M, err)
            if name in ("w8a8", "w4a8_qserve"):
                assert np.array_equal(out[0].cpu().numpy().view(np.uint16), ref.view(np.uint16))


def test_forward_uses_lut_and_counts_switches(gpu, tmp_path):
    from kairos.dynamic_linear import COMP_TYPE_NAME, DynamicLinear
    from kairos.perf_profiler import Profiler
    N, K = 256, 512
    prof = Profiler([(N, K)])
    for r, name in [(4, 'w4a16_gemv'), (64, 'w4a16_gemm'), (512, 'w8a8'), (4096, 'fp16')]:
        prof.record_best_comp((N, K), r, name)
    old = DynamicLinear.prof
    DynamicLinear.prof = prof
    try:
        lin, w = make_linear(N, K, False)
        dl = DynamicLinear.from_module(lin.cuda(), 'cuda')
        prep = O.prepare_weights(w)
        seen = []
        for B, S in [(1, 1), (1, 4), (2, 3), (2, 32), (4, 100), (3, 300), (1, 2)]:
            x = O.synth_acts(B * S, K, seed=B * S)
            out = dl(torch.from_numpy(x).cuda().reshape(B, S, K))
            assert out.shape == (B, S, N)
            m = B * S
            want = prof.get_comp_type((N, K), m)
            assert dl.comp_type == want and dl.pre_m == m
            seen.append(want)
            ref = O.switched_forward(x, prep, want)
            assert O.max_abs_rel(out.reshape(m, N).cpu().numpy(), ref) < 1e-2
        assert seen == [1, 1, 0, 0, 2, 5, 1]
        assert dl.switch_count == 4
    finally:
        DynamicLinear.prof = old


def test_small_m_call_in_forward_agrees_with_the_general_path(gpu):
    """forward() serves decode-sized fp16 calls itself (one allocation, one C call).  Inputs it does not take -- a
    strided view, a tracer installed, a replaced weight tensor -- go the general way; all of them give the same bits,
    with and without a bias, and the cached pointers follow a weight that was replaced."""
    from kairos.dynamic_linear import COMP_TYPE_NAME, DynamicLinear
    from kairos.perf_profiler import Profiler
    from kairos_amd import ops
    N, K = 256, 512
    prof = Profiler([(N, K)])
    prof.record_best_comp((N, K), 64, 'w4a16_gemv')
    prof.record_best_comp((N, K), 4096, 'w8a8')
    old = DynamicLinear.prof
    DynamicLinear.prof = prof
    try:
        for bias in (False, True):
            lin, w = make_linear(N, K, bias)
            dl = DynamicLinear.from_module(lin.cuda(), 'cuda')
            x = torch.from_numpy(O.synth_acts(6, K, seed=3)).cuda().reshape(2, 3, K)
            fast = dl(x)
            assert fast.shape == (2, 3, N) and dl.comp_type == COMP_TYPE_NAME['w4a16_gemv'] and dl._decode_ptrs is not None
            general = dl._forward(x.reshape(-1, K), 6, dl.comp_type).reshape(2, 3, N)
            assert torch.equal(fast, general)
            wide = torch.zeros((2, 3, 2 * K), dtype=torch.float16, device='cuda')
            wide[..., :K] = x
            assert not wide[..., :K].is_contiguous() and torch.equal(dl(wide[..., :K]), fast)      # strided view
            calls = []

            class Tracer:
                def begin(self, name, M, N_, K_):
                    calls.append((name, M, N_, K_))

                def end(self):
                    pass
            ops.set_tracer(Tracer())
            try:
                assert torch.equal(dl(x), fast) and calls == [("gemv_w4a16", 6, N, K)]            # traced: general path
            finally:
                ops.set_tracer(None)
            # a replaced weight: the cached raw pointers must not outlive it
            lin2, _ = make_linear(N, K, bias, seed=99)
            other = DynamicLinear.from_module(lin2.cuda(), 'cuda')
            dl.load_state_dict(other.state_dict())
            assert torch.equal(dl(x), other(x))
    finally:
        DynamicLinear.prof = old


def test_temp_cache_reuse_and_bound(gpu):
    from kairos.dynamic_linear import COMP_TYPE_NAME, DynamicLinear
    from kairos_amd.temp_cache import TempCache
    cache = TempCache()
    a = DynamicLinear.from_module(make_linear(256, 512, False, 1)[0].cuda(), 'cuda')
    b = DynamicLinear.from_module(make_linear(128, 1024, False, 2)[0].cuda(), 'cuda')
    a.temp_cache = b.temp_cache = cache
    x5 = torch.randn(1, 70, 512, dtype=torch.float16, device='cuda')
    xb = torch.randn(1, 70, 1024, dtype=torch.float16, device='cuda')
    o1 = a._forward(x5, 70, COMP_TYPE_NAME['w8a8'])
    o2 = a._forward(x5, 70, COMP_TYPE_NAME['w8a8'])
    assert cache.misses == 1 and cache.hits == 1 and torch.equal(o1, o2)
    o3 = a._forward(x5, 70, COMP_TYPE_NAME['fp16'])              # other format: converts again
    assert cache.misses == 2
    b._forward(xb, 70, COMP_TYPE_NAME['fp16'])                   # other layer evicts
    o4 = a._forward(x5, 70, COMP_TYPE_NAME['fp16'])
    assert cache.misses == 4 and torch.equal(o3, o4)
    assert cache.peak_bytes == 256 * 512 * 2 == max(256 * 512, 128 * 1024) * 2
    assert cache.capacity == cache.peak_bytes                    # one buffer, sized by the largest request


def test_profiler_builds_a_table(gpu, tmp_path):
    from kairos.perf_profiler import Profiler
    prof = Profiler([(256, 512)])
    details = []
    prof.profiling(input_len=[1, 16, 64, 128, 512], n=5, preheat_time=2, details=details)
    seg = prof.seg_perf_list[0]
    assert seg[-1][0] == 512 and all(t[1] in O.COMP_TYPE_NAME for t in seg)
    assert not any(d["comp"] == "w4a16_gemv" and d["m"] > 64 for d in details)
    assert {d["comp"] for d in details} == {'fp16', 'w4a16_gemm', 'w4a16_gemv', 'w8a8', 'w8a16_gemm'}
    prof.save(str(tmp_path) + "/")
    again = Profiler([(256, 512)])
    again.load(str(tmp_path) + "/")
    for m in (1, 16, 17, 100, 512, 5000):
        assert again.get_comp_type((256, 512), m) == prof.get_comp_type((256, 512), m)
    text = open(tmp_path / "seg_perf_list.pt").read()
    assert json.loads(text) == prof.seg_perf_list


@pytest.mark.gpu
def test_graph_replay_matches_eager():
    """A captured layer step replays to the eager bits, several times, with eager work between the replays."""
    import torch
    from kairos_amd.dynamic_linear import DynamicLinear
    from kairos_amd.graphed import GraphedCallable

    class FixedLut:                      # small-M lane for the first linear, W8A8 (conversion in the graph) for the second
        def __init__(self): self.table = {}
        def get_comp_type(self, shape, m): return self.table[shape]

    torch.manual_seed(3)
    l1 = DynamicLinear.from_module(torch.nn.Linear(512, 256, bias=True, dtype=torch.float16), device="cuda")
    l2 = DynamicLinear.from_module(torch.nn.Linear(256, 384, bias=False, dtype=torch.float16), device="cuda")
    l3 = DynamicLinear.from_module(torch.nn.Linear(512, 128, bias=False, dtype=torch.float16), device="cuda")
    lut = FixedLut()
    lut.table = {(256, 512): 1, (384, 256): 2, (128, 512): 2}
    old = DynamicLinear.prof
    DynamicLinear.prof = lut
    try:
        def step(x):
            return l2(l1(x)), l3(x)
        xs = [torch.randn(1, 8, 512, device="cuda", dtype=torch.float16) for _ in range(4)]
        eager = [tuple(t.clone() for t in step(x)) for x in xs]
        g = GraphedCallable(step, [xs[0]])
        for rep in range(3):
            for x, want in zip(xs, eager):
                got = g(x)
                assert all(torch.equal(a, b) for a, b in zip(got, want)), f"replay {rep}"
                # eager work on another layer in between: it overwrites the shared temp cache
                again = step(xs[(rep + 1) % 4])
                assert all(torch.equal(a, b) for a, b in zip(again, eager[(rep + 1) % 4]))
                torch.cuda.synchronize()
        assert g.replays == 12
    finally:
        DynamicLinear.prof = old


@pytest.mark.parametrize("bias", [False, True])
def test_version2_layer_with_the_reference_w4a8_operands(gpu, bias, tmp_path):
    """from_module(..., qserve_factors=True): id 7 multiplies the resident nibbles with the integer factors and the
    per-channel scale of the second quantiser, as kairos/dynamic_linear_v2.py:103,161-179 does -- the oracle's
    restatement of that GEMM bit for bit, the other lanes untouched, and the three extra tensors travel in the state dict."""
    from kairos.dynamic_linear_v2 import COMP_TYPE_NAME, DynamicLinear
    N, K = 256, 1024
    lin, w = make_linear(N, K, bias, seed=31)
    plain = DynamicLinear.from_module(lin.cuda(), 'cuda')
    dl = DynamicLinear.from_module(lin, 'cuda', qserve_factors=True)
    w8, s1 = O.qserve_quantize_int8(w)
    _, si, zi = O.qserve_quantize_int4(w8)
    S, Z = O.qserve_tables(si, zi, N)
    assert np.array_equal(dl.qserve_s2_scales.cpu().numpy(), S) and np.array_equal(dl.qserve_s2_zeros.cpu().numpy(), Z)
    assert np.array_equal(dl.qserve_s1_scales.cpu().numpy().view(np.uint16), s1.reshape(-1).view(np.uint16))
    prep = O.prepare_weights(w)
    b = lin.bias.detach().cpu().numpy() if bias else None
    outs = {}
    for M in (5, 150):
        x = O.synth_acts(M, K, seed=M)
        xd = torch.from_numpy(x).cuda()[None]
        a8, sx = O.quant_act_i8(x)
        ref = O.gemm_w4a8_int(a8, prep["qweight"], S, Z, s1.reshape(-1), sx)[1]
        if b is not None:
            ref = (ref.astype(np.float32) + b.astype(np.float32)).astype(np.float16)
        out = dl._forward(xd, M, COMP_TYPE_NAME['w4a8_qserve'])
        assert np.array_equal(out[0].cpu().numpy().view(np.uint16), ref.view(np.uint16))
        outs[M] = (xd, out.clone())
        # nibbles of one quantiser, factors of another (as in the reference): only roughly the fp16 product -- a sanity
        # bound that a wrong table or a swapped operand would break, not a parity claim
        assert O.max_abs_rel(out[0].cpu().numpy(), O.switched_forward(x, prep, COMP_TYPE_NAME['fp16'], bias=b)) < 0.3
        for cid in (COMP_TYPE_NAME['w8a8'], COMP_TYPE_NAME['w4a16_gemm']):
            assert torch.equal(dl._forward(xd, M, cid), plain._forward(xd, M, cid))
    assert set(dl.state_dict()) - set(plain.state_dict()) == {"qserve_s1_scales", "qserve_s2_scales", "qserve_s2_zeros"}
    path = tmp_path / "v2.pt"
    torch.save(dl.state_dict(), path)
    fresh = DynamicLinear(K, N, bias, 'cuda', 128)                # the plain constructor: shapes come from the file
    fresh.load_state_dict(torch.load(path, weights_only=True))
    for M, (xd, ref) in outs.items():
        assert torch.equal(fresh._forward(xd, M, COMP_TYPE_NAME['w4a8_qserve']), ref)


@pytest.mark.parametrize("cls_name", ["DynamicLinear", "SwitchLinear"])
def test_checkpoint_round_trip_keeps_every_lane(gpu, cls_name, tmp_path):
    """Dump a quantised layer, load it into an init_only module (on the CPU, then moved to the GPU, as
    utils/load_model.py:15-29 does) and into a live module that holds other weights: every lane returns the bits of
    the original, and nothing derived from the replaced weights (temp-cache entries, resident copies) survives."""
    from kairos.dynamic_linear import COMP_TYPE_NAME, DynamicLinear
    from kairos.switch_linear import SwitchLinear
    cls = {"DynamicLinear": DynamicLinear, "SwitchLinear": SwitchLinear}[cls_name]
    N, K = 256, 1024
    lin, _ = make_linear(N, K, True, seed=21)
    src = cls.from_module(lin.cuda(), 'cuda')
    xs = {M: torch.from_numpy(O.synth_acts(M, K, seed=M)).cuda()[None] for M in (3, 70, 300)}
    want = {(M, cid): src._forward(x, M, cid).clone() for M, x in xs.items() for cid in COMP_TYPE_NAME.values()}
    path = tmp_path / "layer.pt"
    torch.save(src.state_dict(), path)

    fresh = cls.from_module(lin, 'cpu', init_only=True)
    fresh.load_state_dict(torch.load(path, weights_only=True))
    fresh = fresh.cuda()
    other, _ = make_linear(N, K, True, seed=22)
    live = cls.from_module(other.cuda(), 'cuda')
    for M, x in xs.items():                                  # fill caches / resident copies with the OTHER weights
        live._forward(x, M, COMP_TYPE_NAME['w8a8'])
        live._forward(x, M, COMP_TYPE_NAME['fp16'])
    live.load_state_dict(torch.load(path, weights_only=True))
    for mod in (fresh, live):
        for (M, cid), ref in want.items():
            out = mod._forward(xs[M], M, cid)
            assert torch.equal(out.view(torch.int16), ref.view(torch.int16)), (cls_name, M, cid)


def test_resident_cache_skips_conversions_and_keeps_results(gpu):
    """Two layers alternating through the W8A8 and fp16 lanes: with the single shared buffer every call converts,
    with an LRU cache that holds all four copies only the first call of each (layer, format) does; same bits."""
    from kairos.dynamic_linear import COMP_TYPE_NAME, DynamicLinear
    from kairos_amd.temp_cache import ResidentCache, TempCache
    layers = [DynamicLinear.from_module(make_linear(256, 512, False, s)[0].cuda(), 'cuda') for s in (31, 32)]
    x = torch.from_numpy(O.synth_acts(70, 512, seed=5)).cuda()[None]
    lanes = (COMP_TYPE_NAME['w8a8'], COMP_TYPE_NAME['fp16'])

    def run(cache, rounds=3):
        outs = []
        for dl in layers:
            dl.temp_cache = cache
        for _ in range(rounds):
            for dl in layers:
                for cid in lanes:
                    outs.append(dl._forward(x, 70, cid).clone())
        return outs

    single = TempCache()
    want = run(single)
    assert single.hits == 0 and single.misses == 12
    lru = ResidentCache(4 * 256 * 512 * 2)
    got = run(lru)
    assert lru.misses == 4 and lru.hits == 8 and lru.capacity <= lru.capacity_limit
    small = ResidentCache(256 * 512 * 3)                     # room for one int8 and one fp16 copy: thrashes, still right
    got_small = run(small)
    assert small.capacity <= small.capacity_limit and small.misses > 4
    for a, b, c in zip(want, got, got_small):
        assert torch.equal(a.view(torch.int16), b.view(torch.int16)) and torch.equal(a.view(torch.int16), c.view(torch.int16))
    for dl in layers:
        dl.temp_cache = None


def test_quantized_llama_matches_dequantised_model(gpu):
    """Model surgery end to end (kairos/quant_model.py:29-56) on a tiny random Llama from transformers: the logits of
    the quantised model, with the table sending a short prompt to the small-M lane and a longer one to the W4A16
    GEMM, match an fp16 model whose linear weights are the oracle's dequantised weights; the W8A8 lane (activations
    quantised as well) stays within the looser bound its int8 activations imply."""
    transformers = pytest.importorskip("transformers")
    from kairos.dynamic_linear import DynamicLinear
    from kairos.perf_profiler import Profiler
    from kairos.quant_model import get_name_linears, quantize_model
    torch.manual_seed(0)
    cfg = transformers.LlamaConfig(hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=4,
                                   num_key_value_heads=2, vocab_size=128, max_position_embeddings=256)
    model = transformers.LlamaForCausalLM(cfg).half().cuda().eval()
    ref = transformers.LlamaForCausalLM(cfg).half().cuda().eval()
    ref.load_state_dict(model.state_dict())
    for layer in ref.model.layers:                       # the reference model computes with what the int4 tensors hold
        for m in get_name_linears(layer).values():
            p = O.prepare_weights(m.weight.detach().cpu().numpy())
            m.weight.data.copy_(torch.from_numpy(O.dequant_to_f16(p["qweight"], p["scales"], p["scaled_zeros"])))
    shapes = sorted({tuple(m.weight.shape) for layer in model.model.layers for m in get_name_linears(layer).values()})
    prof = Profiler(shapes)
    for s in shapes:
        for r, name in [(8, 'w4a16_gemv'), (64, 'w4a16_gemm'), (4096, 'w8a8')]:
            prof.record_best_comp(s, r, name)
    old = DynamicLinear.prof
    DynamicLinear.prof = prof
    try:
        quantize_model(model)
        with torch.no_grad():
            for T, tol in ((5, 1e-2), (40, 1e-2), (100, 6e-2)):
                ids = torch.randint(0, 128, (1, T), device="cuda", generator=torch.Generator(device="cuda").manual_seed(T))
                got = model(ids).logits.float()
                want = ref(ids).logits.float()
                assert torch.isfinite(got).all()
                err = ((got - want).abs().max() / want.abs().max()).item()
                assert err < tol, (T, err)
    finally:
        DynamicLinear.prof = old


def test_split_k_result_does_not_depend_on_the_calling_thread(gpu):
    """The split-K scratch travels with every call, so a GEMM issued from a second host thread splits exactly as
    on the main thread and returns the same bits (fp16 lanes: same fp32 summation order)."""
    import threading
    from kairos_amd import ops
    N, K, M = 1024, 4096, 96
    p = ops.prepare_weight(torch.from_numpy(O.synth_weights(N, K, seed=4)).cuda())
    x = torch.from_numpy(O.synth_acts(M, K, seed=5)).cuda()
    assert ops.gemm_splits_for("w4a16", M, N, K) > 1 and ops.gemm_splits_for("w4a16", M, N, K, 0) == 1
    main = ops.gemm_forward(x, p["qweight"], p["scales"], p["scaled_zeros"])
    torch.cuda.synchronize()
    box = {}

    def worker():
        torch.cuda.set_device(0)
        box["splits"] = ops.gemm_splits_for("w4a16", M, N, K)
        box["out"] = ops.gemm_forward(x, p["qweight"], p["scales"], p["scaled_zeros"])
        torch.cuda.synchronize()

    t = threading.Thread(target=worker)
    t.start()
    t.join()
    assert box["splits"] == ops.gemm_splits_for("w4a16", M, N, K)
    assert torch.equal(box["out"].view(torch.int16), main.view(torch.int16))
    # two streams never share a scratch buffer
    s2 = torch.cuda.Stream()
    with torch.cuda.stream(s2):
        other = ops.gemm_forward(x, p["qweight"], p["scales"], p["scaled_zeros"])
        ws2 = ops.workspace_for(x.device)
    s2.synchronize()
    assert ws2.data_ptr() != ops.workspace_for(x.device).data_ptr()
    assert torch.equal(other.view(torch.int16), main.view(torch.int16))


def test_forward_rejects_a_wrong_input_width(gpu):
    """The decode fast path hands raw pointers to the library: an input whose last dimension is not the layer's K must
    be refused on the host, in both the fast path and the general one, before any kernel reads past the buffer."""
    from kairos.dynamic_linear import DynamicLinear
    from kairos.perf_profiler import Profiler
    N, K = 256, 512
    lin = torch.nn.Linear(K, N, bias=False, dtype=torch.float16)
    dl = DynamicLinear.from_module(lin.cuda(), "cuda")
    prof = Profiler([(N, K)])
    prof.record_best_comp((N, K), 64, "w4a16_gemv")
    prof.record_best_comp((N, K), 1 << 20, "w4a16_gemm")
    old = DynamicLinear.prof
    DynamicLinear.prof = prof
    try:
        assert dl(torch.zeros((1, 4, K), dtype=torch.float16, device="cuda")).shape == (1, 4, N)
        with pytest.raises(ValueError):
            dl(torch.zeros((1, 4, K // 2), dtype=torch.float16, device="cuda"))           # small-M fast path
        from kairos_amd import ops
        with pytest.raises(ValueError):
            ops.gemv_forward(torch.zeros((4, K // 2), dtype=torch.float16, device="cuda"), dl.qweight, dl.scales,
                             dl.scaled_zeros, 4, N, K)
    finally:
        DynamicLinear.prof = old


def test_decoder_harness_two_layers(gpu):
    """The end-to-end decoder harness (GQA attention over a static KV cache, matched norm and SiLU operators, every
    linear a LUT-switched DynamicLinear, decode step replayed from a HIP graph) at reduced width, two layers:
    prefill and decode logits against the same stack computing with the oracle's dequantised fp16 weights in
    PyTorch, and graph-replayed tokens against eagerly generated ones."""
    from kairos.dynamic_linear import DynamicLinear
    from kairos.perf_profiler import Profiler
    from kairos_amd.bench_extra import Decoder
    dev = torch.device("cuda:0")
    hidden, heads, kv, mlp, vocab = 1024, 8, 2, 2048, 2048
    d = hidden // heads
    shapes = [((heads + 2 * kv) * d, hidden), (hidden, hidden), (2 * mlp, hidden), (hidden, mlp)]
    prof = Profiler(shapes)
    for s in shapes:
        for r, name in [(16, 'w4a16_gemv'), (128, 'w4a16_gemm'), (1 << 20, 'w8a8')]:
            prof.record_best_comp(s, r, name)
    old = DynamicLinear.prof
    DynamicLinear.prof = prof

    class Dense(torch.nn.Module):                       # the comparison stack's linear: fp16 matmul on dequantised weights
        def __init__(self, w16):
            super().__init__()
            self.w = w16

        def forward(self, x):
            return x @ self.w.T

    try:
        quant, dense = [], []
        for l in range(2):
            ql, dl_ = [], []
            for i, (N, K) in enumerate(shapes):
                w = O.synth_weights(N, K, seed=100 + 10 * l + i) * np.float16(2.0)
                lin = torch.nn.Linear(K, N, bias=False, dtype=torch.float16)
                with torch.no_grad():
                    lin.weight.copy_(torch.from_numpy(w))
                ql.append(DynamicLinear.from_module(lin.cuda(), "cuda"))
                p = O.prepare_weights(w)
                dl_.append(Dense(torch.from_numpy(O.dequant_to_f16(p["qweight"], p["scales"], p["scaled_zeros"])).cuda()))
            quant.append(ql)
            dense.append(dl_)
        t_max = 160
        dec = Decoder(quant, dev, hidden, heads, kv, vocab, matched=True, t_max=t_max, seed=1)
        ref = Decoder(dense, dev, hidden, heads, kv, vocab, matched=False, t_max=t_max, seed=1)
        assert torch.equal(dec.emb, ref.emb) and torch.equal(dec.head, ref.head)
        B = 2

        def rel(a, b):
            return ((a.float() - b.float()).abs().max() / b.float().abs().max()).item()

        # 48 tokens: W4A16 GEMM prefill (the fp16-output bar); 256 tokens: W8A8 prefill -- int8 activations in all eight
        # linears of the stack, whose bit-exact parity is a kernel- and module-level test; here a sanity bound only
        for prompt, tol in ((24, 1e-2), (128, 0.15)):
            ids = torch.randint(0, vocab, (B, prompt), device=dev, generator=torch.Generator(device=dev).manual_seed(prompt))
            dec.alloc(B)
            ref.alloc(B)
            got, want = dec.prefill_logits(ids), ref.prefill_logits(ids)
            assert torch.isfinite(got).all() and rel(got, want) < tol, (prompt, rel(got, want))
            lanes = {prof.get_comp_type(s, B * prompt) for s in shapes}
            assert lanes == ({0} if prompt == 24 else {2})
            if prompt != 24:
                continue
            # decode: the small-M lane on the quantised stack; both stacks continue from the comparison stack's token
            first = want.argmax(-1)
            dec.start(first, prompt)
            ref.start(first, prompt)
            eager = []
            for t in range(6):
                dec.step()
                ref.step()
                assert rel(dec.logits, ref.logits) < 2e-2, (t, rel(dec.logits, ref.logits))
                eager.append((dec.tok.clone(), dec.logits.clone()))
                ref.x_in.copy_(dec.x_in)                # keep the two sequences on the same tokens
            graph = dec.capture()
            dec.prefill_logits(ids)                     # the capture's warm-up step wrote the cache: refill it
            dec.start(first, prompt)
            for t in range(6):
                graph.replay()
                torch.cuda.synchronize()
                assert torch.equal(dec.tok, eager[t][0]), f"token {t}: graph replay and eager decoding disagree"
                assert torch.equal(dec.logits.view(torch.int16), eager[t][1].view(torch.int16))
            dec.free()
            ref.free()
    finally:
        DynamicLinear.prof = old


def test_decoder_harness_at_8b_width(gpu):
    """The same harness at the true Llama-3-8B layer shapes (hidden 4096, 32 query / 8 key-value heads, MLP 14336), two
    layers that share one set of prepared weights, batch 2, 64 prompt tokens + 4 decoded, with the committed MI355X
    lookup table (so every linear runs the lane the benchmark runs at these token counts: the small-M kernel at M = 2,
    the W4A16 GEMM and the W4A8 lane at M = 128).  Against the same stack on fp16 weights dequantised by the library's
    converter, which is checked against the oracle on a slab of every weight; graph-replayed tokens equal eager ones."""
    import os
    from kairos.dynamic_linear_v2 import DynamicLinear
    from kairos.perf_profiler_v2 import Profiler
    from kairos_amd import ops
    from kairos_amd.bench_extra import Decoder
    dev = torch.device("cuda:0")
    hidden, heads, kv, mlp, vocab = 4096, 32, 8, 14336, 4096
    shapes = [(6144, 4096), (4096, 4096), (28672, 4096), (4096, 14336)]
    prof = Profiler(shapes)
    prof.load(os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "kairos_amd", "prof", "llama3_8b_mi355x_v2") + "/")
    old = DynamicLinear.prof
    DynamicLinear.prof = prof

    class Dense(torch.nn.Module):
        def __init__(self, w16):
            super().__init__()
            self.w = w16

        def forward(self, x):
            return x @ self.w.T

    try:
        ql, dl_ = [], []
        for i, (N, K) in enumerate(shapes):
            w = torch.from_numpy(O.synth_weights(N, K, seed=200 + i) * np.float16(2.0)).cuda()
            prepared = ops.prepare_weight(w)
            q = DynamicLinear(K, N, False, dev, 128)
            for key, val in prepared.items():
                setattr(q, key, val)
            ql.append(q)
            w16 = torch.empty((N, K), dtype=torch.float16, device=dev)
            ops.dequant_interleaved_int4_to_fp16(w16, q.qweight, q.scales, q.scaled_zeros, 128)
            rows = slice(N // 2, N // 2 + 256)                                   # the converter against the oracle on a slab
            want = O.dequant_to_f16(q.qweight[rows.start // 4:rows.stop // 4].cpu().numpy(), q.scales[:, rows].cpu().numpy(),
                                    q.scaled_zeros[:, rows].cpu().numpy())
            assert np.array_equal(w16[rows].cpu().numpy().view(np.uint16), want.view(np.uint16))
            dl_.append(Dense(w16))
        quant, dense = [ql, ql], [dl_, dl_]                                     # two layers, one set of prepared weights
        B, prompt, t_max = 2, 64, 96
        dec = Decoder(quant, dev, hidden, heads, kv, vocab, matched=True, t_max=t_max, seed=3)
        ref = Decoder(dense, dev, hidden, heads, kv, vocab, matched=False, t_max=t_max, seed=3)

        def rel(a, b):
            return ((a.float() - b.float()).abs().max() / b.float().abs().max()).item()

        names = {v: k for k, v in __import__("kairos.dynamic_linear_v2", fromlist=["COMP_TYPE_NAME"]).COMP_TYPE_NAME.items()}
        prefill_lanes = {names[prof.get_comp_type(s, B * prompt)] for s in shapes}
        assert {names[prof.get_comp_type(s, B)] for s in shapes} == {"w4a16_gemv"}
        ids = torch.randint(0, vocab, (B, prompt), device=dev, generator=torch.Generator(device=dev).manual_seed(5))
        dec.alloc(B)
        ref.alloc(B)
        got, want = dec.prefill_logits(ids), ref.prefill_logits(ids)
        # int8 activations (W4A8 / W8A8 lanes) in the prefill: a sanity bound; fp16-activation lanes only: the fp16 bar
        tol = 0.15 if prefill_lanes & {"w4a8_qserve", "w8a8"} else 2e-2
        assert torch.isfinite(got).all() and rel(got, want) < tol, (prefill_lanes, rel(got, want))
        first = want.argmax(-1)
        dec.start(first, prompt)
        ref.start(first, prompt)
        eager = []
        for t in range(4):
            dec.step()
            ref.step()
            # the decode steps (small-M lane) attend over the cache that the prefill's lanes wrote: the prefill's bound
            assert rel(dec.logits, ref.logits) < tol, (t, rel(dec.logits, ref.logits))
            eager.append((dec.tok.clone(), dec.logits.clone()))
            ref.x_in.copy_(dec.x_in)                # keep the two sequences on the same tokens
        graph = dec.capture()
        dec.prefill_logits(ids)
        dec.start(first, prompt)
        for t in range(4):
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(dec.tok, eager[t][0]), f"token {t}: graph replay and eager decoding disagree"
            assert torch.equal(dec.logits.view(torch.int16), eager[t][1].view(torch.int16))
        dec.free()
        ref.free()
    finally:
        DynamicLinear.prof = old


def test_smooth_scale_search_with_the_library_probe(gpu):
    """The smoothing-scale search (kairos/smooth_scale.py:66-176) with its default probe -- the library's own quantised
    linear through the W4A8 lane -- on a tiny fp16 Llama with outlier channels: the scales it finds lower the error of
    the quantised model (every linear a DynamicLinear on the int8-activation lane) against the fp16 model."""
    transformers = pytest.importorskip("transformers")
    from kairos.dynamic_linear_v2 import COMP_TYPE_NAME, DynamicLinear
    from kairos.perf_profiler_v2 import Profiler
    from kairos.quant_model import get_name_linears, quantize_model
    from kairos.smooth_scale import apply_scale, smooth_scale
    torch.manual_seed(0)
    cfg = transformers.LlamaConfig(hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=4,
                                   num_key_value_heads=2, vocab_size=128, max_position_embeddings=256)
    model = transformers.LlamaForCausalLM(cfg).half().cuda().eval()
    with torch.no_grad():
        for layer in model.model.layers:
            layer.input_layernorm.weight[::37] *= 30.0
            layer.post_attention_layernorm.weight[::41] *= 30.0
    ids = torch.randint(0, 128, (2, 48), device="cuda", generator=torch.Generator(device="cuda").manual_seed(1))
    with torch.no_grad():
        want = model(ids).logits.float()
    meta = smooth_scale(model, {"input_ids": ids})
    assert len(meta) == 2 and all(len(b) == 3 for b in meta)
    assert all(type(m) is torch.nn.Linear for layer in model.model.layers for m in get_name_linears(layer).values())
    with torch.no_grad():
        assert torch.equal(model(ids).logits.float(), want)                      # the search left the model as it was

    shapes = sorted({tuple(m.weight.shape) for layer in model.model.layers for m in get_name_linears(layer).values()})
    prof = Profiler(shapes)
    for s in shapes:
        prof.record_best_comp(s, 1 << 20, 'w4a8_qserve')
    old = DynamicLinear.prof
    DynamicLinear.prof = prof

    def quantised_error(smoothed):
        m = transformers.LlamaForCausalLM(cfg).half().cuda().eval()
        m.load_state_dict(model.state_dict())
        if smoothed:
            apply_scale(m, meta)
        quantize_model(m, quant_strategy='DynamicLinear', version='2')
        with torch.no_grad():
            return (m(ids).logits.float() - want).pow(2).mean().item()

    try:
        plain, smoothed = quantised_error(False), quantised_error(True)
    finally:
        DynamicLinear.prof = old
    assert smoothed < plain, (plain, smoothed)
