"""Host-side mirror of the reference interface, on CPU: table files, LUT wrapper, segment
compression, module construction, the import-path aliases, and loud failure without a GPU."""
import json
import os
import shutil

import numpy as np
import pytest
import torch

from oracle import kairos_oracle as O

LLAMA_SHAPES = [(1024, 4096), (4096, 4096), (4096, 14336), (14336, 4096)]
QWEN_SHAPES = [(512, 3584), (3584, 3584), (3584, 18944), (18944, 3584)]


def test_alias_package_exposes_reference_names():
    from kairos.dynamic_linear import COMP_TYPE_NAME, DynamicLinear
    from kairos.dynamic_linear_v2 import COMP_TYPE_NAME as V2, DynamicLinear as D2
    from kairos.switch_linear import SwitchLinear
    from kairos.perf_profiler import LUT, Profiler, test_perf
    from kairos.perf_profiler_v2 import Profiler as P2
    from kairos.quantization import quantize_tensor_int8
    import kairos_amd.dynamic_linear as impl
    assert DynamicLinear is impl.DynamicLinear
    assert COMP_TYPE_NAME == {'w4a16_gemm': 0, 'w4a16_gemv': 1, 'w8a8': 2, 'w8a16_gemm': 3, 'w8a16_gemv': 4, 'fp16': 5}
    assert V2['w4a16_marlin'] == 6 and V2['w4a8_qserve'] == 7 and V2['fp16'] == 5
    assert issubclass(SwitchLinear, D2) and P2.linear_cls is D2
    assert callable(test_perf) and callable(quantize_tensor_int8) and LUT and Profiler


@pytest.mark.parametrize("fixture,shapes", [("prof_llama_seg_perf_list.json", LLAMA_SHAPES),
                                            ("prof_qwen_seg_perf_list.json", QWEN_SHAPES)])
def test_profiler_loads_reference_tables(tmp_path, golden_dir, fixture, shapes):
    from kairos.perf_profiler_v2 import Profiler
    d = tmp_path / "prof"
    d.mkdir()
    shutil.copy(os.path.join(golden_dir, fixture), d / "seg_perf_list.pt")
    prof = Profiler(shapes)
    prof.load(str(d) + "/")
    segs = json.load(open(os.path.join(golden_dir, fixture)))
    for shape, seg in zip(shapes, segs):
        want = O.LUT()
        for r, name, _ in seg:
            want.record(r, O.COMP_TYPE_NAME[name])
        for m in [1, 2, 3, 7, 8, 9, 16, 17, 64, 65, 256, 257, 512, 1024, 1025, 4096, 22528, 22529, 30720, 99999]:
            assert prof.get_comp_type(shape, m) == want.get(m)
    # save writes the same JSON text format back
    out = tmp_path / "out"
    prof.save(str(out) + "/")
    assert json.load(open(out / "seg_perf_list.pt")) == segs


def test_v1_profiler_rejects_v2_only_lane(tmp_path, golden_dir):
    from kairos.perf_profiler import Profiler
    d = tmp_path / "prof"
    d.mkdir()
    shutil.copy(os.path.join(golden_dir, "prof_llama_seg_perf_list.json"), d / "seg_perf_list.pt")
    with pytest.raises(KeyError):        # 'w4a16_marlin' is not in the v1 id table, as upstream
        Profiler(LLAMA_SHAPES).load(str(d) + "/")


def test_compress_segments_matches_reference_rule():
    from kairos.perf_profiler import compress_segments
    perf = [(1, 'w4a16_gemv', 0.0), (2, 'w4a16_gemv', 0.0), (4, 'w4a16_gemm', 0.0), (8, 'w4a16_gemm', 0.0),
            (16, 'w8a8', 12.5), (32, 'w8a8', 30.0)]
    assert compress_segments(perf) == [(2, 'w4a16_gemv', 0.0), (8, 'w4a16_gemm', 0.0), (32, 'w8a8', 30.0)]
    assert compress_segments([(1, 'fp16', 1.0)]) == [(1, 'fp16', 1.0)]


def test_profiler_lane_choice_rules():
    """choose_lane: fastest lane; a lane on the resident int4 weight within the margin goes first; the previous M's
    lane is kept within the stickiness; both margins at zero give the reference's strict minimum
    (kairos/perf_profiler.py:140-147)."""
    from kairos_amd.perf_profiler import choose_lane
    t = {"w8a8": 100.0, "w4a8_qserve": 103.0, "w4a16_gemm": 150.0, "fp16": 170.0}
    assert choose_lane(t, "", 0.0, 0.0) == ("w8a8", 100.0)
    assert choose_lane(t, "", 0.01, 0.04) == ("w4a8_qserve", 103.0)          # within 4 %: no converted copy
    assert choose_lane(t, "", 0.01, 0.02) == ("w8a8", 100.0)                 # beyond the margin: the fastest
    assert choose_lane({**t, "w4a8_qserve": 104.1}, "", 0.01, 0.04) == ("w8a8", 100.0)
    assert choose_lane(t, "fp16", 0.01, 0.0) == ("w8a8", 100.0)              # previous lane far behind: dropped
    assert choose_lane({"w8a8": 100.0, "fp16": 100.5}, "fp16", 0.01, 0.04) == ("fp16", 100.5)   # sticky within 1 %
    assert choose_lane({"w8a8": 100.0, "fp16": 100.5}, "fp16", 0.0, 0.04) == ("w8a8", 100.0)
    # stickiness is measured against the choice after the preference, not against the raw minimum
    assert choose_lane(t, "w8a8", 0.01, 0.04) == ("w8a8", 100.0)
    assert choose_lane({"w4a16_gemv": 10.0, "w4a16_gemm": 12.0, "w8a8": 30.0}, "", 0.01, 0.04) == ("w4a16_gemv", 10.0)
    assert choose_lane({"fp16": 5.0}, "w8a8", 0.01, 0.04) == ("fp16", 5.0)   # no resident lane, previous lane absent


def test_lut_wrapper():
    from kairos.perf_profiler import LUT
    lut = LUT()
    for r, c in [(8, 1), (256, 0), (30720, 2)]:
        lut.record(r, c)
    lut.shrink_to_fit()
    assert len(lut) == 3
    assert [lut.get(m) for m in (1, 8, 9, 256, 257, 10 ** 6, 9, 9)] == [1, 1, 0, 0, 2, 2, 0, 0]
    from kairos_amd._lib import KairosMiError
    with pytest.raises(KairosMiError):
        LUT().get(5)


def test_from_module_on_cpu_matches_oracle_and_refuses_cpu_compute():
    from kairos.dynamic_linear import DynamicLinear
    torch.manual_seed(0)
    lin = torch.nn.Linear(256, 64, bias=True, dtype=torch.float16)
    dl = DynamicLinear.from_module(lin, 'cpu')
    ref = O.prepare_weights(lin.weight.detach().numpy())
    for key in ("qweight", "scales", "scaled_zeros", "scales_to8", "scaled_zeros_to8", "scales_1"):
        assert np.array_equal(getattr(dl, key).numpy().view(np.uint16), ref[key].view(np.uint16)), key
    assert dl.shape == (64, 256) and dl.pre_m == 0 and dl.group_size == 128
    assert torch.equal(dl.bias, lin.bias.detach())
    assert "in_features=256, out_features=64, bias=True" in repr(dl)
    assert DynamicLinear(256, 64, False, 'cpu', 128).qweight is None     # the plain constructor allocates nothing
    with pytest.raises((ValueError, ImportError)):      # no CPU fallback: the HIP path is the only path
        dl._forward(torch.zeros(1, 2, 256, dtype=torch.float16), 2, 1)


def test_state_dict_round_trip_on_cpu(tmp_path):
    """The six resident tensors (and the bias) travel through state_dict / torch.save / load_state_dict; an
    init_only module has the right shapes to receive them (kairos/main.py:85-91, utils/load_model.py:15-29)."""
    from kairos.dynamic_linear import DynamicLinear
    from kairos_amd.dynamic_linear import RESIDENT_KEYS
    torch.manual_seed(1)
    model = torch.nn.Sequential(torch.nn.Linear(256, 64, bias=True, dtype=torch.float16),
                                torch.nn.Linear(128, 64, bias=False, dtype=torch.float16))
    q = torch.nn.Sequential(*[DynamicLinear.from_module(l, 'cpu') for l in model])
    sd = q.state_dict()
    assert set(sd) == {f"{i}.{k}" for i in (0, 1) for k in RESIDENT_KEYS} | {"0.bias"}
    path = tmp_path / "q_model.pt"
    torch.save(sd, path)
    loaded = torch.load(path, weights_only=True)
    fresh = torch.nn.Sequential(*[DynamicLinear.from_module(l, 'cpu', init_only=True) for l in model])
    assert fresh[0].qweight.shape == (16, 256) and fresh[1].scales.shape == (8, 64)
    uid = fresh[0]._uid
    fresh.load_state_dict(loaded)                       # strict
    assert fresh[0]._uid != uid                         # stale temp-cache entries of this layer can no longer hit
    for a, b in zip(q, fresh):
        for k in RESIDENT_KEYS:
            assert torch.equal(getattr(a, k), getattr(b, k)) and getattr(a, k).dtype == getattr(b, k).dtype, k
    assert torch.equal(q[0].bias, fresh[0].bias)
    bare = DynamicLinear(128, 64, False, 'cpu', 128)    # plain constructor: allocated while loading
    bare.load_state_dict({k: getattr(q[1], k) for k in RESIDENT_KEYS})
    assert torch.equal(bare.qweight, q[1].qweight)
    with pytest.raises(RuntimeError):                   # a checkpoint of another shape is refused
        fresh[0].load_state_dict(q[1].state_dict())


def test_temp_cache_is_bounded_and_reuses():
    from kairos_amd.temp_cache import TempCache
    c = TempCache(capacity_limit=1024)
    a, hit = c.get(1, 'i8', (4, 64), torch.int8, 'cpu')
    assert not hit and a.shape == (4, 64) and a.dtype == torch.int8
    b, hit = c.get(1, 'i8', (4, 64), torch.int8, 'cpu')
    assert hit and b.data_ptr() == a.data_ptr()
    d, hit = c.get(2, 'f16', (4, 64), torch.float16, 'cpu')
    assert not hit and d.dtype == torch.float16 and c.capacity == 512 and c.peak_bytes == 512
    _, hit = c.get(1, 'i8', (4, 64), torch.int8, 'cpu')
    assert not hit                                      # evicted by the other layer
    with pytest.raises(MemoryError):
        c.get(3, 'f16', (4, 256), torch.float16, 'cpu')
    assert c.capacity <= 1024


class _FakeStreams:
    """Stand-ins for the stream queries of kairos_amd.temp_cache, so that its capture and multi-stream rules can be
    exercised without a GPU: `current` names the stream, `capturing` says whether it records a graph."""

    def __init__(self, monkeypatch):
        from kairos_amd import temp_cache as tc
        self.current, self.capturing, self.orders = "s0", False, []
        monkeypatch.setattr(tc, "_is_capturing", lambda device: self.capturing)
        monkeypatch.setattr(tc, "_current_stream", lambda device: self.current)
        monkeypatch.setattr(tc, "_order_after", lambda stream, earlier: self.orders.append((stream, earlier)))


def test_temp_cache_never_bakes_a_hit_into_a_graph(monkeypatch):
    """A request made during graph capture is a miss (the conversion must be recorded: at replay time the buffer
    holds whatever ran last) and clears the tag, so the next eager request converts as well."""
    from kairos_amd.temp_cache import TempCache
    st = _FakeStreams(monkeypatch)
    c = TempCache()
    a, hit = c.get(1, 'i8', (4, 64), torch.int8, 'cpu')
    assert not hit and c.get(1, 'i8', (4, 64), torch.int8, 'cpu')[1]          # eager: second call hits
    st.capturing = True
    b, hit = c.get(1, 'i8', (4, 64), torch.int8, 'cpu')
    assert not hit and b.data_ptr() == a.data_ptr()                            # same buffer, but converted in the graph
    assert not c.get(1, 'i8', (4, 64), torch.int8, 'cpu')[1]                   # still capturing: never a hit
    with pytest.raises(RuntimeError, match="eagerly"):                         # growth inside a capture is refused
        c.get(2, 'f16', (64, 64), torch.float16, 'cpu')
    st.capturing = False
    assert not c.get(1, 'i8', (4, 64), torch.int8, 'cpu')[1]                   # the capture left the tag cleared
    assert c.get(1, 'i8', (4, 64), torch.int8, 'cpu')[1]


def test_temp_cache_keeps_a_captured_buffer_alive_when_it_grows(monkeypatch):
    from kairos_amd.temp_cache import TempCache
    st = _FakeStreams(monkeypatch)
    c = TempCache()
    small, _ = c.get(1, 'i8', (4, 64), torch.int8, 'cpu')
    st.capturing = True
    c.get(1, 'i8', (4, 64), torch.int8, 'cpu')                                 # a graph records this address
    st.capturing = False
    storage = small.untyped_storage().data_ptr()
    big, hit = c.get(2, 'f16', (64, 64), torch.float16, 'cpu')                 # eager growth afterwards
    assert not hit and big.untyped_storage().data_ptr() != storage
    assert [b.untyped_storage().data_ptr() for b in c._retired] == [storage]   # still referenced: not freed, not reused
    c2 = TempCache()
    c2.get(1, 'i8', (4, 64), torch.int8, 'cpu')
    c2.get(2, 'f16', (64, 64), torch.float16, 'cpu')                           # no capture in between: nothing kept aside
    assert c2._retired == []


def test_temp_cache_orders_requests_from_different_streams(monkeypatch):
    """The buffer handed out on stream s1 after a use on s0 is ordered behind s0's queue (the earlier conversion and
    the GEMM that reads it), for hits and misses alike; requests on one stream need no event."""
    from kairos_amd.temp_cache import ResidentCache, TempCache
    st = _FakeStreams(monkeypatch)
    c = TempCache()
    c.get(1, 'i8', (4, 64), torch.int8, 'cpu')
    c.get(1, 'i8', (4, 64), torch.int8, 'cpu')
    assert st.orders == []
    st.current = "s1"
    assert c.get(1, 'i8', (4, 64), torch.int8, 'cpu')[1] and st.orders == [("s1", "s0")]     # a safe hit
    c.get(2, 'i8', (4, 64), torch.int8, 'cpu')
    assert st.orders == [("s1", "s0")]
    st.current = "s0"
    assert not c.get(3, 'i8', (4, 64), torch.int8, 'cpu')[1] and st.orders[-1] == ("s0", "s1")
    # a graph replay on s2 uses the buffer behind the cache's back: touch() makes the next request wait for it
    st.current = "s2"
    c.touch('cpu')
    st.current = "s0"
    c.get(3, 'i8', (4, 64), torch.int8, 'cpu')
    assert st.orders[-2:] == [("s2", "s0"), ("s0", "s2")]
    # the many-entry cache keeps one order per copy and converts inside captures without keeping anything
    st.orders.clear()
    r = ResidentCache(4096)
    monkeypatch.setattr(torch.Tensor, "record_stream", lambda self, s: None, raising=False)
    r.get(1, 'i8', (4, 64), torch.int8, 'cpu')
    st.current = "s1"
    assert r.get(1, 'i8', (4, 64), torch.int8, 'cpu')[1] and st.orders == [("s1", "s0")]
    st.capturing = True
    with pytest.raises(RuntimeError, match="prepare_for_capture"):
        r.get(1, 'i8', (4, 64), torch.int8, 'cpu')
    st.capturing = False
    r.prepare_for_capture('cpu')
    st.capturing = True
    assert not r.get(1, 'i8', (4, 64), torch.int8, 'cpu')[1] and not r.get(1, 'i8', (4, 64), torch.int8, 'cpu')[1]
    st.capturing = False
    assert r.get(1, 'i8', (4, 64), torch.int8, 'cpu')[1]                       # the resident copy was left alone


def test_committed_mi355x_tables_load_and_have_three_regimes():
    """Every table shipped under kairos_amd/prof/ has the reference's file format and the small-M / mid-M /
    large-M structure (same schema as the reference's prof_llama / prof_qwen files)."""
    import glob
    import json
    import os
    root = os.path.join(os.path.dirname(os.path.dirname(os.path.abspath(__file__))), "kairos_amd", "prof")
    files = sorted(glob.glob(os.path.join(root, "*", "seg_perf_list.pt")))
    assert len(files) >= 3
    for f in files:
        table = json.load(open(f))
        assert len(table) == 4
        for segs in table:
            edges = [s[0] for s in segs]
            assert edges == sorted(edges) and all(isinstance(e, int) for e in edges)
            assert all(isinstance(s[1], str) and isinstance(s[2], float) for s in segs)
            assert segs[0][1] == "w4a16_gemv" and segs[-1][1] == "w8a8"


def test_resident_cache_lru_and_bound():
    from kairos_amd.temp_cache import ResidentCache, TempCache, default_cache, set_default_cache
    c = ResidentCache(1024)
    a, hit = c.get(1, 'i8', (4, 64), torch.int8, 'cpu')                     # 256 B
    assert not hit and a.shape == (4, 64)
    b, hit = c.get(2, 'f16', (4, 64), torch.float16, 'cpu')                  # 512 B
    assert not hit
    a2, hit = c.get(1, 'i8', (4, 64), torch.int8, 'cpu')
    assert hit and a2.data_ptr() == a.data_ptr()                             # both stay: 768 B <= 1024
    _, hit = c.get(3, 'i8', (8, 64), torch.int8, 'cpu')                      # 512 B: evicts the least recently used (2)
    assert not hit and c.capacity <= 1024
    assert c.get(1, 'i8', (4, 64), torch.int8, 'cpu')[1]
    assert not c.get(2, 'f16', (4, 64), torch.float16, 'cpu')[1]             # was evicted; evicts 3 now
    big, hit = c.get(9, 'f16', (16, 64), torch.float16, 'cpu')               # 2048 B > capacity: served, never kept
    assert not hit and big.shape == (16, 64)
    assert not c.get(9, 'f16', (16, 64), torch.float16, 'cpu')[1]
    assert c.get(1, 'i8', (4, 64), torch.int8, 'cpu')[1]                     # the resident entries are untouched
    ptr = c.get(1, 'i8', (4, 64), torch.int8, 'cpu')[0].data_ptr()
    c.invalidate()
    again, hit = c.get(1, 'i8', (4, 64), torch.int8, 'cpu')
    assert not hit and again.data_ptr() == ptr                               # stale, same buffer, valid afterwards
    assert c.get(1, 'i8', (4, 64), torch.int8, 'cpu')[1]
    assert c.peak_bytes <= 1024 + 2048 and c.hits >= 4 and c.misses >= 6
    old = default_cache()
    try:
        assert set_default_cache(c) is default_cache()
    finally:
        set_default_cache(old)
    assert isinstance(default_cache(), TempCache)


def _tiny_llama(seed=0):
    transformers = pytest.importorskip("transformers")
    torch.manual_seed(seed)
    cfg = transformers.LlamaConfig(hidden_size=256, intermediate_size=512, num_hidden_layers=2, num_attention_heads=4,
                                   num_key_value_heads=2, vocab_size=128, max_position_embeddings=64)
    return transformers.LlamaForCausalLM(cfg).half()


def test_quantize_model_surgery_and_checkpoint_flow(tmp_path):
    """kairos/quant_model.py:29-56 on a tiny random Llama: every decoder linear becomes a DynamicLinear whose tensors
    equal the oracle's preparation of that weight; the dumped state_dict loads into an init_only rebuild
    (kairos/main.py:85-91, utils/load_model.py:15-29)."""
    from kairos.dynamic_linear import DynamicLinear
    from kairos.quant_model import get_name_linears, quantize_model
    from kairos.quant_config import LinearQuantConfig
    from kairos_amd.dynamic_linear import RESIDENT_KEYS
    model = _tiny_llama()
    weights = {(i, n): m.weight.detach().clone() for i, layer in enumerate(model.model.layers)
               for n, m in get_name_linears(layer).items()}
    assert len(weights) == 14
    cfg = quantize_model(model)
    assert cfg == [{n: 'DynamicLinear' for n in ('self_attn.q_proj', 'self_attn.k_proj', 'self_attn.v_proj', 'self_attn.o_proj',
                                                 'mlp.gate_proj', 'mlp.up_proj', 'mlp.down_proj')}] * 2
    assert all(not get_name_linears(layer) for layer in model.model.layers)          # none left inside the layers
    assert isinstance(model.lm_head, torch.nn.Linear)                                # outside the layers: untouched
    for (i, n), w in weights.items():
        q = model.model.layers[i].get_submodule(n)
        assert type(q) is DynamicLinear and q.shape == tuple(w.shape)
        ref = O.prepare_weights(w.numpy())
        for k in RESIDENT_KEYS:
            assert np.array_equal(getattr(q, k).numpy().view(np.uint16), ref[k].view(np.uint16)), (i, n, k)
    path = tmp_path / "q_model.pt"
    torch.save(model.state_dict(), path)
    fresh = _tiny_llama(seed=1)
    assert quantize_model(fresh, init_only=True, _quant_config=cfg) == cfg
    fresh.load_state_dict(torch.load(path, weights_only=True))
    for (i, n) in weights:
        a, b = model.model.layers[i].get_submodule(n), fresh.model.layers[i].get_submodule(n)
        assert all(torch.equal(getattr(a, k), getattr(b, k)) for k in RESIDENT_KEYS)
    with pytest.raises(NotImplementedError):
        LinearQuantConfig('W4A16Linear_Marlin')
    with pytest.raises(ValueError):
        LinearQuantConfig('nonsense')


def test_bench_refuses_more_than_one_gpu():
    """bench.py measures one GPU's share; asking for more must end with a message, not a wrong number."""
    import subprocess
    import sys
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, os.path.join(root, "bench.py"), "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0 and r.stdout.strip() == "" and "--gpus 1" in r.stderr


def test_apply_scale_keeps_the_fp_function():
    """kairos/smooth_scale.py:33-63: folding per-channel scales into the linears (W * s) and into the operator that
    feeds them (norm weight or up_proj rows / s) leaves the layer's function unchanged; fp32 model, so the comparison
    is tight.  The three blocks are the ones the reference's search emits (:107-131)."""
    from kairos.smooth_scale import apply_scale
    model = _tiny_llama(seed=3).float()
    ids = torch.randint(0, 128, (2, 12), generator=torch.Generator().manual_seed(0))
    with torch.no_grad():
        before = model(ids).logits
    g = torch.Generator().manual_seed(1)
    meta = []
    for _ in model.model.layers:
        meta.append([("input_layernorm", ["self_attn.q_proj", "self_attn.k_proj", "self_attn.v_proj"], torch.rand(1, 256, generator=g) + 0.5),
                     ("post_attention_layernorm", ["mlp.gate_proj", "mlp.up_proj"], torch.rand(1, 256, generator=g) + 0.5),
                     ("mlp.up_proj", ["mlp.down_proj"], torch.rand(1, 512, generator=g) + 0.5)])
    w0 = model.model.layers[0].self_attn.q_proj.weight.detach().clone()
    apply_scale(model, meta)
    assert torch.allclose(model.model.layers[0].self_attn.q_proj.weight, w0 * meta[0][0][2])
    with torch.no_grad():
        after = model(ids).logits
    assert torch.allclose(before, after, rtol=1e-4, atol=1e-4)
    with pytest.raises(ValueError):
        apply_scale(model, [[("no_such_op", ["mlp.down_proj"], torch.ones(1, 512))]])


def test_smooth_scale_search_finds_scales_that_help():
    """kairos/smooth_scale.py:66-176 with the plain-torch probe (no GPU): on a tiny Llama whose norm weights give a few
    channels 30x the magnitude of the rest, the search returns one entry per block in the reference's format, prefers a
    non-trivial exponent for the blocks behind the norms, leaves the model untouched, and folding its scales in lowers
    the error of the quantised probes against the unquantised model."""
    from kairos.smooth_scale import apply_scale, fake_quant_probe, smooth_scale
    from kairos.quant_model import get_name_linears, set_op_by_name
    model = _tiny_llama(seed=5).float()
    with torch.no_grad():
        for layer in model.model.layers:
            layer.input_layernorm.weight[::37] *= 30.0
            layer.post_attention_layernorm.weight[::41] *= 30.0
    ids = torch.randint(0, 128, (2, 24), generator=torch.Generator().manual_seed(0))
    state = {k: v.clone() for k, v in model.state_dict().items()}
    with torch.no_grad():
        want = model(ids).logits
    meta = smooth_scale(model, {"input_ids": ids}, make_probe=fake_quant_probe)
    assert all(torch.equal(v, state[k]) for k, v in model.state_dict().items())       # the search restores everything
    assert all(type(m) is torch.nn.Linear for layer in model.model.layers for m in get_name_linears(layer).values())
    assert len(meta) == 2
    for blocks in meta:
        assert [b[0] for b in blocks] == ["input_layernorm", "post_attention_layernorm", "mlp.up_proj"]
        assert [b[1] for b in blocks] == [["self_attn.q_proj", "self_attn.k_proj", "self_attn.v_proj"],
                                          ["mlp.gate_proj", "mlp.up_proj"], ["mlp.down_proj"]]
        assert [tuple(b[2].shape) for b in blocks] == [(1, 256), (1, 256), (1, 512)]
        for _prev, _names, sc in blocks:
            assert torch.isfinite(sc).all() and (sc > 0).all()
            assert abs(float(sc.max() * sc.min()) - 1.0) < 1e-3                        # normalised by sqrt(max * min)
        assert float(blocks[0][2].max() / blocks[0][2].min()) > 2.0                    # outlier channels get scaled down

    def quantised_error(m):
        """logits of `m` with every decoder linear replaced by the fake-quant probe (unit scales) against `want`"""
        originals = []
        for layer in m.model.layers:
            for name, lin in get_name_linears(layer).items():
                originals.append((layer, name, lin))
                set_op_by_name(layer, name, fake_quant_probe(lin, torch.ones(1, lin.in_features)))
        with torch.no_grad():
            err = (m(ids).logits - want).pow(2).mean().item()
        for layer, name, lin in originals:
            set_op_by_name(layer, name, lin)
        return err

    plain = quantised_error(model)
    apply_scale(model, meta)
    with torch.no_grad():
        assert torch.allclose(model(ids).logits, want, rtol=1e-3, atol=1e-3)           # smoothing keeps the function
    smoothed = quantised_error(model)
    assert smoothed < plain, (plain, smoothed)


def test_matched_norm_asks_its_consumers_for_their_lane():
    """Host half of activation matching: the formats a norm emits follow the table lookups of its consumers
    (int8 where a lane is W8A8, fp16 elsewhere, both when consumers disagree); no GPU involved."""
    import torch
    from kairos.act_matching import MatchedActivation, MatchedRMSNorm
    from kairos.dynamic_linear import DynamicLinear
    from kairos.perf_profiler import Profiler
    shapes = [(256, 512), (384, 512)]
    prof = Profiler(shapes)
    for r, name in [(8, 'w4a16_gemv'), (64, 'w4a16_gemm'), (4096, 'w8a8')]:
        prof.record_best_comp(shapes[0], r, name)
    for r, name in [(8, 'w4a16_gemv'), (256, 'w4a16_gemm'), (4096, 'w8a8')]:
        prof.record_best_comp(shapes[1], r, name)
    old = DynamicLinear.prof
    DynamicLinear.prof = prof
    try:
        lins = [DynamicLinear(512, n, False, 'cpu', 128) for n, _ in shapes]
        norm = MatchedRMSNorm(torch.ones(512, dtype=torch.float16), 1e-5, lins)
        assert norm.formats_for(4) == (True, False)
        assert norm.formats_for(64) == (True, False)
        assert norm.formats_for(65) == (True, True)
        assert norm.formats_for(257) == (False, True)
        assert MatchedRMSNorm(norm.weight, 1e-5, [torch.nn.Linear(512, 8)]).formats_for(300) == (True, False)

        class Norm:                                           # the two attribute names of the decoder families
            weight, variance_epsilon = norm.weight, 1e-6
        assert MatchedRMSNorm.from_module(Norm, lins).eps == 1e-6
        act = MatchedActivation(None, torch.zeros(2, 3, 512, dtype=torch.int8), torch.zeros(6, dtype=torch.float16))
        assert act.shape == (2, 3, 512) and act.numel() == 2 * 3 * 512
        with pytest.raises(ValueError):                       # lane for 6 tokens is fp16-fed, the activation is int8 only
            lins[0](act)
    finally:
        DynamicLinear.prof = old


def test_scratch_lookup_rules(monkeypatch):
    """Scratch buffers of the Python layer (host logic, no GPU): one pair per (device, stream handle); a Scratch that
    is active in the thread replaces them whatever the stream; nothing is created while the stream is capturing;
    release forgets one stream's pair."""
    import torch
    from kairos_amd import ops
    made = []

    def fake_new(idx, nbytes, zero, what):
        if capturing[0]:
            return real_new(idx, nbytes, zero, what)
        made.append((idx, nbytes, zero, what))
        return ("buf", len(made))

    real_new = ops._new_scratch
    capturing = [False]
    monkeypatch.setattr(ops, "_new_scratch", fake_new)
    monkeypatch.setattr(torch.cuda, "is_current_stream_capturing", lambda: capturing[0])
    monkeypatch.setattr(ops, "_workspaces", {})
    monkeypatch.setattr(ops, "_gemv_workspaces", {})
    a = ops.workspace_for("cuda:0", stream=111)
    assert ops.workspace_for("cuda:0", stream=111) is a and ops.workspace_for("cuda:0", stream=222) is not a
    g = ops.gemv_workspace_for("cuda:0", stream=111)
    assert g is not a and made[-1][2] is True and made[0][2] is False          # the small-M scratch is created zeroed
    # a stream handle that comes back after its stream was destroyed finds the same buffer (documented), until released
    ops.release_workspace("cuda:0", stream=111)
    assert ops.workspace_for("cuda:0", stream=111) is not a
    # an active Scratch wins over the per-stream buffers, on any stream, and nests
    outer, inner = ops.Scratch.__new__(ops.Scratch), ops.Scratch.__new__(ops.Scratch)
    outer.gemm, outer.gemv, inner.gemm, inner.gemv = "og", "ov", "ig", "iv"
    with outer:
        assert ops.workspace_for("cuda:0", stream=333) == "og" and ops.gemv_workspace_for("cuda:0", stream=444) == "ov"
        with inner:
            assert ops.workspace_for("cuda:0", stream=333) == "ig"
        assert ops.gemv_workspace_for("cuda:0", stream=111) == "ov"
    assert ops.workspace_for("cuda:0", stream=222) not in ("og", "ig")
    # during capture: existing buffers are handed out, missing ones are refused with the remedy
    capturing[0] = True
    assert ops.workspace_for("cuda:0", stream=222) is not None
    with pytest.raises(RuntimeError, match="ensure_workspace"):
        ops.workspace_for("cuda:0", stream=999)
    with pytest.raises(RuntimeError, match="Scratch"):
        ops.gemv_workspace_for("cuda:0", stream=999)
    with outer:
        assert ops.gemv_workspace_for("cuda:0", stream=999) == "ov"            # a graph that owns its scratch needs none
