"""CPU-side checks of the boundary: the shared library loads, exports every symbol the header
declares, reports argument errors without touching a GPU, and its LUT agrees with the oracle."""
import os
import re

import pytest

from oracle import kairos_oracle as O

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def lib():
    from kairos_amd import _lib
    if not os.path.exists(_lib.LIB_PATH):
        from kairos_amd import build
        build.build(verbose=False)
    return _lib.load()


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "kairos_mi.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(kmi_[a-z0-9_]+)\s*\(", text)))


def test_every_declared_symbol_is_exported_and_bound(lib):
    from kairos_amd import _lib
    names = declared_symbols()
    assert len(names) >= 20
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/kairos_mi.h but not exported"
        assert n in _lib.SIGNATURES, f"{n} has no ctypes signature"
    assert set(_lib.SIGNATURES) == set(names)


def test_argument_validation_needs_no_gpu(lib):
    assert lib.kmi_cvt_i4_to_f16(None, None, None, None, 4, 128, 128, None) == -1
    assert b"NULL" in lib.kmi_get_last_error_string()
    assert lib.kmi_cvt_i4_to_i8(16, 16, 16, 16, 4, 128, 64, None) == -3
    assert lib.kmi_cvt_i4_to_i8(16, 16, 16, 16, 6, 128, 128, None) == -2
    assert lib.kmi_cvt_i4_to_i8(16, 8, 16, 16, 4, 128, 128, None) == -5
    assert lib.kmi_gemv_w4a16(16, 16, 16, 16, 16, None, 0, 64, 128, 128, None, 0, None) == -4
    assert lib.kmi_gemv_w4a16(16, 16, 16, 16, 16, None, 65, 64, 128, 128, None, 0, None) == -4
    assert lib.kmi_gemv_w4a16(16, 16, 16, 16, 16, None, 4, 60, 128, 128, None, 0, None) == -2
    assert lib.kmi_gemv_w4a16_cfg(16, 16, 16, 16, 16, None, 4, 64, 1024, 128, 1, 8, 2, None, 0, None) == -2   # a forced K split needs scratch
    assert lib.kmi_gemv_w4a16_ring_cfg(16, 16, 16, 16, 16, None, 4, 64, 1024, 128, 1, 8, 2, 2, None, 0, None) == -2   # the same for the ring form
    assert lib.kmi_gemv_w4a16_ring_cfg(16, 16, 16, 16, 16, None, 4, 64, 1024, 128, 1, 3, 1, 2, None, 0, None) == -2   # 1, 2, 4 or 8 waves
    assert lib.kmi_gemv_w4a16_ring_cfg(16, 16, 16, 18, 16, None, 4, 64, 1024, 128, 1, 8, 1, 2, None, 0, None) == -5   # tables: 4-byte aligned
    assert lib.kmi_gemv_w4a16_ring_cfg(16, 16, 16, 16, 16, None, 40, 64, 1024, 128, 4, 8, 1, 2, None, 0, None) == -2  # 3 x 4 accumulator tiles
    assert lib.kmi_gemv_ws_reset(None, 1 << 20, None) == -1 and lib.kmi_gemv_ws_reset(16, 1024, None) == -2
    assert lib.kmi_gemv_ws_reset(24, 1 << 20, None) == -5
    assert lib.kmi_gemm_w8a8(16, 16, 16, 16, 16, None, 4, 64, 100, None, 0, None) == -2
    assert lib.kmi_gemm_w8a8(16, 16, 16, None, 16, None, 4, 64, 128, None, 0, None) == -1
    assert lib.kmi_quant_act_i8(16, 16, 16, 4, 12, None) == -2
    assert lib.kmi_quant_act_i8(16, 16, 16, 0, 128, None) == 0        # empty batch is a no-op
    assert lib.kmi_gemm_f16(16, 16, 16, None, 0, 64, 128, None, 0, None) == 0
    assert lib.kmi_gemm_f16(16, 16, 16, None, 4, 64, 128, 8, 1024, None) == -5         # misaligned split-K scratch
    # fused preparation launch: same rules as its two halves
    assert lib.kmi_prep_w8a8(None, 0, 16, 16, 16, 4, 128, 128, 16, 16, 16, 2, None) == -1
    assert lib.kmi_prep_w8a8(16, 0, 16, 16, 16, 4, 128, 64, 16, 16, 16, 2, None) == -3
    assert lib.kmi_prep_w8a8(16, 1, 16, 16, 16, 4, 128, 128, 16, 16, 16, 2, None) == -2      # tiled needs N % 128 == 0
    assert lib.kmi_prep_w8a8(16, 0, 16, 16, 16, 4, 128, 128, 8, 16, 16, 2, None) == -5
    assert lib.kmi_prep_w8a8(16, 0, 16, 16, 16, 4, 128, 128, 16, 16, 16, -1, None) == -2
    # variant choice of the W4A16 GEMM is host logic
    assert lib.kmi_gemm_w4a16_wp_rows(16, 4096, 4096) == 32
    assert lib.kmi_gemm_w4a16_wp_rows(4096, 4096, 4096) == 0
    assert lib.kmi_gemm_pick_tile(4096, 4096, 4096) == 256 and lib.kmi_gemm_pick_tile(8, 4096, 4096) == 64
    assert lib.kmi_gemm_pick_tile(512, 4096, 4096) == 64 and lib.kmi_gemm_pick_tile(384, 4096, 14336) == 128
    assert lib.kmi_gemm_pick_tile(768, 8192, 28672) == 256 and lib.kmi_gemm_pick_tile(1024, 4096, 14336) == 128   # split over K counts on long rows only
    assert lib.kmi_gemm_pick_tile(2048, 4096, 14336) == 192 and lib.kmi_gemm_pick_tile(1024, 8192, 28672) == 256   # 256 x 128 tiles, two per CU
    assert lib.kmi_gemm_pick_tile(192, 10240, 8192) == 64 and lib.kmi_gemm_pick_tile(192, 28672, 4096) == 128      # row padding
    # tile choice of the W4A8 GEMM is host logic as well (a cost model fitted to MI355X timings): two wave quartets on
    # 128 x 128 tiles while at most one workgroup per CU, 256 x 128 in between, 512 x 128 from full rounds on, whole rounds
    # plus a tail launch where the last round would be thin; two quartets over K need K % 256 == 0
    picks = {(128, 28672, 4096): 130, (256, 28672, 4096): 192, (512, 28672, 4096): 512, (2048, 28672, 4096): 640,
             (4096, 28672, 4096): 512, (768, 4096, 14336): 130, (2048, 4096, 14336): 192, (4096, 4096, 14336): 512,
             (512, 6144, 4096): 130, (1024, 6144, 4096): 192, (128, 4096, 4224): 192}
    for (M, N, K), want in picks.items():
        assert lib.kmi_gemm_w4a8_pick_tile(M, N, K) == want, (M, N, K)
    # offline weight preparation: same shape rules as the converters; table height is host arithmetic
    assert lib.kmi_prepare_weight(None, 8, 128, 128, 16, 16, 16, 16, 16, 16, None) == -1
    assert lib.kmi_prepare_weight(16, 6, 128, 128, 16, 16, 16, 16, 16, 16, None) == -2
    assert lib.kmi_prepare_weight(16, 8, 192, 128, 16, 16, 16, 16, 16, 16, None) == -2
    assert lib.kmi_prepare_weight(16, 8, 128, 64, 16, 16, 16, 16, 16, 16, None) == -3
    assert lib.kmi_prepare_weight(8, 8, 128, 128, 16, 16, 16, 16, 16, 16, None) == -5
    for K in (128, 1024, 3584, 4096, 14336, 18944, 28672):
        assert lib.kmi_padded_groups(K, 128) == O.padded_groups(K)
    assert lib.kmi_padded_groups(100, 128) == -2 and lib.kmi_padded_groups(128, 64) == -2
    assert lib.kmi_trans_layout_w4a8(None, 16, 32, 64, None) == -1
    assert lib.kmi_trans_layout_w4a8(16, 16, 16, 64, None) == -2 and lib.kmi_trans_layout_w4a8(16, 16, 32, 32, None) == -2
    assert lib.kmi_trans_layout_w4a8(16, 8, 32, 64, None) == -5
    # norm + quantiser: x and gamma always, at least one output, a scale with the int8 output
    assert lib.kmi_rmsnorm_quant_act(16, 16, 16, None, None, None, 16, 1e-5, 2, 128, None) == -1
    assert lib.kmi_rmsnorm_quant_act(None, None, None, None, 16, None, 16, 1e-5, 2, 128, None) == -1
    assert lib.kmi_rmsnorm_quant_act(16, None, None, None, 16, None, 16, 1e-5, 2, 128, None) == -1
    assert lib.kmi_rmsnorm_quant_act(None, None, 16, 16, 16, None, 16, 1e-5, 2, 128, None) == -1    # h_out without a residual
    assert lib.kmi_rmsnorm_quant_act(None, None, 16, None, 16, None, 8, 1e-5, 2, 128, None) == -5
    assert lib.kmi_rmsnorm_quant_act(None, None, 16, None, 16, None, 16, 1e-5, 2, 100, None) == -2
    assert lib.kmi_rmsnorm_quant_act(None, None, 16, None, 16, None, 16, -1.0, 2, 128, None) == -2
    assert lib.kmi_rmsnorm_quant_act(None, None, 16, None, 16, None, 16, 1e-5, 0, 128, None) == 0
    assert lib.kmi_silu_mul_quant_act(16, 16, 16, None, 2, 128, None) == -1
    assert lib.kmi_silu_mul_quant_act(None, None, None, 16, 2, 128, None) == -1
    assert lib.kmi_silu_mul_quant_act(16, None, None, 16, 2, 128, None) == -1
    assert lib.kmi_silu_mul_quant_act(None, None, 8, 16, 2, 128, None) == -5
    assert lib.kmi_silu_mul_quant_act(None, None, 16, 16, 2, 100, None) == -2
    assert lib.kmi_silu_mul_quant_act(None, None, 16, 16, 0, 128, None) == 0
    assert lib.kmi_lut_get(None, 3) == -7


def test_split_choice_depends_on_the_arguments_only(lib):
    """The number of K splits is a function of shape and scratch size: the same on every host thread, whatever other
    threads did before (there is no registration), 1 without scratch, never more than the scratch holds."""
    import threading
    MiB = 1 << 20
    cases = [(0, 96, 1024, 4096), (0, 256, 4096, 14336), (2, 512, 4096, 14336), (2, 384, 4096, 4096), (3, 300, 4096, 4096),
             (1, 128, 6144, 4096)]
    main = [lib.kmi_gemm_splits_for(l, M, N, K, 64 * MiB) for l, M, N, K in cases]
    assert all(s >= 1 for s in main) and any(s > 1 for s in main)
    assert [lib.kmi_gemm_splits_for(l, M, N, K, 0) for l, M, N, K in cases] == [1] * len(cases)
    for (l, M, N, K), s in zip(cases, main):
        assert s == 1 or s * M * N * 4 <= 64 * MiB
        small = lib.kmi_gemm_splits_for(l, M, N, K, 2 * M * N * 4)
        assert small <= 2                                              # a buffer of two slices allows two splits at most
    box = []
    t = threading.Thread(target=lambda: box.append([lib.kmi_gemm_splits_for(l, M, N, K, 64 * MiB) for l, M, N, K in cases]))
    t.start()
    t.join()
    assert box[0] == main
    assert lib.kmi_gemm_splits_for(9, 16, 64, 128, 0) == -2 and lib.kmi_gemm_splits_for(0, 16, 64, 100, 0) == -2


def test_lut_matches_oracle_on_reference_tables(lib, golden_dir):
    for f in ("prof_llama_seg_perf_list.json", "prof_qwen_seg_perf_list.json"):
        for seg in O.load_seg_perf_list(os.path.join(golden_dir, f)):
            h = lib.kmi_lut_new()
            mine = O.LUT()
            for r, name, _ in seg:
                lib.kmi_lut_record(h, r, O.COMP_TYPE_NAME[name])
                mine.record(r, O.COMP_TYPE_NAME[name])
            assert lib.kmi_lut_size(h) == len(seg)
            lib.kmi_lut_shrink_to_fit(h)
            for m in list(range(1, 2500)) + [5, 5, 30720, 30721, 10 ** 6, 1, 1]:
                assert lib.kmi_lut_get(h, m) == mine.get(m)
            lib.kmi_lut_free(h)


def test_small_m_plan_is_host_logic(lib):
    """Which form and split the small-M entry point takes (measured rule, see the kernel file): the ring form beyond 16
    rows everywhere and from 8 rows (1 where K is long) on narrow weights, the register form on wide weights up to 16
    rows; long, narrow weights split K over workgroups only when the caller brought scratch for it."""
    import ctypes
    from kairos_amd import ops

    def plan(M, N, K, ws=ops.GEMV_WORKSPACE_BYTES):
        return ops.gemv_plan(M, N, K, ws)

    assert plan(1, 28672, 4096)["form"] == "register" and plan(16, 28672, 4096)["form"] == "register"
    assert plan(32, 28672, 4096) == {"form": "ring", "nt": 4, "nw": 8, "ks": 1, "depth": 2}
    assert plan(1, 4096, 4096)["form"] == "register" and plan(8, 4096, 4096)["form"] == "ring"
    assert plan(4, 6144, 4096)["form"] == "register" and plan(8, 6144, 4096)["form"] == "ring"
    assert plan(16, 6144, 4096) == {"form": "ring", "nt": 2, "nw": 8, "ks": 1, "depth": 2} and plan(32, 6144, 4096)["nt"] == 2
    assert plan(16, 10240, 8192)["form"] == "ring" and plan(8, 10240, 8192)["form"] == "register"
    assert plan(16, 8192, 28672)["form"] == "register" and plan(32, 8192, 28672)["form"] == "ring"
    assert plan(1, 4096, 14336) == {"form": "ring", "nt": 1, "nw": 8, "ks": 1, "depth": 2}
    assert plan(16, 4096, 14336) == {"form": "ring", "nt": 2, "nw": 8, "ks": 2, "depth": 2}
    assert plan(16, 4096, 14336, 0)["ks"] == 1 and plan(16, 4096, 14336, 0)["form"] == "ring"      # no scratch, no split
    assert plan(32, 8192, 28672) == {"form": "ring", "nt": 4, "nw": 8, "ks": 2, "depth": 2}
    assert plan(64, 57344, 8192) == {"form": "ring", "nt": 2, "nw": 8, "ks": 1, "depth": 2}
    assert plan(4, 4096, 14336 * 2, 1 << 16)["ks"] == 1                                              # scratch too small for a split
    z = ctypes.c_int(0)
    assert lib.kmi_gemv_w4a16_plan(0, 4096, 4096, 0, None, None, None, None, None) == -4
    assert lib.kmi_gemv_w4a16_plan(4, 4090, 4096, 0, ctypes.byref(z), None, None, None, None) == -2
    assert lib.kmi_gemv_w4a16_plan(4, 4096, 4096, 0, None, None, None, None, None) == 0              # outputs are optional


def test_tile_queries_survive_empty_products(lib):
    """The host queries run before the entry points' own M == 0 early return (a tracer asks them): no division by the
    tile count of an empty product."""
    for M, N, K in ((0, 4096, 4096), (4096, 0, 4096), (-3, 4096, 4096)):
        assert lib.kmi_gemm_w4a8_pick_tile(M, N, K) in (128, 130, 192, 256, 448, 512, 640)
        assert lib.kmi_gemm_pick_tile(M, N, K) in (64, 128, 192, 256, 320)
        assert lib.kmi_gemm_w4a16_wp_rows(M, N, K) in (0, 32, 64, 128)
    assert lib.kmi_gemm_w4a8_pick_tile(16, 4096, 0) == 128


def test_w8a8_tile_rule_is_host_logic(lib):
    """kmi_gemm_pick_tile (int8 operands): 256 x 192 tiles (selector 320) where N is a multiple of 384 and they make one
    round or whole rounds while 256 x 256 tiles would leave a ragged one; 256 x 256 when those come in whole rounds; two
    workgroups per CU on 256 x 128 tiles (192) where 256 x 256 tiles are too few and the rows too short to split."""
    pick = lib.kmi_gemm_pick_tile
    assert pick(2048, 6144, 4096) == 320          # 192 tiles of 256 x 256 against 256 of 256 x 192: one round
    assert pick(4096, 6144, 4096) == 320          # 384 against 512: two whole rounds instead of 1.5
    assert pick(8192, 6144, 4096) == 256          # 768 tiles of 256 x 256 are three whole rounds already
    assert pick(4096, 28672, 4096) == 256 and pick(4096, 4096, 14336) == 256
    assert pick(2048, 4096, 14336) == 192
    assert pick(64, 4096, 4096) == 64


def test_conversion_cache_handle_keeps_the_bound(lib):
    """The C-side bookkeeping of the bounded conversion buffer: hits only for the very copy the buffer holds, a request
    beyond the buffer is refused, invalidation forgets."""
    import ctypes
    assert not lib.kmi_cache_create(None, 1024) and not lib.kmi_cache_create(24, 1024) and not lib.kmi_cache_create(4096, 0)
    c = lib.kmi_cache_create(4096, 1 << 20)
    assert c
    ptr = ctypes.c_void_p()
    try:
        assert lib.kmi_cache_acquire(c, 7, 2, 1 << 19, ctypes.byref(ptr)) == 0 and ptr.value == 4096      # miss: convert now
        assert lib.kmi_cache_acquire(c, 7, 2, 1 << 19, ctypes.byref(ptr)) == 1                              # same copy: hit
        assert lib.kmi_cache_acquire(c, 7, 3, 1 << 19, ctypes.byref(ptr)) == 0                              # other format
        assert lib.kmi_cache_acquire(c, 8, 3, 1 << 19, ctypes.byref(ptr)) == 0                              # other layer
        assert lib.kmi_cache_acquire(c, 8, 3, 1 << 19, ctypes.byref(ptr)) == 1
        assert lib.kmi_cache_acquire(c, 8, 3, (1 << 20) + 16, ctypes.byref(ptr)) == -2                      # beyond the bound
        assert b"asked of a buffer" in lib.kmi_get_last_error_string()
        assert lib.kmi_cache_acquire(c, 8, 3, 1 << 19, ctypes.byref(ptr)) == 1                              # a refusal changes nothing
        assert lib.kmi_cache_invalidate(c) == 0 and lib.kmi_cache_acquire(c, 8, 3, 1 << 19, ctypes.byref(ptr)) == 0
        cap, high = ctypes.c_size_t(), ctypes.c_size_t()
        hits, misses = ctypes.c_uint64(), ctypes.c_uint64()
        assert lib.kmi_cache_stats(c, ctypes.byref(cap), ctypes.byref(high), ctypes.byref(hits), ctypes.byref(misses)) == 0
        assert (cap.value, high.value, hits.value, misses.value) == (1 << 20, 1 << 19, 3, 4)
        assert lib.kmi_cache_acquire(None, 1, 1, 16, ctypes.byref(ptr)) == -7 and lib.kmi_cache_acquire(c, 1, 1, 16, None) == -1
    finally:
        lib.kmi_cache_destroy(c)
