"""Pins the LUT oracle against the reference's own C++ class (oracle/_ref, when built) and against
the two table files the reference ships (kept as JSON fixtures under tests/golden)."""
import ctypes
import json
import os

import pytest

from oracle import kairos_oracle as O

HERE = os.path.dirname(os.path.abspath(__file__))
REF_SO = os.path.join(os.path.dirname(HERE), "oracle", "_ref", "libref_lut.so")

LLAMA_SHAPES = [(1024, 4096), (4096, 4096), (4096, 14336), (14336, 4096)]     # kairos/main.py llama list
QWEN_SHAPES = [(512, 3584), (3584, 3584), (3584, 18944), (18944, 3584)]


def build(seg):
    lut = O.LUT()
    for r, name, _gain in seg:
        lut.record(r, O.COMP_TYPE_NAME[name])
    return lut


def test_known_answers_llama(golden_dir):
    segs = O.load_seg_perf_list(os.path.join(golden_dir, "prof_llama_seg_perf_list.json"))
    assert len(segs) == 4
    lut = build(segs[1])            # (4096, 4096): <=8 gemv, <=256 w4a16_gemm, else w8a8
    assert [lut.get(m) for m in (1, 8, 9, 256, 257, 30720, 10 ** 6)] == [1, 1, 0, 0, 2, 2, 2]
    lut = build(segs[2])            # (4096, 14336)
    assert [lut.get(m) for m in (2, 3, 1024, 1025, 22528, 22529, 24576, 24577, 99999)] == [1, 6, 6, 2, 2, 5, 5, 2, 2]
    lut = build(segs[0])
    assert [lut.get(m) for m in (16, 17, 64, 65)] == [1, 0, 0, 5]


def test_file_schema(golden_dir):
    for f in ("prof_llama_seg_perf_list.json", "prof_qwen_seg_perf_list.json"):
        segs = json.load(open(os.path.join(golden_dir, f)))
        assert isinstance(segs, list) and len(segs) == 4
        for per_shape in segs:
            edges = [t[0] for t in per_shape]
            assert edges == sorted(edges) and len(set(edges)) == len(edges)
            for t in per_shape:
                assert isinstance(t[0], int) and t[1] in O.COMP_TYPE_NAME and isinstance(t[2], float)


@pytest.mark.skipif(not os.path.exists(REF_SO), reason="oracle/_ref not built (needs the reference tree)")
def test_oracle_matches_reference_cpp(golden_dir):
    lib = ctypes.CDLL(REF_SO)
    lib.ref_lut_new.restype = ctypes.c_void_p
    lib.ref_lut_free.argtypes = [ctypes.c_void_p]
    lib.ref_lut_record.argtypes = [ctypes.c_void_p, ctypes.c_int, ctypes.c_int]
    lib.ref_lut_get.argtypes = [ctypes.c_void_p, ctypes.c_int]
    lib.ref_lut_get.restype = ctypes.c_int
    for f in ("prof_llama_seg_perf_list.json", "prof_qwen_seg_perf_list.json"):
        for seg in json.load(open(os.path.join(golden_dir, f))):
            ref = lib.ref_lut_new()
            mine = build(seg)
            for r, name, _ in seg:
                lib.ref_lut_record(ref, r, O.COMP_TYPE_NAME[name])
            edges = [t[0] for t in seg]
            probe = sorted(set([1, 2, 3, 10 ** 6] + [e + d for e in edges for d in (-1, 0, 1) if e + d >= 1]))
            probe += list(range(1, 2000))
            for m in probe:
                assert lib.ref_lut_get(ref, m) == mine.get(m), (f, m)
            # repeated query (memo path) and out-of-order queries
            for m in (5, 5, 4000, 5, 1, 1):
                assert lib.ref_lut_get(ref, m) == mine.get(m)
            lib.ref_lut_free(ref)
