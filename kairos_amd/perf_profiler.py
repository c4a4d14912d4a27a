"""Offline profiler and interval lookup table (kairos/perf_profiler.py:17-166).

`Profiler(shape_list)` owns one LUT per (N, K) shape.  `profiling()` times every candidate lane of a
DynamicLinear of that shape over a grid of M on the current GPU -- the timed call is `_forward`, so
weight conversion, activation quantisation and output allocation are inside the measurement -- and
run-length compresses the winners into segments.  `save`/`load` use the reference's file:
`<dir>/seg_perf_list.pt`, JSON text, one list per shape of `[m_right_edge, lane_name, gain_pct]`.
"""
import json
import sys
import os

import torch

from . import _lib
from .dynamic_linear import COMP_TYPE_NAME, DynamicLinear
from .perf_eval import timer

print_flag = False

# M grid of the reference (perf_profiler.py:88-90)
DEFAULT_INPUT_LEN = [1, 2, 4, 8, 16, 24, 32, 48, 64, 128, 256, 512] + \
                    [i for i in range(1024, 1024 * 8, 1024)] + \
                    [i for i in range(1024 * 8, 1024 * 32, 2048)]
# candidate lanes: the reference's four plus W8A16, which exists on this hardware
DEFAULT_COMP_TYPES = ['fp16', 'w4a16_gemm', 'w4a16_gemv', 'w8a8', 'w8a16_gemm']
GEMV_MAX_M = 64


class LUT:
    """Interval table backed by the C ABI (kmi_lut_*); same get/record/shrink_to_fit as LUT_module.LUT."""

    def __init__(self):
        self._lib = _lib.load()
        self._h = self._lib.kmi_lut_new()
        if not self._h:
            raise MemoryError("kmi_lut_new failed")

    def get(self, m):
        return _lib.check(self._lib.kmi_lut_get(self._h, int(m)))

    def record(self, r, comp_type_id):
        _lib.check(self._lib.kmi_lut_record(self._h, int(r), int(comp_type_id)))

    def shrink_to_fit(self):
        _lib.check(self._lib.kmi_lut_shrink_to_fit(self._h))

    def __len__(self):
        return self._lib.kmi_lut_size(self._h)

    def __del__(self):
        h, self._h = getattr(self, "_h", None), None
        if h:
            self._lib.kmi_lut_free(h)


def save_json(save_path, obj):
    os.makedirs(os.path.dirname(save_path) or ".", exist_ok=True)
    with open(save_path, "w") as f:
        f.write(json.dumps(obj))


def load_json(load_path):
    with open(load_path) as f:
        return json.load(f)


class Profiler:
    comp_type_name = COMP_TYPE_NAME
    linear_cls = DynamicLinear
    comp_types = DEFAULT_COMP_TYPES          # candidate lanes profiling() times

    @torch.no_grad()
    def __init__(self, shape_list) -> None:
        self.shape_list = [tuple(s) for s in shape_list]
        self.seg_perf_list = []
        self.lut = {shape: LUT() for shape in self.shape_list}

    def record_best_comp(self, shape, r, comp_type):
        self.lut[tuple(shape)].record(r, self.comp_type_name[comp_type])

    def profiling(self, **kwargs):
        for shape in self.shape_list:
            kwargs.setdefault("comp_type_list", self.comp_types)
            seg = test_perf(str(shape), shape[1], shape[0], False, linear_cls=self.linear_cls,
                            comp_type_name=self.comp_type_name, **kwargs)
            for t in seg:
                self.record_best_comp(shape, t[0], t[1])
            self.seg_perf_list.append([list(t) for t in seg])

    def get_comp_type(self, shape, m):
        return self.lut[shape].get(m)

    def save(self, path='./prof/'):
        save_json(os.path.join(path, 'seg_perf_list.pt'), self.seg_perf_list)

    def load(self, path='./prof/'):
        self.seg_perf_list = load_json(os.path.join(path, 'seg_perf_list.pt'))
        if len(self.seg_perf_list) != len(self.shape_list):
            raise ValueError(f"{path}: table holds {len(self.seg_perf_list)} shapes, profiler has {len(self.shape_list)}")
        for shape, seg in zip(self.shape_list, self.seg_perf_list):
            for t in seg:
                self.record_best_comp(shape, t[0], t[1])


def compress_segments(perf_list):
    """Run-length compression of (m, best, gain) tuples: keep the last tuple of every run of equal
    `best` (perf_profiler.py:150-156), so each kept m is the inclusive right edge of its segment."""
    seg = []
    prev = perf_list[0]
    for t in perf_list:
        if t[1] != prev[1]:
            seg.append(prev)
        prev = t
    seg.append(prev)
    return seg


def choose_lane(times, prev_comp='', stickiness=0.01, prefer_resident=0.0):
    """The lane for one M from the measured times {lane: t}: the fastest; unless a lane that reads only the resident
    int4 weight (names starting with 'w4') is within `prefer_resident` of it; unless the previous M's lane is within
    `stickiness` of that choice.  -> (lane, its time)."""
    best_t, best_comp = min((t, c) for c, t in times.items())
    resident = [(t, c) for c, t in times.items() if c.startswith('w4')]
    if prefer_resident > 0 and resident and not best_comp.startswith('w4'):
        t4, c4 = min(resident)
        if t4 <= best_t * (1.0 + prefer_resident):
            best_t, best_comp = t4, c4
    if prev_comp in times and times[prev_comp] <= best_t * (1.0 + stickiness):
        best_t, best_comp = times[prev_comp], prev_comp
    return best_comp, best_t


def lane_allowed(comp_type, m):
    if 'gemv' in comp_type and m > GEMV_MAX_M:
        return False
    return True


@torch.no_grad()
def test_perf(proj_name, K, N, bias, input_len=None, comp_type_list=None, n=200, preheat_time=20,
              linear_cls=DynamicLinear, comp_type_name=COMP_TYPE_NAME, details=None, stickiness=0.01,
              rotate_bytes=512 << 20, head_start_ms=4.0, prefer_resident=0.0):
    """Times every allowed lane for every M and returns the compressed segment list for one shape.

    stickiness: the lane chosen for the previous M is kept unless another lane is more than this fraction faster
    (the reference takes the strict minimum, perf_profiler.py:140-147; two lanes within timing noise of each other
    then trade places from run to run and split a segment for nothing).  0 restores the strict minimum.

    rotate_bytes: consecutive calls go to copies of the layer whose packed weights add up to at least this many
    bytes (at most 16 copies), so that no call finds its weights in the 256 MiB last-level cache -- in a model
    the next call belongs to another layer.  The reference times one layer over and over (perf_profiler.py:128-132),
    which on this part favours the lanes that stream the packed weight (an 8 MiB weight stays in cache).  0 = one copy.

    head_start_ms: the timed calls are queued behind an idle kernel of this length, so that the device finds them
    waiting and the events bracket device time.  Without it a lane of one 8 us launch and a lane of two 6 us launches
    both read as the ~17 us the host needs per call, although the device (and a replayed HIP graph) tells them
    apart.  0 = time as the reference does.

    prefer_resident: a lane that reads only the resident int4 weight is taken while it is within this fraction of
    the fastest lane (the argument for it: the profile times every lane alone on the device, where the 1.5 N K bytes
    a conversion writes and the GEMM reads back cost only their own time, while in a model they also push the next
    layer's weights out of the last-level cache and occupy the shared buffer).  Default 0 = the fastest lane, always,
    as the reference chooses (perf_profiler.py:133-135): a same-box comparison of tables built with 0.04 and with 0
    showed no difference in the end-to-end figures, so the shipped tables take the measured minimum."""
    torch.manual_seed(10)
    lin = torch.nn.Linear(in_features=K, out_features=N, bias=bias, dtype=torch.float16).cuda()
    dlinear = linear_cls.from_module(lin, 'cuda')
    del lin
    copies = [dlinear]
    weight_bytes = dlinear.qweight.numel() * dlinear.qweight.element_size()
    rotate = rotate_bytes > 0 and not getattr(linear_cls, "resident_copies", False)   # a layer with resident converted copies is not cloned
    for _ in range(min(16, -(-rotate_bytes // weight_bytes)) - 1 if rotate else 0):
        twin = linear_cls(K, N, bias, 'cuda', dlinear.group_size)
        for key, value in dlinear.named_buffers():
            setattr(twin, key, value.clone() if key == 'qweight' else value)
        copies.append(twin)
    # In a model consecutive calls belong to different layers, so a converted weight never survives
    # in the shared temp cache until the next call: the profile must pay the conversion every time.
    cache = dlinear._cache()
    input_len = list(input_len or DEFAULT_INPUT_LEN)
    comp_type_list = list(comp_type_list or DEFAULT_COMP_TYPES)
    perf_list = []
    prev_comp = ''
    for m in input_len:
        x = torch.randn((1, m, K), dtype=torch.float16, device='cuda')
        orig_t = float('inf')
        times = {}
        for comp in comp_type_list:
            if not lane_allowed(comp, m):
                continue
            cid = comp_type_name[comp]
            for i in range(preheat_time):
                cache.invalidate()
                copies[i % len(copies)]._forward(x, m, cid)
            rec = []
            if head_start_ms > 0 and hasattr(torch.cuda, "_sleep"):
                torch.cuda._sleep(int(head_start_ms * 2.4e6))          # ~2.4 counts per nanosecond on this part
            with timer(comp, n=n, recordList=rec, print_flag=print_flag):
                for i in range(n):
                    cache.invalidate()
                    copies[i % len(copies)]._forward(x, m, cid)
            t = rec[-1]
            if details is not None:
                details.append({"shape": [N, K], "m": m, "comp": comp, "ms": t})
            times[comp] = t
            if 'w4' in comp and t < orig_t:
                orig_t = t
        best_comp, best_t = choose_lane(times, prev_comp, stickiness, prefer_resident)
        prev_comp = best_comp
        gain = (orig_t - best_t) * 100 / orig_t if orig_t < float('inf') else 0.0
        perf_list.append((m, best_comp, gain))
        print(f'  N={N} K={K} m={m}: {best_comp} {best_t * 1e3:.1f} us', file=sys.stderr, flush=True)   # progress: a shape takes minutes
    seg = compress_segments(perf_list)
    print('-' * 7 + f'N:{N:5d}  K:{K:5d}' + '-' * 7)
    for t in seg:
        print(f'm: {t[0]:5d}   best: {t[1]:12s}  speed up: {t[2]:4.2f}%')
    return seg


PRESETS = {
    # fused qkv / gate_up shapes of one decoder layer, (N, K)
    "llama3_8b": [(6144, 4096), (4096, 4096), (28672, 4096), (4096, 14336)],
    "llama3_8b_unfused": [(1024, 4096), (4096, 4096), (14336, 4096), (4096, 14336)],
    "llama3_70b": [(10240, 8192), (8192, 8192), (57344, 8192), (8192, 28672)],
    "qwen25_7b": [(4608, 3584), (3584, 3584), (37888, 3584), (3584, 18944)],
}


def main(argv=None):
    import argparse
    ap = argparse.ArgumentParser(description="Rebuild the per-shape M-interval table on this GPU")
    ap.add_argument("--preset", default="llama3_8b", choices=sorted(PRESETS))
    ap.add_argument("--out", required=True, help="directory that receives seg_perf_list.pt (and timings.json)")
    ap.add_argument("--n", type=int, default=200)
    ap.add_argument("--preheat", type=int, default=20)
    ap.add_argument("--max-m", type=int, default=30720)
    ap.add_argument("--v2", action="store_true", help="version-2 id table and candidates (adds the W4A8 lane, id 7)")
    ap.add_argument("--rotate-mb", type=int, default=512,
                    help="rotate over layer copies whose packed weights add up to this many MiB (0 = time one layer over and over, as the reference does)")
    ap.add_argument("--head-start-ms", type=float, default=4.0,
                    help="queue the timed calls behind an idle kernel of this length so that device time is measured (0 = as the reference does)")
    ap.add_argument("--stickiness", type=float, default=0.01, help="keep the previous M's lane within this fraction of the choice (0 = strict minimum)")
    ap.add_argument("--prefer-resident", type=float, default=0.0,
                    help="take a lane that reads only the int4 weight while it is within this fraction of the fastest (0 = strict minimum)")
    args = ap.parse_args(argv)
    # the reference's grid plus the powers of two and the half-way points of the region where the lanes cross
    grid = sorted(set([m for m in DEFAULT_INPUT_LEN if m <= args.max_m] + [1 << i for i in range(13)] + [96, 192, 384, 768, 1536]))
    if args.v2:
        from .perf_profiler_v2 import Profiler as ProfilerCls
    else:
        ProfilerCls = Profiler
    prof = ProfilerCls(PRESETS[args.preset])
    details = []
    prof.profiling(input_len=grid, n=args.n, preheat_time=args.preheat, details=details, prefer_resident=args.prefer_resident,
                   rotate_bytes=args.rotate_mb << 20, head_start_ms=args.head_start_ms, stickiness=args.stickiness)
    out = args.out if args.out.endswith("/") else args.out + "/"
    prof.save(out)
    save_json(os.path.join(out, "timings.json"), details)
    print(f"wrote {out}seg_perf_list.pt")


if __name__ == "__main__":
    main()
