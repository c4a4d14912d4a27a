"""Tensor-level wrappers over the C ABI, named after the native functions of the reference that they
replace (kernels/csrc/pybind.cpp:18-24, thirdparty/AWQ/kernels/csrc/pybind.cpp:21-23).

PyTorch only supplies device memory and the current stream; every computation happens in
libkairos_mi.so.  Outputs are allocated by the caller unless the reference function returns one.
"""
import threading

import torch

from . import _lib

GROUP_SIZE = 128
GEMV_MAX_M = 64

# Optional kernel tracer (profiling tools): an object with begin(name, M, N, K) / end() that is
# called around every kernel launch.  None in normal operation.
_tracer = None


def set_tracer(tracer):
    global _tracer
    _tracer = tracer


def _call(name, M, N, K, fn, *args):
    if _tracer is None:
        return _lib.check(fn(*args))
    _tracer.begin(name, M, N, K)
    try:
        return _lib.check(fn(*args))
    finally:
        _tracer.end()


try:                                       # raw handle of torch's current stream without building a Stream object
    _raw_stream = torch._C._cuda_getCurrentRawStream
except AttributeError:                     # pragma: no cover
    _raw_stream = None


def _stream():
    if _raw_stream is not None:
        return _raw_stream(torch.cuda.current_device())
    return torch.cuda.current_stream().cuda_stream


def _ptr(t):
    return 0 if t is None else t.data_ptr()


def _need(t, dtype, name):
    if t.dtype != dtype:
        raise TypeError(f"{name}: expected {dtype}, got {t.dtype}")
    if not t.is_cuda:
        raise ValueError(f"{name}: expected a GPU tensor (the HIP library is the only compute path)")
    if not t.is_contiguous():
        raise ValueError(f"{name}: expected a contiguous tensor")
    return t


# ---- conversion ---------------------------------------------------------------------------------
def dequant_interleaved_int4_to_fp16(output, qweight, scale, scaled_zero, group_size=GROUP_SIZE, tiled=False):
    """output fp16 [N, K] <- packed int4 [N/4, K] (dequant_i4_to_f16.cu:155-185)."""
    _need(output, torch.float16, "output"); _need(qweight, torch.int16, "qweight")
    _need(scale, torch.float16, "scale"); _need(scaled_zero, torch.float16, "scaled_zero")
    N, K = qweight.shape[0] * 4, qweight.shape[1]
    fn = _lib.load().kmi_cvt_i4_to_f16_tiled if tiled else _lib.load().kmi_cvt_i4_to_f16
    _call("cvt_i4_to_f16", 0, N, K, fn, output.data_ptr(), qweight.data_ptr(), scale.data_ptr(),
          scaled_zero.data_ptr(), N, K, group_size, _stream())


def dequant_interleaved_int4_to_int8(output, qweight, scale, scaled_zero, group_size=GROUP_SIZE, tiled=False):
    """output int8 [N, K] <- packed int4 [N/4, K] (dequant_i4_to_i8.cu:152-180)."""
    _need(output, torch.int8, "output"); _need(qweight, torch.int16, "qweight")
    _need(scale, torch.float16, "scale"); _need(scaled_zero, torch.float16, "scaled_zero")
    N, K = qweight.shape[0] * 4, qweight.shape[1]
    fn = _lib.load().kmi_cvt_i4_to_i8_tiled if tiled else _lib.load().kmi_cvt_i4_to_i8
    _call("cvt_i4_to_i8", 0, N, K, fn, output.data_ptr(), qweight.data_ptr(), scale.data_ptr(),
          scaled_zero.data_ptr(), N, K, group_size, _stream())


def untile(tiled, N, K):
    """Tiled MFMA staging layout -> row-major [N, K] (verification helper)."""
    out = torch.empty((N, K), dtype=tiled.dtype, device=tiled.device)
    _lib.check(_lib.load().kmi_untile(out.data_ptr(), tiled.data_ptr(), N, K, tiled.element_size(), _stream()))
    return out


# ---- activation quantiser -----------------------------------------------------------------------
def quant_fp16_to_int8(out, input, scale):
    """out int8 [..., K], scale fp16 [tokens] <- input fp16 [..., K] (quant_f16_to_i8.cu:86-104)."""
    _need(out, torch.int8, "out"); _need(input, torch.float16, "input"); _need(scale, torch.float16, "scale")
    K = input.shape[-1]
    M = input.numel() // K if K else 0
    _call("quant_act_i8", M, 0, K, _lib.load().kmi_quant_act_i8, out.data_ptr(), scale.data_ptr(), input.data_ptr(),
          M, K, _stream())


def rmsnorm_quant(x, gamma, eps, residual=None, want_f16=True, want_i8=True):
    """RMSNorm of x (of x + residual when given) emitting the activation formats asked for, in one launch.

    x, residual fp16 [..., K]; gamma fp16 [K].  Returns (y, int_x, scale_x, h): y fp16 like x or None; int_x int8
    like x and scale_x fp16 [tokens], or None, None; h = fp16(x + residual), the updated residual stream, or None
    without a residual.  int_x / scale_x equal quant_fp16_to_int8 applied to y bit for bit."""
    _need(x, torch.float16, "x"); _need(gamma, torch.float16, "gamma")
    if not (want_f16 or want_i8):
        raise ValueError("rmsnorm_quant: at least one output format is needed")
    K = x.shape[-1]
    if gamma.numel() != K:
        raise ValueError(f"rmsnorm_quant: gamma has {gamma.numel()} entries, x {K} columns")
    M = x.numel() // K if K else 0
    h = None
    if residual is not None:
        _need(residual, torch.float16, "residual")
        if residual.shape != x.shape:
            raise ValueError("rmsnorm_quant: residual and x differ in shape")
        h = torch.empty_like(x)
    y = torch.empty_like(x) if want_f16 else None
    int_x = torch.empty_like(x, dtype=torch.int8) if want_i8 else None
    scale_x = torch.empty((M,), dtype=torch.float16, device=x.device) if want_i8 else None
    if M == 0:
        return y, int_x, scale_x, h
    _call("rmsnorm_quant_act", M, 0, K, _lib.load().kmi_rmsnorm_quant_act, _ptr(int_x), _ptr(scale_x), _ptr(y), _ptr(h),
          x.data_ptr(), _ptr(residual), gamma.data_ptr(), float(eps), M, K, _stream())
    return y, int_x, scale_x, h


def silu_mul_quant(gate_up, want_f16=True, want_i8=True):
    """SiLU(gate) * up of a fused gate/up output [..., 2*I] (gate first), in the formats asked for, in one launch.
    Returns (y fp16 [..., I] or None, int_x int8 [..., I] or None, scale_x fp16 [tokens] or None); int_x / scale_x equal
    quant_fp16_to_int8 applied to y bit for bit."""
    _need(gate_up, torch.float16, "gate_up")
    if not (want_f16 or want_i8):
        raise ValueError("silu_mul_quant: at least one output format is needed")
    if gate_up.shape[-1] % 2:
        raise ValueError("silu_mul_quant: the last dimension holds gate and up, it must be even")
    I = gate_up.shape[-1] // 2
    M = gate_up.numel() // (2 * I) if I else 0
    shape = gate_up.shape[:-1] + (I,)
    y = torch.empty(shape, dtype=torch.float16, device=gate_up.device) if want_f16 else None
    int_x = torch.empty(shape, dtype=torch.int8, device=gate_up.device) if want_i8 else None
    scale_x = torch.empty((M,), dtype=torch.float16, device=gate_up.device) if want_i8 else None
    if M == 0:
        return y, int_x, scale_x
    _call("silu_mul_quant_act", M, 0, I, _lib.load().kmi_silu_mul_quant_act, _ptr(int_x), _ptr(scale_x), _ptr(y),
          gate_up.data_ptr(), M, I, _stream())
    return y, int_x, scale_x


def prep_w8a8(w8_out, qweight, scale_to8, scaled_zero_to8, int_x, x, scale_x, group_size=GROUP_SIZE, tiled=False):
    """int4 -> int8 weight conversion and per-token activation quantisation in one launch (bit-identical to
    dequant_interleaved_int4_to_int8 followed by quant_fp16_to_int8)."""
    _need(w8_out, torch.int8, "w8_out"); _need(qweight, torch.int16, "qweight")
    _need(scale_to8, torch.float16, "scale_to8"); _need(scaled_zero_to8, torch.float16, "scaled_zero_to8")
    _need(int_x, torch.int8, "int_x"); _need(x, torch.float16, "x"); _need(scale_x, torch.float16, "scale_x")
    N, K = qweight.shape[0] * 4, qweight.shape[1]
    if x.shape[-1] != K:
        raise ValueError(f"prep_w8a8: x has {x.shape[-1]} columns, the weight {K}")
    M = x.numel() // K
    _call("prep_w8a8", M, N, K, _lib.load().kmi_prep_w8a8, w8_out.data_ptr(), 1 if tiled else 0, qweight.data_ptr(),
          scale_to8.data_ptr(), scaled_zero_to8.data_ptr(), N, K, group_size, int_x.data_ptr(), scale_x.data_ptr(),
          x.data_ptr(), M, _stream())


def prepare_weight(weight, group_size=GROUP_SIZE):
    """fp16 [N, K] weight on the GPU -> dict of the six resident tensors (DynamicLinear.from_module,
    kairos/dynamic_linear.py:95-111), computed by one kernel; bit-identical to weight_prep.prepare_linear_weight."""
    _need(weight, torch.float16, "weight")
    if weight.dim() != 2:
        raise ValueError(f"prepare_weight: weight must be 2-D, got {tuple(weight.shape)}")
    N, K = weight.shape
    lib = _lib.load()
    gp = lib.kmi_padded_groups(K, group_size)
    if gp < 0:
        raise ValueError(lib.kmi_get_last_error_string().decode())
    dev = weight.device
    out = {"qweight": torch.empty((max(N // 4, 0), K), dtype=torch.int16, device=dev),
           "scales": torch.empty((gp, N), dtype=torch.float16, device=dev),
           "scaled_zeros": torch.empty((gp, N), dtype=torch.float16, device=dev),
           "scales_to8": torch.empty((gp, N), dtype=torch.float16, device=dev),
           "scaled_zeros_to8": torch.empty((gp, N), dtype=torch.float16, device=dev),
           "scales_1": torch.empty((N,), dtype=torch.float16, device=dev)}
    _call("prepare_weight", 0, N, K, lib.kmi_prepare_weight, weight.data_ptr(), N, K, group_size,
          out["qweight"].data_ptr(), out["scales"].data_ptr(), out["scaled_zeros"].data_ptr(),
          out["scales_to8"].data_ptr(), out["scaled_zeros_to8"].data_ptr(), out["scales_1"].data_ptr(), _stream())
    return out


def trans_layout_c16_to_c8_awq(awq_packed, N, K):
    """Resident packed int4 [N/4, K] -> int8 [N, K/2] in the W4A8 operand layout; allocates and returns the output
    as the reference binding does (trans_layout_marlin_c16_to_c8.cu:183-205)."""
    _need(awq_packed, torch.int16, "awq_packed")
    if awq_packed.numel() != (N // 4) * K:
        raise ValueError(f"trans_layout_c16_to_c8_awq: tensor of {awq_packed.numel()} words does not match N={N} K={K}")
    out = torch.empty((N, K // 2), dtype=torch.int8, device=awq_packed.device)
    _call("trans_layout_w4a8", 0, N, K, _lib.load().kmi_trans_layout_w4a8, out.data_ptr(), awq_packed.data_ptr(), N, K,
          _stream())
    return out


# ---- products -----------------------------------------------------------------------------------
def _flat2d(x):
    return x.reshape(-1, x.shape[-1])


def gemv_forward(x, qweight, scales, scaled_zeros, m, n, k, group_size=GROUP_SIZE, bias=None, cfg=None, ring=None):
    """W4A16 for small m (gemv_cuda.cu:245-463).  Returns fp16 [*x.shape[:-1], n].  Tuning: cfg = (column tiles per wave,
    waves per workgroup[, workgroups over K]) runs the register form, ring = (column tiles, waves, workgroups over K,
    ring depth) the ring form; neither = the library's choice."""
    _need(x, torch.float16, "x"); _need(qweight, torch.int16, "qweight")
    if x.shape[-1] != k or x.numel() != m * k:
        raise ValueError(f"gemv_forward: x of shape {tuple(x.shape)} is not {m} rows of {k}")
    if qweight.shape[0] * 4 != n or qweight.shape[1] != k:
        raise ValueError(f"gemv_forward: packed weight {tuple(qweight.shape)} does not hold {n} x {k}")
    out = torch.empty(x.shape[:-1] + (n,), dtype=torch.float16, device=x.device)
    lib = _lib.load()
    st = _stream()
    ws = gemv_workspace_for(x.device, st)
    try:
        if ring is not None:
            nt, nw, ks, depth = ring
            _call("gemv_w4a16", m, n, k, lib.kmi_gemv_w4a16_ring_cfg, out.data_ptr(), x.data_ptr(), qweight.data_ptr(),
                  scales.data_ptr(), scaled_zeros.data_ptr(), _ptr(bias), m, n, k, group_size, nt, nw, ks, depth,
                  ws.data_ptr(), ws.numel(), st)
        else:
            nt, nw, ks = (tuple(cfg) + (1,))[:3] if cfg is not None else (0, 0, 0)
            _call("gemv_w4a16", m, n, k, lib.kmi_gemv_w4a16_cfg, out.data_ptr(), x.data_ptr(), qweight.data_ptr(),
                  scales.data_ptr(), scaled_zeros.data_ptr(), _ptr(bias), m, n, k, group_size, nt, nw, ks, ws.data_ptr(),
                  ws.numel(), st)
    except _lib.KairosMiError as e:
        if e.code == -6:                   # the runtime rejected a launch: leave the counters in a known state
            lib.kmi_gemv_ws_reset(ws.data_ptr(), ws.numel(), st)
        raise
    return out


WORKSPACE_BYTES = 64 << 20
GEMV_WORKSPACE_BYTES = 65536 + (32 << 20)      # arrival counters (KMI_GEMV_WS_HEADER) + fp32 partial sums
_workspaces = {}                 # (device index, raw stream handle) -> uint8 tensor; never resized
_gemv_workspaces = {}            # the same for the small-M kernel's scratch (zeroed counter header first)
_override = threading.local()    # .scratch: a Scratch that replaces the per-stream buffers in this thread, or None


class Scratch:
    """One owner's pair of scratch buffers: split-K partial sums of the GEMMs (`gemm`) and the small-M kernel's
    arrival counters + partial sums (`gemv`, counters zeroed here).  Work that shares a Scratch must be ordered (one
    stream, or replays that wait for each other): two launches using it at the same time race on the partial sums.
    `with scratch:` makes every call of this thread use it instead of the per-stream buffers -- a graph captured inside
    the block owns its scratch, whatever stream it is replayed on."""

    def __init__(self, device="cuda"):
        dev = torch.device(device)
        idx = dev.index if dev.index is not None else torch.cuda.current_device()
        self.device_index = idx
        self.gemm = torch.empty(WORKSPACE_BYTES, dtype=torch.uint8, device=torch.device("cuda", idx))
        self.gemv = torch.zeros(GEMV_WORKSPACE_BYTES, dtype=torch.uint8, device=torch.device("cuda", idx))

    def __enter__(self):
        self._prev = getattr(_override, "scratch", None)
        _override.scratch = self
        return self

    def __exit__(self, *exc):
        _override.scratch = self._prev
        return False

    def reset(self):
        """Arrival counters back to zero (after a call on this scratch that did not run to completion)."""
        _lib.check(_lib.load().kmi_gemv_ws_reset(self.gemv.data_ptr(), self.gemv.numel(), _stream()))


def _index_of(device):
    dev = torch.device(device)
    return dev.index if dev.index is not None else torch.cuda.current_device()


def _new_scratch(idx, nbytes, zero, what):
    # Allocating under stream capture would take the buffer from the graph's private pool (and, zeroed, record a
    # memset node) and then hand it to eager calls as well: refuse, and say what to do instead.
    if torch.cuda.is_current_stream_capturing():
        raise RuntimeError(f"the {what} scratch of this stream does not exist yet and cannot be created during graph "
                           "capture: call kairos_amd.ops.ensure_workspace(device, stream) before capturing, or capture "
                           "inside `with kairos_amd.ops.Scratch(device):`")
    make = torch.zeros if zero else torch.empty
    return make(nbytes, dtype=torch.uint8, device=torch.device("cuda", idx))


def workspace_for(device, stream=None):
    """Split-K scratch for a GEMM call: the active Scratch of this thread if there is one, else one fixed-size buffer
    per (device, stream), created on first use.  Streams are told apart by their raw handle; a handle that the runtime
    hands out again after its stream was destroyed finds the old buffer, which is harmless as long as the destroyed
    stream's work has finished.  A pointer baked into a captured graph stays valid until release_workspace /
    drop_workspaces; a graph that must not share scratch with eager work on the same stream captures under a Scratch."""
    ov = getattr(_override, "scratch", None)
    if ov is not None:
        return ov.gemm
    idx = _index_of(device)
    if stream is None:
        stream = _stream()
    ws = _workspaces.get((idx, stream))
    if ws is None:
        ws = _workspaces[(idx, stream)] = _new_scratch(idx, WORKSPACE_BYTES, False, "split-K")
    return ws


def gemv_workspace_for(device, stream=None):
    """Scratch of the small-M kernel's split over K, chosen like workspace_for, but ZEROED at creation: its first 64 KiB
    are arrival counters that the kernels return to zero themselves.  Kept apart from the GEMM scratch, whose partial
    sums would overwrite the counters."""
    ov = getattr(_override, "scratch", None)
    if ov is not None:
        return ov.gemv
    idx = _index_of(device)
    if stream is None:
        stream = _stream()
    ws = _gemv_workspaces.get((idx, stream))
    if ws is None:
        ws = _gemv_workspaces[(idx, stream)] = _new_scratch(idx, GEMV_WORKSPACE_BYTES, True, "small-M")
    return ws


def gemv_workspace_reset(device="cuda", stream=None):
    """Zeroes the arrival counters of the calling (or given) stream's small-M scratch with a small kernel: after a
    call that raised, or whenever the buffer's history is in doubt."""
    ws = gemv_workspace_for(device, stream)
    _lib.check(_lib.load().kmi_gemv_ws_reset(ws.data_ptr(), ws.numel(), _stream() if stream is None else stream))


def ensure_workspace(device="cuda", stream=None):
    """Creates the calling (or given) stream's scratch buffers ahead of time, e.g. before a graph capture on it."""
    gemv_workspace_for(device, stream)
    return workspace_for(device, stream)


def release_workspace(device="cuda", stream=None):
    """Forgets the scratch of one (device, stream); the memory returns to the allocator once no tensor refers to it.
    Not while work that uses it is pending or a captured graph that used it is alive."""
    idx = _index_of(device)
    if stream is None:
        stream = _stream()
    _workspaces.pop((idx, stream), None)
    _gemv_workspaces.pop((idx, stream), None)


def drop_workspaces():
    """Forgets every per-stream scratch buffer (tests).  Not while a captured graph that used one is still alive."""
    _workspaces.clear()
    _gemv_workspaces.clear()


def gemv_plan(M, N, K, workspace_bytes=GEMV_WORKSPACE_BYTES):
    """What the small-M entry point does for this shape (host only): dict with form ('register' / 'ring'), nt (16-column
    tiles per wave), nw (waves per workgroup), ks (workgroups sharing a strip's K range), depth (ring slots asked for)."""
    import ctypes
    v = [ctypes.c_int(0) for _ in range(5)]
    _lib.check(_lib.load().kmi_gemv_w4a16_plan(int(M), int(N), int(K), int(workspace_bytes), *[ctypes.byref(c) for c in v]))
    return {"form": "ring" if v[0].value == 1 else "register", "nt": v[1].value, "nw": v[2].value, "ks": v[3].value,
            "depth": v[4].value}


def gemm_splits_for(lane, M, N, K, workspace_bytes=WORKSPACE_BYTES):
    """K splits a GEMM call of `lane` ('w4a16', 'w8a16', 'w8a8', 'f16') would use with that much scratch (host only)."""
    return _lib.check(_lib.load().kmi_gemm_splits_for({"w4a16": 0, "w8a16": 1, "w8a8": 2, "f16": 3}[lane], int(M), int(N),
                                                      int(K), int(workspace_bytes)))


def gemm_forward(x, qweight, scales, scaled_zeros, bias=None):
    """W4A16 MFMA GEMM for any m (gemm_cuda.cu:1126-1235).  Returns fp16 [*x.shape[:-1], N]."""
    _need(x, torch.float16, "x"); _need(qweight, torch.int16, "qweight")
    N, K = qweight.shape[0] * 4, qweight.shape[1]
    x2 = _flat2d(x)
    out = torch.empty(x.shape[:-1] + (N,), dtype=torch.float16, device=x.device)
    st = _stream()
    ws = workspace_for(x.device, st)
    _call("gemm_w4a16", x2.shape[0], N, K, _lib.load().kmi_gemm_w4a16, out.data_ptr(), x2.data_ptr(),
          qweight.data_ptr(), scales.data_ptr(), scaled_zeros.data_ptr(), _ptr(bias), x2.shape[0], N, K,
          GROUP_SIZE, ws.data_ptr(), ws.numel(), st)
    return out


def w8a8_gemm_forward(in_feats, kernel, wscales, ascales, out_feats, bias=None, tiled=False):
    """out_feats fp16 [M, N] <- int8 [M, K] x int8 [N, K] (w8a8_gemm_cuda.cu:909-954)."""
    _need(in_feats, torch.int8, "in_feats"); _need(kernel, torch.int8, "kernel"); _need(out_feats, torch.float16, "out_feats")
    M, K = in_feats.shape
    N = out_feats.shape[-1]
    fn = _lib.load().kmi_gemm_w8a8_tiled if tiled else _lib.load().kmi_gemm_w8a8
    st = _stream()
    ws = workspace_for(in_feats.device, st)
    _call("gemm_w8a8", M, N, K, fn, out_feats.data_ptr(), in_feats.data_ptr(), kernel.data_ptr(), wscales.data_ptr(),
          ascales.data_ptr(), _ptr(bias), M, N, K, ws.data_ptr(), ws.numel(), st)


def w4a8_gemm_forward(in_feats, qweight, scales_to8, scaled_zeros_to8, wscales, ascales, out_feats, bias=None):
    """out_feats fp16 [M, N] <- int8 [M, K] x packed int4 [N/4, K]: the W8A8 product of the weight the int4 -> int8
    converter would write, decoded inside the GEMM (bit-identical to dequant_interleaved_int4_to_int8 +
    w8a8_gemm_forward; takes the place of the version-2 candidate, kairos/dynamic_linear_v2.py:161-179)."""
    _need(in_feats, torch.int8, "in_feats"); _need(qweight, torch.int16, "qweight"); _need(out_feats, torch.float16, "out_feats")
    _need(scales_to8, torch.float16, "scales_to8"); _need(scaled_zeros_to8, torch.float16, "scaled_zeros_to8")
    M, K = in_feats.shape
    N = qweight.shape[0] * 4
    if qweight.shape[1] != K or out_feats.shape[-1] != N:
        raise ValueError(f"w4a8_gemm_forward: activations [{M}, {K}], weight [{N}, {qweight.shape[1]}], output {tuple(out_feats.shape)}")
    st = _stream()
    ws = workspace_for(in_feats.device, st)
    _call("gemm_w4a8", M, N, K, _lib.load().kmi_gemm_w4a8, out_feats.data_ptr(), in_feats.data_ptr(), qweight.data_ptr(),
          scales_to8.data_ptr(), scaled_zeros_to8.data_ptr(), wscales.data_ptr(), ascales.data_ptr(), _ptr(bias), M, N, K,
          GROUP_SIZE, ws.data_ptr(), ws.numel(), st)


def w4a8_gemm_acc_i32(in_feats, qweight, scales_to8, scaled_zeros_to8):
    """Raw int32 accumulators [M, N] of the W4A8 product."""
    _need(in_feats, torch.int8, "in_feats"); _need(qweight, torch.int16, "qweight")
    M, K = in_feats.shape
    N = qweight.shape[0] * 4
    acc = torch.empty((M, N), dtype=torch.int32, device=in_feats.device)
    st = _stream()
    ws = workspace_for(in_feats.device, st)
    _lib.check(_lib.load().kmi_gemm_w4a8_acc_i32(acc.data_ptr(), in_feats.data_ptr(), qweight.data_ptr(), scales_to8.data_ptr(),
                                                 scaled_zeros_to8.data_ptr(), M, N, K, GROUP_SIZE, ws.data_ptr(), ws.numel(), st))
    return acc


def _need_int_tables(name, s2_scales, s2_zeros, N, K):
    for t, what in ((s2_scales, "s2_scales"), (s2_zeros, "s2_zeros")):
        _need(t, torch.int8, what)
        if t.dim() != 2 or t.shape[0] < K // GROUP_SIZE or t.shape[1] != N:
            raise ValueError(f"{name}: {what} must be int8 [K/{GROUP_SIZE}, N] = [{K // GROUP_SIZE}, {N}], got {tuple(t.shape)}")


def w4a8_int_gemm_forward(in_feats, qweight, s2_scales, s2_zeros, wscales, ascales, out_feats, bias=None):
    """out_feats fp16 [M, N] <- int8 [M, K] x packed int4 [N/4, K] with integer per-group factors: the arithmetic of
    omniserve_backend.qgemm_w4a8_per_group.gemm_forward_cuda as the version-2 layer calls it
    (kairos/dynamic_linear_v2.py:161-179), on the resident weight (no re-pack) and with the int8 tables [K/128, N] in
    plain column order: weight byte = (q * s2_scales + s2_zeros) mod 256."""
    _need(in_feats, torch.int8, "in_feats"); _need(qweight, torch.int16, "qweight"); _need(out_feats, torch.float16, "out_feats")
    M, K = in_feats.shape
    N = qweight.shape[0] * 4
    if qweight.shape[1] != K or out_feats.shape[-1] != N:
        raise ValueError(f"w4a8_int_gemm_forward: activations [{M}, {K}], weight [{N}, {qweight.shape[1]}], output {tuple(out_feats.shape)}")
    _need_int_tables("w4a8_int_gemm_forward", s2_scales, s2_zeros, N, K)
    st = _stream()
    ws = workspace_for(in_feats.device, st)
    _call("gemm_w4a8_int", M, N, K, _lib.load().kmi_gemm_w4a8_int, out_feats.data_ptr(), in_feats.data_ptr(), qweight.data_ptr(),
          s2_scales.data_ptr(), s2_zeros.data_ptr(), wscales.data_ptr(), ascales.data_ptr(), _ptr(bias), M, N, K,
          GROUP_SIZE, ws.data_ptr(), ws.numel(), st)


def w4a8_int_gemm_acc_i32(in_feats, qweight, s2_scales, s2_zeros):
    """Raw int32 accumulators [M, N] of the integer-factor W4A8 product."""
    _need(in_feats, torch.int8, "in_feats"); _need(qweight, torch.int16, "qweight")
    M, K = in_feats.shape
    N = qweight.shape[0] * 4
    _need_int_tables("w4a8_int_gemm_acc_i32", s2_scales, s2_zeros, N, K)
    acc = torch.empty((M, N), dtype=torch.int32, device=in_feats.device)
    st = _stream()
    ws = workspace_for(in_feats.device, st)
    _lib.check(_lib.load().kmi_gemm_w4a8_int_acc_i32(acc.data_ptr(), in_feats.data_ptr(), qweight.data_ptr(), s2_scales.data_ptr(),
                                                     s2_zeros.data_ptr(), M, N, K, GROUP_SIZE, ws.data_ptr(), ws.numel(), st))
    return acc


def w8a8_gemm_acc_i32(in_feats, kernel, N):
    """Raw int32 accumulators [M, N] of the W8A8 product."""
    _need(in_feats, torch.int8, "in_feats"); _need(kernel, torch.int8, "kernel")
    M, K = in_feats.shape
    acc = torch.empty((M, N), dtype=torch.int32, device=in_feats.device)
    st = _stream()
    ws = workspace_for(in_feats.device, st)
    _lib.check(_lib.load().kmi_gemm_w8a8_acc_i32(acc.data_ptr(), in_feats.data_ptr(), kernel.data_ptr(), M, N, K,
                                                 ws.data_ptr(), ws.numel(), st))
    return acc


def w8a16_gemm_forward(x, w8, wscales, N, bias=None):
    """fp16 [M, N] <- fp16 [M, K] x int8 [N, K] (row-major), per-channel scale in the epilogue."""
    _need(x, torch.float16, "x"); _need(w8, torch.int8, "w8")
    x2 = _flat2d(x)
    M, K = x2.shape
    out = torch.empty(x.shape[:-1] + (N,), dtype=torch.float16, device=x.device)
    st = _stream()
    ws = workspace_for(x.device, st)
    _call("gemm_w8a16", M, N, K, _lib.load().kmi_gemm_w8a16, out.data_ptr(), x2.data_ptr(), w8.data_ptr(),
          wscales.data_ptr(), _ptr(bias), M, N, K, ws.data_ptr(), ws.numel(), st)
    return out


def f16_gemm_forward(x, w16, N, bias=None, tiled=False):
    """fp16 [M, N] <- fp16 [M, K] x fp16 [N, K] (`input @ tmp_weight.T`, dynamic_linear.py:163)."""
    _need(x, torch.float16, "x"); _need(w16, torch.float16, "w16")
    x2 = _flat2d(x)
    M, K = x2.shape
    out = torch.empty(x.shape[:-1] + (N,), dtype=torch.float16, device=x.device)
    fn = _lib.load().kmi_gemm_f16_tiled if tiled else _lib.load().kmi_gemm_f16
    st = _stream()
    ws = workspace_for(x.device, st)
    _call("gemm_f16", M, N, K, fn, out.data_ptr(), x2.data_ptr(), w16.data_ptr(), _ptr(bias), M, N, K,
          ws.data_ptr(), ws.numel(), st)
    return out


def gemm_tile_for(M, N, K=4096):
    """Workgroup tile (64/128/256) the automatic choice uses for an M x N output over int8 rows of K bytes."""
    return _lib.load().kmi_gemm_pick_tile(int(M), int(N), int(K))


def gemm_w4a8_tile_for(M, N, K=4096):
    """Tile selector of the W4A8 GEMM for an M x N x K product: 128 (128 x 128), 130 (the same on two wave quartets),
    192 (256 x 128), 256 (256 x 256), 512 (512 x 128), 448 / 640 (256 x 256 / 512 x 128 in whole rounds, the remaining
    columns as 256 x 128 tiles in a second launch)."""
    return _lib.load().kmi_gemm_w4a8_pick_tile(int(M), int(N), int(K))


def gemm_w4a16_wp_rows(M, N, K=4096):
    """Rows per tile of the small-M W4A16 GEMM variant used for an M x N x K product (0: the LDS-staged variant)."""
    return _lib.load().kmi_gemm_w4a16_wp_rows(int(M), int(N), int(K))


def force_gemm_splits(splits):
    """Test hook of the calling thread: 0 = automatic, else the number of K splits."""
    _lib.load().kmi_gemm_force_splits(int(splits))


def force_gemm_group_m(group_m):
    """Test hook of the calling thread: tile rows per group of the GEMM kernels' workgroup -> tile order (0 = default)."""
    _lib.load().kmi_gemm_force_group_m(int(group_m))


def force_gemm_tile(tile):
    """Test hook of the calling thread: 0 = automatic, else 64 / 128 / 192 / 256 (and the 1xxx / 2xxx selectors of the
    small-M W4A16 variant)."""
    _lib.load().kmi_gemm_force_tile(int(tile))
