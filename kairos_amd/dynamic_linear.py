"""DynamicLinear: the LUT-switched mixed-precision linear layer (kairos/dynamic_linear.py:39-175).

Weights are resident only as packed int4 (+ fp16 scale tables).  Each call looks M = tokens up in
the offline-profiled interval table of this layer's shape and runs one of the HIP kernel lanes:

    w4a16_gemv (1)  small-M MFMA streaming kernel            kmi_gemv_w4a16
    w4a16_gemm (0)  LDS-staged MFMA GEMM, int4 decoded on the fly   kmi_gemm_w4a16
    w8a8       (2)  int4->int8 conversion + per-token int8 activations + int8 MFMA GEMM
    w8a16_*  (3,4)  int4->int8 conversion + fp16 activations, fp16 MFMA GEMM (declared but unused upstream)
    fp16       (5)  int4->fp16 conversion + fp16 MFMA GEMM
    w4a16 alt  (6)  version-2 tables only: the W4A16 MFMA GEMM again (one W4A16 GEMM exists here)
    w4a8       (7)  version-2 tables only: per-token int8 activations x int4 weights decoded inside the int8 MFMA
                    GEMM; same results as w8a8, no converted copy                  kmi_gemm_w4a8

Same constructor, class attribute `prof`, `from_module`, `forward`, `_forward` and tensor attributes
as the reference module.
"""
import itertools

import torch

from . import ops
from .ops import GEMV_MAX_M as _GEMV_MAX_M, _gemv_workspaces, _override, _raw_stream
from .temp_cache import default_cache
from .weight_prep import calculate_zeros_width, prepare_linear_weight

COMP_TYPE_NAME = {'w4a16_gemm': 0, 'w4a16_gemv': 1, 'w8a8': 2,
                  'w8a16_gemm': 3, 'w8a16_gemv': 4, 'fp16': 5}

_W4A16_GEMM, _W4A16_GEMV, _W8A8, _W8A16_GEMM, _W8A16_GEMV, _FP16 = 0, 1, 2, 3, 4, 5
_W4A16_ALT, _W4A8 = 6, 7          # ids of the version-2 table (kairos/dynamic_linear_v2.py:11-13)
_uids = itertools.count(1)
RESIDENT_KEYS = ("qweight", "scales", "scaled_zeros", "scales_to8", "scaled_zeros_to8", "scales_1")


class DynamicLinear(torch.nn.Module):
    prof = None                 # Profiler shared by every instance, set by the caller (kairos/main.py:52)
    tiled_weights = True        # converted weights are written in the tiled MFMA staging layout
    temp_cache = None           # None -> the process-wide default cache
    resident_copies = False     # True (SwitchLinear): converted weights are kept per layer, no lane converts

    @torch.no_grad()
    def __init__(self, in_features, out_features, bias, device, group_size):
        super().__init__()
        self.enable_accel = False
        self.return_dtype = torch.float16
        self.in_features = in_features
        self.out_features = out_features
        self.group_size = group_size
        if bias:
            self.register_buffer("bias", torch.empty((out_features,), device=device, dtype=torch.float16))
        else:
            self.bias = None
        self.shape = (out_features, in_features)
        self.pre_m = 0
        self.pre_comp_type = ''
        self.comp_type = None
        self._uid = next(_uids)     # identifies this layer's entries in the temp cache
        self._decode_ptrs = None
        self.switch_count = 0       # times the selected lane changed between consecutive forward calls
        # The six resident tensors are buffers, so state_dict() / load_state_dict() carry the quantised layer
        # (the reference keeps them as plain attributes, which torch.save(model.state_dict()) silently drops,
        # kairos/main.py:85-91).  None until from_module fills or allocates them.
        for key in RESIDENT_KEYS:
            self.register_buffer(key, None)

    def _allocate_resident(self, device):
        """Uninitialised resident tensors of the right shapes: the target of load_state_dict (init_only modules)."""
        N, K = self.shape
        gp = calculate_zeros_width(K, self.group_size) * 8
        self.qweight = torch.empty((N // 4, K), dtype=torch.int16, device=device)
        for key in ("scales", "scaled_zeros", "scales_to8", "scaled_zeros_to8"):
            setattr(self, key, torch.empty((gp, N), dtype=torch.float16, device=device))
        self.scales_1 = torch.empty((N,), dtype=torch.float16, device=device)

    def init(self):
        """After the resident tensors changed in place or moved (load_state_dict, .to()): forget everything derived
        from the old ones -- cached pointers, the lane memo and this layer's entries in the temp cache
        (kairos/dynamic_linear.py:81-83 is the reference's hook of the same name)."""
        self._decode_ptrs = None
        self.pre_m = 0
        self.comp_type = None
        self._uid = next(_uids)

    def _apply(self, fn, *args, **kwargs):
        out = super()._apply(fn, *args, **kwargs)
        self.init()
        return out

    def _load_from_state_dict(self, state_dict, prefix, *args, **kwargs):
        if self.qweight is None and prefix + "qweight" in state_dict:      # plain constructor: allocate on the fly
            dev = state_dict[prefix + "qweight"].device if self.bias is None else self.bias.device
            self._allocate_resident(dev)
        super()._load_from_state_dict(state_dict, prefix, *args, **kwargs)
        self.init()

    @classmethod
    @torch.no_grad()
    def from_module(cls, linear, device, return_dtype=torch.float16, init_only=False, name=''):
        q_linear = cls(linear.in_features, linear.out_features, linear.bias is not None, device, group_size=128)
        if init_only:
            q_linear._allocate_resident(device)
            return q_linear
        # On a GPU the whole chain (int8 per channel -> uint4 per group -> packed words and tables) is one kernel
        # of the library.  The same torch ops on a ROCm device would not do: PyTorch's elementwise fp32 division
        # there is not correctly rounded, which flips round-half-even ties against the reference arithmetic.
        # A CPU target keeps the host chain (weight_prep), which yields the same bits.
        if torch.device(device).type == 'cuda':
            w = linear.weight.data.detach().to(device=device, dtype=torch.float16).contiguous()
            prepared = ops.prepare_weight(w, group_size=128)
        else:
            prepared = prepare_linear_weight(linear.weight.data.detach().cpu(), group_size=128)
        for key, value in prepared.items():
            setattr(q_linear, key, value.to(device))
        if linear.bias is not None:
            q_linear.bias = linear.bias.detach().clone().half().to(device)
        return q_linear

    # ------------------------------------------------------------------------------------------
    def _cache(self):
        return self.temp_cache if self.temp_cache is not None else default_cache()

    def _tileable(self):
        return self.tiled_weights and self.out_features % 128 == 0

    def _converted(self, fmt, tiled=None):
        """int8 or fp16 copy of the weight in the temp cache; converts only if it is not there."""
        tiled = self._tileable() if tiled is None else tiled
        dtype = torch.int8 if fmt == 'i8' else torch.float16
        buf, hit = self._cache().get(self._uid, (fmt, tiled), self.shape, dtype, self.qweight.device)
        if not hit:
            if fmt == 'i8':
                ops.dequant_interleaved_int4_to_int8(buf, self.qweight, self.scales_to8, self.scaled_zeros_to8,
                                                     self.group_size, tiled=tiled)
            else:
                ops.dequant_interleaved_int4_to_fp16(buf, self.qweight, self.scales, self.scaled_zeros,
                                                     self.group_size, tiled=tiled)
        return buf, tiled

    def _select(self, m):
        if m != self.pre_m:
            self.pre_m = m
            comp = type(self).prof.get_comp_type(self.shape, m)
            if self.comp_type is not None and comp != self.comp_type:
                self.switch_count += 1
            self.comp_type = comp
        return self.comp_type

    def forward(self, input) -> torch.Tensor:
        # Decode-sized calls are host-bound (the kernels take 5-13 us, a Python call with a launch about as long), so
        # the small-M lane is served right here: one allocation, one C call, cached pointers, no context managers.
        # Nothing on it records autograd history (the output is a fresh tensor filled by the library).
        if type(input) is torch.Tensor:
            shape = input.shape
            m = input.numel() // shape[-1]
            if m != self.pre_m:
                self._select(m)
            if (self.comp_type == _W4A16_GEMV and m <= _GEMV_MAX_M and ops._tracer is None
                    and input.dtype is torch.float16 and input.is_cuda and input.is_contiguous()):
                ptrs = self._decode_ptrs
                if ptrs is None or ptrs[0] != self._buffers['qweight'].data_ptr():
                    ptrs = self._decode_ptrs = self._decode_pointers()
                if shape[-1] != ptrs[7] or input.device.index != ptrs[5]:
                    raise ValueError(f"DynamicLinear: input of shape {tuple(shape)} on {input.device} for a layer with "
                                     f"{ptrs[7]} input features on cuda:{ptrs[5]}")
                out = torch.empty(shape[:-1] + (ptrs[6],), dtype=torch.float16, device=input.device)
                st = _raw_stream(ptrs[5]) if _raw_stream is not None else ops._stream()
                ws = getattr(_override, "scratch", None)
                ws = _gemv_workspaces.get((ptrs[5], st)) if ws is None else ws.gemv
                if ws is None:
                    ws = ops.gemv_workspace_for(input.device, st)
                rc = ptrs[4](out.data_ptr(), input.data_ptr(), ptrs[0], ptrs[1], ptrs[2], ptrs[3], m, ptrs[6], ptrs[7], ptrs[8],
                             ws.data_ptr(), ws.numel(), st)
                if rc < 0:
                    if rc == -6:               # the runtime rejected the launch: leave the counters in a known state
                        ops._lib.load().kmi_gemv_ws_reset(ws.data_ptr(), ws.numel(), st)
                    ops._lib.check(rc)
                return out
        return self._forward_any(input)

    def _decode_pointers(self):
        N, K = self.shape
        dev = self.qweight.device
        return (self.qweight.data_ptr(), self.scales.data_ptr(), self.scaled_zeros.data_ptr(),
                0 if self.bias is None else self.bias.data_ptr(), ops._lib.load().kmi_gemv_w4a16,
                dev.index if dev.index is not None else torch.cuda.current_device(), N, K, self.group_size)

    @torch.no_grad()
    def _forward_any(self, input) -> torch.Tensor:
        shape = input.shape
        K = shape[-1]
        m = input.numel() // K
        self._select(m)
        if not isinstance(input, torch.Tensor):              # a MatchedActivation from the operator in front
            if self.comp_type == _W8A8 and input.int_x is not None:
                return self._w8a8(None, input.int_x.reshape(-1, K), input.scale_x).reshape(*shape[:-1], -1)
            if self.comp_type == _W4A8 and input.int_x is not None:
                return self._w4a8(None, input.int_x.reshape(-1, K), input.scale_x).reshape(*shape[:-1], -1)
            if input.f16 is None:
                raise ValueError("the matched activation holds no fp16 form, but this layer's lane for "
                                 f"{m} tokens (id {self.comp_type}) needs one")
            input = input.f16
        return self._forward(input.reshape(-1, K), m, self.comp_type).reshape(*shape[:-1], -1)

    def _w8a8(self, x, int_x, scale_x):
        """The W8A8 lane on fp16 activations x [m, K], or on activations that arrive quantised (x None)."""
        N, K = self.shape
        quantise = int_x is None
        if quantise:
            int_x = torch.empty_like(x, dtype=torch.int8)
            scale_x = torch.empty((x.shape[0],), device=x.device, dtype=torch.float16)
        m = int_x.shape[0]
        if self.resident_copies:
            (w8, tiled), hit = self._converted('i8'), True
        else:
            tiled = self._tileable()
            w8, hit = self._cache().get(self._uid, ('i8', tiled), self.shape, torch.int8, self.qweight.device)
        if not quantise:
            if not hit:
                ops.dequant_interleaved_int4_to_int8(w8, self.qweight, self.scales_to8, self.scaled_zeros_to8,
                                                     self.group_size, tiled=tiled)
        elif hit:
            ops.quant_fp16_to_int8(int_x, x, scale_x)
        else:                                                # conversion and quantisation share one launch
            ops.prep_w8a8(w8, self.qweight, self.scales_to8, self.scaled_zeros_to8, int_x, x, scale_x,
                          self.group_size, tiled=tiled)
        out = torch.empty((m, N), device=int_x.device, dtype=torch.float16)
        ops.w8a8_gemm_forward(int_x, w8, self.scales_1, scale_x, out, bias=self.bias, tiled=tiled)
        return out

    def _w4a8(self, x, int_x, scale_x):
        """The W4A8 lane on fp16 activations x [m, K], or on activations that arrive quantised (x None): the
        activation quantiser, then the int8 GEMM that decodes the resident int4 weight on the fly."""
        N, K = self.shape
        if int_x is None:
            int_x = torch.empty_like(x, dtype=torch.int8)
            scale_x = torch.empty((x.shape[0],), device=x.device, dtype=torch.float16)
            ops.quant_fp16_to_int8(int_x, x, scale_x)
        out = torch.empty((int_x.shape[0], N), device=int_x.device, dtype=torch.float16)
        ops.w4a8_gemm_forward(int_x, self.qweight, self.scales_to8, self.scaled_zeros_to8, self.scales_1, scale_x, out,
                              bias=self.bias)
        return out

    @torch.no_grad()
    def _forward(self, input: torch.Tensor, batch_token_len, comp_type) -> torch.Tensor:
        N, K = self.shape
        lead = input.shape[:-1]
        x = input.reshape(-1, K)
        if not x.is_contiguous():
            x = x.contiguous()
        m = x.shape[0]
        if comp_type == _W4A16_GEMV and m <= ops.GEMV_MAX_M:
            out = ops.gemv_forward(x, self.qweight, self.scales, self.scaled_zeros, m, N, K,
                                   self.group_size, bias=self.bias)
        elif comp_type in (_W4A16_GEMM, _W4A16_GEMV, _W4A16_ALT):
            out = ops.gemm_forward(x, self.qweight, self.scales, self.scaled_zeros, bias=self.bias)
        elif comp_type == _W8A8:
            out = self._w8a8(x, None, None)
        elif comp_type == _W4A8:
            out = self._w4a8(x, None, None)
        elif comp_type in (_W8A16_GEMM, _W8A16_GEMV):
            w8, _ = self._converted('i8', tiled=False)       # this lane widens int8 in registers: row-major source
            out = ops.w8a16_gemm_forward(x, w8, self.scales_1, N, bias=self.bias)
        elif comp_type == _FP16:
            w16, tiled = self._converted('f16')
            out = ops.f16_gemm_forward(x, w16, N, bias=self.bias, tiled=tiled)
        else:
            raise ValueError(f"unknown comp_type id {comp_type}")
        return out.reshape(*lead, N)

    def extra_repr(self) -> str:
        return f"in_features={self.in_features}, out_features={self.out_features}, bias={self.bias is not None}"
