"""ctypes binding of ``libll_nvfp4.so`` (the C ABI declared in ``include/ll_nvfp4.h``).

The library is the only implementation of the hot path: if it is missing, every
call raises.  Nothing here falls back to PyTorch arithmetic.  PyTorch is used
for device memory and the current HIP stream only.
"""
from __future__ import annotations

import ctypes
import os
import re
from ctypes import c_char_p, c_float, c_int, c_int64, c_size_t, c_void_p

import torch

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "csrc", "libll_nvfp4.so")
HEADER_PATH = os.path.join(os.path.dirname(_HERE), "include", "ll_nvfp4.h")

RULE_IDS = {"static_6": 0, "static_4": 1, "mae": 2, "mse": 3, "abs_max": 4}
# looks (1-2 us each) a workgroup of a launch whose workgroups exchange their maxima waits for the others
NORM_QUANTIZE_SPIN_LIMIT = 64
DTYPE_CODES = {torch.bfloat16: 0, torch.float16: 1, torch.float32: 2}
ACTIVATION_IDS = {"gelu_tanh": 1}

_lib = None

_SIGNATURES = {
    "ll_last_error": (c_char_p, []),
    "ll_version": (c_int, []),
    "ll_nvfp4_quantize_workspace_floats": (c_size_t, []),
    "ll_nvfp4_quantize": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_int, c_void_p, c_void_p, c_void_p, c_int,
                                  c_void_p, c_void_p]),
    "ll_nvfp4_quantize_from_sink": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_int, c_void_p, c_void_p, c_void_p,
                                            c_void_p, c_void_p]),
    "ll_nvfp4_quantize_pair_from_sinks": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_int64, c_int, c_void_p, c_void_p,
                                                  c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]),
    "ll_nvfp4_dequantize": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int64, c_int64, c_int64, c_int64,
                                    c_void_p, c_int, c_int64, c_void_p]),
    "ll_nvfp4_gemm_tnt": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_float,
                                  c_float, c_int64, c_int64, c_int64, c_int64, c_int64, c_void_p, c_int64, c_void_p,
                                  c_void_p]),
    "ll_nvfp4_gemm_tnt_act": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_float,
                                      c_float, c_int64, c_int64, c_int64, c_int64, c_int64, c_void_p, c_int64,
                                      c_void_p, c_int, c_void_p]),
    "ll_nvfp4_gemm_tnt_fused": (c_int, [c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_float,
                                        c_float, c_int64, c_int64, c_int64, c_int64, c_int64, c_void_p, c_int64,
                                        c_void_p, c_void_p]),
    "ll_nvfp4_gemm_tnt_grouped": (c_int, [c_void_p, c_void_p, c_void_p, c_float, c_int64, c_int64, c_int64, c_int64,
                                          c_int64, c_int, c_void_p, c_void_p]),
    "ll_kv_dequantize_blocks": (c_int, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_float, c_float,
                                        c_void_p, c_void_p]),
    "ll_kv_attention": (c_int, [c_void_p, c_int64, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                c_int64, c_int, c_float, c_float, c_void_p, c_void_p, c_int64, c_float, c_void_p,
                                c_void_p]),
    "ll_kv_attention_amax": (c_int, [c_void_p, c_int64, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                     c_void_p, c_int64, c_int, c_float, c_float, c_void_p, c_void_p, c_int64, c_float,
                                     c_void_p, c_void_p, c_void_p]),
    "ll_attention_bf16": (c_int, [c_void_p, c_void_p, c_void_p, c_int64, c_int64, c_int, c_float, c_void_p, c_void_p]),
    "ll_amax_epoch_advance": (c_int, [c_void_p, ctypes.c_uint32, c_void_p, c_void_p]),
    "ll_kv_attention_set_policy": (c_int, [c_int]),
    "ll_kv_attention_get_policy": (c_int, []),
    "ll_kv_attention_plan": (c_int, [c_int64, c_int, c_int64, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p]),
    "ll_rope_apply": (c_int, [c_void_p, c_int64, c_int, c_int, c_int64, c_int64, c_void_p, c_void_p, c_int64,
                              c_void_p, c_void_p]),
    "ll_adaln_modulate": (c_int, [c_void_p, c_int64, c_int64, c_int, c_void_p, c_void_p, c_int64, c_int64, c_int64,
                                  c_int64, c_int64, c_float, c_int, c_void_p, c_void_p]),
    "ll_adaln_modulate_amax": (c_int, [c_void_p, c_int64, c_int64, c_int, c_void_p, c_void_p, c_int64, c_int64,
                                       c_int64, c_int64, c_int64, c_float, c_int, c_void_p, c_void_p, c_void_p]),
    "ll_qk_norm_rope": (c_int, [c_void_p, c_int64, c_int, c_void_p, c_float, c_void_p, c_void_p, c_int64, c_void_p,
                                c_void_p, c_void_p]),
    "ll_qk_norm_rope_pair": (c_int, [c_void_p, c_void_p, c_int64, c_int, c_void_p, c_void_p, c_float, c_void_p,
                                     c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p]),
    "ll_qk_norm_rope_pair_amax": (c_int, [c_void_p, c_void_p, c_int64, c_int, c_void_p, c_void_p, c_float, c_void_p,
                                     c_void_p, c_int64, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p]),
    "ll_gate_residual": (c_int, [c_void_p, c_void_p, c_int64, c_int64, c_int, c_void_p, c_int64, c_int64, c_int64,
                                 c_void_p, c_void_p]),
    "ll_rms_norm": (c_int, [c_void_p, c_int64, c_int, c_void_p, c_float, c_void_p, c_void_p]),
    "ll_adaln_quantize": (c_int, [c_void_p, c_int64, c_int64, c_int, c_void_p, c_void_p, c_int64, c_int64, c_int64,
                                  c_int64, c_int64, c_float, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p,
                                  c_int64, c_void_p]),
    "ll_layer_norm_quantize": (c_int, [c_void_p, c_int64, c_int, c_void_p, c_void_p, c_float, c_int, c_void_p,
                                       c_void_p, c_void_p, c_void_p, c_int64, c_void_p]),
    "ll_layer_norm": (c_int, [c_void_p, c_int64, c_int, c_void_p, c_void_p, c_float, c_void_p, c_void_p, c_void_p]),
    "ll_release_stream_memory": (c_int, [c_void_p]),
    "ll_nvfp4_gemm_set_schedule": (c_int, [c_int]),
    "ll_nvfp4_gemm_get_schedule": (c_int, []),
    "ll_nvfp4_gemm_reserve": (c_int, [c_int64, c_int64, c_int64, c_int, c_void_p]),
    "ll_nvfp4_gemm_plan": (c_int, [c_int64, c_int64, c_int64, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_void_p]),
    "ll_nvfp4_gemm_kernel": (c_int, [c_int64, c_int64, c_int64, c_int, c_int, c_int, c_void_p, c_void_p]),
    "ll_kv_attention_reserve": (c_int, [c_int64, c_int, c_int64, c_void_p]),
    "ll_kv_attention_release": (c_int, [c_void_p]),
    "ll_nvfp4_quantize_noalloc_max_elements": (c_int64, []),
    "ll_nvfp4_quantize_noalloc": (c_int, [c_void_p, c_int64, c_int64, c_int64, c_int, c_void_p, c_void_p, c_void_p,
                                          c_void_p]),
}


def declared_symbols() -> list[str]:
    """Entry points declared in include/ll_nvfp4.h."""
    with open(HEADER_PATH) as f:
        text = f.read()
    return sorted(set(re.findall(r"\b(ll_[a-z0-9_]+)\s*\(", text)))


def load():
    """Load the shared library (once).  Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(LIB_PATH):
        raise RuntimeError(
            f"{LIB_PATH} is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
            "(or `make -C longlive_amd/csrc`). There is no fallback implementation."
        )
    lib = ctypes.CDLL(LIB_PATH)
    for name, (res, args) in _SIGNATURES.items():
        fn = getattr(lib, name)
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def _check(code: int, what: str) -> None:
    if code != 0:
        msg = load().ll_last_error().decode()
        if code == -1:
            raise ValueError(msg or what)
        raise RuntimeError(msg or what)


def _stream() -> int:
    return torch.cuda.current_stream().cuda_stream


def _ptr(t: torch.Tensor | None) -> int | None:
    return None if t is None else t.data_ptr()


def _require_cuda(*tensors: torch.Tensor) -> None:
    for t in tensors:
        if t is not None and t.device.type != "cuda":
            raise ValueError("the NVFP4 kernels run on the GPU only; got a tensor on " + str(t.device))


_workspaces: dict[tuple[int, int], torch.Tensor] = {}


def _workspace(device: torch.device) -> torch.Tensor:
    key = (device.index if device.index is not None else torch.cuda.current_device(), _stream())
    ws = _workspaces.get(key)
    if ws is None:
        ws = torch.empty(load().ll_nvfp4_quantize_workspace_floats(), dtype=torch.float32, device=device)
        _workspaces[key] = ws
    return ws


def padded_shape(shape: tuple[int, int]) -> tuple[int, int]:
    return (-(-shape[0] // 128) * 128, -(-shape[1] // 64) * 64)


# --------------------------------------------------------------------------- amax sink
AMAX_PARTS = 1024


class AmaxSinkStruct(ctypes.Structure):
    """struct ll_amax_sink of include/ll_nvfp4.h."""
    _fields_ = [("parts", c_void_p), ("epoch", ctypes.c_uint32), ("epoch_offset", c_void_p)]


class AmaxTicket:
    """One use of a device's amax sink: handed to the kernel that writes a tensor (``amax_out=``) and then to
    the quantization of that tensor (``amax=``), which reads the maximum the producer left."""

    __slots__ = ("parts", "epoch", "entry", "offset")

    def __init__(self, parts: torch.Tensor, epoch: int, entry=None, offset: torch.Tensor | None = None) -> None:
        # entry: the bookkeeping of the sink the ticket belongs to, [buffer, last epoch issued, (epoch, stream) of
        # the last producer launch]; it lives as long as the sink or any of its tickets
        self.parts, self.epoch, self.entry, self.offset = parts, epoch, entry, offset

    def struct(self) -> AmaxSinkStruct:
        return AmaxSinkStruct(self.parts.data_ptr(), self.epoch, None if self.offset is None else self.offset.data_ptr())


# the devices' shared sinks, (device type, index) -> [sink buffer, last epoch issued, (epoch, stream) of the last
# producer launch]; private and graph sinks keep their entry themselves and go away with their owner
_sinks: dict = {}
# device key -> the ReplayableAmaxSink whose tickets amax_ticket hands out at the moment
_active_graph_sinks: dict = {}


def _device_key(device: torch.device):
    index = device.index if device.index is not None else (torch.cuda.current_device() if device.type == "cuda" else 0)
    return (device.type, index)


class PrivateAmaxSink:
    """An amax sink buffer of its own for one producer / consumer pair whose two ends lie far apart in the launch
    sequence (the K and V of a chunk are produced early in a forward and quantized into the cache after it): the
    tickets of the device's shared sink are good only until the next producer launch."""

    def __init__(self, device) -> None:
        self.parts = torch.zeros(AMAX_PARTS, dtype=torch.int64, device=torch.device(device))
        self.entry = [self.parts, 0, None]

    def ticket(self) -> "AmaxTicket | None":
        """The next ticket, or None while launches are being recorded into a graph: a recording has one sink for
        all its producers, whose slots the next producer overwrites, and no place for a maximum that is consumed
        after the forward.  Without a ticket the producer leaves nothing behind and the consumer reduces the tensor
        itself."""
        if _device_key(self.parts.device) in _active_graph_sinks:
            return None
        if self.entry[1] >= 0xFFFFFFFE:
            self.parts.zero_()
            self.entry[1] = 0
        self.entry[1] += 1
        return AmaxTicket(self.parts, self.entry[1], self.entry)


class ReplayableAmaxSink:
    """An amax sink for launches that are recorded into a HIP graph and replayed.  A recorded launch runs again
    with the epoch it was recorded with, so every kernel adds a device word to its epoch, and the first recorded
    launch (``__enter__``) raises that word by more than the number of tickets one replay uses: every replay
    works with fresh epochs on a buffer of its own.  Use: create it ahead of the capture (it allocates), then

        with torch.cuda.graph(g, stream=s), sink:
            y = block(...)

    Inside the ``with`` every ``amax_ticket`` of the device comes from this sink."""

    STEP = 1 << 16  # epochs per replay; a replay may use at most STEP - 1 tickets

    def __init__(self, device) -> None:
        self.device = torch.device(device)
        self.parts = torch.zeros(AMAX_PARTS, dtype=torch.int64, device=self.device)
        self.offset = torch.zeros(1, dtype=torch.int32, device=self.device)
        self.entry = [self.parts, 0, None]

    def __enter__(self):
        dkey = _device_key(self.device)
        if dkey in _active_graph_sinks:
            raise RuntimeError("another replayable amax sink is active on this device")
        self.entry[1], self.entry[2] = 0, None
        _active_graph_sinks[dkey] = self
        with torch.cuda.device(self.device):
            _check(load().ll_amax_epoch_advance(self.offset.data_ptr(), self.STEP, self.parts.data_ptr(), _stream()),
                   "ll_amax_epoch_advance")
        return self

    def __exit__(self, *exc):
        del _active_graph_sinks[_device_key(self.device)]
        if self.entry[1] >= self.STEP:
            raise RuntimeError(f"{self.entry[1]} amax tickets in one recording; at most {self.STEP - 1} are supported")
        return False

    def ticket(self) -> "AmaxTicket":
        self.entry[1] += 1
        return AmaxTicket(self.parts, self.entry[1], self.entry, self.offset)


def amax_ticket(device: torch.device) -> AmaxTicket:
    """A fresh epoch on the device's amax sink buffer.  Epochs only grow, which is what lets the buffer go
    uncleared between uses.  All tickets of a device share the one buffer, so a ticket is good for exactly one
    producer launch followed by the quantization(s) of its output, on one stream, with no other producer launch
    in between: a later producer overwrites the slots.  The host side checks this (see ``_check_consumer``)."""
    device = torch.device(device)
    key = _device_key(device)
    if key in _active_graph_sinks:
        return _active_graph_sinks[key].ticket()
    entry = _sinks.get(key)
    if entry is None or entry[1] >= 0xFFFFFFFE:
        entry = [torch.zeros(AMAX_PARTS, dtype=torch.int64, device=device), 0, None]
        _sinks[key] = entry
    entry[1] += 1
    return AmaxTicket(entry[0], entry[1], entry)


def _stream_of(ticket: AmaxTicket) -> int:
    return _stream() if ticket.parts.is_cuda else 0


def _sink_struct(ticket):
    """The struct a producer kernel is given; notes the launch as the sink's latest producer."""
    if ticket is None:
        return AmaxSinkStruct(None, 0)
    if not isinstance(ticket, AmaxTicket):
        raise TypeError("amax_out must be an AmaxTicket (see amax_ticket)")
    entry = ticket.entry
    if entry is not None and entry[0] is ticket.parts:
        entry[2] = (ticket.epoch, _stream_of(ticket))
    return ticket.struct()


def _check_consumer(ticket: AmaxTicket) -> None:
    """A quantization may read a ticket's amax only while that ticket's producer is the latest producer launch
    on the device's sink, and on the stream the producer ran on.  Anything else (another producer launched in
    between, the producer never launched, a different stream) would make the kernel read partial maxima of
    another tensor or none at all and quantize against a wrong amax without any error, so it is refused here."""
    entry = ticket.entry
    if entry is None or entry[0] is not ticket.parts:
        raise RuntimeError("this amax ticket belongs to a sink buffer that has been replaced")
    last = entry[2]
    if last is None or last[0] != ticket.epoch:
        raise RuntimeError(
            f"amax ticket {ticket.epoch} is not the latest producer on its sink (latest: "
            f"{'none' if last is None else last[0]}): between the kernel that was given this ticket as amax_out and "
            "the quantization of its output no other kernel may be given a ticket of the same device")
    if last[1] != _stream_of(ticket):
        raise RuntimeError("the producer of this amax ticket ran on another stream than the quantization that "
                           "reads it; both must be issued on one stream")


# --------------------------------------------------------------------------- quantize / dequantize
def quantize(x: torch.Tensor, rule: str, amax: torch.Tensor | None = None, out=None):
    """x bf16 [M, K] -> (values u8 [Mp, Kp/2], scales float8_e4m3fn [Mp*Kp/16] blocked, amax f32[1]).
    ``out`` = (values, scale_factors, amax) buffers of exactly those shapes to write into (KV slots).
    ``amax``: a float32[1] tensor to quantize against, or the :class:`AmaxTicket` the producer of ``x`` was
    given, in which case the bytes equal those of ``amax=None``."""
    ticket = amax if isinstance(amax, AmaxTicket) else None
    if ticket is not None:
        _check_consumer(ticket)
        amax = None
    _require_cuda(x, amax)
    if x.ndim != 2:
        raise ValueError("quantize expects a 2-D tensor")
    if x.dtype != torch.bfloat16:
        raise ValueError(f"the NVFP4 quantizer takes bfloat16 input, got {x.dtype}")
    if x.stride(1) != 1:
        x = x.contiguous()
    M, K = x.shape
    Mp, Kp = padded_shape((M, K))
    given = amax is not None
    if out is not None:
        values, scales, amax_t = out
        if (values.shape != (Mp, Kp // 2) or values.dtype != torch.uint8 or scales.numel() != Mp * Kp // 16
                or scales.element_size() != 1 or amax_t.numel() != 1 or amax_t.dtype != torch.float32
                or not (values.is_contiguous() and scales.is_contiguous())):
            raise ValueError("out buffers do not match the padded NVFP4 shape of x")
        if given:
            amax_t.copy_(amax.reshape(amax_t.shape))
    else:
        values = torch.empty((Mp, Kp // 2), dtype=torch.uint8, device=x.device)
        scales = torch.empty(Mp * Kp // 16, dtype=torch.uint8, device=x.device)
        amax_t = amax.reshape(1).to(torch.float32).contiguous() if given else torch.empty(
            1, dtype=torch.float32, device=x.device)
    ws = None if given or ticket is not None else _workspace(x.device)
    with torch.cuda.device(x.device):
        if ticket is not None:
            sink = ticket.struct()
            code = load().ll_nvfp4_quantize_from_sink(x.data_ptr(), M, K, x.stride(0), RULE_IDS[rule],
                                                      values.data_ptr(), scales.data_ptr(), amax_t.data_ptr(),
                                                      ctypes.byref(sink), _stream())
        else:
            code = load().ll_nvfp4_quantize(x.data_ptr(), M, K, x.stride(0), RULE_IDS[rule], values.data_ptr(),
                                            scales.data_ptr(), amax_t.data_ptr(), int(given), _ptr(ws), _stream())
    _check(code, "ll_nvfp4_quantize")
    if out is not None:
        return out
    return values, scales.view(torch.float8_e4m3fn), amax_t


def quantize_pair(x0: torch.Tensor, x1: torch.Tensor, rule: str, ticket0: AmaxTicket, ticket1: AmaxTicket, out0, out1):
    """``quantize(x0, rule, amax=ticket0, out=out0)`` and ``quantize(x1, rule, amax=ticket1, out=out1)`` as one
    launch (the K and the V of a chunk on their way into the cache): two bf16 [M, K] tensors of the same shape and
    row stride, each with the amax ticket of its producer (tickets of two different sink buffers) and its
    (values, scale_factors, amax) buffers.  The bytes equal those of the two calls."""
    for t in (ticket0, ticket1):
        if not isinstance(t, AmaxTicket):
            raise TypeError("quantize_pair needs the amax tickets of the two producers")
        _check_consumer(t)
    if ticket0.parts.data_ptr() == ticket1.parts.data_ptr():
        raise ValueError("the two tickets must belong to two sink buffers")
    _require_cuda(x0, x1)
    if x0.ndim != 2 or x0.shape != x1.shape or x0.dtype != torch.bfloat16 or x1.dtype != torch.bfloat16:
        raise ValueError("quantize_pair expects two 2-D bfloat16 tensors of the same shape")
    if x0.stride(1) != 1:
        x0 = x0.contiguous()
    if x1.stride(1) != 1 or x1.stride(0) != x0.stride(0):
        x1 = x1.contiguous()
        if x1.stride(0) != x0.stride(0):
            x0 = x0.contiguous()
    M, K = x0.shape
    Mp, Kp = padded_shape((M, K))
    for values, scales, amax_t in (out0, out1):
        if (values.shape != (Mp, Kp // 2) or values.dtype != torch.uint8 or scales.numel() != Mp * Kp // 16
                or scales.element_size() != 1 or amax_t.numel() != 1 or amax_t.dtype != torch.float32
                or not (values.is_contiguous() and scales.is_contiguous())):
            raise ValueError("out buffers do not match the padded NVFP4 shape of the inputs")
    s0, s1 = ticket0.struct(), ticket1.struct()
    with torch.cuda.device(x0.device):
        code = load().ll_nvfp4_quantize_pair_from_sinks(
            x0.data_ptr(), x1.data_ptr(), M, K, x0.stride(0), RULE_IDS[rule], out0[0].data_ptr(), out1[0].data_ptr(),
            out0[1].data_ptr(), out1[1].data_ptr(), out0[2].data_ptr(), out1[2].data_ptr(), ctypes.byref(s0),
            ctypes.byref(s1), _stream())
    _check(code, "ll_nvfp4_quantize_pair_from_sinks")
    return out0, out1


def dequantize(values, scales, amax, rule: str, padded, original, dtype: torch.dtype) -> torch.Tensor:
    _require_cuda(values, scales, amax)
    out = torch.empty(original, dtype=dtype, device=values.device)
    with torch.cuda.device(values.device):
        code = load().ll_nvfp4_dequantize(values.data_ptr(), scales.data_ptr(), amax.data_ptr(), RULE_IDS[rule],
                                          padded[0], padded[1], original[0], original[1], out.data_ptr(),
                                          DTYPE_CODES[dtype], out.stride(0), _stream())
    _check(code, "ll_nvfp4_dequantize")
    return out


# --------------------------------------------------------------------------- GEMM
class GemmEpilogue(ctypes.Structure):
    """struct ll_gemm_epilogue of include/ll_nvfp4.h."""
    _fields_ = [("bias", c_void_p), ("activation", c_int), ("gate", c_void_p), ("gate_rows", c_int64),
                ("gate_stride", c_int64), ("residual", c_void_p), ("ldr", c_int64), ("amax_sink", AmaxSinkStruct)]


def gemm(a_values, a_scales, b_values, b_scales, M: int, N: int, *, alpha=None, amax_a=None, amax_b=None,
         denom_a: float = 1536.0, denom_b: float = 1536.0, bias=None, out=None, activation=None,
         residual=None, gate=None, gate_rows: int = 0, amax_out=None) -> torch.Tensor:
    """D = A @ B^T with the epilogue of ll_nvfp4_gemm_tnt_fused: bias, activation, then
    ``residual + y * gate[m // gate_rows]`` (gate [G, N], rows may be strided) or ``residual + y``, and the
    absolute maximum of the result left in ``amax_out`` (an :class:`AmaxTicket`)."""
    if activation is not None and activation not in ACTIVATION_IDS:
        raise ValueError(f"unknown epilogue activation {activation!r}")
    _require_cuda(a_values, a_scales, b_values, b_scales, alpha, amax_a, amax_b, bias, residual, gate)
    Mp, Kb = a_values.shape
    Np, Kb2 = b_values.shape
    if Kb != Kb2:
        raise ValueError(f"inner dimensions differ: {Kb * 2} vs {Kb2 * 2}")
    if out is None:
        out = torch.empty((M, N), dtype=torch.bfloat16, device=a_values.device)
    if bias is not None and (bias.dtype != torch.bfloat16 or bias.numel() != N or not bias.is_contiguous()):
        raise ValueError("bias must be a contiguous bfloat16 vector of length N")
    epi = GemmEpilogue(_ptr(bias), ACTIVATION_IDS[activation] if activation else 0, None, 0, 0, None, 0,
                       _sink_struct(amax_out))
    if residual is not None:
        if residual.dtype != torch.bfloat16 or residual.shape != (M, N) or residual.stride(1) != 1:
            raise ValueError("residual must be bfloat16 [M, N] with contiguous rows")
        epi.residual, epi.ldr = residual.data_ptr(), residual.stride(0)
        if gate is not None:
            if gate.dtype != torch.bfloat16 or gate.dim() != 2 or gate.shape[1] != N or gate.stride(1) != 1 \
                    or gate_rows <= 0 or gate.shape[0] * gate_rows < M:
                raise ValueError("gate must be bfloat16 [G, N] with contiguous rows and G * gate_rows >= M")
            epi.gate, epi.gate_rows, epi.gate_stride = gate.data_ptr(), gate_rows, gate.stride(0)
    elif gate is not None:
        raise ValueError("a gate needs a residual")
    with torch.cuda.device(a_values.device):
        code = load().ll_nvfp4_gemm_tnt_fused(
            a_values.data_ptr(), a_scales.data_ptr(), b_values.data_ptr(), b_scales.data_ptr(), _ptr(alpha),
            _ptr(amax_a), _ptr(amax_b), denom_a, denom_b, M, N, Mp, Np, Kb * 2, out.data_ptr(), out.stride(0),
            ctypes.byref(epi), _stream())
    _check(code, "ll_nvfp4_gemm_tnt")
    return out


class GemmProduct(ctypes.Structure):
    """struct ll_gemm_product of include/ll_nvfp4.h."""
    _fields_ = [("B_values", c_void_p), ("B_scales", c_void_p), ("alpha", c_void_p), ("amax_b", c_void_p),
                ("denom_b", ctypes.c_float), ("D", c_void_p), ("ldd", c_int64), ("bias", c_void_p),
                ("amax_sink", AmaxSinkStruct)]


def gemm_grouped(a_values, a_scales, amax_a, denom_a: float, M: int, N: int, products) -> list[torch.Tensor]:
    """Several products ``A @ B_i^T`` with the same A operand and the same N and K in one launch
    (ll_nvfp4_gemm_tnt_grouped).  ``products``: one dict per product with ``values``, ``scales``, ``amax``,
    ``denom`` and optionally ``bias`` and ``amax_out`` (an :class:`AmaxTicket`).  Each output equals what
    :func:`gemm` returns for that product alone, bit for bit."""
    Mp, Kb = a_values.shape
    sinks = [pr["amax_out"].parts.data_ptr() for pr in products if pr.get("amax_out") is not None]
    if len(set(sinks)) != len(sinks):
        raise ValueError("the products of one launch need amax sinks with buffers of their own (a later epoch hides an "
                         "earlier one on a shared buffer)")
    outs, structs = [], (GemmProduct * len(products))()
    for i, pr in enumerate(products):
        bias = pr.get("bias")
        _require_cuda(pr["values"], pr["scales"], pr["amax"], bias)
        if pr["values"].shape[1] != Kb or pr["values"].shape[0] != products[0]["values"].shape[0]:
            raise ValueError("the products of one launch must have the same N and K")
        if bias is not None and (bias.dtype != torch.bfloat16 or bias.numel() != N or not bias.is_contiguous()):
            raise ValueError("bias must be a contiguous bfloat16 vector of length N")
        out = torch.empty((M, N), dtype=torch.bfloat16, device=a_values.device)
        outs.append(out)
        structs[i] = GemmProduct(pr["values"].data_ptr(), pr["scales"].data_ptr(), None, pr["amax"].data_ptr(),
                                 float(pr["denom"]), out.data_ptr(), out.stride(0), _ptr(bias),
                                 _sink_struct(pr.get("amax_out")))
    with torch.cuda.device(a_values.device):
        code = load().ll_nvfp4_gemm_tnt_grouped(a_values.data_ptr(), a_scales.data_ptr(), amax_a.data_ptr(), float(denom_a),
                                                M, N, Mp, products[0]["values"].shape[0], Kb * 2, len(products),
                                                ctypes.cast(structs, c_void_p), _stream())
    _check(code, "ll_nvfp4_gemm_tnt_grouped")
    return outs


GEMM_SCHEDULES = {"auto": -1, "tiles": 0, "persistent": 1, "tiles_compiled": 2}


def gemm_plan(M: int, N: int, Kp: int, n_products: int = 1, compute_units: int = 256, schedule: str = "auto") -> dict:
    """What a GEMM launch of these sizes would do on a device with ``compute_units`` CUs (host arithmetic only):
    whether it runs as one persistent launch, and then its workgroups, output tiles and K steps per tile."""
    persistent, groups, tiles, steps = c_int(), ctypes.c_uint32(), ctypes.c_uint32(), ctypes.c_uint32()
    _check(load().ll_nvfp4_gemm_plan(M, N, Kp, n_products, compute_units, GEMM_SCHEDULES[schedule], ctypes.byref(persistent),
                                     ctypes.byref(groups), ctypes.byref(tiles), ctypes.byref(steps)), "ll_nvfp4_gemm_plan")
    return {"persistent": bool(persistent.value), "workgroups": groups.value, "tiles": tiles.value, "k_steps": steps.value}


GEMM_KERNELS = ("64x64", "128x128", "128x256", "256x128", "eight_waves", "persistent")


def gemm_kernel(M: int, N: int, Kp: int, n_products: int = 1, compute_units: int = 256, schedule: str = "auto") -> dict:
    """Which kernel a GEMM launch of these sizes runs on a device with ``compute_units`` CUs (host arithmetic only):
    one of GEMM_KERNELS, and whether its main loop is the hand-scheduled one."""
    kernel, generated = c_int(), c_int()
    _check(load().ll_nvfp4_gemm_kernel(M, N, Kp, n_products, compute_units, GEMM_SCHEDULES[schedule], ctypes.byref(kernel),
                                       ctypes.byref(generated)), "ll_nvfp4_gemm_kernel")
    return {"kernel": GEMM_KERNELS[kernel.value], "hand_scheduled": bool(generated.value)}


def gemm_reserve(M: int, N: int, Kp: int, n_products: int = 1, device=None) -> None:
    """Set up, on the current stream, the memory through which a GEMM launch of these sizes would pass partial
    tiles (nothing if it would run one workgroup per tile), so that the launch itself allocates nothing."""
    with torch.cuda.device(device if device is not None else torch.cuda.current_device()):
        _check(load().ll_nvfp4_gemm_reserve(M, N, Kp, n_products, _stream()), "ll_nvfp4_gemm_reserve")


class gemm_schedule:
    """``with gemm_schedule("tiles"): ...`` - which kernel the GEMM entry points run ("auto", "tiles": one workgroup
    per output tile, its large tiles with the hand-scheduled main loop, "tiles_compiled": the same with the compiled
    loop everywhere, "persistent": one workgroup per compute unit wherever the shapes allow; process-wide, restored
    on exit)."""

    def __init__(self, name: str):
        if name not in GEMM_SCHEDULES:
            raise ValueError(f"unknown GEMM schedule {name!r}; one of {sorted(GEMM_SCHEDULES)}")
        self.value = GEMM_SCHEDULES[name]

    def __enter__(self):
        self.previous = load().ll_nvfp4_gemm_get_schedule()
        _check(load().ll_nvfp4_gemm_set_schedule(self.value), "ll_nvfp4_gemm_set_schedule")
        return self

    def __exit__(self, *exc):
        _check(load().ll_nvfp4_gemm_set_schedule(self.previous), "ll_nvfp4_gemm_set_schedule")
        return False


def release_stream_memory(device=None) -> None:
    """Free the memory the library holds for the current stream (partial tiles of the attention and the GEMM)."""
    with torch.cuda.device(device if device is not None else torch.cuda.current_device()):
        _check(load().ll_release_stream_memory(_stream()), "ll_release_stream_memory")


# --------------------------------------------------------------------------- KV cache
def kv_dequantize_blocks(values_ptrs, scales_ptrs, amax_ptrs, n_blocks, num_heads, block_token_size, dtype,
                         e2m1_max, e4m3_max) -> torch.Tensor:
    out = torch.empty((1, n_blocks * block_token_size, num_heads, 128), dtype=dtype, device=values_ptrs.device)
    with torch.cuda.device(values_ptrs.device):
        code = load().ll_kv_dequantize_blocks(values_ptrs.data_ptr(), scales_ptrs.data_ptr(), amax_ptrs.data_ptr(),
                                              n_blocks, num_heads, block_token_size, DTYPE_CODES[dtype],
                                              float(e2m1_max), float(e4m3_max), out.data_ptr(), _stream())
    _check(code, "ll_kv_dequantize_blocks")
    return out


def kv_attention(q, tables, n_cached, block_token_size, e2m1_max, e4m3_max, k_new, v_new, softmax_scale,
                 amax_out=None):
    """q [Lq, H, 128] bf16; tables = six int64 device tensors of slot pointers (or None when n_cached == 0).
    ``amax_out`` (an :class:`AmaxTicket`) receives the absolute maximum of the result."""
    _require_cuda(q, k_new, v_new)
    sink = _sink_struct(amax_out)
    if q.dtype != torch.bfloat16 or q.ndim != 3 or q.shape[-1] != 128 or not q.is_contiguous():
        raise ValueError("q must be a contiguous bfloat16 [Lq, H, 128] tensor")
    Lq, H, _ = q.shape
    n_new = 0
    if k_new is not None:
        if k_new.shape != v_new.shape or k_new.shape[1:] != (H, 128) or k_new.dtype != torch.bfloat16:
            raise ValueError("k_new / v_new must be bfloat16 [n_new, H, 128]")
        k_new = k_new.contiguous()
        v_new = v_new.contiguous()
        n_new = k_new.shape[0]
    out = torch.empty_like(q)
    t = [None] * 6 if tables is None else [x.data_ptr() for x in tables]
    with torch.cuda.device(q.device):
        code = load().ll_kv_attention_amax(q.data_ptr(), Lq, H, *t, n_cached, block_token_size, float(e2m1_max),
                                           float(e4m3_max), _ptr(k_new), _ptr(v_new), n_new, float(softmax_scale),
                                           out.data_ptr(), ctypes.byref(sink), _stream())
    _check(code, "ll_kv_attention")
    return out


def attention_bf16(q, k, v, softmax_scale, amax_out=None):
    return kv_attention(q, None, 0, 0, 6.0, 256.0, k, v, softmax_scale, amax_out=amax_out)


ATTENTION_POLICIES = {"auto": -1, "narrow": 0, "wide": 1, "split": 2}


def attention_plan(Lq: int, num_heads: int, n_keys: int, compute_units: int = 256, policy: str = "auto") -> dict:
    """How an attention launch of these sizes would be divided between workgroups on a device with
    ``compute_units`` CUs (host arithmetic only): division name, workgroups, whole tiles per workgroup and the
    number of tiles cut into shares."""
    division, groups, rounds = c_int(), ctypes.c_uint32(), ctypes.c_uint32()
    split = c_int64()
    _check(load().ll_kv_attention_plan(Lq, num_heads, n_keys, compute_units, ATTENTION_POLICIES[policy],
                                       ctypes.byref(division), ctypes.byref(groups), ctypes.byref(rounds),
                                       ctypes.byref(split)), "ll_kv_attention_plan")
    names = {v: k for k, v in ATTENTION_POLICIES.items()}
    return {"division": names[division.value], "workgroups": groups.value, "whole_rounds": rounds.value,
            "split_tiles": split.value}


def attention_reserve(Lq: int, num_heads: int, n_keys: int, device=None) -> None:
    """Set up, on the current stream, the memory an attention launch of these sizes would pass partial tiles
    through (nothing if it would not split), so that the launch itself - for instance inside a graph recording -
    allocates nothing."""
    with torch.cuda.device(device if device is not None else torch.cuda.current_device()):
        _check(load().ll_kv_attention_reserve(Lq, num_heads, n_keys, _stream()), "ll_kv_attention_reserve")


def attention_release(device=None) -> None:
    """Free the memory the split division holds for the current stream, if any."""
    with torch.cuda.device(device if device is not None else torch.cuda.current_device()):
        _check(load().ll_kv_attention_release(_stream()), "ll_kv_attention_release")


class attention_policy:
    """``with attention_policy("narrow"): ...`` - how the attention launches inside the block divide their work
    between workgroups ("auto", "narrow", "wide" or "split"; process-wide, restored on exit)."""

    def __init__(self, name: str):
        if name not in ATTENTION_POLICIES:
            raise ValueError(f"unknown attention policy {name!r}; one of {sorted(ATTENTION_POLICIES)}")
        self.value = ATTENTION_POLICIES[name]

    def __enter__(self):
        self.previous = load().ll_kv_attention_get_policy()
        _check(load().ll_kv_attention_set_policy(self.value), "ll_kv_attention_set_policy")
        return self

    def __exit__(self, *exc):
        _check(load().ll_kv_attention_set_policy(self.previous), "ll_kv_attention_set_policy")
        return False


# --------------------------------------------------------------------------- elementwise
def rope_apply(x, cos, sin, seq_len=None):
    _require_cuda(x, cos, sin)
    if x.ndim != 3 or x.dtype != torch.bfloat16 or x.stride(2) != 1:
        raise ValueError("x must be bfloat16 [S, N, D] with a contiguous last dimension")
    S, N, D = x.shape
    seq_len = S if seq_len is None else seq_len
    if cos.shape != (seq_len, D // 2) or sin.shape != cos.shape or cos.dtype != torch.float32:
        raise ValueError(f"cos/sin must be float32 [{seq_len}, {D // 2}]")
    cos = cos.contiguous()
    sin = sin.contiguous()
    out = torch.empty((S, N, D), dtype=x.dtype, device=x.device)
    with torch.cuda.device(x.device):
        code = load().ll_rope_apply(x.data_ptr(), S, N, D, x.stride(0), x.stride(1), cos.data_ptr(), sin.data_ptr(),
                                    seq_len, out.data_ptr(), _stream())
    _check(code, "ll_rope_apply")
    return out


def qk_norm_rope(x, weight, eps, cos, sin, num_heads, seq_len=None, smooth=False):
    """RMSNorm over rows of x bf16 [S, num_heads*128], RoPE per head -> bf16 [S, num_heads, 128]; with
    ``smooth`` also returns that tensor minus its per-head mean over the 128 channels."""
    _require_cuda(x, weight, cos, sin)
    if x.ndim != 2 or x.dtype != torch.bfloat16 or not x.is_contiguous() or x.shape[1] != num_heads * 128:
        raise ValueError("x must be a contiguous bfloat16 [S, num_heads * 128] tensor")
    if weight.dtype != torch.bfloat16 or weight.numel() != x.shape[1]:
        raise ValueError("weight must be bfloat16 with one entry per channel")
    S = x.shape[0]
    seq_len = S if seq_len is None else seq_len
    if cos.shape != (seq_len, 64) or sin.shape != cos.shape or cos.dtype != torch.float32:
        raise ValueError(f"cos/sin must be float32 [{seq_len}, 64]")
    cos = cos.contiguous()
    sin = sin.contiguous()
    out = torch.empty((S, num_heads, 128), dtype=x.dtype, device=x.device)
    out_s = torch.empty_like(out) if smooth else None
    with torch.cuda.device(x.device):
        code = load().ll_qk_norm_rope(x.data_ptr(), S, num_heads, weight.contiguous().data_ptr(), float(eps),
                                      cos.data_ptr(), sin.data_ptr(), seq_len, out.data_ptr(), _ptr(out_s), _stream())
    _check(code, "ll_qk_norm_rope")
    return (out, out_s) if smooth else out


def qk_norm_rope_pair(q, k, q_weight, k_weight, eps, cos, sin, num_heads, seq_len=None, k_amax_out=None):
    """:func:`qk_norm_rope` of q and of k (with the smoothed second output) in one launch:
    returns (roped_q, roped_k, smoothed_k), each bf16 [S, num_heads, 128].  ``k_amax_out`` (an
    :class:`AmaxTicket`) receives the absolute maximum of roped_k."""
    _require_cuda(q, k, q_weight, k_weight, cos, sin)
    sink = _sink_struct(k_amax_out)
    for x in (q, k):
        if x.ndim != 2 or x.dtype != torch.bfloat16 or not x.is_contiguous() or x.shape[1] != num_heads * 128:
            raise ValueError("q and k must be contiguous bfloat16 [S, num_heads * 128] tensors")
    if q.shape != k.shape:
        raise ValueError("q and k must have the same shape")
    for w in (q_weight, k_weight):
        if w.dtype != torch.bfloat16 or w.numel() != q.shape[1]:
            raise ValueError("weights must be bfloat16 with one entry per channel")
    S = q.shape[0]
    seq_len = S if seq_len is None else seq_len
    if cos.shape != (seq_len, 64) or sin.shape != cos.shape or cos.dtype != torch.float32:
        raise ValueError(f"cos/sin must be float32 [{seq_len}, 64]")
    cos = cos.contiguous()
    sin = sin.contiguous()
    out_q = torch.empty((S, num_heads, 128), dtype=q.dtype, device=q.device)
    out_k, out_s = torch.empty_like(out_q), torch.empty_like(out_q)
    with torch.cuda.device(q.device):
        code = load().ll_qk_norm_rope_pair_amax(q.data_ptr(), k.data_ptr(), S, num_heads,
                                                q_weight.contiguous().data_ptr(), k_weight.contiguous().data_ptr(),
                                                float(eps), cos.data_ptr(), sin.data_ptr(), seq_len,
                                                out_q.data_ptr(), out_k.data_ptr(), out_s.data_ptr(),
                                                ctypes.byref(sink), _stream())
    _check(code, "ll_qk_norm_rope_pair")
    return out_q, out_k, out_s


def adaln_modulate(x, e_scale, e_shift, frame_seqlen, eps=1e-6, add_one_to_scale=True, amax_out=None):
    """``amax_out`` (an :class:`AmaxTicket`) receives the absolute maximum of the result."""
    _require_cuda(x, e_scale, e_shift)
    sink = _sink_struct(amax_out)
    if x.ndim != 3 or x.dtype != torch.bfloat16 or not x.is_contiguous():
        raise ValueError("x must be a contiguous bfloat16 [B, L, C] tensor")
    B, L, C = x.shape
    F = L // frame_seqlen
    for name, e in (("e_scale", e_scale), ("e_shift", e_shift)):
        if e.shape != (B, F, 1, C) or e.dtype != torch.bfloat16 or e.stride(3) != 1:
            raise ValueError(f"{name} must be bfloat16 [B, F, 1, C] = {(B, F, 1, C)}, got {tuple(e.shape)}")
    out = torch.empty_like(x)
    with torch.cuda.device(x.device):
        code = load().ll_adaln_modulate_amax(x.data_ptr(), B, L, C, e_scale.data_ptr(), e_shift.data_ptr(),
                                             e_scale.stride(0), e_scale.stride(1), e_shift.stride(0),
                                             e_shift.stride(1), frame_seqlen, float(eps), int(add_one_to_scale),
                                             out.data_ptr(), ctypes.byref(sink), _stream())
    _check(code, "ll_adaln_modulate")
    return out


def _norm_quantize_outputs(M: int, C: int, device):
    Mp, Kp = padded_shape((M, C))
    return (torch.empty((Mp, Kp // 2), dtype=torch.uint8, device=device),
            torch.empty(Mp * Kp // 16, dtype=torch.uint8, device=device),
            torch.empty(1, dtype=torch.float32, device=device))


def _norm_quantize_result(code: int, what: str, values, scales, amax):
    """None when the kernel does not take the shape (the caller runs the separate operations)."""
    if code == -3:
        return None
    _check(code, what)
    return values, scales.view(torch.float8_e4m3fn), amax


def adaln_quantize(x, e_scale, e_shift, frame_seqlen, rule: str, eps=1e-6, add_one_to_scale=True, spin_limit=None):
    """``quantize(adaln_modulate(x, ...).reshape(-1, C), rule)`` as one launch that never writes the modulated
    tensor: (values, scales, amax) with the same bytes, or None when the kernel does not take the shape."""
    _require_cuda(x, e_scale, e_shift)
    if x.ndim != 3 or x.dtype != torch.bfloat16 or not x.is_contiguous():
        raise ValueError("x must be a contiguous bfloat16 [B, L, C] tensor")
    B, L, C = x.shape
    F = L // frame_seqlen
    for name, e in (("e_scale", e_scale), ("e_shift", e_shift)):
        if e.shape != (B, F, 1, C) or e.dtype != torch.bfloat16 or e.stride(3) != 1:
            raise ValueError(f"{name} must be bfloat16 [B, F, 1, C] = {(B, F, 1, C)}, got {tuple(e.shape)}")
    values, scales, amax = _norm_quantize_outputs(B * L, C, x.device)
    sink = _sink_struct(amax_ticket(x.device))
    with torch.cuda.device(x.device):
        code = load().ll_adaln_quantize(x.data_ptr(), B, L, C, e_scale.data_ptr(), e_shift.data_ptr(),
                                        e_scale.stride(0), e_scale.stride(1), e_shift.stride(0), e_shift.stride(1),
                                        frame_seqlen, float(eps), int(add_one_to_scale), RULE_IDS[rule],
                                        values.data_ptr(), scales.data_ptr(), amax.data_ptr(), ctypes.byref(sink),
                                        NORM_QUANTIZE_SPIN_LIMIT if spin_limit is None else int(spin_limit), _stream())
    return _norm_quantize_result(code, "ll_adaln_quantize", values, scales, amax)


def layer_norm_quantize(x, weight, bias, rule: str, eps=1e-6, spin_limit=None):
    """``quantize(layer_norm(x, weight, bias).reshape(-1, C), rule)`` as one launch, like :func:`adaln_quantize`."""
    _require_cuda(x, weight, bias)
    if x.dtype != torch.bfloat16 or any(t is not None and t.dtype != torch.bfloat16 for t in (weight, bias)):
        raise ValueError("layer_norm takes bfloat16 input, weight and bias")
    C = x.shape[-1]
    x2 = x.reshape(-1, C)
    if not x2.is_contiguous():
        x2 = x2.contiguous()
    w = None if weight is None else weight.contiguous()
    b = None if bias is None else bias.contiguous()
    values, scales, amax = _norm_quantize_outputs(x2.shape[0], C, x.device)
    sink = _sink_struct(amax_ticket(x.device))
    with torch.cuda.device(x.device):
        code = load().ll_layer_norm_quantize(x2.data_ptr(), x2.shape[0], C, _ptr(w), _ptr(b), float(eps), RULE_IDS[rule],
                                             values.data_ptr(), scales.data_ptr(), amax.data_ptr(), ctypes.byref(sink),
                                             NORM_QUANTIZE_SPIN_LIMIT if spin_limit is None else int(spin_limit),
                                             _stream())
    return _norm_quantize_result(code, "ll_layer_norm_quantize", values, scales, amax)


def gate_residual(x, y, gate, frame_seqlen):
    """x + y * gate, x / y bf16 [B, L, C] contiguous, gate bf16 [B, F, 1, C] (per frame)."""
    _require_cuda(x, y, gate)
    if x.ndim != 3 or x.dtype != torch.bfloat16 or y.dtype != torch.bfloat16 or x.shape != y.shape \
            or not (x.is_contiguous() and y.is_contiguous()):
        raise ValueError("x and y must be contiguous bfloat16 [B, L, C] tensors of the same shape")
    B, L, C = x.shape
    F = L // frame_seqlen
    if gate.shape != (B, F, 1, C) or gate.dtype != torch.bfloat16 or gate.stride(3) != 1:
        raise ValueError(f"gate must be bfloat16 [B, F, 1, C] = {(B, F, 1, C)}, got {tuple(gate.shape)}")
    out = torch.empty_like(x)
    with torch.cuda.device(x.device):
        code = load().ll_gate_residual(x.data_ptr(), y.data_ptr(), B, L, C, gate.data_ptr(), gate.stride(0),
                                       gate.stride(1), frame_seqlen, out.data_ptr(), _stream())
    _check(code, "ll_gate_residual")
    return out


def rms_norm(x, weight, eps=1e-6):
    _require_cuda(x, weight)
    if x.dtype != torch.bfloat16 or weight.dtype != torch.bfloat16:
        raise ValueError("rms_norm takes bfloat16 input and weight")
    C = x.shape[-1]
    x2 = x.reshape(-1, C)
    if not x2.is_contiguous():
        x2 = x2.contiguous()
    out = torch.empty_like(x2)
    with torch.cuda.device(x.device):
        code = load().ll_rms_norm(x2.data_ptr(), x2.shape[0], C, weight.contiguous().data_ptr(), float(eps),
                                  out.data_ptr(), _stream())
    _check(code, "ll_rms_norm")
    return out.view(x.shape)


def layer_norm(x, weight, bias, eps=1e-6, amax_out=None):
    """LayerNorm over the last dimension with optional bf16 weight / bias (fp32 statistics, one rounding);
    ``amax_out`` (an :class:`AmaxTicket`) receives the absolute maximum of the result."""
    _require_cuda(x, weight, bias)
    if x.dtype != torch.bfloat16 or any(t is not None and t.dtype != torch.bfloat16 for t in (weight, bias)):
        raise ValueError("layer_norm takes bfloat16 input, weight and bias")
    C = x.shape[-1]
    x2 = x.reshape(-1, C)
    if not x2.is_contiguous():
        x2 = x2.contiguous()
    out = torch.empty_like(x2)
    sink = _sink_struct(amax_out)
    w = None if weight is None else weight.contiguous()
    b = None if bias is None else bias.contiguous()
    with torch.cuda.device(x.device):
        code = load().ll_layer_norm(x2.data_ptr(), x2.shape[0], C, _ptr(w), _ptr(b), float(eps), out.data_ptr(),
                                    ctypes.byref(sink), _stream())
    _check(code, "ll_layer_norm")
    return out.view(x.shape)
