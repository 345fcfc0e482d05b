"""ctypes binding of libmldhip.so (the C-ABI in include/mldhip.h).

The library is the product; there is no fallback path.  Importing works anywhere the
shared library exists; anything that launches needs a GPU.
"""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(os.path.dirname(_HERE), "libmldhip.so")

OK, INVALID_ARGUMENT, FAILED_PRECONDITION, OUT_OF_RANGE, UNIMPLEMENTED, INTERNAL = 0, 3, 9, 11, 12, 13
NOT_FOUND = 5
FLOAT16, FLOAT32, UINT8, INT8, INT32, UINT4 = 1, 2, 5, 6, 10, 15
PACKED_UINT8C4, PACKED_INT8C4, PACKED_INT8C16, PACKED_UINT8C16 = 1, 2, 5, 6
PACKED_UINT8W4C4, PACKED_INT8W4C4, PACKED_INT4C32, PACKED_UINT4C32 = 3, 4, 7, 8
LAYOUT_UNKNOWN, LAYOUT_I4O4, LAYOUT_O4I4, LAYOUT_2D_I4O4, LAYOUT_CUSTOM = 0, 1, 2, 6, 7
PRECISION_F32, PRECISION_F32_F16, PRECISION_F16 = 0, 1, 2
AXIS_O, AXIS_H, AXIS_W, AXIS_I = 0, 1, 2, 3
MAX_CUSTOM_GROUPS = 8

SYMBOLS = [
    "mldhip_last_error", "mldhip_version", "mldhip_fc_int8_weights_desc",
    "mldhip_fc_int4_weights_desc", "mldhip_conv_int8_weights_desc", "mldhip_total_elements",
    "mldhip_packed_bytes", "mldhip_rearrange_int8_as_uint8", "mldhip_rearrange_int8_as_uint4",
    "mldhip_rearrange_int8", "mldhip_rearrange_uint4_packed", "mldhip_weights_sum_i",
    "mldhip_scale_to_tensor", "mldhip_fc_is_recommended", "mldhip_fc_create",
    "mldhip_quantization_create", "mldhip_conv_int8_src_type", "mldhip_conv_int8_create",
    "mldhip_op_src_count", "mldhip_op_dst_count", "mldhip_op_src_name", "mldhip_op_dst_name",
    "mldhip_op_set_src", "mldhip_op_set_dst", "mldhip_op_set_shape", "mldhip_op_launch",
    "mldhip_op_kernel_name", "mldhip_op_cost", "mldhip_op_destroy", "mldhip_fc_launch_fused",
    "mldhip_checkpoint_fc_probe", "mldhip_checkpoint_fc_read", "mldhip_fc_launch_gated",
    "mldhip_scale_to_tensor_batched", "mldhip_fc_batch_ids_create",
    "mldhip_fc_int4_weights_desc_reference", "mldhip_fc_int4_weights_desc_decode", "mldhip_fc_int8_weights_desc_decode", "mldhip_set_tuning", "mldhip_fc_int4_decode_noalloc",
]


class WeightsDesc(C.Structure):
    _fields_ = [("type", C.c_int32), ("layout", C.c_int32), ("output_group_size", C.c_int32),
                ("n_groups", C.c_int32), ("group_axis", C.c_int32 * MAX_CUSTOM_GROUPS),
                ("group_size", C.c_int32 * MAX_CUSTOM_GROUPS)]


class FcDesc(C.Structure):
    _fields_ = [("precision", C.c_int32), ("src_type", C.c_int32), ("dst_type", C.c_int32),
                ("o", C.c_int32), ("i", C.c_int32), ("weights", WeightsDesc),
                ("scale_o", C.c_int32), ("scale_i", C.c_int32), ("scalar_scale", C.c_float),
                ("has_zero_point_tensor", C.c_int32), ("has_scalar_zero_point", C.c_int32),
                ("scalar_zero_point", C.c_float), ("has_bias", C.c_int32),
                ("max_tokens", C.c_int32), ("has_runtime_check", C.c_int32),
                ("src_end_ch_index", C.c_int32), ("dst_end_ch_index", C.c_int32),
                ("ring_o_offset_index", C.c_int32), ("ring_i_offset_index", C.c_int32), ("ring_size", C.c_int32),
                ("packed_params_offset", C.c_int32), ("packed_num_groups", C.c_int32),
                ("packed_max_group_size", C.c_int32), ("src_channels", C.c_int32), ("dst_channels", C.c_int32)]


class QuantDesc(C.Structure):
    _fields_ = [("src_type", C.c_int32), ("packed_type", C.c_int32), ("channels", C.c_int32),
                ("calculate_sum", C.c_int32), ("symmetric", C.c_int32), ("max_tokens", C.c_int32),
                ("round_to_nearest_even", C.c_int32)]


class ConvInt8Desc(C.Structure):
    _fields_ = [("src_packed_type", C.c_int32), ("dst_type", C.c_int32), ("o", C.c_int32),
                ("i", C.c_int32), ("weights", WeightsDesc), ("has_zero_point", C.c_int32),
                ("has_bias", C.c_int32), ("max_tokens", C.c_int32)]


class CheckpointFc(C.Structure):
    _fields_ = [("weights", WeightsDesc), ("o", C.c_int32), ("i", C.c_int32), ("weight_bits", C.c_int32),
                ("group_size", C.c_int32), ("scale_i", C.c_int32), ("has_zero_point", C.c_int32),
                ("weights_bytes", C.c_size_t), ("scale_elements", C.c_size_t)]


class MldhipError(RuntimeError):
    def __init__(self, code, message):
        super().__init__("mldhip status %d: %s" % (code, message))
        self.code = code
        self.message = message


_lib = None


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise ImportError(
                "libmldhip.so is not built (expected at %s); run `make -C ml-drift_amd/csrc` or "
                "__graft_entry__.build()" % LIB_PATH)
        # torch, where it is installed, is the device allocator of the tests and the bench, and it
        # ships a HIP runtime of its own: it has to be in the process first, so that this library
        # binds to the same runtime (loaded the other way round, launches from here fail with
        # "no ROCm-capable device is detected").
        try:
            import torch  # noqa: F401
        except ImportError:
            pass
        _lib = C.CDLL(LIB_PATH)
        _lib.mldhip_last_error.restype = C.c_char_p
        _lib.mldhip_version.restype = C.c_char_p
        _lib.mldhip_op_src_name.restype = C.c_char_p
        _lib.mldhip_op_dst_name.restype = C.c_char_p
        _lib.mldhip_op_kernel_name.restype = C.c_char_p
        _lib.mldhip_op_src_name.argtypes = [C.c_void_p, C.c_int]
        _lib.mldhip_op_dst_name.argtypes = [C.c_void_p, C.c_int]
        _lib.mldhip_op_kernel_name.argtypes = [C.c_void_p]
        _lib.mldhip_op_src_count.argtypes = [C.c_void_p]
        _lib.mldhip_op_dst_count.argtypes = [C.c_void_p]
        _lib.mldhip_op_set_src.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_size_t]
        _lib.mldhip_op_set_dst.argtypes = [C.c_void_p, C.c_int, C.c_void_p, C.c_size_t]
        _lib.mldhip_op_set_shape.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_int]
        _lib.mldhip_op_launch.argtypes = [C.c_void_p, C.c_void_p]
        _lib.mldhip_op_cost.argtypes = [C.c_void_p, C.POINTER(C.c_uint64), C.POINTER(C.c_uint64)]
        _lib.mldhip_op_destroy.argtypes = [C.c_void_p]
        _lib.mldhip_op_destroy.restype = None
        _lib.mldhip_set_tuning.argtypes = [C.c_char_p, C.c_int]
        _lib.mldhip_fc_int4_decode_noalloc.argtypes = [C.c_void_p] * 5 + [C.c_int] * 5 + [C.c_void_p]
    return _lib


def check(code):
    if code != OK:
        raise MldhipError(code, lib().mldhip_last_error().decode())


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def div_up(a, b):
    return (a + b - 1) // b


# ---- weight descriptions / packers (host) ----
def fc_int8_weights_desc(o, i, decode=False):
    """The reference's layout (one output group); with `decode` the layout for ops that run one token
    per launch (output groups of one slice)."""
    d = WeightsDesc()
    check((lib().mldhip_fc_int8_weights_desc_decode if decode else lib().mldhip_fc_int8_weights_desc)(o, i, C.byref(d)))
    return d


def fc_int4_weights_desc(o, i, reference=False, decode=False):
    """The layout this library asks for (output groups of 16 slices where the shape allows), with
    `reference` the reference's own choice (one output group), with `decode` the layout for ops that
    run one token per launch (output groups of 2 slices for layers of a few thousand channels)."""
    d = WeightsDesc()
    fn = (lib().mldhip_fc_int4_weights_desc_reference if reference else
          lib().mldhip_fc_int4_weights_desc_decode if decode else lib().mldhip_fc_int4_weights_desc)
    check(fn(o, i, C.byref(d)))
    return d


_forced_generic = [False]


def get_tuning_forced_generic():
    """True inside a `tuning(force_generic=1)` block."""
    return _forced_generic[0]


class tuning:
    """Context manager: overrides launch heuristics (mldhip_set_tuning) inside the block."""

    def __init__(self, **knobs):
        self.knobs = knobs

    def __enter__(self):
        for name, value in self.knobs.items():
            check(lib().mldhip_set_tuning(name.encode(), int(value)))
        if int(self.knobs.get("force_generic", 0)) > 0:
            _forced_generic[0] = True
        return self

    def __exit__(self, *exc):
        for name in self.knobs:
            check(lib().mldhip_set_tuning(name.encode(), -1))
        if "force_generic" in self.knobs:
            _forced_generic[0] = False
        return False


def conv_int8_weights_desc(o, i):
    d = WeightsDesc()
    check(lib().mldhip_conv_int8_weights_desc(o, i, C.byref(d)))
    return d


def make_desc(type_, layout, group=1, custom=None):
    d = WeightsDesc()
    d.type, d.layout, d.output_group_size = type_, layout, group
    if custom:
        d.n_groups = len(custom)
        for k, (axis, size) in enumerate(custom):
            d.group_axis[k] = axis
            d.group_size[k] = size
    return d


def _ohwi(w):
    w = np.ascontiguousarray(w)
    if w.ndim == 2:
        w = w.reshape(w.shape[0], 1, 1, w.shape[1])
    return w


def total_elements(desc, o, h, w, i):
    n = C.c_size_t()
    check(lib().mldhip_total_elements(C.byref(desc), o, h, w, i, C.byref(n)))
    return n.value


def packed_bytes(desc, o, h, w, i):
    n = C.c_size_t()
    check(lib().mldhip_packed_bytes(C.byref(desc), o, h, w, i, C.byref(n)))
    return n.value


def rearrange_int8_as_uint8(w, desc, shift=128, pad=128):
    w = _ohwi(np.asarray(w, np.int8))
    o, h, ww, i = w.shape
    out = np.empty(total_elements(desc, o, h, ww, i), np.uint8)
    check(lib().mldhip_rearrange_int8_as_uint8(_p(w), o, h, ww, i, C.byref(desc), _p(out),
                                               C.c_size_t(out.nbytes), shift, C.c_uint(pad)))
    return out


def rearrange_int8_as_uint4(w, desc, shift=8, pad=8):
    w = _ohwi(np.asarray(w, np.int8))
    o, h, ww, i = w.shape
    out = np.empty(total_elements(desc, o, h, ww, i) // 2, np.uint8)
    check(lib().mldhip_rearrange_int8_as_uint4(_p(w), o, h, ww, i, C.byref(desc), _p(out),
                                               C.c_size_t(out.nbytes), shift, C.c_uint(pad)))
    return out


def rearrange_int8(w, desc):
    w = _ohwi(np.asarray(w, np.int8))
    o, h, ww, i = w.shape
    out = np.empty(total_elements(desc, o, h, ww, i), np.int8)
    check(lib().mldhip_rearrange_int8(_p(w), o, h, ww, i, C.byref(desc), _p(out),
                                      C.c_size_t(out.nbytes)))
    return out


def rearrange_uint4_packed(src, shape_ohwi, desc, pad=8, swap_dims=False, sum_len=None,
                           sum_init=None):
    src = np.ascontiguousarray(src, np.uint8)
    o, h, w, i = shape_ohwi
    out = np.empty(total_elements(desc, o, h, w, i) // 2, np.uint8)
    sum_len = o if sum_len is None else sum_len
    sums = (np.zeros(sum_len, np.int32) if sum_init is None
            else np.ascontiguousarray(sum_init, np.int32).copy())
    check(lib().mldhip_rearrange_uint4_packed(_p(src), o, h, w, i, C.byref(desc), _p(out),
                                              C.c_size_t(out.nbytes), _p(sums), C.c_size_t(sum_len),
                                              C.c_uint(pad), int(swap_dims)))
    return out, sums


def weights_sum_i(w):
    w = _ohwi(np.asarray(w, np.int8))
    o, h, ww, i = w.shape
    out = np.empty(o, np.int32)
    check(lib().mldhip_weights_sum_i(_p(w), o, h, ww, i, _p(out)))
    return out


def scale_to_tensor(scale, dst_type):
    """scale: (o,) or (o, groups) float32 -> padded tensor buffer (uint16 bits or float32)."""
    s = np.ascontiguousarray(scale, np.float32)
    if s.ndim == 1:
        s = s.reshape(-1, 1)
    o, groups = s.shape
    dt = np.uint16 if dst_type == FLOAT16 else np.float32
    out = np.empty(groups * div_up(o, 4) * 4, dt)
    check(lib().mldhip_scale_to_tensor(_p(s), o, groups, dst_type, _p(out), C.c_size_t(out.nbytes)))
    return out


def scale_to_tensor_batched(scale, dst_type):
    """scale: (o, batch, groups) float32 -> [groups][batch][ceil(o/4)][4] tensor buffer."""
    s = np.ascontiguousarray(scale, np.float32)
    o, batch, groups = s.shape
    dt = np.uint16 if dst_type == FLOAT16 else np.float32
    out = np.empty(groups * batch * div_up(o, 4) * 4, dt)
    check(lib().mldhip_scale_to_tensor_batched(_p(s), o, batch, groups, dst_type, _p(out), C.c_size_t(out.nbytes)))
    return out


# ---- checkpoint files (host) ----
def checkpoint_fc_probe(directory, weights_name, base_name, o, i, weight_bits):
    """-> CheckpointFc (weights description, group size, zero-point presence, buffer sizes)."""
    info = CheckpointFc()
    check(lib().mldhip_checkpoint_fc_probe(directory.encode(), weights_name.encode(), base_name.encode(),
                                           o, i, weight_bits, C.byref(info)))
    return info


def checkpoint_fc_read(directory, weights_name, base_name, info, tensor_type, swap_dims=False):
    """-> dict(weights=uint8 buffer, scale=tensor buffer, zero_point=tensor buffer or None,
    weights_sum_i=int32[o])."""
    dt = np.uint16 if tensor_type == FLOAT16 else np.float32
    weights = np.empty(info.weights_bytes, np.uint8)
    scale = np.empty(info.scale_elements, dt)
    zp = np.empty(info.scale_elements, dt) if info.has_zero_point else None
    sums = np.empty(info.o, np.int32)
    check(lib().mldhip_checkpoint_fc_read(directory.encode(), weights_name.encode(), base_name.encode(),
                                          C.byref(info), int(bool(swap_dims)), tensor_type, _p(weights),
                                          C.c_size_t(weights.nbytes), _p(scale),
                                          _p(zp) if zp is not None else None, C.c_size_t(scale.nbytes), _p(sums)))
    return dict(weights=weights, scale=scale, zero_point=zp, weights_sum_i=sums)


# ---- ops ----
class Op:
    """Owns an mldhip_op handle.  Device buffers are torch tensors (or anything with
    data_ptr()/numel()/element_size()); they are kept alive by the caller."""

    def __init__(self, handle):
        self.handle = handle

    def __del__(self):
        if _lib is not None:  # (module globals are already cleared at interpreter shutdown)
            self.destroy()

    def destroy(self):
        if getattr(self, "handle", None):
            _lib.mldhip_op_destroy(self.handle)
            self.handle = None

    @property
    def src_names(self):
        n = lib().mldhip_op_src_count(self.handle)
        return [lib().mldhip_op_src_name(self.handle, k).decode() for k in range(n)]

    @property
    def dst_names(self):
        n = lib().mldhip_op_dst_count(self.handle)
        return [lib().mldhip_op_dst_name(self.handle, k).decode() for k in range(n)]

    def set_src(self, index, tensor):
        check(lib().mldhip_op_set_src(self.handle, index, C.c_void_p(tensor.data_ptr()),
                                      tensor.numel() * tensor.element_size()))

    def set_dst(self, index, tensor):
        check(lib().mldhip_op_set_dst(self.handle, index, C.c_void_p(tensor.data_ptr()),
                                      tensor.numel() * tensor.element_size()))

    def set_src_raw(self, index, ptr, nbytes):
        check(lib().mldhip_op_set_src(self.handle, index, C.c_void_p(ptr), nbytes))

    def set_dst_raw(self, index, ptr, nbytes):
        check(lib().mldhip_op_set_dst(self.handle, index, C.c_void_p(ptr), nbytes))

    def bind(self, srcs, dsts):
        for k, t in enumerate(srcs):
            self.set_src(k, t)
        for k, t in enumerate(dsts):
            self.set_dst(k, t)

    def set_shape(self, b, h, w):
        check(lib().mldhip_op_set_shape(self.handle, b, h, w))

    def launch(self, stream=0):
        check(lib().mldhip_op_launch(self.handle, C.c_void_p(stream)))

    @property
    def kernel_name(self):
        return lib().mldhip_op_kernel_name(self.handle).decode()

    def cost(self):
        b, f = C.c_uint64(), C.c_uint64()
        check(lib().mldhip_op_cost(self.handle, C.byref(b), C.byref(f)))
        return b.value, f.value


def fc_launch_fused(ops, stream=0):
    """One launch for FC ops that read the same source tensor; raises MldhipError with
    FAILED_PRECONDITION when they cannot share a launch."""
    arr = (C.c_void_p * len(ops))(*[op.handle for op in ops])
    check(lib().mldhip_fc_launch_fused(arr, len(ops), C.c_void_p(stream)))


GATE_GELU_TANH, GATE_SILU = 1, 2


def fc_launch_gated(gate, up, activation, dst, stream=0):
    """dst = activation(gate(x)) * up(x) in one launch; MldhipError(FAILED_PRECONDITION) when the
    pair is not served (launch the ops and the elementwise step separately then)."""
    check(lib().mldhip_fc_launch_gated(gate.handle, up.handle, activation,
                                       C.c_void_p(dst.data_ptr()), C.c_size_t(dst.numel() * dst.element_size()),
                                       C.c_void_p(stream)))


def fc_create(precision, src_type, dst_type, o, i, weights_desc, scale_shape=(1, 1),
              scalar_scale=1.0, has_zero_point_tensor=False, scalar_zero_point=None,
              has_bias=False, max_tokens=1, weights_batch=None, shared_src=False, src_end_ch_index=None,
              dst_end_ch_index=None, ring_o_offset_index=None, ring_i_offset_index=None, ring_size=0,
              packed_groups=None, src_channels=0, dst_channels=0):
    """weights_batch: number of weight matrices of a batch-ids op (mldhip_fc_batch_ids_create).
    src_end_ch_index / dst_end_ch_index: ConvRuntimeCheckDesc indices into the "params" object.
    ring_o_offset_index / ring_i_offset_index, ring_size: ringed weights (src_channels / dst_channels:
    channels of the tensors where they differ from the weights' i / o).
    packed_groups: (params_offset, num_groups, max_group_size) of ConvRuntimeCheckDesc::PackedGroups."""
    d = FcDesc()
    d.precision, d.src_type, d.dst_type, d.o, d.i = precision, src_type, dst_type, o, i
    d.weights = weights_desc
    d.scale_o, d.scale_i = scale_shape
    d.scalar_scale = scalar_scale
    d.has_zero_point_tensor = int(has_zero_point_tensor)
    d.has_scalar_zero_point = int(scalar_zero_point is not None)
    d.scalar_zero_point = 0.0 if scalar_zero_point is None else scalar_zero_point
    d.has_bias = int(has_bias)
    d.max_tokens = max_tokens
    checks = (src_end_ch_index, dst_end_ch_index, ring_o_offset_index, ring_i_offset_index)
    d.has_runtime_check = int(any(v is not None for v in checks) or packed_groups is not None)
    if packed_groups is not None:
        d.packed_params_offset, d.packed_num_groups, d.packed_max_group_size = packed_groups
    d.src_end_ch_index, d.dst_end_ch_index, d.ring_o_offset_index, d.ring_i_offset_index = [
        -1 if v is None else v for v in checks]
    d.ring_size = ring_size
    d.src_channels, d.dst_channels = src_channels, dst_channels
    h = C.c_void_p()
    if weights_batch is not None:
        check(lib().mldhip_fc_batch_ids_create(C.byref(d), weights_batch, int(shared_src), C.byref(h)))
    else:
        check(lib().mldhip_fc_create(C.byref(d), C.byref(h)))
    return Op(h)


def quantization_create(src_type, packed_type, channels, calculate_sum=False, symmetric=False,
                        max_tokens=1, round_to_nearest_even=False):
    d = QuantDesc(src_type, packed_type, channels, int(calculate_sum), int(symmetric), max_tokens,
                  int(round_to_nearest_even))
    h = C.c_void_p()
    check(lib().mldhip_quantization_create(C.byref(d), C.byref(h)))
    return Op(h)


def conv_int8_create(dst_type, o, i, weights_desc, has_zero_point=False, has_bias=False,
                     max_tokens=1, src_packed_type=PACKED_INT8C16):
    d = ConvInt8Desc()
    d.src_packed_type, d.dst_type, d.o, d.i = src_packed_type, dst_type, o, i
    d.weights = weights_desc
    d.has_zero_point, d.has_bias, d.max_tokens = int(has_zero_point), int(has_bias), max_tokens
    h = C.c_void_p()
    check(lib().mldhip_conv_int8_create(C.byref(d), C.byref(h)))
    return Op(h)


def fc_int4_decode_noalloc(src, weights, scale, bias, dst, o, i, scale_groups, output_group_size, tokens, stream=0):
    """mldhip_fc_int4_decode_noalloc over torch tensors (or None for `bias`)."""
    ptr = lambda t: None if t is None else C.c_void_p(t.data_ptr())
    check(lib().mldhip_fc_int4_decode_noalloc(ptr(src), ptr(weights), ptr(scale), ptr(bias), ptr(dst), o, i,
                                              scale_groups, output_group_size, tokens, C.c_void_p(stream)))
