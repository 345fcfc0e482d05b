"""ctypes binding of the CPU oracle (TEST INFRASTRUCTURE ONLY).

Only tests, the smoke check and the benchmark's cpu_baseline leg import this module; the
product package never does.  Functions take and return numpy arrays.

The restatements written here in numpy on top of the C kernel restatement, and what pins each
(the C functions' pins are listed in mld_oracle.c):
  fc_kernel_runtime_check   literal end-slice values and the reference's four runtime-channel cases
                            (K = 171, N = 533) against the float product over the aligned bounds
  fc_batch_ids_kernel       the reference's own test shapes against FullyConnectedWeightsBatchIdsReference
                            restated per row, and the id-permutation property
  fc_packed_groups_kernel   the reference test's flow (sort by matrix, run, unsort) against per-token
                            float64 products
  ringed_gather / fc_ringed_kernel
                            what the mathematics fixes: a ring offset r equals the plain FullyConnected
                            over the weights rolled by r along I (ring_i) or O (ring_o), computed in
                            float64 from the unpacked values, on the sizes and offsets of the
                            reference's FullyConnectedRingedITest / RingedOTest (72 / 20 / 56 channels,
                            offsets 0, 17, 20, 33, 49, one and three matrices), plus negative and
                            beyond-the-ring offsets and the composition with src_end_ch
  gated_activation          closed forms (0 at 0, g * u for large g, the clamps)
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "libmld_oracle.so")

LAYOUT_I4O4 = 1
LAYOUT_O4I4 = 2
LAYOUT_2D_I4O4 = 6
PREC_F32, PREC_F32F16, PREC_F16 = 0, 1, 2
SCALE_SCALAR, SCALE_LINEAR, SCALE_BLOCK = 0, 1, 2
PACKED_UINT8C4, PACKED_INT8C4, PACKED_INT8C16, PACKED_UINT8C16 = 1, 2, 5, 6
PACKED_UINT8W4C4, PACKED_INT8W4C4, PACKED_INT4C32, PACKED_UINT4C32 = 3, 4, 7, 8
AXIS_O, AXIS_H, AXIS_W, AXIS_I = 0, 1, 2, 3


def build(force=False):
    if force or not os.path.exists(_LIB_PATH):
        subprocess.check_call(["make", "-C", _HERE, "-B" if force else "-s"],
                              stdout=subprocess.DEVNULL)
    return _LIB_PATH


class FcParams(C.Structure):
    _fields_ = [("m", C.c_int), ("k", C.c_int), ("n", C.c_int), ("precision", C.c_int),
                ("weight_bits", C.c_int), ("scale_kind", C.c_int), ("groups", C.c_int),
                ("has_zero_point", C.c_int), ("has_bias", C.c_int), ("use_fma", C.c_int),
                ("wg_y", C.c_int), ("scalar_scale", C.c_float),
                ("scalar_zero_point", C.c_float), ("threads", C.c_int)]


_lib = None


def lib():
    global _lib
    if _lib is None:
        build()
        _lib = C.CDLL(_LIB_PATH)
        _lib.mldo_total_elements.restype = C.c_size_t
        _lib.mldo_custom_total_elements.restype = C.c_size_t
        _lib.mldo_f32_to_f16.restype = C.c_uint16
        _lib.mldo_f32_to_f16.argtypes = [C.c_float]
        _lib.mldo_f16_to_f32.restype = C.c_float
        _lib.mldo_f16_to_f32.argtypes = [C.c_uint16]
    return _lib


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _c(a, dtype):
    return np.ascontiguousarray(a, dtype=dtype)


def div_up(a, b):
    return (a + b - 1) // b


# ---- fp16 ----
def f32_to_f16_bits(x):
    x = _c(x, np.float32)
    out = np.empty(x.shape, np.uint16)
    lib().mldo_convert_f32_f16(_p(x), _p(out), C.c_size_t(x.size))
    return out


def f16_bits_to_f32(h):
    h = _c(h, np.uint16)
    out = np.empty(h.shape, np.float32)
    lib().mldo_convert_f16_f32(_p(h), _p(out), C.c_size_t(h.size))
    return out


# ---- tensor layout ----
def to_slices(x):
    """[tokens][channels] -> slice-major [ceil(C/4)][tokens][4], zero padded."""
    x = np.ascontiguousarray(x)
    t, c = x.shape
    out = np.empty((div_up(c, 4), t, 4), x.dtype)
    lib().mldo_bhwc_to_slices(_p(x), t, c, x.dtype.itemsize, _p(out))
    return out


def from_slices(x, channels):
    x = np.ascontiguousarray(x)
    s, t, four = x.shape
    assert four == 4 and s == div_up(channels, 4)
    out = np.empty((t, channels), x.dtype)
    lib().mldo_slices_to_bhwc(_p(x), t, channels, x.dtype.itemsize, _p(out))
    return out


# ---- packers.  weights are numpy arrays shaped (O, H, W, I) or (O, I) ----
def _ohwi(w):
    w = np.ascontiguousarray(w)
    if w.ndim == 2:
        w = w.reshape(w.shape[0], 1, 1, w.shape[1])
    return w


def total_elements(layout, o, h, w, i, group):
    return lib().mldo_total_elements(layout, o, h, w, i, group)


def rearrange_u8(w, layout, group, pad, reshape_path=False):
    w = _ohwi(_c(w, np.uint8))
    o, h, ww, i = w.shape
    out = np.empty(total_elements(layout, o, h, ww, i, group), np.uint8)
    fn = lib().mldo_rearrange_u8_reshape if reshape_path else lib().mldo_rearrange_u8
    rc = fn(_p(w), o, h, ww, i, layout, group, C.c_uint8(pad), _p(out))
    if rc:
        raise ValueError("unsupported layout")
    return out


def rearrange_i8(w, layout, group):
    w = _ohwi(_c(w, np.int8))
    o, h, ww, i = w.shape
    out = np.empty(total_elements(layout, o, h, ww, i, group), np.int8)
    if lib().mldo_rearrange_i8(_p(w), o, h, ww, i, layout, group, _p(out)):
        raise ValueError("unsupported layout")
    return out


def int8_as_uint8(w, layout, group, shift=128, pad=128):
    w = _ohwi(_c(w, np.int8))
    o, h, ww, i = w.shape
    out = np.empty(total_elements(layout, o, h, ww, i, group), np.uint8)
    if lib().mldo_int8_as_uint8(_p(w), o, h, ww, i, layout, group, shift, C.c_uint(pad), _p(out)):
        raise ValueError("unsupported layout")
    return out


def int8_as_uint4(w, layout, group, shift=8, pad=8):
    w = _ohwi(_c(w, np.int8))
    o, h, ww, i = w.shape
    out = np.empty(total_elements(layout, o, h, ww, i, group) // 2, np.uint8)
    if lib().mldo_int8_as_uint4(_p(w), o, h, ww, i, layout, group, shift, C.c_uint(pad), _p(out)):
        raise ValueError("unsupported layout")
    return out


def uint4_packed(src_packed, shape_ohwi, layout, group, pad=8, swap_dims=False, sum_len=None,
                 sum_init=None):
    src = _c(src_packed, np.uint8)
    o, h, w, i = shape_ohwi
    out = np.empty(total_elements(layout, o, h, w, i, group) // 2, np.uint8)
    sum_len = o if sum_len is None else sum_len
    sums = np.zeros(sum_len, np.int32) if sum_init is None else _c(sum_init, np.int32).copy()
    rc = lib().mldo_uint4_packed(_p(src), o, h, w, i, layout, group, _p(out), _p(sums),
                                 C.c_size_t(sum_len), C.c_uint(pad), int(swap_dims))
    if rc:
        raise NotImplementedError("Unsupported layout")
    return out, sums


def weights_sum_i(w):
    w = _ohwi(_c(w, np.int8))
    o, h, ww, i = w.shape
    out = np.empty(o, np.int32)
    lib().mldo_weights_sum_i(_p(w), o, h, ww, i, _p(out))
    return out


def rearrange_custom_i8(w, groups, pad=0):
    """groups: list of (axis, size), fastest-varying first; size <= 0 = rest of the axis."""
    w = _ohwi(_c(w, np.int8))
    o, h, ww, i = w.shape
    axes = np.array([g[0] for g in groups], np.int32)
    sizes = np.array([g[1] for g in groups], np.int32)
    n = lib().mldo_custom_total_elements(o, h, ww, i, _p(axes), _p(sizes), len(groups))
    out = np.empty(n, np.int8)
    lib().mldo_rearrange_custom_i8(_p(w), o, h, ww, i, _p(axes), _p(sizes), len(groups),
                                   C.c_int8(pad), _p(out))
    return out


def scale_to_hoio4(scale_ohi):
    """(O, I) float scales -> [I groups][ceil(O/4)][4] float, zero padded."""
    s = _c(scale_ohi, np.float32)
    o, i = s.shape
    out = np.empty((div_up(o, 4), 4 * i), np.float32)
    lib().mldo_scale_to_hoio4(_p(s), o, 1, i, _p(out))
    # HWC (1, os, 4*i) with channel index i*4+ch -> slice-major [i][os][4]
    return np.ascontiguousarray(out.reshape(div_up(o, 4), i, 4).transpose(1, 0, 2))


def scale_to_hoio4_batched(scale_obi):
    """(O, batch, I) float scales -> [I groups][batch][ceil(O/4)][4] float, zero padded: the HWC
    tensor (h = batch, w = O slices, c = 4*I) of OHIToHOIO4 (common/task/tensor_desc.cc:267-292) in
    the buffer order [slice of c][h][w][4] (task/tensor_desc.cc:1841-1873)."""
    s = _c(scale_obi, np.float32)
    o, b, i = s.shape
    out = np.empty((b, div_up(o, 4), 4 * i), np.float32)
    lib().mldo_scale_to_hoio4(_p(s), o, b, i, _p(out))
    return np.ascontiguousarray(out.reshape(b, div_up(o, 4), i, 4).transpose(2, 0, 1, 3))


# ---- FullyConnected ----
def fc_kernel(act_slices, weights, m, k, n, precision, weight_bits, scale_kind=SCALE_LINEAR,
              scale=None, zero_point=None, bias=None, groups=1, use_fma=True, wg_y=1,
              scalar_scale=1.0, scalar_zero_point=0.0, threads=0):
    """act_slices / scale / zero_point / bias / result are in the tensor dtype of the
    precision: float32 for PREC_F32, uint16 (binary16 bits) otherwise."""
    tdt = np.float32 if precision == PREC_F32 else np.uint16
    act = _c(act_slices, tdt)
    assert act.size == div_up(k, 4) * m * 4
    w = _c(weights, np.uint8)
    p = FcParams(m, k, n, precision, weight_bits, scale_kind, groups,
                 int(zero_point is not None or (scale_kind == SCALE_SCALAR and scalar_zero_point != 0.0)),
                 int(bias is not None), int(use_fma), wg_y, scalar_scale, scalar_zero_point,
                 threads)
    sc = None if scale is None else _c(scale, tdt)
    zp = None if zero_point is None else _c(zero_point, tdt)
    bi = None if bias is None else _c(bias, tdt)
    out = np.empty((div_up(n, 4), m, 4), tdt)
    global last_fc_path
    last_fc_path = lib().mldo_fc_kernel(C.byref(p), _p(act), _p(w), _p(sc), _p(zp), _p(bi), _p(out))
    return out


last_fc_path = None  # what the last fc_kernel call ran: 0 one channel at a time, 1 eight at a time (AVX2 + F16C)


def set_fast_path(enabled):
    """Switches the vector path of fc_kernel (bit-identical to the scalar one) on or off."""
    lib().mldo_set_fast_path(int(bool(enabled)))


def runtime_end_slices(src_end_ch, dst_end_ch, k, n, block_quantized):
    """(K-slices the loop covers, dst slices written) under runtime channel bounds:
    src_end_ch = min(params value, src channels), src_end_slices = (src_end_ch + 3) / 4
    (common/kernels/fully_connected.cc:750-755, 795; the group-wise loop runs over all groups,
    :784-794); dst_end_slice = min(round_up(params value, 32) / 4, dst slices)
    (ConvRuntimeCheckDesc::GetRuntimeEndSlice, common/task/gpu_operation.cc:1832-1836, with
    kChannelsAlignment = 32; fully_connected_util.cc:231-243)."""
    ks, ns = div_up(k, 4), div_up(n, 4)
    ks_end = ks
    if src_end_ch is not None and not block_quantized:
        ks_end = max(0, min(ks, (min(int(src_end_ch), k) + 3) // 4))
    ns_end = ns
    if dst_end_ch is not None:
        ns_end = max(0, min(ns, ((int(dst_end_ch) + 31) // 32) * 32 // 4))
    return ks_end, ns_end


def fc_kernel_runtime_check(act_slices, weights, m, k, n, precision, weight_bits, scale_kind=SCALE_LINEAR, scale=None,
                            zero_point=None, bias=None, groups=1, src_end_ch=None, dst_end_ch=None, dst_before=None):
    """The generated kernel with ConvRuntimeCheckDesc channel bounds (fully_connected.cc:644-652: work
    items of slices >= dst_end_slice return before they write; :750-755, 795: the K loop stops at
    src_end_slices).  The K loop over the first src_end_slices slices is the kernel on the leading
    rows of the packed buffer (the one-group I4O4 layout has the K-slice outermost), so this
    restatement runs `fc_kernel` on that prefix; dst slices that are not written keep `dst_before`
    (zeros when not given).  `weights`: packed in the reference's one-group layout."""
    tdt = np.float32 if precision == PREC_F32 else np.uint16
    ks, ns = div_up(k, 4), div_up(n, 4)
    ks_end, ns_end = runtime_end_slices(src_end_ch, dst_end_ch, k, n, scale_kind == SCALE_BLOCK)
    out = np.zeros((ns, m, 4), tdt) if dst_before is None else _c(dst_before, tdt).reshape(ns, m, 4).copy()
    if ns_end == 0:
        return out
    block_bytes = 16 if weight_bits == 8 else 8
    act = _c(act_slices, tdt).reshape(ks, m, 4)
    w = _c(weights, np.uint8).reshape(ks, ns * block_bytes)
    if ks_end == 0:
        # no K-slice: the result is the bias alone (0 without one), converted like any result
        zero_act = np.zeros((1, m, 4), tdt)
        full = fc_kernel(zero_act, w[:1].copy(), m, 4, n, precision, weight_bits, scale_kind, scale, zero_point, bias,
                         1 if scale_kind != SCALE_BLOCK else groups)
    else:
        full = fc_kernel(np.ascontiguousarray(act[:ks_end]), np.ascontiguousarray(w[:ks_end]), m, ks_end * 4, n, precision,
                         weight_bits, scale_kind, scale, zero_point, bias, groups)
    out[:ns_end] = full[:ns_end]
    return out


def ringed_gather(weights, ring_axis, ring_size, ring_offset, src_slices, dst_slices, batch_id=0):
    """The 16-byte I4O4 blocks (word i = input channel i of the K-slice, byte c = output channel c of the
    dst slice) that the generated kernel assembles from ringed uint8 weights, for every (src_s, dst_s),
    by the reference's own address arithmetic on 4-byte words (ReadRingedWeightsAsFloat,
    common/kernels/fully_connected.cc:443-471):
      ring_axis "i" (kOSpatialIOGroupI4O4 buffer, GetRingedIAddresses :424-441 with :699-706):
        ring_i_offset = ((offset % ring_size) + ring_size) % ring_size; i0 = (src_s * 4 + ring_i_offset) %
        ring_size, i1..i3 = i0 + 1..3 wrapped once; word j at (ij >> 2) * dst_stride + (ij & 3) + ring_i_base,
        dst_stride = 4 * dst slices, ring_i_base = dst_s * 4 + w_batch_id * ring_size * dst slices;
      ring_axis "o" (kOSpatialIOGroupO4I4 buffer, GetRingedOAddresses :411-422 with :676-697):
        o0 = (dst_s * 4 + ring_o_offset) % ring_size, o1..o3 wrapped once; word c at src_s * ring_size + oc
        + w_batch_id * ring_size * src slices holds the 4 input channels of output oc, so the I4O4 block is
        its byte transpose.
    Returns uint8 [src_slices][dst_slices][16]: the packed buffer (one output group) of an unringed
    FullyConnected with the same results."""
    w32 = _c(weights, np.uint8).view(np.uint32)
    off = ((int(ring_offset) % ring_size) + ring_size) % ring_size
    if ring_axis == "i":
        src_s = np.arange(src_slices)[:, None, None]
        dst_s = np.arange(dst_slices)[None, :, None]
        j = np.arange(4)[None, None, :]
        i0 = (src_s * 4 + off) % ring_size
        ij = i0 + j
        ij = np.where(ij >= ring_size, ij - ring_size, ij)
        addr = (ij >> 2) * (dst_slices * 4) + (ij & 3) + dst_s * 4 + batch_id * ring_size * dst_slices
        words = w32[addr]  # [src_s][dst_s][word j]
        return np.ascontiguousarray(words).view(np.uint8).reshape(src_slices, dst_slices, 16)
    assert ring_axis == "o"
    src_s = np.arange(src_slices)[:, None, None]
    dst_s = np.arange(dst_slices)[None, :, None]
    c = np.arange(4)[None, None, :]
    o0 = (dst_s * 4 + off) % ring_size
    oc = o0 + c
    oc = np.where(oc >= ring_size, oc - ring_size, oc)
    addr = src_s * ring_size + oc + batch_id * ring_size * src_slices
    words = np.ascontiguousarray(w32[addr]).view(np.uint8).reshape(src_slices, dst_slices, 4, 4)  # [c][i]
    return np.ascontiguousarray(words.transpose(0, 1, 3, 2)).reshape(src_slices, dst_slices, 16)  # [i][c]


def fc_ringed_kernel(act_slices, weights, m, src_channels, dst_channels, ring_axis, ring_size, ring_offset, precision,
                     scale_kind=SCALE_LINEAR, scale=None, zero_point=None, bias=None, groups=1, src_end_ch=None,
                     dst_end_ch=None, batch_id=0, dst_before=None, scalar_scale=1.0, scalar_zero_point=0.0):
    """The generated kernel over ringed uint8 weights (ConvRuntimeCheckDesc::ring_i_offset_index /
    ring_o_offset_index, common/kernels/fully_connected.cc:676-706, 411-471): it differs from the plain
    kernel only in where the four weight words of a (src_s, dst_s) step come from, so this restatement
    gathers them (`ringed_gather`) and runs `fc_kernel_runtime_check` on the result.  Scales, zero points
    and biases are read at the dst slice (fully_connected.cc:762-776), i.e. they belong to the dst channel,
    not to the ring position.  For ring_axis "o" the reference accumulates `r.c += dot(v, w_c)` per output
    (fully_connected_util.cc:186-199), whose summation order inside dot() is the compiler's; the I4O4
    order used here is one valid choice (results agree within the FullyConnected tolerance, not bit for
    bit).  `weights`: the packed ring buffer (all matrices); `batch_id`: the matrix of this dst row."""
    ks, ns = div_up(src_channels, 4), div_up(dst_channels, 4)
    blocks = ringed_gather(weights, ring_axis, ring_size, ring_offset, ks, ns, batch_id)
    if scale_kind == SCALE_SCALAR:
        tdt = np.float32 if precision == PREC_F32 else np.uint16
        out = fc_kernel(act_slices, blocks, m, src_channels, dst_channels, precision, 8, scale_kind, None, None, bias, 1,
                        scalar_scale=scalar_scale, scalar_zero_point=scalar_zero_point)
        assert src_end_ch is None and dst_end_ch is None
        return out.astype(tdt)
    return fc_kernel_runtime_check(act_slices, blocks, m, src_channels, dst_channels, precision, 8, scale_kind, scale,
                                   zero_point, bias, groups, src_end_ch=src_end_ch, dst_end_ch=dst_end_ch,
                                   dst_before=dst_before)


def fc_batch_ids_kernel(act_slices, ids, weights, rows, row_tokens, src_rows, weights_batch, k, n, precision,
                        weight_bits, scale_kind=SCALE_LINEAR, scale=None, zero_point=None, bias=None, groups=1):
    """The generated kernel with batched weights and runtime batch ids
    (common/kernels/fully_connected.cc:654-665 w_batch_id, :482-560 the weight address offset
    w_batch_id * Ks * Ns, :804-822 source row min(dst_h, Height - 1);
    fully_connected_util.cc:80-125 scale / zero point read at (o_slice, w_batch_id, group),
    :279-290 GetWeightsBatchId): every dst row is the plain kernel on that row's source tokens with
    the selected matrix, so this restatement runs `fc_kernel` per row on views of the buffers.
    act_slices [Ks][src_rows * row_tokens][4], result [Ns][rows * row_tokens][4];
    weights: `weights_batch` packed matrices one after the other; scale / zero_point:
    [groups][weights_batch][Ns][4]."""
    tdt = np.float32 if precision == PREC_F32 else np.uint16
    ks, ns = div_up(k, 4), div_up(n, 4)
    act = _c(act_slices, tdt).reshape(ks, src_rows * row_tokens, 4)
    w = _c(weights, np.uint8).reshape(weights_batch, -1)
    sc = None if scale is None else _c(scale, tdt).reshape(groups, weights_batch, ns * 4)
    zp = None if zero_point is None else _c(zero_point, tdt).reshape(groups, weights_batch, ns * 4)
    out = np.empty((ns, rows * row_tokens, 4), tdt)
    for y in range(rows):
        e = int(ids[y])
        sy = min(y, src_rows - 1)
        a = np.ascontiguousarray(act[:, sy * row_tokens:(sy + 1) * row_tokens, :])
        r = fc_kernel(a, w[e], row_tokens, k, n, precision, weight_bits, scale_kind,
                      None if sc is None else np.ascontiguousarray(sc[:, e, :]),
                      None if zp is None else np.ascontiguousarray(zp[:, e, :]), bias, groups)
        out[:, y * row_tokens:(y + 1) * row_tokens, :] = r
    return out


def fc_packed_groups_kernel(act_slices, sizes, offsets, weights, tokens, k, n, precision, weight_bits,
                            scale_kind=SCALE_LINEAR, scale=None, zero_point=None, bias=None, groups=1,
                            max_group_size=None, dst_before=None):
    """The generated kernel with ConvRuntimeCheckDesc::PackedGroups (common/kernels/fully_connected_util.cc:
    263-277: w_group_size / w_group_offset read per weight matrix, work-groups beyond the size return;
    fully_connected.cc:810-816: source and destination token = w_group_offset + local token, row 0;
    fully_connected_util.cc:382-386: written only below w_group_offset + w_group_size): matrix g on the
    `sizes[g]` tokens from token `offsets[g]`, i.e. `fc_kernel` on that run of tokens with matrix g of
    the batched buffers.  Tokens in no group keep `dst_before` (zeros when not given).
    act [Ks][tokens][4] -> [Ns][tokens][4]; weights / scale / zero_point as for fc_batch_ids_kernel."""
    tdt = np.float32 if precision == PREC_F32 else np.uint16
    ks, ns = div_up(k, 4), div_up(n, 4)
    nb = len(sizes)
    act = _c(act_slices, tdt).reshape(ks, tokens, 4)
    w = _c(weights, np.uint8).reshape(nb, -1)
    sc = None if scale is None else _c(scale, tdt).reshape(groups, nb, ns * 4)
    zp = None if zero_point is None else _c(zero_point, tdt).reshape(groups, nb, ns * 4)
    out = np.zeros((ns, tokens, 4), tdt) if dst_before is None else _c(dst_before, tdt).reshape(ns, tokens, 4).copy()
    for g in range(nb):
        size, off = int(sizes[g]), int(offsets[g])
        if max_group_size is not None:
            size = min(size, max_group_size)
        size = min(size, tokens - off)
        if size <= 0 or off < 0:
            continue
        a = np.ascontiguousarray(act[:, off:off + size, :])
        out[:, off:off + size, :] = fc_kernel(a, w[g], size, k, n, precision, weight_bits, scale_kind,
                                              None if sc is None else np.ascontiguousarray(sc[:, g, :]),
                                              None if zp is None else np.ascontiguousarray(zp[:, g, :]), bias, groups)
    return out


def fc_batch_ids_int8_kernel(act_slices_i8, ids, weights, rows, row_tokens, src_rows, weights_batch, k, n, weight_bits):
    """The integer-math variant with batched weights (the same generator with int8 sources:
    common/kernels/fully_connected.cc:543-621 with the w_batch_id offsets of :549-557, rows as in
    :804-822): `fc_int8_kernel` per dst row on views of the buffers.  act [Ks][src_rows *
    row_tokens][4] int8 -> [Ns][rows * row_tokens][4] int32."""
    ks, ns = div_up(k, 4), div_up(n, 4)
    act = _c(act_slices_i8, np.int8).reshape(ks, src_rows * row_tokens, 4)
    w = _c(weights, np.uint8).reshape(weights_batch, -1)
    out = np.empty((ns, rows * row_tokens, 4), np.int32)
    for y in range(rows):
        sy = min(y, src_rows - 1)
        a = np.ascontiguousarray(act[:, sy * row_tokens:(sy + 1) * row_tokens, :])
        out[:, y * row_tokens:(y + 1) * row_tokens, :] = fc_int8_kernel(a, w[int(ids[y])], row_tokens, k, n, weight_bits)
    return out


def fc_batch_ids_reference_f32(src, weights_obi, ids):
    """FullyConnectedWeightsBatchIdsReference (common/task/testing_ref_ops.cc:1042-1067): src
    (src_rows, tokens, K) float, weights (O, batch, K) float -> (rows, tokens, O); a source with one
    row is read by every dst row."""
    src = np.asarray(src, np.float32)
    w = np.asarray(weights_obi, np.float32)
    rows = len(ids)
    out = np.zeros((rows, src.shape[1], w.shape[0]), np.float32)
    for y in range(rows):
        sy = 0 if src.shape[0] == 1 else y
        wm = w[:, int(ids[y]), :]
        for x in range(src.shape[1]):
            for d in range(w.shape[0]):
                acc = np.float32(0.0)
                for c in range(w.shape[2]):
                    acc = np.float32(acc + src[sy, x, c] * wm[d, c])
                out[y, x, d] = acc
    return out


def fc_int8_kernel(act_slices_i8, weights, m, k, n, weight_bits):
    act = _c(act_slices_i8, np.int8)
    w = _c(weights, np.uint8)
    out = np.empty((div_up(n, 4), m, 4), np.int32)
    lib().mldo_fc_int8_kernel(m, k, n, weight_bits, _p(act), _p(w), _p(out))
    return out


def fc_reference_f32(src, weights, bias=None):
    src = _c(src, np.float32)
    w = _c(weights, np.float32)
    m, k = src.shape
    n = w.shape[0]
    b = None if bias is None else _c(bias, np.float32)
    out = np.empty((m, n), np.float32)
    lib().mldo_fc_reference_f32(m, k, n, _p(src), _p(w), _p(b), _p(out))
    return out


def fc_reference_i8(src, weights):
    src = _c(src, np.int8)
    w = _c(weights, np.int8)
    m, k = src.shape
    n = w.shape[0]
    out = np.empty((m, n), np.int32)
    lib().mldo_fc_reference_i8(m, k, n, _p(src), _p(w), _p(out))
    return out


def make_weights_from_int8(w, scale, zero_point=None):
    w = _c(w, np.int8)
    n, k = w.shape
    s = _c(scale, np.float32).reshape(-1, 1) if np.ndim(scale) == 1 else _c(scale, np.float32)
    z = None
    if zero_point is not None:
        z = _c(zero_point, np.float32).reshape(s.shape)
    out = np.empty((n, k), np.float32)
    lib().mldo_make_weights_from_int8(n, k, _p(w), _p(s), _p(z), s.shape[0], s.shape[1], _p(out))
    return out


# ---- quantization ----
def quantize(src_slices, tokens, channels, packed_type=PACKED_INT8C4, symmetric=False,
             calculate_sum=False, batch=1, height=1):
    """tokens = height * width * batch, flattened as (y * width + x) * batch + b.  Returns (codes,
    params): codes as bytes, C4 [S][tokens][4]; C16 [ceil(S/4)][tokens][16]; C32 (4-bit codes,
    uint8 bytes of two nibbles) [ceil(S/8)][tokens][16]; W4C4 [S][height][ceil(width/4)][batch][16]."""
    src = np.ascontiguousarray(src_slices)
    is_f16 = src.dtype == np.uint16
    assert is_f16 or src.dtype == np.float32
    slices = div_up(channels, 4)
    assert src.size == slices * tokens * 4 and tokens % (batch * height) == 0
    width = tokens // (batch * height)
    signed = packed_type in (PACKED_INT8C4, PACKED_INT8C16, PACKED_INT8W4C4)
    cdt = np.int8 if signed else np.uint8
    if packed_type in (PACKED_INT8C16, PACKED_UINT8C16):
        codes = np.empty((div_up(slices, 4), tokens, 16), cdt)
    elif packed_type in (PACKED_INT4C32, PACKED_UINT4C32):
        codes = np.empty((div_up(slices, 8), tokens, 16), np.uint8)
    elif packed_type in (PACKED_INT8W4C4, PACKED_UINT8W4C4):
        codes = np.empty((slices, height, div_up(width, 4), batch, 16), cdt)
    else:
        codes = np.empty((slices, tokens, 4), cdt)
    params = np.empty((tokens, 4), np.float32)
    lib().mldo_quantize_packed(height, width, batch, channels, int(is_f16), _p(src), packed_type,
                               int(symmetric), int(calculate_sum), _p(codes), _p(params))
    return codes, params


def dequantize(acc_slices, params, weights_sum, weights_scale, n, k, weights_zero_point=None,
               bias=None, dst_f16=True):
    acc = _c(acc_slices, np.int32)
    ns, tokens, _ = acc.shape
    pr = _c(params, np.float32)

    def padded(a, dt):
        a = _c(a, dt).ravel()
        out = np.zeros(ns * 4, dt)
        out[:a.size] = a
        return out
    ws = padded(weights_sum, np.int32)
    sc = padded(weights_scale, np.float32)
    zp = None if weights_zero_point is None else padded(weights_zero_point, np.float32)
    bdt = np.uint16 if dst_f16 else np.float32
    bi = None if bias is None else padded(bias, bdt)
    out = np.empty((ns, tokens, 4), bdt)
    lib().mldo_dequantize(tokens, n, k, _p(acc), _p(pr), _p(ws), _p(sc), _p(zp), _p(bi),
                          int(dst_f16), _p(out))
    return out


def dequantize_weights(weights, n, k, weight_bits, scale_bits, scale_kind=SCALE_LINEAR, groups=1,
                       zero_point_bits=None):
    w = _c(weights, np.uint8)
    sc = _c(scale_bits, np.uint16)
    zp = None if zero_point_bits is None else _c(zero_point_bits, np.uint16)
    out = np.empty((n, k), np.uint16)
    lib().mldo_dequantize_weights(n, k, weight_bits, _p(w), scale_kind, groups, _p(sc), _p(zp),
                                  _p(out))
    return out


# ---- gated MLP step (samples/llm/gemma3_model_builder.cc:1054-1075, qwen3_model_builder.cc:850-863) ----
def gated_activation(gate_f16, up_f16, kind):
    """The sample's elementwise kernels on fp16 tensors, in fp32, in their operation order.
    kind: "gelu_tanh" or "silu".  Returns fp16.  (tanh / exp are numpy's float32 routines: the
    result is pinned up to the accuracy of those, a few ulp of fp32.)"""
    g = np.asarray(gate_f16, np.float16).astype(np.float32)
    u = np.asarray(up_f16, np.float16).astype(np.float32)
    f32 = np.float32
    if kind == "gelu_tanh":
        gate_sq = g * g
        tanh_in = g * (f32(0.7978845608) + f32(0.03567740813) * gate_sq)
        clamped = np.clip(tanh_in, f32(-10.0), f32(10.0))
        tanh_val = np.tanh(clamped).astype(np.float32)
        gate_up_half = f32(0.5) * g * u
        res = np.clip(gate_up_half * (f32(1.0) + tanh_val), f32(-65504.0), f32(65504.0))
    elif kind == "silu":
        with np.errstate(over="ignore"):  # exp(-g) = inf for very negative g: sig = 0, as on the device
            sig = f32(1.0) / (f32(1.0) + np.exp(-g).astype(np.float32))
        res = np.clip((g * sig) * u, f32(-65504.0), f32(65504.0))
    else:
        raise ValueError(kind)
    return res.astype(np.float16)
