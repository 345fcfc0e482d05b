"""CPU restatement of the LLM sample's checkpoint files and their loader (TEST INFRASTRUCTURE
ONLY: tests import it, the product never does).

Writer side, samples/llm/extract_weights_hf.py (read as text, not imported):
  quantize_int8_sym   :137-164, the `optimize_scale=False` branch (scale = absmax / 127,
                      np.round = half to even, clip to [-128, 127], zero rows get scale 1)
  quantize_int4_sym   :167-229, the `optimize_scale=False` branches, channel-wise and block-wise
                      (scale = absmax / 7, clip to [-8, 7])
  pack_int4           :232-241 (low nibble = even element)
  optimize_scale_search :78-134, the grid search of the `optimize_scale=True` branches (the extractor's
                      default): per block / channel, of the candidate scales absmax * alpha / qmax
                      (alpha = linspace(1.0, 0.5, 7) for int4, linspace(1.0, 0.7, 7) for int8, float32),
                      the first one that minimises the mean squared reconstruction error
  quantize_int8_sym / quantize_int4_sym take `optimize_scale=True` for those branches (:148-159, :188-201,
                      :211-219)
Pinned by: the closed forms themselves are checked in tests/test_checkpoint.py through what the
mathematics fixes (|w - q*s| <= s/2 away from the clip, q = +-7 / +-127 at the extreme of every
row, scale 1 for zero rows, round-half-even on exact ties, nibble order against a hand-written
byte string).  The grid search: the chosen scale is one of the seven candidates and no candidate
reconstructs the block with a smaller mean squared error (checked in float64, block by block, by
plain loops), ties go to the larger alpha, a block whose extreme is an outlier takes a smaller scale
than absmax / qmax and clips the outlier, a block of evenly spread values keeps alpha = 1 where the
closed form is optimal, zero blocks get scale 1 and codes 0.  Not checked against the extractor's
output bit for bit (it is not run here): the last-place rounding of the float32 error sums could
break a near-tie differently; parity for such near-ties is unpinned.

Loader side, samples/llm/llm_file_tensor_loader.cc:
  group_size          :399-452 GetQuantizationIGroupSize
  load_scale_or_zp    :54-148 (raw fp32, or int32 header + int8 / int16 values / 1024)
  load_fc             :262-302, :350-395, :454-496 and llm_weights_loader.cc:29-117: packed weights
                      (through the oracle's packers, pinned by the reference's golden vectors),
                      scale tensor, zero point = file / scale, weights_sum_i
Pinned by: hand-computed files in tests/test_checkpoint.py (sizes that select each format,
headers, the 1/1024 factor, the zero-scale rule).
"""
import os

import numpy as np

from . import oracle as O


# ---- writer side -------------------------------------------------------------------------
def optimize_scale_search(blocks, bound, scale_bound, min_q, max_q, alphas):
    """_optimize_scale_search (samples/llm/extract_weights_hf.py:78-134) without its chunking (which
    only bounds memory): blocks (N, D), bound (N, 1) = max |block| -> (int8 codes (N, D), float32 scales
    (N, 1)).  Candidate scales bound * alpha / scale_bound (zero -> 1), codes clip(round(x / scale)),
    error = mean over the block of (x - code * scale)^2, argmin over the candidates (first on ties), all
    in the arrays' own float type as numpy evaluates the reference's expressions."""
    blocks = np.asarray(blocks)
    cand = (bound[:, None, :] * alphas[None, :, None]) / scale_bound
    cand = np.where(cand == 0.0, 1.0, cand)
    cq = np.clip(np.round(blocks[:, None, :] / cand), min_q, max_q)
    err = np.mean((blocks[:, None, :] - cq * cand) ** 2, axis=-1)
    best = np.argmin(err, axis=1)
    scales = np.take_along_axis(cand[:, :, 0], best[:, None], axis=1).astype(np.float32)
    q = np.take_along_axis(cq, best[:, None, None], axis=1)[:, 0, :].astype(np.int8)
    return q, scales


def quantize_int8_sym(w, optimize_scale=False):
    """w: (o, i) float -> (int8 (o, i), float32 scale (o,))."""
    w = np.asarray(w)
    if optimize_scale:
        bound = np.max(np.abs(w), axis=-1, keepdims=True)
        q, scale = optimize_scale_search(w, bound, 127.0, -128, 127, np.linspace(1.0, 0.7, num=7, dtype=np.float32))
        return q, scale.reshape(-1).astype(np.float32)
    bound = np.max(np.abs(w), axis=1, keepdims=True)
    scale = bound / 127.0
    scale = np.where(scale == 0.0, 1.0, scale)
    q = np.clip(np.round(w / scale), -128, 127).astype(np.int8)
    return q, np.squeeze(scale, axis=1).astype(np.float32)


def quantize_int4_sym(w, block_size=0, optimize_scale=False):
    """w: (o, i) float -> (int8-held int4 (o, i), float32 scale (o,) or (o, i / block_size))."""
    w = np.asarray(w)
    if optimize_scale:
        o, i = w.shape
        if block_size > 0 and i % block_size:
            raise ValueError("not divisible by block_size")
        blocks = w.reshape(-1, block_size) if block_size > 0 else w
        bound = np.max(np.abs(blocks), axis=-1, keepdims=True)
        q, scale = optimize_scale_search(blocks, bound, 7.0, -8, 7, np.linspace(1.0, 0.5, num=7, dtype=np.float32))
        return q.reshape(o, i), (scale.reshape(o, i // block_size) if block_size > 0 else scale.reshape(o)).astype(np.float32)
    if block_size > 0:
        o, i = w.shape
        if i % block_size:
            raise ValueError("not divisible by block_size")
        r = w.reshape(o, i // block_size, block_size)
        bound = np.max(np.abs(r), axis=2, keepdims=True)
        scale = bound / 7.0
        scale = np.where(scale == 0.0, 1.0, scale)
        q = np.clip(np.round(r / scale), -8, 7).astype(np.int8).reshape(o, i)
        return q, np.squeeze(scale, axis=2).astype(np.float32)
    bound = np.max(np.abs(w), axis=1, keepdims=True)
    scale = bound / 7.0
    scale = np.where(scale == 0.0, 1.0, scale)
    q = np.clip(np.round(w / scale), -8, 7).astype(np.int8)
    return q, np.squeeze(scale, axis=1).astype(np.float32)


def pack_int4(q):
    flat = np.asarray(q).ravel().astype(np.uint8)
    if flat.size % 2:
        raise ValueError("odd number of elements")
    return (flat[0::2] & 0x0F) | ((flat[1::2] & 0x0F) << 4)


def write_scale_file(path, values, fmt="f32", group_size=0):
    """values: (o, scale_i).  fmt f32: raw float32; i8 / i16: int32 header (group size) followed
    by round(value * 1024) as int8 / int16 (the format llm_file_tensor_loader.cc:54-97 reads)."""
    v = np.ascontiguousarray(values, np.float32)
    with open(path, "wb") as f:
        if fmt == "f32":
            v.tofile(f)
        else:
            np.array([group_size], np.int32).tofile(f)
            np.round(v * 1024.0).astype(np.int8 if fmt == "i8" else np.int16).tofile(f)


def write_fc_files(directory, base, q, scale, bits, zero_point=None, scale_fmt="f32", group_size=0,
                   swap_dims=False):
    """Writes `<base>.weight`, `<base>.weight_quantized_scale` [, `<base>.weight_quantized_zp`]."""
    q = np.asarray(q, np.int8)
    stored = np.ascontiguousarray(q.T) if swap_dims else q
    data = pack_int4(stored) if bits == 4 else stored
    with open(os.path.join(directory, base + ".weight"), "wb") as f:
        data.tofile(f)
    s = np.asarray(scale, np.float32)
    write_scale_file(os.path.join(directory, base + ".weight_quantized_scale"), s.reshape(q.shape[0], -1),
                     scale_fmt, group_size)
    if zero_point is not None:
        write_scale_file(os.path.join(directory, base + ".weight_quantized_zp"),
                         np.asarray(zero_point, np.float32).reshape(q.shape[0], -1), scale_fmt, group_size)


# ---- loader side -------------------------------------------------------------------------
def group_size(scale_path, o, i):
    if not os.path.exists(scale_path):
        return i
    size = os.path.getsize(scale_path)
    if size < 4:
        return i
    if size % 4 == 0:
        elements = size // 4
        if elements > 0 and elements % o == 0:
            scale_i = elements // o
            if i % scale_i == 0:
                return i // scale_i
    header = int(np.fromfile(scale_path, np.int32, 1)[0])
    if 0 < header <= i and i % header == 0:
        elements = o * (i // header)
        if size in (4 + elements, 4 + 2 * elements):
            return header
    return i


def _read_prefix(path, dtype, count, offset=0):
    out = np.zeros(count, dtype)
    got = np.fromfile(path, dtype, count, offset=offset)
    out[:got.size] = got
    return out


def load_scale_or_zp(path, o, scale_i):
    count = o * scale_i
    size = os.path.getsize(path)
    grouped = False
    if size >= 4:
        header = int(np.fromfile(path, np.int32, 1)[0])
        grouped = 0 < header < 65536 and (size - 4) in (count, 2 * count)
    if not grouped:
        return _read_prefix(path, np.float32, count).reshape(o, scale_i)
    per = (size - 4) // count
    raw = _read_prefix(path, np.int8 if per == 1 else np.int16, count, offset=4)
    return (raw.astype(np.float32) / np.float32(1024.0)).reshape(o, scale_i)


def load_fc(directory, base, o, i, bits, tensor_dtype, swap_dims=False, output_group=None):
    """-> dict(group_size, scale_i, weights, scale, zero_point, weights_sum_i): what the FC op binds.
    `output_group`: output_group_size of the WeightsDescription the loader is handed (the reference
    passes the FullyConnected's own description, llm_weights_loader.cc:29-71); default one group."""
    w_path = os.path.join(directory, base + ".weight")
    s_path = os.path.join(directory, base + ".weight_quantized_scale")
    z_path = os.path.join(directory, base + ".weight_quantized_zp")
    g = group_size(s_path, o, i)
    scale_i = i // g
    ns = O.div_up(o, 4)
    if bits == 4:
        raw = _read_prefix(w_path, np.uint8, o * i // 2)
        weights, sums = O.uint4_packed(raw, (o, 1, 1, i), O.LAYOUT_I4O4, output_group or ns, pad=8,
                                       swap_dims=swap_dims)
    else:
        raw = _read_prefix(w_path, np.int8, o * i)
        q = raw.reshape(i, o).T if swap_dims else raw.reshape(o, i)
        q = np.ascontiguousarray(q)
        weights = O.int8_as_uint8(q, O.LAYOUT_I4O4, ns, 128, 128)
        sums = O.weights_sum_i(q)

    def tensor(v):
        t = O.scale_to_hoio4(v).reshape(-1) if scale_i > 1 else np.pad(v[:, 0], (0, ns * 4 - o))
        return t.astype(tensor_dtype)
    s = load_scale_or_zp(s_path, o, scale_i)
    out = dict(group_size=g, scale_i=scale_i, weights=weights, weights_sum_i=sums, scale=tensor(s),
               scale_f32=s, zero_point=None, zero_point_f32=None)
    if os.path.exists(z_path):
        z = load_scale_or_zp(z_path, o, scale_i)
        with np.errstate(divide="ignore", invalid="ignore"):
            z = np.where(s == 0.0, np.float32(0.0), z / s).astype(np.float32)
        out.update(zero_point=tensor(z), zero_point_f32=z)
    return out
