"""Checkpoint files of the LLM sample: the extractor's closed-form quantizers (oracle only), the
oracle's restatement of the loader against hand-made files, and the C-ABI loader
(mldhip_checkpoint_fc_probe / _read) against the oracle, byte for byte.  CPU only."""
import os
import struct

import numpy as np
import pytest

import mldhip as M
from oracle import checkpoint as CK


# ---- the writer's closed forms (samples/llm/extract_weights_hf.py:137-241) ----
def test_pack_int4_nibble_order():
    q = np.array([1, -1, 7, -8, 0, 3], np.int8)
    assert CK.pack_int4(q).tobytes() == bytes([0xF1, 0x87, 0x30])
    with pytest.raises(ValueError):
        CK.pack_int4(np.zeros(3, np.int8))


@pytest.mark.parametrize("block", [0, 32])
def test_quantize_int4_closed_form(block):
    rng = np.random.default_rng(3)
    w = rng.standard_normal((12, 64)).astype(np.float32)
    w[5] = 0.0
    q, s = CK.quantize_int4_sym(w, block)
    assert q.dtype == np.int8 and q.min() >= -8 and q.max() <= 7
    sf = s.reshape(12, -1)
    groups = sf.shape[1]
    wr = w.reshape(12, groups, -1)
    qr = q.reshape(12, groups, -1)
    assert np.array_equal(sf, np.where(np.abs(wr).max(axis=2) == 0, 1.0, np.abs(wr).max(axis=2) / 7.0).astype(np.float32))
    assert np.all(sf[5] == 1.0) and np.all(q[5] == 0)
    # the extreme of every group maps to +-7, everything is within half a step
    assert np.all(np.abs(qr).max(axis=2)[np.abs(wr).max(axis=2) > 0] == 7)
    assert np.all(np.abs(wr - qr * sf[:, :, None]) <= sf[:, :, None] * 0.5 + 1e-6)


def test_quantize_rounds_half_to_even():
    # scale = 7/7 = 1: the values 0.5, 1.5, 2.5, -0.5, -2.5 are exact ties
    w = np.array([[7.0, 0.5, 1.5, 2.5, -0.5, -2.5, 6.5, -7.0]], np.float32)
    q, s = CK.quantize_int4_sym(w)
    assert s[0] == 1.0
    assert q.tolist() == [[7, 0, 2, 2, 0, -2, 6, -7]]
    w8 = np.array([[127.0, 0.5, 1.5, -126.5, 126.5]], np.float32)
    q8, s8 = CK.quantize_int8_sym(w8)
    assert s8[0] == 1.0 and q8.tolist() == [[127, 0, 2, -126, 126]]


# ---- the loader's file formats (samples/llm/llm_file_tensor_loader.cc:54-148, 399-452) ----
def test_group_size_rules(tmp_path):
    d = str(tmp_path)
    p = os.path.join(d, "s")
    o, i = 8, 64
    assert CK.group_size(p, o, i) == i                       # no file
    open(p, "wb").write(b"\x00\x00")
    assert CK.group_size(p, o, i) == i                       # shorter than a header
    np.zeros(o, np.float32).tofile(p)
    assert CK.group_size(p, o, i) == i                       # raw fp32, one scale per channel
    np.zeros(o * 4, np.float32).tofile(p)
    assert CK.group_size(p, o, i) == 16                      # raw fp32, 4 scales per channel
    np.zeros(o * 3, np.float32).tofile(p)
    assert CK.group_size(p, o, i) == i                       # 64 % 3 != 0 and no valid header
    open(p, "wb").write(struct.pack("<i", 32) + bytes(o * 2))
    assert CK.group_size(p, o, i) == 32                      # header + int8 (4 + 16 bytes: 20 % 4 == 0 but 5 % 8 != 0)
    open(p, "wb").write(struct.pack("<i", 32) + bytes(o * 2 * 2))
    assert CK.group_size(p, o, i) == 32                      # header + int16
    open(p, "wb").write(struct.pack("<i", 48) + bytes(o * 2))
    assert CK.group_size(p, o, i) == i                       # 64 % 48 != 0


def test_load_scale_formats(tmp_path):
    p = str(tmp_path / "s")
    vals = np.array([[0.5, -0.25], [0.125, 0.0]], np.float32)
    vals.tofile(p)
    assert np.array_equal(CK.load_scale_or_zp(p, 2, 2), vals)
    open(p, "wb").write(struct.pack("<i", 16) + np.array([64, -32, 127, -128], np.int8).tobytes())
    assert np.array_equal(CK.load_scale_or_zp(p, 2, 2), np.array([[0.0625, -0.03125], [127 / 1024, -0.125]], np.float32))
    open(p, "wb").write(struct.pack("<i", 16) + np.array([1024, -3, 32767, 0], np.int16).tobytes())
    assert np.array_equal(CK.load_scale_or_zp(p, 2, 2), np.array([[1.0, -3 / 1024], [32767 / 1024, 0.0]], np.float32))
    # a short raw file reads as zeros beyond its end
    np.array([2.0], np.float32).tofile(p)
    assert np.array_equal(CK.load_scale_or_zp(p, 2, 1), np.array([[2.0], [0.0]], np.float32))


# ---- the C-ABI loader against the oracle ----
def _make(tmp_path, o, i, bits, block, zp, fmt, swap, seed=0):
    rng = np.random.default_rng(seed)
    w = (rng.standard_normal((o, i)) * 0.05).astype(np.float32)
    q, s = (CK.quantize_int4_sym(w, block) if bits == 4 else CK.quantize_int8_sym(w))
    s = s.reshape(o, -1)
    if fmt != "f32":
        s = np.maximum(np.round(s * 1024.0), 1.0) / 1024.0   # representable in the integer formats
    z = None
    if zp:
        z = (rng.integers(-3, 4, size=s.shape) * s).astype(np.float32)
        z[0, 0] = 0.0
    d = str(tmp_path) + os.sep
    gs = block if block else i
    CK.write_fc_files(d, "layer", q, s, bits, zero_point=z, scale_fmt=fmt, group_size=gs, swap_dims=swap)
    return d, q, s.astype(np.float32), z


@pytest.mark.parametrize("o,i,bits,block,zp,fmt,swap", [
    (16, 64, 4, 0, False, "f32", False),
    (16, 64, 4, 32, False, "f32", False),
    (20, 96, 4, 32, True, "f32", False),
    (7, 40, 4, 0, False, "f32", True),
    (533, 176, 4, 16, True, "i16", False),
    (16, 64, 8, 0, False, "f32", False),
    (12, 72, 8, 0, True, "f32", True),
    (24, 128, 4, 64, False, "i8", False),
    (128, 64, 4, 32, True, "f32", False),   # two output groups of 16 slices
    (192, 96, 4, 0, False, "f32", True),
])
@pytest.mark.parametrize("tensor_type", [M.FLOAT16, M.FLOAT32])
def test_loader_matches_oracle(oracle, tmp_path, o, i, bits, block, zp, fmt, swap, tensor_type):
    d, q, s, z = _make(tmp_path, o, i, bits, block, zp, fmt, swap, seed=o + i)
    info = M.checkpoint_fc_probe(d, "layer.weight", "layer", o, i, bits)
    td = np.float16 if tensor_type == M.FLOAT16 else np.float32
    ref = CK.load_fc(d, "layer", o, i, bits, td, swap_dims=swap, output_group=info.weights.output_group_size)
    assert info.group_size == ref["group_size"] == (block if block else i)
    assert info.scale_i == ref["scale_i"]
    assert bool(info.has_zero_point) == zp
    got = M.checkpoint_fc_read(d, "layer.weight", "layer", info, tensor_type, swap_dims=swap)
    assert got["weights"].tobytes() == ref["weights"].tobytes()
    assert np.array_equal(got["weights_sum_i"], ref["weights_sum_i"])
    assert np.array_equal(got["weights_sum_i"], q.astype(np.int64).sum(axis=1))
    assert got["scale"].tobytes() == ref["scale"].tobytes()
    if zp:
        assert got["zero_point"].tobytes() == ref["zero_point"].tobytes()
        # file / scale gives back the integral zero points the files were made from
        assert np.allclose(ref["zero_point_f32"], np.round(ref["zero_point_f32"]), atol=1e-3)
    else:
        assert got["zero_point"] is None
    # the packed weights are what the packers give for the quantized values themselves
    desc = M.fc_int4_weights_desc(o, i) if bits == 4 else M.fc_int8_weights_desc(o, i)
    direct = (M.rearrange_int8_as_uint4 if bits == 4 else M.rearrange_int8_as_uint8)(q, desc)
    assert got["weights"].tobytes() == direct.tobytes()


def test_loader_errors(tmp_path):
    d = str(tmp_path) + os.sep
    with pytest.raises(M.MldhipError) as e:
        M.checkpoint_fc_probe(d, "missing.weight", "missing", 8, 32, 4)
    assert e.value.code == M.NOT_FOUND and "Failed to load weights" in e.value.message
    with pytest.raises(M.MldhipError) as e:
        M.checkpoint_fc_probe(d, "x", "x", 8, 32, 2)
    assert e.value.code == M.INVALID_ARGUMENT
    # zero scale: the zero point becomes 0
    q = np.zeros((4, 8), np.int8)
    CK.write_fc_files(d, "z", q, np.array([0.0, 1.0, 2.0, 0.5], np.float32), 4,
                      zero_point=np.array([3.0, 3.0, 3.0, 3.0], np.float32))
    info = M.checkpoint_fc_probe(d, "z.weight", "z", 4, 8, 4)
    got = M.checkpoint_fc_read(d, "z.weight", "z", info, M.FLOAT32)
    assert got["zero_point"].tolist() == [0.0, 3.0, 1.5, 6.0]


# ---- the extractor's scale search (samples/llm/extract_weights_hf.py:78-134) -------------------------
def _mse(block, scale, lo, hi):
    """float64, plain loop: mean squared error of the block quantized with `scale`."""
    total = 0.0
    for x in block:
        q = min(max(float(np.round(np.float64(x) / scale)), lo), hi)
        total += (float(x) - q * scale) ** 2
    return total / len(block)


@pytest.mark.parametrize("bits,block", [(4, 32), (4, 0), (8, 0)])
def test_scale_search_picks_the_best_candidate(bits, block):
    """The chosen scale is one of the seven candidates absmax * alpha / qmax and no candidate gives a
    smaller mean squared error (float64, block by block); the codes are the rounding with that scale."""
    rng = np.random.default_rng(bits + block)
    o, i = 12, 64
    w = rng.standard_normal((o, i)).astype(np.float32)
    w[3, 5] = 9.0      # an outlier: a smaller scale that clips it wins
    w[7] = 0.0         # a zero row
    qmax, lo, hi = (7.0, -8, 7) if bits == 4 else (127.0, -128, 127)
    alphas = np.linspace(1.0, 0.5 if bits == 4 else 0.7, num=7, dtype=np.float32)
    if bits == 4:
        q, scale = CK.quantize_int4_sym(w, block, optimize_scale=True)
    else:
        q, scale = CK.quantize_int8_sym(w, optimize_scale=True)
    blocks = w.reshape(-1, block) if block else w
    qb = q.reshape(blocks.shape)
    sb = scale.reshape(-1)
    assert q.dtype == np.int8 and scale.dtype == np.float32 and q.shape == w.shape
    assert scale.shape == ((o, i // block) if block else (o,))
    for b in range(blocks.shape[0]):
        bound = float(np.max(np.abs(blocks[b])))
        if bound == 0.0:
            assert sb[b] == 1.0 and not qb[b].any()
            continue
        cands = [float(np.float32(np.float32(bound) * a) / np.float32(qmax)) for a in alphas]
        assert any(abs(float(sb[b]) - c) <= 1e-7 * c for c in cands), (b, sb[b], cands)
        errs = [_mse(blocks[b], c, lo, hi) for c in cands]
        mine = _mse(blocks[b], float(sb[b]), lo, hi)
        assert mine <= min(errs) * (1 + 1e-5) + 1e-12, (b, mine, errs)
        want = np.clip(np.round(blocks[b] / sb[b]), lo, hi).astype(np.int8)
        assert np.array_equal(qb[b], want)
    if bits == 4 and block:
        # the outlier's block clips it: a scale below absmax / 7, the outlier at the top code
        k = 3 * (i // block) + 5 // block
        assert sb[k] < 9.0 / 7.0 * (1 - 1e-6) and q[3, 5] == 7


def test_scale_search_ties_and_spread_blocks():
    """A block that the largest scale reconstructs exactly keeps alpha = 1 (the first candidate wins a
    tie at zero error, and nothing beats zero); an evenly spread block of codes -7..7 times a scale s
    is reproduced with scale s."""
    s = np.float32(0.25)
    block = (np.arange(-7, 8, dtype=np.float32) * s)[None, :]
    q, scale = CK.quantize_int4_sym(np.concatenate([block, block[:, ::-1]], axis=1), 15, optimize_scale=True)
    assert np.allclose(scale, s) and np.array_equal(q[0, :15], np.arange(-7, 8))
    # the closed form is the alpha = 1 candidate
    q1, s1 = CK.quantize_int4_sym(block, 0, optimize_scale=False)
    q2, s2 = CK.quantize_int4_sym(block, 0, optimize_scale=True)
    assert np.array_equal(q1, q2) and np.allclose(s1, s2)


def test_scale_search_files_load_like_any_other(tmp_path):
    """Scales from the grid search are ordinary loader input: write, load, compare."""
    rng = np.random.default_rng(9)
    o, i, block = 16, 64, 32
    w = rng.standard_normal((o, i)).astype(np.float32)
    q, scale = CK.quantize_int4_sym(w, block, optimize_scale=True)
    d = str(tmp_path) + "/"
    CK.write_fc_files(d, "layer", q, scale, 4)
    got = CK.load_fc(d, "layer", o, i, 4, np.float32)
    assert got["group_size"] == block
