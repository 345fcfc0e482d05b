"""Product packers (host code of libmldhip.so) against the oracle, bit for bit, and against
the reference's literal golden vectors (common/task/weights_conversion_test.cc:50-479)."""
import numpy as np
import pytest

import mldhip as M


def pack_nibbles(vals):
    vals = np.asarray(vals, np.uint8)
    return (vals[0::2] | (vals[1::2] << 4)).astype(np.uint8)


def counting(n_bytes=8):
    return np.array([(((2 * i + 1) << 4) | (2 * i)) & 0xFF for i in range(n_bytes)], np.uint8)


BASE = pack_nibbles([0, 4, 8, 12, 1, 5, 9, 13, 2, 6, 10, 14, 3, 7, 11, 15]) ^ 0x88


@pytest.mark.parametrize("layout", [M.LAYOUT_I4O4, M.LAYOUT_2D_I4O4])
def test_golden_base_and_stale_sums(layout):
    d = M.make_desc(M.UINT8, layout, 1)
    out, sums = M.rearrange_uint4_packed(counting(), (4, 1, 1, 4), d, sum_init=[1, 0, 0, 0])
    assert out.tolist() == BASE.tolist() and sums.tolist() == [6, 22, -26, -10]


@pytest.mark.parametrize("layout", [M.LAYOUT_I4O4, M.LAYOUT_2D_I4O4])
def test_golden_pad(layout):
    d = M.make_desc(M.UINT8, layout, 1)
    expected = pack_nibbles([0, 4, 8, 0, 1, 5, 9, 0, 2, 6, 10, 0, 3, 7, 11, 0]) ^ 0x88
    out, sums = M.rearrange_uint4_packed(counting(6), (3, 1, 1, 4), d, sum_len=4)
    assert out.tolist() == expected.tolist() and sums.tolist() == [6, 22, -26, 0]


def test_golden_double_pad_and_swap_dims():
    d2 = M.make_desc(M.UINT8, M.LAYOUT_2D_I4O4, 1)
    expected = pack_nibbles([0, 2, 4, 6, 1, 3, 5, 7] + [0] * 8) ^ 0x88
    out, sums = M.rearrange_uint4_packed(counting(4), (4, 1, 1, 2), d2)
    assert out.tolist() == expected.tolist() and sums.tolist() == [1, 5, 9, 13]
    d1 = M.make_desc(M.UINT8, M.LAYOUT_I4O4, 1)
    expected = np.array([((2 * i) | ((2 * i + 1) << 4)) ^ 0x88 for i in range(8)], np.uint8)
    out, sums = M.rearrange_uint4_packed(counting(), (4, 1, 1, 4), d1, swap_dims=True)
    assert out.tolist() == expected.tolist() and sums.tolist() == [-8, -4, 0, 4]


SHAPES = [(4, 1, 1, 4), (3, 1, 1, 5), (171, 1, 1, 533), (533, 1, 1, 171), (39, 2, 3, 23),
          (256, 1, 1, 512), (16, 2, 1, 8)]


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("layout", [M.LAYOUT_I4O4, M.LAYOUT_O4I4, M.LAYOUT_2D_I4O4])
@pytest.mark.parametrize("group", [1, 2, 4, None])
def test_packers_match_oracle(oracle, shape, layout, group):
    o, h, w, i = shape
    g = (o + 3) // 4 if group is None else group
    rng = np.random.default_rng(o * 31 + i + g)
    w8 = rng.integers(-128, 128, size=shape, dtype=np.int8)
    w4 = rng.integers(-8, 8, size=shape, dtype=np.int8)
    d8 = M.make_desc(M.UINT8, layout, g)
    d4 = M.make_desc(M.UINT4, layout, g)
    assert M.total_elements(d8, o, h, w, i) == oracle.total_elements(layout, o, h, w, i, g)
    assert np.array_equal(M.rearrange_int8_as_uint8(w8, d8), oracle.int8_as_uint8(w8, layout, g))
    assert np.array_equal(M.rearrange_int8_as_uint4(w4, d4), oracle.int8_as_uint4(w4, layout, g))
    assert np.array_equal(M.rearrange_int8(w8, M.make_desc(M.INT8, layout, g)),
                          oracle.rearrange_i8(w8, layout, g))
    assert np.array_equal(M.weights_sum_i(w8), oracle.weights_sum_i(w8))
    if layout != M.LAYOUT_O4I4:
        flat = (w4.astype(np.int16).ravel() & 0xF).astype(np.uint8)
        if flat.size % 2:
            flat = np.append(flat, 0)
        packed_src = pack_nibbles(flat)
        for swap in (False, True):
            src = packed_src
            if swap:
                t = np.ascontiguousarray(w4.transpose(3, 1, 2, 0))
                flat_t = (t.astype(np.int16).ravel() & 0xF).astype(np.uint8)
                if flat_t.size % 2:
                    flat_t = np.append(flat_t, 0)
                src = pack_nibbles(flat_t)
            got, gs = M.rearrange_uint4_packed(src, shape, d4, swap_dims=swap, sum_len=o + 3,
                                               sum_init=np.full(o + 3, 7))
            ref, rs = oracle.uint4_packed(src, shape, layout, g, swap_dims=swap, sum_len=o + 3,
                                          sum_init=np.full(o + 3, 7))
            assert np.array_equal(got, ref)
            assert np.array_equal(gs, rs)
            assert np.array_equal(got, oracle.int8_as_uint4(w4, layout, g))
            assert np.array_equal(gs[:o], w4.astype(np.int64).sum(axis=(1, 2, 3)))


def test_custom_groups_match_oracle(oracle):
    rng = np.random.default_rng(8)
    w = rng.integers(-128, 128, size=(39, 2, 3, 23), dtype=np.int8)
    O, H, W, I = M.AXIS_O, M.AXIS_H, M.AXIS_W, M.AXIS_I
    for groups in ([(O, 4), (I, 4), (O, 4), (I, 0), (W, 0), (H, 0), (O, 0)],
                   [(I, 4), (O, 4), (O, 4), (I, 0), (W, 0), (H, 0), (O, 0)],
                   [(I, 16), (O, 0), (I, 0), (W, 0), (H, 0)]):
        d = M.make_desc(M.INT8, M.LAYOUT_CUSTOM, 1, custom=groups)
        assert np.array_equal(M.rearrange_int8(w, d), oracle.rearrange_custom_i8(w, groups))


def test_conv_int8_layout_closed_form():
    # [ceil(i/16)][o][16], zero padded
    rng = np.random.default_rng(9)
    n, k = 37, 40
    w = rng.integers(-127, 128, size=(n, k), dtype=np.int8)
    got = M.rearrange_int8(w, M.conv_int8_weights_desc(n, k)).reshape(3, n, 16)
    full = np.zeros((n, 48), np.int8)
    full[:, :k] = w
    assert np.array_equal(got, full.reshape(n, 3, 16).transpose(1, 0, 2))


def test_scale_tensor_matches_oracle(oracle):
    rng = np.random.default_rng(10)
    s = (np.abs(rng.standard_normal((533, 7))) * 0.01).astype(np.float32)
    got32 = M.scale_to_tensor(s, M.FLOAT32)
    assert np.array_equal(got32.reshape(7, 134, 4), oracle.scale_to_hoio4(s))
    got16 = M.scale_to_tensor(s, M.FLOAT16)
    assert np.array_equal(got16, oracle.f32_to_f16_bits(oracle.scale_to_hoio4(s)).ravel())
    lin = M.scale_to_tensor(s[:, 0], M.FLOAT16)
    assert lin.size == 536 and np.array_equal(lin[:533], s[:, 0].astype(np.float16).view(np.uint16))
    assert np.all(lin[533:] == 0)


@pytest.mark.parametrize("o,i,group", [(64, 32, 16), (128, 64, 4), (14336, 64, 16), (192, 36, 8), (4096, 32, 8),
                                       (192, 36, 16)])
def test_int4_library_layout_matches_oracle(oracle, o, i, group):
    """The layouts mldhip_fc_int4_weights_desc asks for (kOSpatialIOGroupI4O4 in output groups of 16,
    8 or 4 slices): the product packers against the oracle's restatement of the reference's packer
    for the same description, from int8-held values and from nibble-packed input, and against the
    closed form block index ((slice / G) * Ks + ks) * G + slice % G."""
    rng = np.random.default_rng(o + i)
    w = rng.integers(-8, 8, size=(o, i), dtype=np.int8)
    with M.tuning(fc_group=group):
        desc = M.fc_int4_weights_desc(o, i)
    assert desc.output_group_size == group
    got = M.rearrange_int8_as_uint4(w, desc)
    ref = oracle.int8_as_uint4(w, oracle.LAYOUT_I4O4, group)
    assert np.array_equal(got, ref)
    nib = ((w[:, 0::2] & 0xF) | ((w[:, 1::2] & 0xF) << 4)).astype(np.uint8)  # two's complement, low nibble first
    got2, sums = M.rearrange_uint4_packed(nib, (o, 1, 1, i), desc)
    ref2, ref_sums = oracle.uint4_packed(nib, (o, 1, 1, i), oracle.LAYOUT_I4O4, group)
    assert np.array_equal(got2, ref2) and np.array_equal(got2, got)
    assert np.array_equal(sums, ref_sums) and np.array_equal(sums, w.astype(np.int64).sum(axis=1))
    # closed form: block (ks, slice) holds element (ii, oo) in nibble ii * 4 + oo
    ks_n, ns = (i + 3) // 4, o // 4
    blocks = got.reshape(-1, 8)
    for ks in (0, ks_n - 1):
        for sl in sorted({0, group - 1, min(group, ns - 1), ns - 1}):
            blk = blocks[((sl // group) * ks_n + ks) * group + sl % group]
            for ii in range(4):
                for oo in range(4):
                    e = ii * 4 + oo
                    nibble = (blk[e // 2] >> (4 * (e & 1))) & 0xF
                    ic = ks * 4 + ii
                    want = (int(w[sl * 4 + oo, ic]) + 8) if ic < i else 8
                    assert nibble == want
