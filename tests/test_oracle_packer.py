"""Pins the oracle's weight packers against the golden vectors the reference's own tests
hold (common/task/weights_conversion_test.cc:50-479), against a second formulation, and
by brute force over every (o, i) on ragged shapes."""
import numpy as np
import pytest

I4O4, O4I4, TWO_D = 1, 2, 6


def pack_nibbles(vals):
    vals = np.asarray(vals, np.uint8)
    return (vals[0::2] | (vals[1::2] << 4)).astype(np.uint8)


def counting_4x4_packed(n_bytes=8):
    # weights_conversion_test.cc:54-58: byte i = ((2i+1) << 4) | 2i
    return np.array([(((2 * i + 1) << 4) | (2 * i)) & 0xFF for i in range(n_bytes)], np.uint8)


EXPECTED_BASE = pack_nibbles([0, 4, 8, 12, 1, 5, 9, 13, 2, 6, 10, 14, 3, 7, 11, 15]) ^ 0x88


@pytest.mark.parametrize("layout", [I4O4, TWO_D])
def test_uint4_packed_base(oracle, layout):
    # :50-91 and :264-305
    out, sums = oracle.uint4_packed(counting_4x4_packed(), (4, 1, 1, 4), layout, 1)
    assert out.tolist() == EXPECTED_BASE.tolist()
    assert sums.tolist() == [6, 22, -26, -10]


@pytest.mark.parametrize("layout", [I4O4, TWO_D])
def test_uint4_packed_zeroes_sums(oracle, layout):
    # :93-179: a stale value in weights_sum_i[0] is cleared
    out, sums = oracle.uint4_packed(counting_4x4_packed(), (4, 1, 1, 4), layout, 1,
                                    sum_init=[1, 0, 0, 0])
    assert out.tolist() == EXPECTED_BASE.tolist()
    assert sums.tolist() == [6, 22, -26, -10]


@pytest.mark.parametrize("layout", [I4O4, TWO_D])
def test_uint4_packed_pad_output_channels(oracle, layout):
    # :307-393: O=3, pad nibble (8 ^ 8 = 0) then ^0x88; the padded sum stays 0
    pad = 8 ^ 8
    expected = pack_nibbles([0, 4, 8, pad, 1, 5, 9, pad, 2, 6, 10, pad, 3, 7, 11, pad]) ^ 0x88
    out, sums = oracle.uint4_packed(counting_4x4_packed(6), (3, 1, 1, 4), layout, 1, sum_len=4)
    assert out.tolist() == expected.tolist()
    assert sums.tolist() == [6, 22, -26, 0]


def test_uint4_packed_double_pad(oracle):
    # :395-438: I=2, missing input channels become 0x88 bytes
    pad = 8 ^ 8
    expected = pack_nibbles([0, 2, 4, 6, 1, 3, 5, 7] + [pad] * 8) ^ 0x88
    out, sums = oracle.uint4_packed(counting_4x4_packed(4), (4, 1, 1, 2), TWO_D, 1)
    assert out.tolist() == expected.tolist()
    assert sums.tolist() == [1, 5, 9, 13]


def test_uint4_packed_swap_dims(oracle):
    # :440-479: input is IHWO, so the transpose cancels
    expected = np.array([((2 * i) | ((2 * i + 1) << 4)) ^ 0x88 for i in range(8)], np.uint8)
    out, sums = oracle.uint4_packed(counting_4x4_packed(), (4, 1, 1, 4), I4O4, 1, swap_dims=True)
    assert out.tolist() == expected.tolist()
    assert sums.tolist() == [-8, -4, 0, 4]


def test_uint4_packed_unsupported_layout(oracle):
    with pytest.raises(NotImplementedError):
        oracle.uint4_packed(counting_4x4_packed(), (4, 1, 1, 4), O4I4, 1)


def twos_complement_pack(w_i8):
    flat = (np.asarray(w_i8, np.int16).ravel() & 0xF).astype(np.uint8)
    return pack_nibbles(flat)


def test_packed_path_equals_int8_path_4x4(oracle):
    # :183-219
    w = np.arange(-8, 8, dtype=np.int8).reshape(4, 4)
    out, sums = oracle.uint4_packed(twos_complement_pack(w), (4, 1, 1, 4), I4O4, 1)
    ref = oracle.int8_as_uint4(w, I4O4, 1)
    assert out.tolist() == ref.tolist()
    assert sums.tolist() == oracle.weights_sum_i(w).tolist()


def test_packed_path_equals_int8_path_2d_group2(oracle):
    # :221-262: OHWI(16,2,1,8), output_group_size 2
    w = ((np.arange(16 * 2 * 1 * 8) % 16) - 8).astype(np.int8).reshape(16, 2, 1, 8)
    out, sums = oracle.uint4_packed(twos_complement_pack(w), (16, 2, 1, 8), TWO_D, 2)
    ref = oracle.int8_as_uint4(w, TWO_D, 2)
    assert out.tolist() == ref.tolist()
    assert sums.tolist() == oracle.weights_sum_i(w).tolist()


SHAPES = [(4, 1, 1, 4), (3, 1, 1, 5), (171, 1, 1, 533), (533, 1, 1, 171), (39, 2, 3, 23),
          (64, 1, 1, 128), (8, 1, 1, 4)]


@pytest.mark.parametrize("shape", SHAPES)
@pytest.mark.parametrize("layout", [I4O4, O4I4, TWO_D])
@pytest.mark.parametrize("group", [1, 2, 4, None])
def test_loop_and_transpose_formulations_agree(oracle, shape, layout, group):
    o, h, w, i = shape
    g = (o + 3) // 4 if group is None else group
    rng = np.random.default_rng(o * 1000 + i)
    src = rng.integers(0, 256, size=shape, dtype=np.uint8)
    a = oracle.rearrange_u8(src, layout, g, 77)
    b = oracle.rearrange_u8(src, layout, g, 77, reshape_path=True)
    assert a.size == oracle.total_elements(layout, o, h, w, i, g)
    assert np.array_equal(a, b)


@pytest.mark.parametrize("n,k", [(4, 4), (3, 5), (533, 171), (171, 533), (64, 96), (5, 3)])
@pytest.mark.parametrize("bits", [4, 8])
def test_fc_layout_brute_force(oracle, n, k, bits):
    """Every (o, i): reading the packed buffer with the kernel's block/nibble order
    (block = i_slice * Ns + o_slice, element i%4*4 + o%4, low nibble first) returns w + shift;
    padding elements hold the shift (a zero weight)."""
    rng = np.random.default_rng(n * 7 + k)
    ns, ks = (n + 3) // 4, (k + 3) // 4
    if bits == 4:
        w = rng.integers(-8, 8, size=(n, k), dtype=np.int8)
        packed = oracle.int8_as_uint4(w, I4O4, ns)
        elems = np.stack([packed & 0xF, packed >> 4], axis=1).ravel()
        shift = 8
    else:
        w = rng.integers(-128, 128, size=(n, k), dtype=np.int8)
        elems = oracle.int8_as_uint8(w, I4O4, ns)
        shift = 128
    assert elems.size == ks * ns * 16
    blocks = elems.reshape(ks, ns, 4, 4)  # [i_slice][o_slice][i%4][o%4]
    full = np.full((ns * 4, ks * 4), shift, np.int32)
    full[:n, :k] = w.astype(np.int32) + shift
    expect = full.reshape(ns, 4, ks, 4).transpose(2, 0, 3, 1)
    assert np.array_equal(blocks.astype(np.int32), expect)


def test_closed_form_element_index(oracle):
    # e(o,i) = ((i/4 * Ns + o/4) * 4 + i%4) * 4 + o%4
    n, k = 20, 12
    ns = 5
    w = np.arange(n * k, dtype=np.int32).reshape(n, k)
    packed = oracle.rearrange_u8((w % 251).astype(np.uint8), I4O4, ns, 0)
    for o in range(n):
        for i in range(k):
            e = ((i // 4 * ns + o // 4) * 4 + i % 4) * 4 + o % 4
            assert packed[e] == w[o, i] % 251


def test_o4i4_signed_int8_closed_form(oracle):
    # conv int8 route: [Og][Is][G][4o][4i], pad 0 (weights_conversion.cc:1374-1376)
    n, k, g = 24, 12, 4
    rng = np.random.default_rng(3)
    w = rng.integers(-127, 128, size=(n, k), dtype=np.int8)
    out = oracle.rearrange_i8(w, O4I4, g)
    og = (n + 4 * g - 1) // (4 * g)
    assert out.size == og * g * 4 * k
    full = np.zeros((og * g * 4, k), np.int8)
    full[:n] = w
    expect = full.reshape(og, g, 4, k // 4, 4).transpose(0, 3, 1, 2, 4).ravel()
    assert np.array_equal(out, expect)


def test_custom_groups_equal_named_layouts(oracle):
    # weights_conversion_test.cc:1196-1251: these group lists are I4O4 / O4I4 with group 4
    O, H, W, I = 0, 1, 2, 3
    shape = (39, 2, 3, 23)
    rng = np.random.default_rng(11)
    w = rng.integers(-128, 128, size=shape, dtype=np.int8)
    i4o4 = oracle.rearrange_custom_i8(w, [(O, 4), (I, 4), (O, 4), (I, 0), (W, 0), (H, 0), (O, 0)])
    o4i4 = oracle.rearrange_custom_i8(w, [(I, 4), (O, 4), (O, 4), (I, 0), (W, 0), (H, 0), (O, 0)])
    assert np.array_equal(i4o4, oracle.rearrange_i8(w, I4O4, 4))
    assert np.array_equal(o4i4, oracle.rearrange_i8(w, O4I4, 4))


def test_total_elements(oracle):
    assert oracle.total_elements(I4O4, 14336, 1, 1, 4096, 3584) == 14336 * 4096
    assert oracle.total_elements(I4O4, 3, 1, 1, 5, 1) == 4 * 8
    assert oracle.total_elements(O4I4, 39, 2, 3, 23, 4) == 24 * 48 * 6
    assert oracle.total_elements(TWO_D, 16, 2, 1, 8, 2) == 2 * 4 * 16 * 2


def test_weights_sum(oracle):
    rng = np.random.default_rng(5)
    w = rng.integers(-128, 128, size=(37, 2, 2, 19), dtype=np.int8)
    assert np.array_equal(oracle.weights_sum_i(w), w.astype(np.int64).sum(axis=(1, 2, 3)))


def test_fp16_conversion_exhaustive(oracle):
    bits = np.arange(65536, dtype=np.uint16)
    f = oracle.f16_bits_to_f32(bits)
    ref = bits.view(np.float16).astype(np.float32)
    nan = np.isnan(ref)
    assert np.array_equal(f[~nan], ref[~nan]) and np.all(np.isnan(f[nan]))
    back = oracle.f32_to_f16_bits(f[~nan])
    assert np.array_equal(back, bits[~nan])
    # weights_conversion_test.cc:43-48
    src = np.array([0.1, 0.2, 0.3, 0.4], np.float32)
    assert np.array_equal(oracle.f32_to_f16_bits(src), src.astype(np.float16).view(np.uint16))
    rng = np.random.default_rng(0)
    x = np.concatenate([rng.standard_normal(200000).astype(np.float32) * 100,
                        (rng.standard_normal(100000) * 1e-6).astype(np.float32),
                        np.array([65504, 65519.99, 65520, 1e30, -1e30, 2.0 ** -25, 2.0 ** -24 * 1.5,
                                  2.0 ** -25 * 1.0000001], np.float32)])
    with np.errstate(over="ignore"):
        assert np.array_equal(oracle.f32_to_f16_bits(x), x.astype(np.float16).view(np.uint16))


def test_scale_layout(oracle):
    # tensor_desc.cc:267-292: [group][o_slice][4]
    o, groups = 10, 3
    s = np.arange(o * groups, dtype=np.float32).reshape(o, groups)
    out = oracle.scale_to_hoio4(s)
    assert out.shape == (groups, 3, 4)
    for g in range(groups):
        for oc in range(12):
            expect = s[oc, g] if oc < o else 0.0
            assert out[g, oc // 4, oc % 4] == expect
