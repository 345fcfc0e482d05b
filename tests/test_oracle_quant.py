"""Pins the oracle's per-token quantization and the int32->float rescale against the CPU
mirrors and edge rows inside the reference's tests
(common/kernels/tests/quantize_and_dequantize_test_util.cc) and against algebra that does
not depend on the oracle's own formulas."""
import numpy as np
import pytest

K_MAX_HALF = 65504.0
K_MIN_NORMAL_HALF = 2.0 ** -14


def symmetric_test_tensor(rng, h, w, c):
    """tests/quantize_and_dequantize_test_util.cc:554-585 (rows: all zero, +-65504, [-12,4] / [-4,12])."""
    x = rng.uniform(-1, 1, size=(h, w, c)).astype(np.float32)
    for y in range(h):
        bias = -4.0 if y % 2 == 0 else 4.0
        for xx in range(w):
            if y == 0 and xx == 0:
                x[y, xx] = 0
            elif y == 0 and xx == 1:
                row = x[y, xx] * K_MAX_HALF
                row[0], row[1] = K_MAX_HALF, -K_MAX_HALF
                x[y, xx] = row
            else:
                x[y, xx] = x[y, xx] * 8 + bias
    return x.astype(np.float16).astype(np.float32).reshape(h * w, c)


@pytest.mark.parametrize("shape", [(13, 15, 237), (5, 7, 64)])
@pytest.mark.parametrize("signed", [True, False])
@pytest.mark.parametrize("f16", [True, False])
@pytest.mark.parametrize("calc_sum", [False, True])
def test_symmetric_against_reference_mirror(oracle, shape, signed, f16, calc_sum):
    o = oracle
    h, w, c = shape
    rng = np.random.default_rng(c + signed)
    x = symmetric_test_tensor(rng, h, w, c)
    tokens = h * w
    src = o.to_slices(x)
    src = o.f32_to_f16_bits(src) if f16 else src
    ptype = o.PACKED_INT8C4 if signed else o.PACKED_UINT8C4
    codes, params = o.quantize(src, tokens, c, ptype, symmetric=True, calculate_sum=calc_sum)
    codes = o.from_slices(codes, c).astype(np.int32)
    shift = 128 if signed else 0
    # mirror: :633-673
    min_scale = K_MIN_NORMAL_HALF if f16 else np.float32(1.0e-30)
    for t in range(tokens):
        abs_max = np.abs(x[t]).max()
        inv = np.float32(0); sc = np.float32(0); off = np.float32(0)
        if abs_max > 0:
            inv = max(np.float32(min_scale), np.float32(abs_max) / np.float32(127))
            if f16 and not signed:
                inv = min(inv, np.float32(K_MAX_HALF / 128))
            sc = np.float32(1) / inv
            if not signed:
                off = -inv * np.float32(128)
        assert params[t, 0] == inv and params[t, 1] == off
        ref = np.clip(np.floor(x[t] * sc + np.float32(128.5)), 0, 255).astype(np.int32) - shift
        assert np.array_equal(codes[t], ref), t
        if calc_sum:
            assert params[t, 2] == ref.sum()
        # contract x ~= q*inv_scale + offset within 0.51 step (:611-616, 687-698)
        deq = codes[t] * params[t, 0] + params[t, 1]
        expect = x[t]
        if f16 and not signed:
            expect = np.minimum(x[t], (255 - shift) * params[t, 0] + params[t, 1])
        assert np.all(np.abs(deq - expect) <= 0.51 * params[t, 0] + 1e-30)
    # all-zero row: params exactly 0, midpoint codes (:708-714)
    assert params[0, 0] == 0 and params[0, 1] == 0
    assert np.all(codes[0] == 128 - shift)


@pytest.mark.parametrize("f16", [True, False])
@pytest.mark.parametrize("calc_sum", [False, True])
def test_asymmetric_against_reference_mirror(oracle, f16, calc_sum):
    """Unsigned codes against the mirror the reference runs (:49-151: truncation, hence its
    +-1 code allowance; :522-541: BHWC(1,13,15,237), values in [-16, 48]).  The signed
    mirror (:153-255) is not called by any reference test and disagrees with the kernel's
    offset (min + range*128/255, quantize_and_dequantize.cc:397-399, 786-787), so signed
    codes are pinned as unsigned codes - 128 with that offset."""
    o = oracle
    h, w, c = 13, 15, 237
    rng = np.random.default_rng(1)
    x = (rng.uniform(-1, 1, size=(h * w, c)) * 32 + 16).astype(np.float32)
    if f16:
        x = x.astype(np.float16).astype(np.float32)
    src = o.to_slices(x)
    src = o.f32_to_f16_bits(src) if f16 else src
    ucodes, uparams = o.quantize(src, h * w, c, o.PACKED_UINT8C4, calculate_sum=calc_sum)
    scodes, sparams = o.quantize(src, h * w, c, o.PACKED_INT8C4, calculate_sum=calc_sum)
    ucodes = o.from_slices(ucodes, c).astype(np.int32)
    scodes = o.from_slices(scodes, c).astype(np.int32)
    assert np.array_equal(scodes, ucodes - 128)
    eps = 0.005 if f16 else 0.00005
    for t in range(h * w):
        mn = min(x[0, 0], x[t].min()); mx = max(x[0, 0], x[t].max())
        rng_ = np.float32(mx - mn)
        if f16:  # the kernel subtracts in the source type (quantize_and_dequantize.cc:392)
            rng_ = np.float32(np.float16(rng_))
        scale = np.float32(255.0) / rng_
        ref = np.clip((x[t] - mn) * scale, 0, 255).astype(np.int32)  # truncation
        assert abs(uparams[t, 0] - 1 / scale) <= eps
        assert abs(uparams[t, 1] - mn) <= eps
        assert np.abs(ucodes[t] - ref).max() <= 1
        assert sparams[t, 0] == uparams[t, 0]
        assert abs(sparams[t, 1] - (mn + rng_ * 128.0 / 255.0)) <= 1e-5
        if calc_sum:
            assert abs(uparams[t, 2] - ref.sum()) <= c
            assert sparams[t, 2] == uparams[t, 2] - 128 * c
        # round trip: x ~= q*inv_scale + offset within 0.51 of a step
        for codes, params in ((ucodes, uparams), (scodes, sparams)):
            deq = codes[t] * params[t, 0] + params[t, 1]
            assert np.all(np.abs(deq - x[t]) <= 0.51 * params[t, 0] + 1e-4)


def test_asymmetric_exact_small_case(oracle):
    # hand-computed: token 0 = [0, 255] -> range 255, scale 1, codes x - 128
    o = oracle
    x = np.array([[0.0, 255.0, 100.0, 17.0], [0.0, 51.0, 25.4, 25.6]], np.float32)
    codes, params = o.quantize(o.to_slices(x), 2, 4, o.PACKED_INT8C4, calculate_sum=True)
    codes = o.from_slices(codes, 4)
    assert codes[0].tolist() == [-128, 127, -28, -111]
    assert params[0, 0] == 1.0 and params[0, 1] == np.float32(255.0) * np.float32(128.0 / 255.0)
    assert params[0, 2] == -128 + 127 - 28 - 111
    # token 1: min 0 (also the seed element), max 51 -> scale 5: 25.4*5+.5=127.5->127 ; 25.6*5+.5=128.5->128
    assert codes[1].tolist() == [-128, 127, -1, 0]
    assert params[1, 0] == np.float32(51.0) / np.float32(255.0)


def test_asymmetric_seed_element_quirk(oracle):
    # the search starts from element (b, 0, 0, 0), so token 1's range includes token 0's
    # first channel (quantize_and_dequantize.cc:288; mirrored at test_util.cc:168)
    o = oracle
    x = np.array([[100.0, 1.0, 2.0, 3.0], [0.0, 1.0, 2.0, 3.0]], np.float32)
    _, params = o.quantize(o.to_slices(x), 2, 4, o.PACKED_INT8C4)
    assert params[1, 0] == np.float32(100.0) / np.float32(255.0)


def test_c16_layout_is_a_permutation_of_c4(oracle):
    o = oracle
    rng = np.random.default_rng(2)
    tokens, c = 7, 72
    x = rng.standard_normal((tokens, c)).astype(np.float32)
    src = o.f32_to_f16_bits(o.to_slices(x))
    c4, p4 = o.quantize(src, tokens, c, o.PACKED_INT8C4, symmetric=True)
    c16, p16 = o.quantize(src, tokens, c, o.PACKED_INT8C16, symmetric=True)
    assert np.array_equal(p4, p16)
    flat4 = o.from_slices(c4, c)
    # [S/4][tokens][16] -> k = 16*s16 + j
    flat16 = c16.transpose(1, 0, 2).reshape(tokens, -1)[:, :c]
    assert np.array_equal(flat4, flat16)


@pytest.mark.parametrize("with_zp", [False, True])
def test_dequantize_algebra(oracle, with_zp):
    """quantize_and_dequantize.cc:844-866: the epilogue applied to the exact integer dot
    product equals the float product of the dequantised operands."""
    o = oracle
    rng = np.random.default_rng(4)
    m, k, n = 5, 96, 22
    x = rng.standard_normal((m, k)).astype(np.float32)
    w = rng.integers(-127, 128, size=(n, k), dtype=np.int8)
    ws = (np.abs(rng.standard_normal(n)) * 0.02 / 127).astype(np.float32)
    wzp = rng.integers(-5, 6, size=n).astype(np.float32) if with_zp else None
    codes, params = o.quantize(o.to_slices(x), m, k, o.PACKED_INT8C4, symmetric=False,
                               calculate_sum=True)
    q = o.from_slices(codes, k)
    acc = o.to_slices(o.fc_reference_i8(q, w))
    out = o.dequantize(acc, params, o.weights_sum_i(w), ws, n, k, weights_zero_point=wzp,
                       dst_f16=False)
    got = o.from_slices(out, n)
    a_deq = q.astype(np.float64) * params[:, 0:1] + params[:, 1:2]
    # reference convention here: Wi = Iw * Wsc + Wzp (:856-858)
    w_deq = w.astype(np.float64) * ws[:, None] + (0 if wzp is None else wzp[:, None])
    ref = a_deq @ w_deq.T
    assert np.abs(got - ref).max() <= 1e-4 * max(1.0, np.abs(ref).max())


LITERAL_TIE_ROW = np.array([127.0, 0.5, -0.5, 1.5, -1.5, 2.4, -2.6, -127.0], np.float32)
# absmax 127 -> inv_scale = scale = 1 exactly, so code = floor(x + 128.5) - 128: ties go up
# (0.5 -> 1, -0.5 -> 0, 1.5 -> 2, -1.5 -> -1), 2.4 -> 2, -2.6 -> -3.  Worked by hand from
# common/kernels/quantize_and_dequantize.cc:363-377, 423-429; round-to-nearest-even would give
# 0, 0, 2, -2 for the four ties.
LITERAL_TIE_CODES = np.array([127, 1, 0, 2, -1, 2, -3, -127], np.int32)


@pytest.mark.parametrize("f16", [True, False])
def test_symmetric_literal_tie_vector(oracle, f16):
    o = oracle
    src = o.to_slices(LITERAL_TIE_ROW[None])
    src = o.f32_to_f16_bits(src) if f16 else src
    codes, params = o.quantize(src, 1, 8, o.PACKED_INT8C4, symmetric=True, calculate_sum=True)
    assert params[0, 0] == 1.0 and params[0, 1] == 0.0
    assert np.array_equal(o.from_slices(codes, 8).astype(np.int32)[0], LITERAL_TIE_CODES)
    assert params[0, 2] == LITERAL_TIE_CODES.sum()
    # unsigned codes: the same + 128, offset -128 * inv_scale
    codes_u, params_u = o.quantize(src, 1, 8, o.PACKED_UINT8C4, symmetric=True)
    assert np.array_equal(o.from_slices(codes_u, 8).astype(np.int32)[0], LITERAL_TIE_CODES + 128)
    assert params_u[0, 0] == 1.0 and params_u[0, 1] == -128.0


# ---- packed outputs beyond C4 / C16: 4-bit codes (C32) and four columns per element (W4C4) ----
# hand-computed: abs_max 7 -> inv_scale 7 / 7 = 1; code = clamp(floor(x + 8.5), 0, 15) (- 8 signed)
INT4_ROW = np.array([7.0, -7.0, 3.5, 0.5, -0.5, -3.5, 6.49, 0.0], np.float32)
INT4_CODES = np.array([7, -7, 4, 1, 0, -3, 6, 0], np.int32)
# nibble j of the 16 bytes = channel j, two's complement, low nibble first; the 8 channels are two
# slices, the six slices that complete the group of 32 channels repeat the last one
INT4_BYTES = bytes([0x97, 0x14, 0xD0, 0x06] + [0xD0, 0x06] * 6)
UINT4_BYTES = bytes([0x1F, 0x9C, 0x58, 0x8E] + [0x58, 0x8E] * 6)


def unpack_c32(codes, channels, signed):
    """[G][tokens][16] bytes -> [tokens][channels] integer codes."""
    g, tokens, _ = codes.shape
    b = codes.astype(np.int32)
    nib = np.stack([b & 15, b >> 4], axis=-1).reshape(g, tokens, 32)
    flat = nib.transpose(1, 0, 2).reshape(tokens, g * 32)[:, :channels]
    return np.where(flat >= 8, flat - 16, flat) if signed else flat


@pytest.mark.parametrize("f16", [True, False])
def test_int4_symmetric_literal(oracle, f16):
    o = oracle
    src = o.to_slices(INT4_ROW[None])
    src = o.f32_to_f16_bits(src) if f16 else src   # 6.49 rounds to 6.4883 in half: same code
    codes, params = o.quantize(src, 1, 8, o.PACKED_INT4C32, symmetric=True, calculate_sum=True)
    assert codes.shape == (1, 1, 16) and codes.tobytes() == INT4_BYTES
    assert params[0].tolist() == [1.0, 0.0, float(INT4_CODES.sum()), 0.0]
    assert np.array_equal(unpack_c32(codes, 8, True)[0], INT4_CODES)
    codes_u, params_u = o.quantize(src, 1, 8, o.PACKED_UINT4C32, symmetric=True)
    assert codes_u.tobytes() == UINT4_BYTES
    assert params_u[0, 0] == 1.0 and params_u[0, 1] == -8.0   # offset = -inv_scale * 8


def test_int4_asymmetric_literal(oracle):
    # [0, 15]: range 15, scale 15 / 15 = 1, code = trunc(x + 0.5): 7.4 -> 7, 7.6 -> 8
    o = oracle
    x = np.array([[0.0, 15.0, 7.4, 7.6]], np.float32)
    codes, params = o.quantize(o.to_slices(x), 1, 4, o.PACKED_UINT4C32, calculate_sum=True)
    assert unpack_c32(codes, 4, False)[0].tolist() == [0, 15, 7, 8]
    assert params[0].tolist() == [1.0, 0.0, 30.0, 0.0]
    codes, params = o.quantize(o.to_slices(x), 1, 4, o.PACKED_INT4C32, calculate_sum=True)
    assert unpack_c32(codes, 4, True)[0].tolist() == [-8, 7, -1, 0]
    # signed offset = min + range * (8 / 15), quantize_and_dequantize.cc:397-399, 786-787
    assert params[0, 0] == 1.0 and params[0, 1] == np.float32(15.0) * (np.float32(8.0) / np.float32(15.0))
    assert params[0, 2] == -2.0


@pytest.mark.parametrize("signed", [True, False])
@pytest.mark.parametrize("f16", [True, False])
@pytest.mark.parametrize("c", [237, 64, 20])
def test_int4_symmetric_contract_and_padding(oracle, signed, f16, c):
    """4-bit codes on the reference's symmetric test tensor: the dequantization contract
    x ~= q * inv_scale + offset within 0.51 step (tests/quantize_and_dequantize_test_util.cc:611-616),
    the all-zero row (params 0, mid-point codes, :708-714), inv_scale = abs_max / 7 and the slices that
    pad the last group of 32 channels."""
    o = oracle
    h, w = 5, 7
    x = symmetric_test_tensor(np.random.default_rng(c), h, w, c)
    tokens = h * w
    src = o.to_slices(x)
    src = o.f32_to_f16_bits(src) if f16 else src
    codes, params = o.quantize(src, tokens, c, o.PACKED_INT4C32 if signed else o.PACKED_UINT4C32, symmetric=True,
                               calculate_sum=True)
    q = unpack_c32(codes, c, signed)
    lo, hi = (-8, 7) if signed else (0, 15)
    assert q.min() >= lo and q.max() <= hi
    for t in range(tokens):
        abs_max = np.abs(x[t]).max()
        if abs_max == 0:
            assert params[t, 0] == 0 and params[t, 1] == 0 and np.all(q[t] == (0 if signed else 8))
            continue
        inv = np.float32(abs_max) / np.float32(7)
        if f16 and not signed:
            inv = min(inv, np.float32(K_MAX_HALF / 8))
        assert params[t, 0] == inv and params[t, 2] == q[t].sum()
        deq = q[t] * params[t, 0] + params[t, 1]
        expect = np.minimum(x[t], hi * params[t, 0] + params[t, 1])
        assert np.all(np.abs(deq - expect) <= 0.51 * params[t, 0])
    # padding: channels c .. 4*slices-1 are the codes of 0.0, slices beyond the last repeat it
    slices = (c + 3) // 4
    full = unpack_c32(codes, codes.shape[0] * 32, signed)
    last = full[:, (slices - 1) * 4: slices * 4]
    for s in range(slices, codes.shape[0] * 8):
        assert np.array_equal(full[:, s * 4: s * 4 + 4], last)


@pytest.mark.parametrize("symmetric", [True, False])
def test_c32_and_c16_hold_the_c4_codes_of_a_narrower_range(oracle, symmetric):
    """Layout only: the 8-bit C16 bytes against the C4 bytes (slice s of group s / 4 at byte 4 * (s % 4),
    the host-side packing of the reference's int8 convolution test, conv_generic_test_util.cc:1176-1200),
    including the repeated last slice."""
    o = oracle
    rng = np.random.default_rng(5)
    tokens, c = 6, 44   # 11 slices: the last C16 group holds 3 slices + 1 repeat
    x = rng.standard_normal((tokens, c)).astype(np.float32)
    src = o.to_slices(x)
    c4, p4 = o.quantize(src, tokens, c, o.PACKED_INT8C4, symmetric=symmetric)
    c16, p16 = o.quantize(src, tokens, c, o.PACKED_INT8C16, symmetric=symmetric)
    assert np.array_equal(p4, p16)
    for s in range(12):
        assert np.array_equal(c16[s // 4, :, (s % 4) * 4:(s % 4) * 4 + 4], c4[min(s, 10)])


@pytest.mark.parametrize("signed", [True, False])
@pytest.mark.parametrize("h,w,b", [(1, 8, 1), (3, 7, 1), (2, 5, 3), (1, 1, 2)])
def test_w4c4_layout(oracle, signed, h, w, b):
    """W4C4: element (x / 4, y, s) of the int32x4 tensor holds the four char4 of columns x..x+3
    (quantize_and_dequantize.cc:461-483).  With batch 1 and a width that is a multiple of 4 the bytes are
    those of the C4 tensor (how the reference's convolution test uploads one as the other,
    conv_generic_test_util.cc:1168-1175); columns beyond the width repeat the last one; with a batch
    the four columns of one batch element sit together."""
    o = oracle
    c = 24
    tokens = h * w * b
    rng = np.random.default_rng(h * 100 + w * 10 + b)
    x = rng.standard_normal((tokens, c)).astype(np.float32)
    src = o.to_slices(x)
    p_c4, p_w4 = (o.PACKED_INT8C4, o.PACKED_INT8W4C4) if signed else (o.PACKED_UINT8C4, o.PACKED_UINT8W4C4)
    c4, params4 = o.quantize(src, tokens, c, p_c4, calculate_sum=True, batch=b, height=h)
    w4, params = o.quantize(src, tokens, c, p_w4, calculate_sum=True, batch=b, height=h)
    assert np.array_equal(params, params4)
    assert w4.shape == (6, h, (w + 3) // 4, b, 16)
    if b == 1 and w % 4 == 0:
        assert w4.tobytes() == c4.tobytes()
    c4 = c4.reshape(6, h, w, b, 4)
    for xx in range(4 * ((w + 3) // 4)):
        got = w4[:, :, xx // 4, :, (xx % 4) * 4:(xx % 4) * 4 + 4]
        assert np.array_equal(got, c4[:, :, min(xx, w - 1)]), xx
