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
