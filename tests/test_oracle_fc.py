"""Pins the oracle's FullyConnected restatements: literal known answers held by the
reference tests (common/kernels/tests/fully_connected_test_util.cc), closed-form integer
results, and kernel-vs-textbook agreement under the reference's tolerance rule."""
import numpy as np
import pytest

I4O4 = 1


def tensor(o, x, precision):
    """float array -> tensor dtype of the precision (float32, or binary16 bits)."""
    x = np.asarray(x, np.float32)
    return x if precision == o.PREC_F32 else o.f32_to_f16_bits(x)


def to_f32(o, x, precision):
    return x if precision == o.PREC_F32 else o.f16_bits_to_f32(x)


def run_fc(o, src, w_i8, bits, precision, scale_kind, scale=None, zero_point=None, bias=None,
           scalar_scale=1.0, use_fma=True, wg_y=1):
    m, k = src.shape
    n = w_i8.shape[0]
    ns = (n + 3) // 4
    packed = (o.int8_as_uint8 if bits == 8 else o.int8_as_uint4)(w_i8, I4O4, ns)
    act = tensor(o, o.to_slices(src.astype(np.float32)), precision)
    groups = 1
    sc = zp = None
    if scale_kind == o.SCALE_LINEAR:
        sc = np.zeros(ns * 4, np.float32); sc[:n] = scale
        sc = tensor(o, sc, precision)
        if zero_point is not None:
            zp = np.zeros(ns * 4, np.float32); zp[:n] = zero_point
            zp = tensor(o, zp, precision)
    elif scale_kind == o.SCALE_BLOCK:
        groups = scale.shape[1]
        sc = tensor(o, o.scale_to_hoio4(scale), precision)
        if zero_point is not None:
            zp = tensor(o, o.scale_to_hoio4(zero_point), precision)
    bi = None
    if bias is not None:
        bi = np.zeros(ns * 4, np.float32); bi[:n] = bias
        bi = tensor(o, bi, precision)
    out = o.fc_kernel(act, packed, m, k, n, precision, bits, scale_kind, sc, zp, bi, groups,
                      use_fma, wg_y, scalar_scale)
    return o.from_slices(to_f32(o, out, precision), n)


PRECS = [0, 1, 2]


@pytest.mark.parametrize("precision", PRECS)
@pytest.mark.parametrize("use_fma", [True, False])
def test_known_answer_scalar_scale_bias(oracle, precision, use_fma):
    # fully_connected_test_util.cc:49-103
    src = np.array([[0.0, 1.0, 2.0, 3.0]])
    w = np.array([[2, 4, 6, 8], [10, 12, -14, 16]], np.int8)
    out = run_fc(oracle, src, w, 8, precision, oracle.SCALE_SCALAR, bias=[0.5, -0.5],
                 scalar_scale=0.5, use_fma=use_fma)
    eps = 1e-6 if precision == 0 else 1e-3
    assert np.allclose(out, [[20.5, 15.5]], atol=eps, rtol=0)


@pytest.mark.parametrize("precision", PRECS)
def test_known_answer_blockwise(oracle, precision):
    # :105-175
    src = np.arange(8, dtype=np.float32)[None]
    w = np.array([[1, 1, 1, 1, 2, 2, 2, 2], [3, 3, 3, 3, 4, 4, 4, 4]], np.int8)
    scale = np.array([[0.5, 2.0], [1.0, 0.1]], np.float32)
    out = run_fc(oracle, src, w, 8, precision, oracle.SCALE_BLOCK, scale=scale, bias=[0.0, 0.0])
    eps = 1e-5 if precision == 0 else 0.05
    assert np.allclose(out, [[91.0, 26.8]], atol=eps, rtol=0)


@pytest.mark.parametrize("precision", PRECS)
def test_known_answer_blockwise_zero_points(oracle, precision):
    # :177-249
    src = np.arange(1, 9, dtype=np.float32)[None]
    w = np.array([[1, 2, 3, 4, 5, 6, 7, 8], [-8, -7, -6, -5, -4, -3, -2, -1]], np.int8)
    scale = np.array([[0.5, 2.0], [1.5, 0.1]], np.float32)
    zp = np.array([[2, -3], [1, 4]], np.float32)
    out = run_fc(oracle, src, w, 8, precision, oracle.SCALE_BLOCK, scale=scale, zero_point=zp,
                 bias=[0.0, 0.0])
    eps = 1e-5 if precision == 0 else 0.1
    assert np.allclose(out, [[509.0, -121.4]], atol=eps, rtol=0)


def test_known_answer_int4_blockwise_all_ones(oracle):
    # :1541-1614: K=16, N=4, all-ones int4 weights and activations, two blocks of scale 0.5,
    # zero bias -> every output 8.0
    k, n, groups = 16, 4, 2
    src = np.ones((1, k), np.float32)
    w = np.ones((n, k), np.int8)
    scale = np.full((n, groups), 0.5, np.float32)
    for precision in PRECS:
        out = run_fc(oracle, src, w, 4, precision, oracle.SCALE_BLOCK, scale=scale,
                     bias=np.zeros(n, np.float32))
        eps = 1e-6 if precision == 0 else 1e-2
        assert np.allclose(out, np.full((1, n), 8.0), atol=eps, rtol=0)


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("m", [1, 4])
@pytest.mark.parametrize("kind", ["linear", "block", "block_zp"])
def test_kernel_matches_textbook_reference(oracle, bits, m, kind):
    """Shapes of the reference's 'Big' tests (:935-1001, 1616-1788): K = 11*4*7 or 171,
    N = 533; tolerance GetEpsilon(precision) * (K + 1) (common/task/testing_util.cc:328-331,
    common/util.cc:192-203)."""
    o = oracle
    rng = np.random.default_rng(bits * 10 + m)
    n = 533
    k = 171 if kind == "linear" else 11 * 4 * 7
    lo, hi = (-8, 8) if bits == 4 else (-128, 128)
    w = rng.integers(lo, hi, size=(n, k), dtype=np.int8)
    src = rng.uniform(-1, 1, size=(m, k)).astype(np.float32)
    bias = rng.uniform(-1, 1, size=n).astype(np.float32)
    groups = 1 if kind == "linear" else 7
    scale = (rng.uniform(-1, 1, size=(n, groups)) / 128).astype(np.float32)
    zp = rng.integers(-3, 4, size=(n, groups)).astype(np.float32) if kind == "block_zp" else None
    for precision, eps in [(o.PREC_F32, 1.1920929e-7), (o.PREC_F32F16, 9.7656e-4),
                           (o.PREC_F16, 9.7656e-4)]:
        if precision != o.PREC_F32:
            # what the fp16 tensors actually hold
            src_q = o.f16_bits_to_f32(o.f32_to_f16_bits(src))
            scale_q = o.f16_bits_to_f32(o.f32_to_f16_bits(scale))
            bias_q = o.f16_bits_to_f32(o.f32_to_f16_bits(bias))
        else:
            src_q, scale_q, bias_q = src, scale, bias
        wf = o.make_weights_from_int8(w, scale_q, zp)
        ref = o.fc_reference_f32(src_q, wf, bias_q)
        exact = src_q.astype(np.float64) @ wf.astype(np.float64).T + bias_q
        assert np.abs(ref - exact).max() < 1e-4
        for wg_y in (1, 4):
            out = run_fc(o, src_q, w, bits, precision,
                         o.SCALE_LINEAR if kind == "linear" else o.SCALE_BLOCK,
                         scale=scale_q[:, 0] if kind == "linear" else scale_q,
                         zero_point=zp, bias=bias_q, wg_y=wg_y)
            tol = eps * (k + 1) * (4 if precision != o.PREC_F32 else 1)
            assert np.abs(out - ref).max() <= tol, (precision, wg_y, np.abs(out - ref).max(), tol)


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("m,k,n", [(1, 112, 152), (3, 171, 533), (2, 8, 4)])
def test_int8_math_kernel_is_exact(oracle, bits, m, k, n):
    # :1426-1486: int8 activations x int8 weights -> int32, ContainerEq
    rng = np.random.default_rng(k + n)
    lo, hi = (-8, 8) if bits == 4 else (-128, 128)
    w = rng.integers(lo, hi, size=(n, k), dtype=np.int8)
    src = (rng.uniform(-1, 1, size=(m, k)) * 128).astype(np.int8)
    ns = (n + 3) // 4
    packed = (oracle.int8_as_uint8 if bits == 8 else oracle.int8_as_uint4)(w, I4O4, ns)
    out = oracle.fc_int8_kernel(oracle.to_slices(src), packed, m, k, n, bits)
    got = oracle.from_slices(out, n)
    ref = oracle.fc_reference_i8(src, w)
    assert np.array_equal(ref, src.astype(np.int64) @ w.astype(np.int64).T)
    assert np.array_equal(got, ref)


def test_int8_math_extremes(oracle):
    k, n = 64, 8
    w = np.full((n, k), -128, np.int8); w[1] = 127
    src = np.full((1, k), -128, np.int8)
    packed = oracle.int8_as_uint8(w, I4O4, 2)
    out = oracle.from_slices(oracle.fc_int8_kernel(oracle.to_slices(src), packed, 1, k, n, 8), n)
    assert out[0, 0] == 128 * 128 * k and out[0, 1] == -128 * 127 * k


def test_dequantize_weights_matches_make_weights(oracle):
    o = oracle
    rng = np.random.default_rng(9)
    n, k, groups = 37, 96, 3
    w = rng.integers(-8, 8, size=(n, k), dtype=np.int8)
    scale = o.f16_bits_to_f32(o.f32_to_f16_bits(rng.uniform(0.001, 0.01, size=(n, groups))))
    packed = o.int8_as_uint4(w, I4O4, (n + 3) // 4)
    sc_bits = o.f32_to_f16_bits(o.scale_to_hoio4(scale))
    got = o.f16_bits_to_f32(o.dequantize_weights(packed, n, k, 4, sc_bits, o.SCALE_BLOCK, groups))
    ref = o.make_weights_from_int8(w, scale)
    # fp16 rounding of (q-8)*s: relative error 2^-11
    assert np.abs(got - ref).max() <= np.abs(ref).max() * 2.0 ** -10


def test_gated_activation_known_values(oracle):
    """gelu_tanh(g) * u and silu(g) * u against closed forms: 0 at g = 0, ~g*u for large g,
    ~0 for very negative g, silu(g) = g / (1 + e^-g), the tanh argument clamp at +-10, the
    fp16 range clamp."""
    g = np.array([0.0, 8.0, -8.0, 1.0, -1.0, 300.0], np.float16)
    u = np.array([3.0, 2.0, 2.0, 1.0, 1.0, 300.0], np.float16)
    gelu = oracle.gated_activation(g, u, "gelu_tanh").astype(np.float64)
    assert gelu[0] == 0.0 and gelu[1] == 16.0 and abs(gelu[2]) < 1e-6
    assert abs(gelu[3] - 0.5 * (1 + np.tanh(0.7978845608 * (1 + 0.044715)))) < 1e-3
    assert abs(gelu[4] + 0.5 * (1 - np.tanh(0.7978845608 * (1 + 0.044715)))) < 1e-3
    assert gelu[5] == 65504.0  # 300 * 300 clamps to the fp16 range
    silu = oracle.gated_activation(g, u, "silu").astype(np.float64)
    assert silu[0] == 0.0 and abs(silu[3] - 1 / (1 + np.exp(-1.0))) < 1e-3 and abs(silu[4] + 1 / (1 + np.exp(1.0))) < 1e-3
    assert abs(silu[1] - 16.0) < 2e-2 and abs(silu[2]) < 1e-2 and silu[5] == 65504.0
