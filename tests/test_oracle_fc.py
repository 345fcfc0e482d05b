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


# ---- batched weights selected by runtime ids (mixture-of-experts FullyConnected) ----
def make_batch_ids_case(seed, rows, row_tokens, src_rows, k, n, batch, bits=8, groups=1, with_zp=False):
    """Shapes of FullyConnectedInt8BatchedWeightsIdsBigTest (fully_connected_test_util.cc:1338-1380):
    weights OHWI(n, batch, 1, k), scales OHWI(n, batch, 1, groups), ids random in [0, batch)."""
    rng = np.random.default_rng(seed)
    lim = 127 if bits == 8 else 7
    w = rng.integers(-lim - (bits == 4), lim + 1, size=(n, batch, 1, k), dtype=np.int8)
    scale = (np.abs(rng.normal(0.0, 1.0, size=(n, batch, groups))) / 128.0 + 1e-3).astype(np.float32)
    zp = rng.integers(-3, 4, size=(n, batch, groups)).astype(np.float32) if with_zp else None
    src = rng.uniform(-1, 1, size=(src_rows, row_tokens, k)).astype(np.float32)
    ids = rng.integers(0, batch, size=rows).astype(np.int32)
    return dict(w=w, scale=scale, zp=zp, src=src, ids=ids, rows=rows, row_tokens=row_tokens, src_rows=src_rows,
                k=k, n=n, batch=batch, bits=bits, groups=groups)


def batch_ids_float_weights(o, c):
    """(n, batch, k) dequantized weights (MakeWeightsFromInt8 per matrix)."""
    out = np.empty((c["n"], c["batch"], c["k"]), np.float32)
    for e in range(c["batch"]):
        zp = None if c["zp"] is None else c["zp"][:, e, :]
        out[:, e, :] = o.make_weights_from_int8(c["w"][:, e, 0, :], c["scale"][:, e, :], zp)
    return out


def run_batch_ids_oracle(o, c, precision):
    ns = (c["n"] + 3) // 4
    pack = o.int8_as_uint8 if c["bits"] == 8 else o.int8_as_uint4
    packed = pack(c["w"], I4O4, ns)
    src2 = c["src"].reshape(c["src_rows"] * c["row_tokens"], c["k"])
    act = tensor(o, o.to_slices(src2), precision)
    kind = o.SCALE_LINEAR if c["groups"] == 1 else o.SCALE_BLOCK
    sc = tensor(o, o.scale_to_hoio4_batched(c["scale"]), precision)
    zp = None if c["zp"] is None else tensor(o, o.scale_to_hoio4_batched(c["zp"]), precision)
    out = o.fc_batch_ids_kernel(act, c["ids"], packed, c["rows"], c["row_tokens"], c["src_rows"], c["batch"], c["k"],
                                c["n"], precision, c["bits"], kind, sc, zp, None, c["groups"])
    return o.from_slices(to_f32(o, out, precision), c["n"]).reshape(c["rows"], c["row_tokens"], c["n"])


def test_batched_packing_is_one_matrix_after_the_other(oracle):
    """kOSpatialIOGroupI4O4 with one output group: the spatial index (the weights batch) is the
    outermost, so a batched buffer is the single-matrix buffers concatenated - what the kernel's
    address offset w_batch_id * Ks * Ns (fully_connected.cc:493-496) assumes."""
    rng = np.random.default_rng(5)
    for bits, n, k, batch in ((8, 32, 64, 16), (4, 20, 40, 3), (8, 7, 12, 2)):
        lim = 127 if bits == 8 else 7
        w = rng.integers(-lim, lim + 1, size=(n, batch, 1, k), dtype=np.int8)
        ns = (n + 3) // 4
        pack = oracle.int8_as_uint8 if bits == 8 else oracle.int8_as_uint4
        whole = pack(w, I4O4, ns)
        parts = np.concatenate([pack(np.ascontiguousarray(w[:, e, 0, :]), I4O4, ns) for e in range(batch)])
        assert np.array_equal(whole, parts)


def test_batched_packing_in_output_groups(oracle):
    """With output groups of G slices the spatial index lies between the output group and the K-slice
    ([Og][HW][Is][G] blocks, weights_conversion.cc:139-185): the run of output group g of matrix b in
    the batched buffer is that group's run of matrix b packed alone, at run index g * batch + b."""
    rng = np.random.default_rng(6)
    for bits, n, k, batch, group in ((4, 128, 64, 3, 16), (8, 32, 20, 4, 2), (4, 24, 40, 5, 3), (8, 16, 8, 2, 1)):
        lim = 127 if bits == 8 else 7
        w = rng.integers(-lim, lim + 1, size=(n, batch, 1, k), dtype=np.int8)
        ns, ks = (n + 3) // 4, (k + 3) // 4
        pack = oracle.int8_as_uint8 if bits == 8 else oracle.int8_as_uint4
        run = ks * group * (16 if bits == 8 else 8)  # bytes of one output group of one matrix
        whole = pack(w, I4O4, group).reshape(ns // group, batch, run)
        for e in range(batch):
            single = pack(np.ascontiguousarray(w[:, e, 0, :]), I4O4, group).reshape(ns // group, run)
            assert np.array_equal(whole[:, e, :], single), (bits, n, k, batch, group, e)


def test_batched_scale_tensor_layout(oracle):
    """[group][batch][slice][4], zero padded: element (o, b, g) found where the kernel reads it
    (weights_scale.Read(o_slice, w_batch_id, group), fully_connected_util.cc:80-98)."""
    o_ch, batch, groups = 10, 3, 2
    s = np.arange(o_ch * batch * groups, dtype=np.float32).reshape(o_ch, batch, groups) + 1
    t = oracle.scale_to_hoio4_batched(s)
    assert t.shape == (groups, batch, 3, 4)
    for oc in range(o_ch):
        for b in range(batch):
            for g in range(groups):
                assert t[g, b, oc // 4, oc % 4] == s[oc, b, g]
    assert np.all(t[:, :, 2, 2:] == 0)
    # one matrix: the same bytes as the unbatched conversion
    assert np.array_equal(oracle.scale_to_hoio4_batched(s[:, :1, :])[:, 0], oracle.scale_to_hoio4(s[:, 0, :]))


@pytest.mark.parametrize("src_shape,ids_count", [((1, 1, 32), 1), ((8, 1, 32), 8), ((128, 1, 64), 128),
                                                 ((1, 1, 32), 4)])
@pytest.mark.parametrize("precision", [0, 1])
def test_batch_ids_reference_test_shapes(oracle, src_shape, ids_count, precision):
    """fully_connected_test.cc:227-250: 32 output channels, a batch of 16 int8 matrices, sources
    (1,1,1,32), (1,8,1,32), (1,128,1,64) with as many ids as rows, and the broadcast case of one
    source row read by 4 ids.  Checked like the reference does: kernel against the float
    reference over dequantized weights."""
    src_rows, row_tokens, k = src_shape
    c = make_batch_ids_case(ids_count + k, ids_count, row_tokens, src_rows, k, 32, 16)
    got = run_batch_ids_oracle(oracle, c, precision)
    ref = oracle.fc_batch_ids_reference_f32(c["src"], batch_ids_float_weights(oracle, c), c["ids"])
    eps = 2e-5 * k if precision == 0 else 2e-2
    assert np.abs(got - ref).max() <= eps * max(1.0, np.abs(ref).max())
    # a row's result depends on its id: permuting two different ids changes those rows
    if ids_count >= 8:
        c2 = dict(c, ids=c["ids"].copy())
        a, b = 0, int(np.argmax(c["ids"] != c["ids"][0]))
        c2["ids"][[a, b]] = c["ids"][[b, a]]
        got2 = run_batch_ids_oracle(oracle, c2, precision)
        assert not np.array_equal(got2[a], got[a])
        others = [y for y in range(ids_count) if y not in (a, b)]
        assert np.array_equal(got2[others], got[others])


def test_batch_ids_int4_groups_zero_points(oracle):
    c = make_batch_ids_case(3, rows=5, row_tokens=3, src_rows=5, k=64, n=20, batch=4, bits=4, groups=2, with_zp=True)
    got = run_batch_ids_oracle(oracle, c, 0)
    ref = oracle.fc_batch_ids_reference_f32(c["src"], batch_ids_float_weights(oracle, c), c["ids"])
    assert np.abs(got - ref).max() <= 1e-4 * max(1.0, np.abs(ref).max())


def make_batch_ids_int8_case(seed, rows, row_tokens, src_rows, k, n, batch, bits):
    rng = np.random.default_rng(seed)
    lim = 127 if bits == 8 else 7
    w = rng.integers(-lim - 1, lim + 1, size=(n, batch, 1, k), dtype=np.int8)
    src = rng.integers(-128, 128, size=(src_rows, row_tokens, k), dtype=np.int8)
    ids = rng.integers(0, batch, size=rows).astype(np.int32)
    return dict(w=w, src=src, ids=ids, rows=rows, row_tokens=row_tokens, src_rows=src_rows, k=k, n=n, batch=batch, bits=bits)


def batch_ids_int8_exact(c):
    """The closed form: int32 products of the selected matrix with the row's tokens."""
    out = np.empty((c["rows"], c["row_tokens"], c["n"]), np.int64)
    for y in range(c["rows"]):
        sy = 0 if c["src_rows"] == 1 else y
        out[y] = c["src"][sy].astype(np.int64) @ c["w"][:, int(c["ids"][y]), 0, :].astype(np.int64).T
    return out


def run_batch_ids_int8_oracle(o, c):
    ns = (c["n"] + 3) // 4
    packed = (o.int8_as_uint8 if c["bits"] == 8 else o.int8_as_uint4)(c["w"], I4O4, ns)
    act = o.to_slices(c["src"].reshape(-1, c["k"]))
    out = o.fc_batch_ids_int8_kernel(act, c["ids"], packed, c["rows"], c["row_tokens"], c["src_rows"], c["batch"],
                                     c["k"], c["n"], c["bits"])
    return o.from_slices(out, c["n"]).reshape(c["rows"], c["row_tokens"], c["n"])


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("rows,row_tokens,src_rows,k,n,batch", [(8, 1, 8, 32, 32, 16), (4, 1, 1, 32, 32, 16),
                                                                 (5, 3, 5, 171, 20, 3)])
def test_batch_ids_int8_math_exact(oracle, bits, rows, row_tokens, src_rows, k, n, batch):
    c = make_batch_ids_int8_case(rows + k + bits, rows, row_tokens, src_rows, k, n, batch, bits)
    assert np.array_equal(run_batch_ids_int8_oracle(oracle, c), batch_ids_int8_exact(c))


# ------------------------------------------------------------------------------------------
# Runtime channel bounds (ConvRuntimeCheckDesc): the reference's FullyConnectedRuntimeChWi8Test
# (common/kernels/tests/fully_connected_test_util.cc:1260-1300): K = 171, N = 533, int8
# per-channel weights + bias, runtime channels {src_end 4, dst_end 8}, {src_end 8},
# {src_end K + 4}, {dst_end 14}, against FullyConnectedReference with runtime channels
# (common/task/testing_ref_ops.cc:961-988: sum over s < src_end_ch for d < dst_end_ch), the first
# dst_end_ch values compared (fully_connected_test_util.cc:1208-1222).
# ------------------------------------------------------------------------------------------
RUNTIME_CHANNEL_CASES = [dict(src_end_ch=4, dst_end_ch=8), dict(src_end_ch=8), dict(src_end_ch=171 + 4), dict(dst_end_ch=14)]


def test_runtime_end_slices_literals(oracle):
    o = oracle
    # round_up(dst_end_ch, 32) / 4, capped at the slice count; (src_end_ch + 3) / 4 after the cap at K
    assert o.runtime_end_slices(4, 8, 171, 533, False) == (1, 8)
    assert o.runtime_end_slices(8, None, 171, 533, False) == (2, 134)
    assert o.runtime_end_slices(175, None, 171, 533, False) == (43, 134)
    assert o.runtime_end_slices(None, 14, 171, 533, False) == (43, 8)
    assert o.runtime_end_slices(None, 33, 171, 533, False) == (43, 16)
    assert o.runtime_end_slices(None, 532, 171, 533, False) == (43, 134)   # 544 / 4 = 136 -> capped
    assert o.runtime_end_slices(5, None, 171, 533, False) == (2, 134)
    assert o.runtime_end_slices(5, None, 176, 533, True) == (44, 134)      # group-wise scales: all groups
    assert o.runtime_end_slices(-3, -1, 171, 533, False) == (0, 0)


@pytest.mark.parametrize("precision", ["f32", "f16"])
@pytest.mark.parametrize("rc", RUNTIME_CHANNEL_CASES)
def test_runtime_channels_reference_test(oracle, precision, rc):
    o = oracle
    k, n = 171, 533
    rng = np.random.default_rng(5)
    w = rng.integers(-128, 128, size=(n, k), dtype=np.int8)
    scale = (rng.uniform(0.1, 1.0, size=n) / 128.0).astype(np.float32)
    bias = rng.uniform(-1, 1, size=n).astype(np.float32)
    src = rng.uniform(-1, 1, size=(1, k)).astype(np.float32)
    prec = o.PREC_F32 if precision == "f32" else o.PREC_F32F16
    if precision == "f16":
        scale, bias, src = [x.astype(np.float16).astype(np.float32) for x in (scale, bias, src)]
    ns = (n + 3) // 4
    packed = o.int8_as_uint8(w, o.LAYOUT_I4O4, ns)
    pad = lambda v: np.concatenate([v, np.zeros(ns * 4 - n, np.float32)])
    sentinel = np.full((ns, 1, 4), 7.0, np.float32)
    out = o.fc_kernel_runtime_check(tensor(o, o.to_slices(src), prec), packed, 1, k, n, prec, 8, o.SCALE_LINEAR,
                                    tensor(o, pad(scale), prec), None, tensor(o, pad(bias), prec),
                                    dst_before=tensor(o, sentinel, prec), **rc)
    got = o.from_slices(to_f32(o, out, prec), ns * 4)[0]
    src_end = min(rc.get("src_end_ch", k), k)
    dst_end = rc.get("dst_end_ch", n)
    ref = (src[0, :src_end].astype(np.float64) @ (w[:, :src_end].astype(np.float64) * scale[:, None].astype(np.float64)).T) + bias
    eps = (1e-6 if precision == "f32" else 2e-3) * (k + 1)
    assert np.all(np.abs(got[:dst_end] - ref[:dst_end]) <= eps)
    # slices from dst_end_slice on are not written
    ns_end = o.runtime_end_slices(rc.get("src_end_ch"), rc.get("dst_end_ch"), k, n, False)[1]
    assert np.all(got[ns_end * 4:] == 7.0)
    if ns_end < ns:
        assert np.all(got[dst_end:ns_end * 4] != 7.0)


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("m,k,n,groups,bias,use_fma", [
    (1, 256, 128, 1, False, True), (3, 172, 536, 1, True, True), (2, 171, 533, 1, True, False), (1, 512, 68, 4, False, True),
    (5, 1024, 260, 32, True, True), (1, 64, 4, 1, True, True), (1, 2048, 2044, 64, False, False)])
def test_vector_path_is_bit_identical_to_scalar_path(oracle, bits, m, k, n, groups, bias, use_fma):
    """fc_kernel's eight-channels-at-a-time path (AVX2 + F16C, used for the CPU baseline) against the
    one-channel-at-a-time restatement: same bits, on unaligned shapes, odd slice counts, wide-range
    scales (down to half's subnormals) and both dequantization forms."""
    o = oracle
    rng = np.random.default_rng(k * 7 + n + bits)
    ks, ns = o.div_up(k, 4), o.div_up(n, 4)
    lim = 127 if bits == 8 else 7
    w = rng.integers(-lim - 1, lim + 1, size=(n, k), dtype=np.int8)
    packed = (o.int8_as_uint8 if bits == 8 else o.int8_as_uint4)(w, o.LAYOUT_I4O4, ns)
    act = o.f32_to_f16_bits(o.to_slices(rng.standard_normal((m, k)).astype(np.float32)))
    sc = (rng.standard_normal((n, groups)) * np.exp2(rng.integers(-20, 3, size=(n, groups)))).astype(np.float32)
    if groups == 1:
        flat = np.zeros(ns * 4, np.float32); flat[:n] = sc[:, 0]
        kind = o.SCALE_LINEAR
    else:
        flat = o.scale_to_hoio4(sc); kind = o.SCALE_BLOCK
    flat = o.f32_to_f16_bits(flat)
    b = o.f32_to_f16_bits(np.pad(rng.standard_normal(n).astype(np.float32), (0, ns * 4 - n))) if bias else None
    try:
        o.set_fast_path(False)
        slow = o.fc_kernel(act, packed, m, k, n, o.PREC_F32F16, bits, kind, flat, None, b, groups, use_fma=use_fma)
        assert o.last_fc_path == 0
        o.set_fast_path(True)
        fast = o.fc_kernel(act, packed, m, k, n, o.PREC_F32F16, bits, kind, flat, None, b, groups, use_fma=use_fma)
        path = o.last_fc_path
    finally:
        o.set_fast_path(True)
    if path != 1:
        pytest.skip("this CPU has no AVX2 + FMA + F16C: the vector path was not taken")
    assert np.array_equal(slow, fast)


def test_vector_path_declines_what_it_cannot_state_exactly(oracle):
    """A scale whose shift * scale leaves half's range (here 8 * 2^-24 is fine, 8 * 60000 overflows) and a
    zero point both fall back to the scalar path."""
    o = oracle
    k, n = 64, 8
    w = np.ones((n, k), np.int8)
    packed = o.int8_as_uint4(w, o.LAYOUT_I4O4, 2)
    act = o.f32_to_f16_bits(o.to_slices(np.ones((1, k), np.float32)))
    big = o.f32_to_f16_bits(np.full(8, 60000.0, np.float32))
    o.fc_kernel(act, packed, 1, k, n, o.PREC_F32F16, 4, o.SCALE_LINEAR, big)
    assert o.last_fc_path == 0
    ok = o.f32_to_f16_bits(np.full(8, 0.01, np.float32))
    o.fc_kernel(act, packed, 1, k, n, o.PREC_F32F16, 4, o.SCALE_LINEAR, ok, zero_point=ok)
    assert o.last_fc_path == 0
    o.fc_kernel(act, packed, 1, k, n, o.PREC_F32, 4, o.SCALE_LINEAR, np.full(8, 0.01, np.float32))
    assert o.last_fc_path == 0


# ---- packed groups (the grouped FullyConnected of a mixture-of-experts prefill) ----
def make_packed_groups_case(seed, width, per_item, k, n, batch, bits=8, groups=1, with_zp=False):
    """The set-up of FullyConnectedPackedGroupsTest (fully_connected_test_util.cc:2487-2530): every one of
    `width` tokens goes to `per_item` distinct matrices of `batch`; GroupsMapReference /
    PackedGroupsMapReference (common/task/testing_ref_ops.cc:2765-2816) sort the (slot, token) pairs by
    matrix (tokens ascending, slots inner), RemapToReference (:2819-2833) gathers the source rows in that
    order.  Returns the batch-ids style case plus ids [width][per_item], the packed (slot, token) list,
    sizes and offsets."""
    c = make_batch_ids_case(seed, 1, 1, 1, k, n, batch, bits, groups, with_zp)
    rng = np.random.default_rng(seed + 1)
    src = rng.uniform(-1, 1, size=(width, k)).astype(np.float32)
    ids = np.stack([rng.permutation(batch)[:per_item] for _ in range(width)]).astype(np.int32)
    lists = [[] for _ in range(batch)]
    for w in range(width):
        for slot in range(per_item):
            lists[int(ids[w, slot])].append((slot, w))
    sizes = np.array([len(l) for l in lists], np.int32)
    offsets = np.concatenate([[0], np.cumsum(sizes)[:-1]]).astype(np.int32)
    packed_map = [p for l in lists for p in l]
    c.update(tokens_src=src, ids2=ids, packed_map=packed_map, sizes=sizes, offsets=offsets, width=width, per_item=per_item,
             packed_src=np.stack([src[w] for _, w in packed_map]))
    return c


def packed_groups_expected(o, c, dtype=np.float32):
    """ConvolutionWithIds (common/task/testing_ref_ops.cc:2853-2880) in float64 over the dequantized
    matrices: result[slot][token] = W[ids[token][slot]] . src[token]."""
    wf = batch_ids_float_weights(o, c).astype(np.float64)
    src = c["tokens_src"].astype(dtype).astype(np.float64)
    out = np.empty((c["per_item"], c["width"], c["n"]))
    for w in range(c["width"]):
        for slot in range(c["per_item"]):
            out[slot, w] = wf[:, int(c["ids2"][w, slot]), :] @ src[w]
    return out


def unpack_groups(c, packed_rows):
    """RemapFromReference (common/task/testing_ref_ops.cc:2835-2851)."""
    out = np.full((c["per_item"], c["width"], packed_rows.shape[1]), np.nan)
    for i, (slot, w) in enumerate(c["packed_map"]):
        out[slot, w] = packed_rows[i]
    return out


def run_packed_groups_oracle(o, c, precision, max_group_size=None, dst_before=None, sizes=None, offsets=None):
    ns = (c["n"] + 3) // 4
    pack = o.int8_as_uint8 if c["bits"] == 8 else o.int8_as_uint4
    packed = pack(c["w"], I4O4, ns)
    tokens = c["packed_src"].shape[0]
    act = tensor(o, o.to_slices(c["packed_src"]), precision)
    kind = o.SCALE_LINEAR if c["groups"] == 1 else o.SCALE_BLOCK
    sc = tensor(o, o.scale_to_hoio4_batched(c["scale"]), precision)
    zp = None if c["zp"] is None else tensor(o, o.scale_to_hoio4_batched(c["zp"]), precision)
    out = o.fc_packed_groups_kernel(act, c["sizes"] if sizes is None else sizes, c["offsets"] if offsets is None else offsets,
                                    packed, tokens, c["k"], c["n"], precision, c["bits"], kind, sc, zp, None, c["groups"],
                                    max_group_size, dst_before)
    return o.from_slices(to_f32(o, out, precision), c["n"])


@pytest.mark.parametrize("bits,groups,zp", [(8, 1, False), (4, 2, True)])
def test_packed_groups_reference_test_flow(oracle, bits, groups, zp):
    """The reference test's shape (64 -> 32 channels, 64 tokens, 16 matrices, 4 per token) through the
    reference test's own flow: pack by matrix, run the grouped kernel, unpack, compare with the
    per-token products; its tolerance eps * 2 * K (fully_connected_test_util.cc:2594-2595)."""
    o = oracle
    c = make_packed_groups_case(3 + bits, 64, 4, 64, 32, 16, bits, groups, zp)
    assert c["sizes"].sum() == 64 * 4 and c["packed_src"].shape == (256, 64)
    got = unpack_groups(c, run_packed_groups_oracle(o, c, o.PREC_F32))
    ref = packed_groups_expected(o, c)
    assert not np.isnan(got).any()
    assert np.abs(got - ref).max() <= 1e-6 * 2.0 * 64 * max(1.0, np.abs(ref).max())


def test_packed_groups_leaves_other_tokens_alone(oracle):
    """Tokens that no group covers keep what the tensor held; a group is cut at max_group_size and at
    the end of the tensor; a group of size 0 writes nothing."""
    o = oracle
    c = make_packed_groups_case(11, 16, 2, 32, 8, 4)
    tokens = c["packed_src"].shape[0]  # 32
    sizes = np.array([5, 0, 9, 40], np.int32)
    offsets = np.array([2, 7, 10, 28], np.int32)
    before = np.full((2, tokens, 4), 7.0, np.float32)
    got = run_packed_groups_oracle(o, c, o.PREC_F32, max_group_size=6, dst_before=before, sizes=sizes, offsets=offsets)
    written = np.zeros(tokens, bool)
    written[2:7] = True      # group 0: 5 tokens
    written[10:16] = True    # group 2: 9 cut to max_group_size 6
    written[28:32] = True    # group 3: cut at the end of the tensor
    assert np.all(got[~written] == 7.0) and not np.any(got[written] == 7.0)
    wf = batch_ids_float_weights(o, c).astype(np.float64)
    for g, (a, b) in {0: (2, 7), 2: (10, 16), 3: (28, 32)}.items():
        ref = c["packed_src"][a:b].astype(np.float64) @ wf[:, g, :].T
        assert np.abs(got[a:b] - ref).max() <= 1e-5
