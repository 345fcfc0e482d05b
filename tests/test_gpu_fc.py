"""GPU parity of the FullyConnected kernels, through the C-ABI, against the CPU oracle.

Bars: int32 results bit-exact; fp16-output paths max|err| <= 2e-2 * RMS(reference output)
(the tolerance the north star states); fp32 paths eps_f32 * (K+1), the reference tests'
own rule (common/task/testing_util.cc:328-331)."""
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

import mldhip as M
import workloads as W
from refmath import textbook  # noqa: F401  (re-exported: the other GPU tests import it from here)

FP16_TOL = 2e-2
# The int4 GEMV kernels: the streaming kernel (any layout) and the contiguous-strip kernel, which
# serves one token over weights packed in output groups of 16 slices.
W4_GEMV = ("fc_w4_stream_kernel", "fc_w4_strip_kernel")


def torch_cuda():
    import torch
    assert torch.cuda.is_available()
    return torch


def oracle_fc(o, case, precision=None, use_kernel=True, wg_y=1):
    """Oracle output [m][n] float32 for a workloads case."""
    m, k, n, bits, groups = case["m"], case["k"], case["n"], case["weight_bits"], case["groups"]
    f16 = case["tensor_dtype"] == np.float16
    if precision is None:
        precision = o.PREC_F32F16 if f16 else o.PREC_F32
    ns = (n + 3) // 4
    packed = (o.int8_as_uint4 if bits == 4 else o.int8_as_uint8)(case["w"], o.LAYOUT_I4O4, ns)
    conv = (lambda a: o.f32_to_f16_bits(a)) if f16 else (lambda a: np.asarray(a, np.float32))
    act = conv(o.to_slices(case["act"]))
    if groups == 1:
        sc = np.zeros(ns * 4, np.float32); sc[:n] = case["scale"][:, 0]
        kind = o.SCALE_LINEAR
        zp = None
        if case["zero_point"] is not None:
            zp = np.zeros(ns * 4, np.float32); zp[:n] = case["zero_point"][:, 0]
    else:
        sc = o.scale_to_hoio4(case["scale"]); kind = o.SCALE_BLOCK
        zp = None if case["zero_point"] is None else o.scale_to_hoio4(case["zero_point"])
    bias = None
    if case["bias"] is not None:
        bias = np.zeros(ns * 4, np.float32); bias[:n] = case["bias"]
        bias = conv(bias)
    out = o.fc_kernel(act, packed, m, k, n, precision, bits, kind, conv(sc),
                      None if zp is None else conv(zp), bias, groups, True, wg_y)
    out = o.f16_bits_to_f32(out) if f16 else out
    return o.from_slices(out, n)


def check_fp(got, ref, case, label=""):
    err = np.abs(got.astype(np.float64) - ref).max()
    rms = np.sqrt(np.mean(ref.astype(np.float64) ** 2))
    if case["tensor_dtype"] == np.float16:
        assert err <= FP16_TOL * rms, (label, err, rms)
    else:
        tol = 1.1920929e-7 * (case["k"] + 1) * max(1.0, np.abs(ref).max())
        assert err <= tol, (label, err, tol)
    return err / rms


def restatement_affordable(case, tokens=None):
    """The oracle's eight-channel path (fp16 tensors, no zero points) restates about 5e9 multiply-adds
    per second on 8 cores, the one-channel path 30 times fewer."""
    work = (case["m"] if tokens is None else tokens) * case["k"] * case["n"]
    fast = case["tensor_dtype"] == np.float16 and case["zero_point"] is None
    return work <= (1 << 33 if fast else 1 << 27)


def check_as_accurate_as(got, restatement, exact, case, label=""):
    """The sharp bar beside the stated tolerance: measured against the float64 result, the GPU's
    error (RMS and maximum over the outputs) is no larger than 1.5 x the error of the reference's own
    kernel, as the oracle restates it operation by operation (measured on this suite: 0.5-0.7 x in
    RMS, at most 1.11 x; at most 1.00 x in the maximum).  A kernel that rounds where the reference
    does not, or sums in a narrower type, fails this long before it fails 2e-2 x RMS.  The floor
    (a quarter of an output ulp at the RMS) keeps cases the restatement gets exactly right."""
    eg = np.abs(got.astype(np.float64) - exact)
    er = np.abs(restatement.astype(np.float64) - exact)
    rms = np.sqrt(np.mean(exact ** 2))
    floor = (2.0 ** -12 if case["tensor_dtype"] == np.float16 else 2.0 ** -25) * rms
    assert np.sqrt(np.mean(eg ** 2)) <= 1.5 * np.sqrt(np.mean(er ** 2)) + floor, (label, "rms", np.sqrt(np.mean(eg ** 2)), np.sqrt(np.mean(er ** 2)))
    assert eg.max() <= 1.5 * er.max() + floor, (label, "max", eg.max(), er.max())


def native_layout_differs(case):
    """True when the library asks for another int4 layout than the reference's (output groups)."""
    if case["weight_bits"] != 4:
        return False
    a = M.fc_int4_weights_desc(case["n"], case["k"])
    b = M.fc_int4_weights_desc(case["n"], case["k"], reference=True)
    return a.output_group_size != b.output_group_size


def run_case(oracle, case, expect_kernel=None, tune=None, layouts=None):
    """Runs the case through the C-ABI and checks it against the textbook reference and the oracle's
    restatement of the reference kernel.  int4 cases run in both weight layouts (the one the
    library asks for and the reference's) where they differ; `tune` = tuning knobs for the run."""
    torch_cuda()
    if layouts is None:
        layouts = [False, True] if native_layout_differs(case) else [True]
    got = None
    for reference_layout in layouts:
        print("case", {k: case[k] for k in ("m", "k", "n", "weight_bits", "groups")}, tune,
              "reference layout" if reference_layout else "library layout", flush=True)
        with M.tuning(**(tune or {})):
            dev = W.FcDevice(case, reference_layout=reference_layout)
            dev.run()
            got = dev.result()
            if expect_kernel:
                names = (expect_kernel,) if isinstance(expect_kernel, str) else tuple(expect_kernel)
                assert dev.op.kernel_name in names, dev.op.kernel_name
            # a second launch must reproduce the first bit for bit
            dev.run()
            assert np.array_equal(got, dev.result())
        ref_tb = textbook(case)
        check_fp(got, ref_tb, case, "textbook")
        if restatement_affordable(case):
            rest = oracle_fc(oracle, case).astype(np.float64)
            check_fp(got, rest, case, "kernel restatement")
            check_as_accurate_as(got, rest, ref_tb, case, dev.op.kernel_name)
    return got


def test_config1_int8_fp32(oracle):
    case = W.make_fc_case(**W.CONFIGS["c1"])
    run_case(oracle, case, "fc_w8_stream_kernel")


def test_config2_int4_decode(oracle):
    case = W.make_fc_case(**W.CONFIGS["c2"])
    run_case(oracle, case, W4_GEMV)


@pytest.mark.parametrize("lpr", [8, 16])
@pytest.mark.parametrize("waves", [4, 8, 16])
@pytest.mark.parametrize("ksplit", [1, 3, 16])
def test_stream_kernel_shapes(oracle, lpr, waves, ksplit):
    case = W.make_fc_case(seed=3, m=1, k=4096, n=1536, weight_bits=4, tensor_dtype=np.float16)
    run_case(oracle, case, "fc_w4_stream_kernel", dict(gemv_lpr=lpr, gemv_waves=waves, gemv_ksplit=ksplit, gemv_fast=0))


@pytest.mark.parametrize("m", [1, 2, 3, 4])
@pytest.mark.parametrize("groups", [1, 32])
def test_stream_kernel_variants_ragged(oracle, m, groups):
    # N = 8*129: the last 4-column block of the strip is partly outside the matrix
    case = W.make_fc_case(seed=17 + m, m=m, k=1024, n=1032, weight_bits=4, tensor_dtype=np.float16,
                          groups=groups, with_bias=True)
    run_case(oracle, case, W4_GEMV)


@pytest.mark.parametrize("m", [1, 2, 3, 4])
@pytest.mark.parametrize("groups", [1, 64])
def test_stream_kernel_tokens_and_groups(oracle, m, groups):
    case = W.make_fc_case(seed=5 + m, m=m, k=2048, n=2048, weight_bits=4, tensor_dtype=np.float16,
                          groups=groups, with_bias=True)
    run_case(oracle, case, W4_GEMV)


@pytest.mark.parametrize("m", [1, 3, 4])
@pytest.mark.parametrize("groups", [1, 64])
def test_stream_kernel_zero_points(oracle, m, groups):
    """Asymmetric int4 weights (a zero-point tensor shaped like the scales) on the streaming kernel."""
    case = W.make_fc_case(seed=23 + m, m=m, k=2048, n=1032, weight_bits=4, tensor_dtype=np.float16,
                          groups=groups, with_bias=True, with_zero_point=True)
    run_case(oracle, case, W4_GEMV)


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("m,k,n,groups,zp", [(1, 2048, 2048, 1, False), (4, 1000, 1030, 1, True), (3, 2048, 516, 64, True),
                                             (2, 4096, 8192, 16, False), (1, 64, 8, 1, False)])
def test_w8_stream_kernel(oracle, dtype, m, k, n, groups, zp):
    """int8 weights on the streaming kernel: both tensor types, per-channel and group-wise scales,
    zero points, ragged K (1000) and N (1030), tiny layers."""
    case = W.make_fc_case(seed=31 + m, m=m, k=k, n=n, weight_bits=8, tensor_dtype=dtype, groups=groups,
                          with_bias=True, with_zero_point=zp)
    run_case(oracle, case, "fc_w8_stream_kernel")


@pytest.mark.parametrize("name,k,n", W.C5_LAYER)
def test_config5_decode_layer_shapes(oracle, name, k, n):
    case = W.make_fc_case(seed=7, m=1, k=k, n=n, weight_bits=4, tensor_dtype=np.float16, groups=k // 32)
    run_case(oracle, case, W4_GEMV)


def test_stream_kernel_ragged(oracle):
    # K not a multiple of 32 (partial chunk), N = 8*odd (partial strip)
    case = W.make_fc_case(seed=11, m=2, k=1000, n=1032, weight_bits=4, tensor_dtype=np.float16)
    run_case(oracle, case, W4_GEMV)


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("kind", ["linear", "block", "block_zp"])
def test_generic_kernel_reference_test_shapes(oracle, bits, dtype, kind):
    """Shapes of the reference's big tests: K=171 or 11*4*7, N=533, tokens 1/4/15."""
    k = 171 if kind == "linear" else 11 * 4 * 7
    groups = 1 if kind == "linear" else 7
    for m in (1, 4, 15):
        case = W.make_fc_case(seed=13 + m, m=m, k=k, n=533, weight_bits=bits, tensor_dtype=dtype,
                              groups=groups, with_bias=True, with_zero_point=kind == "block_zp",
                              act_uniform=True)
        # (N=533 gives an even slice count, so the symmetric fp16 int4 cases take the streaming kernel)
        fast = bits == 4 and dtype == np.float16 and kind == "linear"
        expect = "fc_generic_kernel"
        if fast:  # symmetric fp16 int4: streaming GEMV up to 4 tokens, MFMA GEMM beyond
            expect = W4_GEMV if m <= 4 else "fc_w4_mfma_gemm_kernel"
        if bits == 8 and kind == "linear" and m <= 4:  # per-channel int8, either tensor type
            expect = "fc_w8_stream_kernel"
        if bits == 8 and kind == "linear" and m > 4 and dtype == np.float16:
            expect = "fc_w8_mfma_gemm_kernel"
        run_case(oracle, case, expect)


def test_known_answers_on_gpu():
    """Literal cases of common/kernels/tests/fully_connected_test_util.cc:49-249, 1541-1614."""
    torch = torch_cuda()
    # scalar scale 0.5 + bias -> {20.5, 15.5}
    case = dict(m=1, k=4, n=2, weight_bits=8, tensor_dtype=np.float32, groups=1,
                act=np.array([[0, 1, 2, 3]], np.float32),
                w=np.array([[2, 4, 6, 8], [10, 12, -14, 16]], np.int8),
                scale=np.ones((2, 1), np.float32), bias=np.array([0.5, -0.5], np.float32), zero_point=None)
    dev = W.FcDevice(case, scalar_scale=0.5)
    dev.run()
    assert np.allclose(dev.result(), [[20.5, 15.5]], atol=1e-6)
    # block-wise -> {91.0, 26.8}
    case = dict(m=1, k=8, n=2, weight_bits=8, tensor_dtype=np.float32, groups=2,
                act=np.arange(8, dtype=np.float32)[None],
                w=np.array([[1, 1, 1, 1, 2, 2, 2, 2], [3, 3, 3, 3, 4, 4, 4, 4]], np.int8),
                scale=np.array([[0.5, 2.0], [1.0, 0.1]], np.float32), bias=np.zeros(2, np.float32),
                zero_point=None)
    dev = W.FcDevice(case); dev.run()
    assert np.allclose(dev.result(), [[91.0, 26.8]], atol=1e-5)
    # block-wise with zero points -> {509.0, -121.4}
    case.update(act=np.arange(1, 9, dtype=np.float32)[None],
                w=np.array([[1, 2, 3, 4, 5, 6, 7, 8], [-8, -7, -6, -5, -4, -3, -2, -1]], np.int8),
                scale=np.array([[0.5, 2.0], [1.5, 0.1]], np.float32),
                zero_point=np.array([[2, -3], [1, 4]], np.float32))
    dev = W.FcDevice(case); dev.run()
    assert np.allclose(dev.result(), [[509.0, -121.4]], atol=1e-4)
    # int4 block-wise all ones -> 8.0
    for dtype, eps in ((np.float32, 1e-6), (np.float16, 1e-2)):
        case = dict(m=1, k=16, n=4, weight_bits=4, tensor_dtype=dtype, groups=2,
                    act=np.ones((1, 16), np.float32), w=np.ones((4, 16), np.int8),
                    scale=np.full((4, 2), 0.5, np.float32), bias=np.zeros(4, np.float32), zero_point=None)
        dev = W.FcDevice(case); dev.run()
        assert np.allclose(dev.result(), np.full((1, 4), 8.0), atol=eps)


@pytest.mark.parametrize("m,k,n,zp,bias", [(2, 4096, 14336, False, False), (16, 4096, 8192, True, True),
                                            (3, 1000, 8200, False, True), (7, 171, 8200, True, False),
                                            (5, 4104, 8228, False, False), (9, 16384, 8192, False, False)])
def test_w4_mfma_stream_kernel(oracle, m, k, n, zp, bias):
    """2..16 tokens on wide per-channel int4 layers run on the matrix-core GEMV: ragged K (the last
    step, the last wave's share), ragged N, zero points, more than one chunk of steps per wave."""
    case = W.make_fc_case(seed=m + n, m=m, k=k, n=n, weight_bits=4, tensor_dtype=np.float16, groups=1,
                          with_zero_point=zp, with_bias=bias)
    print("w4 mfma stream", m, k, n, zp, bias, flush=True)
    # (2..4 tokens in whole strips with one chunk per thread would take the token form of the strip
    # kernel: switched off here, this test is about the 16-token matrix-core GEMV)
    with M.tuning(gemv_one_chunk=0):
        dev = W.FcDevice(case)
        dev.run()
        got = dev.result()
    assert dev.op.kernel_name == "fc_w4_mfma_stream_kernel", dev.op.kernel_name
    check_fp(got, textbook(case), case, "textbook")
    if m * k * n <= 1 << 26:
        check_fp(got, oracle_fc(oracle, case).astype(np.float64), case, "kernel restatement")
    with M.tuning(gemv_one_chunk=0):
        dev.run()
        assert np.array_equal(got, dev.result())


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("m,k,n", [(1, 112, 152), (5, 171, 533), (1, 2048, 2048), (16, 4096, 1024),
                                   (2, 171, 533), (3, 100, 8), (4, 1000, 4104), (1, 4096, 14336), (1, 36, 20)])
def test_int8_math_bit_exact(oracle, bits, m, k, n):
    """int8 activations x packed weights -> int32, exact (fully_connected_test_util.cc:1446-1448)."""
    torch = torch_cuda()
    rng = np.random.default_rng(k + n + bits)
    lo, hi = (-8, 8) if bits == 4 else (-128, 128)
    w = rng.integers(lo, hi, size=(n, k), dtype=np.int8)
    src = rng.integers(-128, 128, size=(m, k), dtype=np.int8)
    desc = M.fc_int4_weights_desc(n, k) if bits == 4 else M.fc_int8_weights_desc(n, k)
    packed = (M.rearrange_int8_as_uint4 if bits == 4 else M.rearrange_int8_as_uint8)(w, desc)
    act = torch.from_numpy(W.to_slices(src)).cuda()
    wt = torch.from_numpy(packed).cuda()
    out = torch.zeros(((n + 3) // 4, m, 4), dtype=torch.int32, device="cuda")
    op = M.fc_create(M.PRECISION_F32, M.INT8, M.INT32, n, k, desc, max_tokens=m)
    op.bind([act, wt], [out])
    op.set_shape(1, 1, m)
    print("int8 math", bits, m, k, n, flush=True)
    op.launch(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    got = W.from_slices(out.cpu().numpy(), n)
    ref = oracle.fc_reference_i8(src, w)
    assert np.array_equal(got, ref)
    # 1..4 tokens stream (uint4 rows with an odd number of slices keep the tiled kernel)
    streams = m <= 4 and (bits == 8 or ((n + 3) // 4) % 2 == 0)
    # one token over at least 128 whole strips of 64 channels and whole chunks of K: the strip form
    strips = bits == 4 and m == 1 and n % 64 == 0 and n // 64 >= 128 and k % 32 == 0
    assert op.kernel_name == ("fc_i8math_strip_kernel" if strips else "fc_i8math_stream_kernel" if streams
                              else "fc_int8_math_kernel"), op.kernel_name
    if m * k * n <= 1 << 24:  # the restatement reads the reference's layout
        ns = (n + 3) // 4
        packed_ref = (oracle.int8_as_uint4 if bits == 4 else oracle.int8_as_uint8)(w, oracle.LAYOUT_I4O4, ns)
        mimic = oracle.from_slices(oracle.fc_int8_kernel(oracle.to_slices(src), packed_ref, m, k, n, bits), n)
        assert np.array_equal(got, mimic)


@pytest.mark.parametrize("reference_layout", [False, True])
@pytest.mark.parametrize("k,n", [(4096, 14336), (1024, 8192), (2048, 8192), (3072, 8256), (8192, 8192), (32, 8192),
                                 (544, 16384)])
def test_int8_math_strip_kernel(oracle, k, n, reference_layout):
    """One token of int8 activations over uint4 weights in whole strips of 64 channels: one chunk per
    thread at K = 1024 / 2048 / 4096, the chunk loop otherwise (also with idle rows), output groups of
    16 slices and the reference's one group; exact."""
    torch = torch_cuda()
    rng = np.random.default_rng(k + n)
    w = rng.integers(-8, 8, size=(n, k), dtype=np.int8)
    src = rng.integers(-128, 128, size=(1, k), dtype=np.int8)
    desc = M.fc_int4_weights_desc(n, k, reference=reference_layout)
    packed = M.rearrange_int8_as_uint4(w, desc)
    act = torch.from_numpy(W.to_slices(src)).cuda()
    wt = torch.from_numpy(packed).cuda()
    out = torch.zeros((n // 4, 1, 4), dtype=torch.int32, device="cuda")
    op = M.fc_create(M.PRECISION_F32, M.INT8, M.INT32, n, k, desc, max_tokens=1)
    op.bind([act, wt], [out])
    op.set_shape(1, 1, 1)
    print("int8 math strips", k, n, reference_layout, desc.output_group_size, flush=True)
    op.launch(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert op.kernel_name == "fc_i8math_strip_kernel", op.kernel_name
    got = W.from_slices(out.cpu().numpy(), n)
    assert np.array_equal(got, oracle.fc_reference_i8(src, w))
    with M.tuning(gemv_one_chunk=0):
        out.zero_()
        op.launch(torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        assert op.kernel_name == "fc_i8math_stream_kernel", op.kernel_name
        assert np.array_equal(W.from_slices(out.cpu().numpy(), n), got)


@pytest.mark.parametrize("m,k,n,groups,bias", [(1, 2048, 16384, 64, False), (2, 2048, 16384, 64, True),
                                               (1, 4096, 14336, 1, False), (2, 1000, 1032, 1, True),
                                               (1, 512, 72, 16, False)])
@pytest.mark.parametrize("kind", ["gelu_tanh", "silu"])
def test_gated_pair(oracle, m, k, n, groups, bias, kind):
    run_gated_pair(oracle, m, k, n, groups, bias, kind, "fc_w4_gated_stream_kernel")


def run_gated_pair(oracle, m, k, n, groups, bias, kind, expect_kernel, ulp_check=True, bits=4):
    """dst = activation(gate(x)) * up(x) in one launch against the three separate steps: the two
    FullyConnected launches on the GPU, then the oracle's restatement of the sample's elementwise
    kernel on their fp16 outputs.  Bar: the FullyConnected bar, 2e-2 of the output RMS (the fused
    kernel adds K in another order, so a gate value can differ by an fp16 ulp); besides, 99 % of
    the elements must agree to 2 fp16 ulp."""
    torch = torch_cuda()
    gate_case = W.make_fc_case(seed=11 + n, m=m, k=k, n=n, weight_bits=bits, tensor_dtype=np.float16, groups=groups,
                               with_bias=bias)
    up_case = W.make_fc_case(seed=12 + n, m=m, k=k, n=n, weight_bits=bits, tensor_dtype=np.float16, groups=groups,
                             with_bias=bias)
    up_case["act"] = gate_case["act"]
    # gate values of a few units so that the activation is in its curved range
    gate_case["scale"] = gate_case["scale"] * np.float32(40.0)
    gate = W.FcDevice(gate_case)
    up = W.FcDevice(up_case)
    srcs = [gate.act, up.weights, up.scale] + ([up.bias] if bias else [])
    up.op.bind(srcs, [up.out])  # both read the same tensor
    print("gated", m, k, n, groups, bias, kind, flush=True)
    gate.run(); up.run()
    torch.cuda.synchronize()
    g16 = gate.out.cpu().numpy()
    u16 = up.out.cpu().numpy()
    ref = W.from_slices(oracle.gated_activation(g16, u16, kind).astype(np.float32), n).astype(np.float64)
    dst = torch.zeros_like(gate.out)
    M.fc_launch_gated(gate.op, up.op, M.GATE_GELU_TANH if kind == "gelu_tanh" else M.GATE_SILU, dst,
                      torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert gate.op.kernel_name == expect_kernel, gate.op.kernel_name
    got = W.from_slices(dst.cpu().numpy().astype(np.float32), n).astype(np.float64)
    rms = np.sqrt(np.mean(ref ** 2))
    assert rms > 0
    assert np.abs(got - ref).max() <= 2e-2 * rms
    if ulp_check:
        close = np.abs(got - ref) <= 2 * np.maximum(np.abs(ref), 2.0 ** -14) * 2.0 ** -10
        assert close.mean() >= 0.99, close.mean()
    # the two ops' own outputs are untouched by the gated launch
    assert np.array_equal(gate.out.cpu().numpy(), g16) and np.array_equal(up.out.cpu().numpy(), u16)


@pytest.mark.parametrize("m,k,n,groups,bias", [(3, 512, 72, 16, False), (16, 2048, 2048, 1, True),
                                               (64, 1024, 1032, 32, True), (77, 352, 200, 11, False),
                                               (128, 2048, 16384, 64, False), (130, 96, 260, 1, True),
                                               (2048, 256, 4096, 1, True),
                                               (129, 128, 8192, 4, True)])  # odd token count on the 64-token tile
@pytest.mark.parametrize("kind", ["gelu_tanh", "silu"])
def test_gated_pair_prefill(oracle, m, k, n, groups, bias, kind):
    """The same step at prefill token counts: the matrix-core GEMM with the gated epilogue (tiles of
    64 channels of both matrices), every token tile, ragged channel and token edges."""
    # Up to 4 tokens the separate launches run the streaming GEMV, which keeps the weights in fp32
    # where the matrix-core kernel rounds them to fp16: gate values then differ by a few fp16 ulp
    # (inside the FullyConnected bar) and the ulp-level comparison says nothing there.
    run_gated_pair(oracle, m, k, n, groups, bias, kind, "fc_w4_gated_mfma_gemm_kernel", ulp_check=m > 4)


@pytest.mark.parametrize("m,k,n,groups,bias", [(5, 512, 72, 16, False), (64, 1024, 1032, 32, True),
                                               (130, 96, 260, 1, True), (1024, 256, 4096, 1, False)])
@pytest.mark.parametrize("kind", ["gelu_tanh", "silu"])
def test_gated_pair_prefill_uint8(oracle, m, k, n, groups, bias, kind):
    """uint8 weights on the same gated matrix-core kernel (above the GEMV token counts)."""
    run_gated_pair(oracle, m, k, n, groups, bias, kind, "fc_w8_gated_mfma_gemm_kernel", bits=8)


def test_gated_pair_refused(oracle):
    torch = torch_cuda()
    a = W.FcDevice(W.make_fc_case(seed=1, m=3, k=256, n=64, weight_bits=4, tensor_dtype=np.float16, groups=1))
    b = W.FcDevice(W.make_fc_case(seed=2, m=3, k=256, n=64, weight_bits=4, tensor_dtype=np.float16, groups=1))
    dst = torch.zeros_like(a.out)
    with pytest.raises(M.MldhipError) as e:   # two different source tensors
        M.fc_launch_gated(a.op, b.op, M.GATE_SILU, dst, torch.cuda.current_stream().cuda_stream)
    assert e.value.code == M.FAILED_PRECONDITION
    # uint8 weights at GEMV token counts: left to the two streaming GEMVs and the host's elementwise node
    c8 = W.make_fc_case(seed=3, m=3, k=256, n=64, weight_bits=8, tensor_dtype=np.float16, groups=1)
    g8, u8 = W.FcDevice(c8), W.FcDevice(c8)
    u8.op.set_src(0, g8.act)
    with pytest.raises(M.MldhipError) as e:
        M.fc_launch_gated(g8.op, u8.op, M.GATE_SILU, torch.zeros_like(g8.out), torch.cuda.current_stream().cuda_stream)
    assert e.value.code == M.FAILED_PRECONDITION
    # a uint4 gate with a uint8 up
    c48 = W.make_fc_case(seed=3, m=8, k=256, n=64, weight_bits=8, tensor_dtype=np.float16, groups=1)
    c44 = W.make_fc_case(seed=3, m=8, k=256, n=64, weight_bits=4, tensor_dtype=np.float16, groups=1)
    gm, um = W.FcDevice(c44), W.FcDevice(c48)
    um.op.set_src(0, gm.act)
    with pytest.raises(M.MldhipError) as e:
        M.fc_launch_gated(gm.op, um.op, M.GATE_SILU, torch.zeros_like(gm.out), torch.cuda.current_stream().cuda_stream)
    assert e.value.code == M.FAILED_PRECONDITION
    # a destination that is too small
    c4 = W.make_fc_case(seed=4, m=8, k=256, n=64, weight_bits=4, tensor_dtype=np.float16, groups=1)
    g4, u4 = W.FcDevice(c4), W.FcDevice(c4)
    u4.op.set_src(0, g4.act)
    with pytest.raises(M.MldhipError) as e:
        M.fc_launch_gated(g4.op, u4.op, M.GATE_SILU, torch.zeros(16, dtype=torch.float16, device="cuda"),
                          torch.cuda.current_stream().cuda_stream)
    assert e.value.code == M.INVALID_ARGUMENT


def test_random_shapes_sweep(oracle):
    """Seeded sweep over token counts, ragged K / N and scale groupings, whatever kernel the
    dispatcher picks: every result against the textbook reference at the fp16 bar.  Covers the
    tile-plane edges of the kernels (odd tile counts per XCD rectangle, strips and K shares that
    end inside a work-group, token counts at the kernel boundaries)."""
    rng = np.random.default_rng(2024)
    seen = {}
    for it in range(48):
        m = int(rng.choice([1, 2, 3, 4, 5, 7, 16, 17, 31, 33, 64, 65, 100, 128, 129, 200, 257, 300]))
        bits = int(rng.choice([4, 4, 4, 8]))
        k = int(rng.choice([64, 96, 171, 256, 512, 1000, 1024, 2048, 4096])) if m > 4 else int(
            rng.choice([64, 171, 512, 1000, 2048, 4096, 8192]))
        n = int(rng.choice([8, 20, 64, 152, 533, 1024, 2050, 4096, 8200, 8228]))
        groups = 1
        if k % 32 == 0 and rng.random() < 0.6:
            groups = k // int(rng.choice([32, 64, k])) if k >= 64 else 1
        zp = bool(rng.random() < 0.3)
        bias = bool(rng.random() < 0.5)
        if m * k * n > 300 * 1024 * 8228:
            n = 1024
        case = W.make_fc_case(seed=1000 + it, m=m, k=k, n=n, weight_bits=bits, tensor_dtype=np.float16, groups=groups,
                              with_zero_point=zp, with_bias=bias)
        print("sweep", it, dict(m=m, k=k, n=n, bits=bits, groups=groups, zp=zp, bias=bias), flush=True)
        dev = W.FcDevice(case)
        dev.run()
        got = dev.result()
        seen[dev.op.kernel_name] = seen.get(dev.op.kernel_name, 0) + 1
        check_fp(got, textbook(case), case, "sweep %d (%s)" % (it, dev.op.kernel_name))
    print("kernels exercised:", seen)
    assert len(seen) >= 4


def test_random_layouts_sweep(oracle):
    """Seeded sweep over the weights layouts the op accepts (output groups of any size that divides
    the output slices: 1 is the FullyConnectedOI layout, 2 the decode layout, all slices the
    reference's FullyConnected layout), crossed with token counts, ragged K / N and scale
    groupings: every result against the textbook reference at the fp16 bar."""
    rng = np.random.default_rng(77)
    seen = {}
    for it in range(40):
        m = int(rng.choice([1, 1, 1, 2, 3, 4, 5, 16, 33, 64, 130]))
        bits = int(rng.choice([4, 4, 4, 8]))
        k = int(rng.choice([64, 100, 171, 512, 1000, 2048, 4096]))
        n = int(rng.choice([8, 24, 64, 152, 536, 1024, 2056, 4096, 8200]))
        ns = -(-n // 4)
        divisors = [g for g in range(1, ns + 1) if ns % g == 0]
        group = int(rng.choice([1, 2, ns, divisors[int(rng.integers(len(divisors)))]]))
        groups = 1
        if k % 32 == 0 and rng.random() < 0.6:
            groups = k // int(rng.choice([32, 64, k])) if k >= 64 else 1
        zp = bool(rng.random() < 0.3)
        bias = bool(rng.random() < 0.5)
        case = W.make_fc_case(seed=3000 + it, m=m, k=k, n=n, weight_bits=bits, tensor_dtype=np.float16, groups=groups,
                              with_zero_point=zp, with_bias=bias)
        print("layout sweep", it, dict(m=m, k=k, n=n, bits=bits, group=group, of=ns, groups=groups, zp=zp, bias=bias),
              flush=True)
        dev = W.FcDevice(case, output_group=group)
        dev.run()
        got = dev.result()
        seen[dev.op.kernel_name] = seen.get(dev.op.kernel_name, 0) + 1
        check_fp(got, textbook(case), case, "layout sweep %d (group %d, %s)" % (it, group, dev.op.kernel_name))
    print("kernels exercised:", seen)
    assert len(seen) >= 4


@pytest.mark.parametrize("group", [4, 8, 16])
@pytest.mark.parametrize("k,n,groups,zp,bias", [(2048, 2048, 64, False, True), (16384, 2048, 512, False, False),
                                               (4096, 1536, 1, True, True), (512, 256, 1, False, False),
                                               (2048, 16384, 64, True, False), (96, 64, 3, False, True)])
def test_strip_kernel_group_sizes(oracle, group, k, n, groups, zp, bias):
    """One token on the contiguous-strip kernel over weights packed in output groups of 4, 8 and 16
    slices: K inside the work-group and split across work-groups, per-channel and group-wise scales,
    zero points, a single chunk per wave row and several."""
    case = W.make_fc_case(seed=k + n + group, m=1, k=k, n=n, weight_bits=4, tensor_dtype=np.float16, groups=groups,
                          with_bias=bias, with_zero_point=zp)
    with M.tuning(fc_group=group):
        assert M.fc_int4_weights_desc(n, k).output_group_size == group
        got = run_case(oracle, case, "fc_w4_strip_kernel", layouts=[False])
    # K split across work-groups (a second kernel adds the sums in split order): inside the bar too
    for ksplit in (4, 7):
        if k // 32 >= ksplit:
            with M.tuning(fc_group=group, gemv_ksplit=ksplit):
                run_case(oracle, case, "fc_w4_strip_kernel", layouts=[False])


@pytest.mark.parametrize("reference_layout", [False, True])
@pytest.mark.parametrize("k,n,groups,bias", [(4096, 14336, 1, False), (2048, 16384, 64, True), (256, 8192, 1, True),
                                             (1024, 8192, 8, False), (512, 24576, 1, False)])
def test_strip_kernel_one_chunk_forms(oracle, k, n, groups, bias, reference_layout):
    """One token over at least 128 strips of 64 channels with K = 256 ... 4096: every thread owns exactly one
    chunk, and the strip kernel runs without a chunk loop, over contiguous strips (output groups of 16
    slices) and over strided ones (the reference's one output group).  With the form switched off the
    older kernels serve the same case; both are held to the oracle."""
    case = W.make_fc_case(seed=k + n, m=1, k=k, n=n, weight_bits=4, tensor_dtype=np.float16, groups=groups,
                          with_bias=bias)
    got = run_case(oracle, case, "fc_w4_strip_kernel", layouts=[reference_layout])
    other = run_case(oracle, case, "fc_w4_strip_kernel" if not reference_layout else "fc_w4_stream_kernel",
                     tune=dict(gemv_one_chunk=0), layouts=[reference_layout])
    # (another order of the K sum: a result may land on the neighbouring fp16 value)
    assert np.abs(got.astype(np.float64) - other).max() <= 2.0 ** -9 * np.abs(other).max()


@pytest.mark.parametrize("reference_layout", [False, True])
def test_strip_kernel_fused_launch_one_chunk_forms(oracle, reference_layout):
    """Two and three matrices that read one source tensor in one launch (one list of strips): the
    one-chunk forms give the bytes of the single launches, in both layouts."""
    torch = torch_cuda()
    shapes = [(1024, 8192, 32, True), (1024, 8256, 32, False), (1024, 8192, 32, False)]
    devs = []
    for i, (k, n, groups, bias) in enumerate(shapes):
        case = W.make_fc_case(seed=90 + i, m=1, k=k, n=n, weight_bits=4, tensor_dtype=np.float16, groups=groups, with_bias=bias)
        devs.append(W.FcDevice(case, reference_layout=reference_layout))
    for d in devs[1:]:  # the same source tensor for all
        d.op.bind([devs[0].act, d.weights, d.scale] + ([d.bias] if d.case["bias"] is not None else []), [d.out])
        d.case["act"] = devs[0].case["act"]
    single = []
    for d in devs:
        d.run()
        assert d.op.kernel_name == "fc_w4_strip_kernel", d.op.kernel_name
        single.append(d.result())
        check_fp(single[-1], textbook(d.case), d.case, "single launch")
        d.out.zero_()
    for count in (2, 3):
        print("fused one-chunk launch of", count, "matrices, reference layout" if reference_layout else "", flush=True)
        M.fc_launch_fused([d.op for d in devs[:count]], torch.cuda.current_stream().cuda_stream)
        for d, want in zip(devs[:count], single):
            assert d.op.kernel_name == "fc_w4_strip_kernel", d.op.kernel_name
            assert np.array_equal(d.result(), want)
            d.out.zero_()


def test_split_k_launches_repeat_bit_for_bit(oracle):
    """50 launches in a row of a K-split GEMV (the down projection of the decoder stack): the same
    bits every time."""
    case = W.make_fc_case(seed=77, m=1, k=16384, n=2048, weight_bits=4, tensor_dtype=np.float16, groups=512)
    dev = W.FcDevice(case)
    dev.run()
    assert dev.op.kernel_name == "fc_w4_strip_kernel"
    first = dev.result()
    check_fp(first, textbook(case), case, "textbook")
    import torch
    stream = torch.cuda.current_stream().cuda_stream
    for i in range(50):
        dev.out.zero_()
        dev.op.launch(stream)
        if i % 10 == 9:
            assert np.array_equal(dev.result(), first), i


@pytest.mark.parametrize("bits,k,n,groups", [(4, 4096, 2048, 1), (4, 1024, 1032, 32), (8, 2048, 2048, 1), (4, 171, 533, 1)])
@pytest.mark.parametrize("b,w", [(2, 4), (2, 1), (10, 3)])
def test_fc_tensor_batch(oracle, bits, k, n, groups, b, w):
    """Activation tensors with batch > 1 (the reference's big tests use B in {2, 10, 20},
    fully_connected_test_util.cc:935-1001): the token index of the buffer layout is
    (y*W + x)*B + b, so BHWC(b, 1, w, k) is b*w tokens; the result must be that of the same
    tokens given as BHWC(1, 1, b*w, k), bit for bit, and meet the FullyConnected bar."""
    import torch
    m = b * w
    case = W.make_fc_case(seed=b + w + n, m=m, k=k, n=n, weight_bits=bits, tensor_dtype=np.float16, groups=groups,
                          with_bias=True)
    print("fc batch", bits, k, n, groups, b, w, flush=True)
    dev = W.FcDevice(case)
    dev.op.set_shape(1, 1, m)
    dev.run()
    flat = dev.result()
    dev.out.zero_()
    dev.op.set_shape(b, 1, w)
    dev.run()
    batched = dev.result()
    assert np.array_equal(flat, batched)
    check_fp(batched, textbook(case), case, "textbook")
    if m * k * n <= 1 << 27:
        check_fp(batched, oracle_fc(oracle, case).astype(np.float64), case, "kernel restatement")


@pytest.mark.parametrize("bits,m,k,n,groups", [(4, 1, 4096, 2048, 1), (4, 3, 1024, 1032, 32), (8, 1, 2048, 2048, 16),
                                               (4, 64, 512, 384, 4), (8, 5, 171, 533, 1)])
def test_precision_f16_runs_with_float_accumulators(oracle, bits, m, k, n, groups):
    """CalculationsPrecision::kF16 (all arithmetic in half in the reference,
    common/kernels/fully_connected_util.cc:167-203) is accepted and computed like kF32_F16, with fp32
    accumulators: bit-identical to the op created with kF32_F16, hence inside the tolerance, and
    closer to the float64 result than the reference's all-half kernel as the oracle restates it."""
    case = W.make_fc_case(seed=bits + m + k, m=m, k=k, n=n, weight_bits=bits, tensor_dtype=np.float16, groups=groups,
                          with_bias=True)
    print("precision F16", bits, m, k, n, groups, flush=True)
    a = W.FcDevice(case, precision=M.PRECISION_F16)
    a.run()
    b = W.FcDevice(case, precision=M.PRECISION_F32_F16)
    b.run()
    got = a.result()
    assert a.op.kernel_name == b.op.kernel_name and np.array_equal(got, b.result())
    ref = textbook(case)
    check_fp(got, ref, case, "textbook")
    half = oracle_fc(oracle, case, precision=oracle.PREC_F16).astype(np.float64)
    assert np.sqrt(np.mean((got - ref) ** 2)) <= np.sqrt(np.mean((half - ref) ** 2)) + 2.0 ** -12 * np.sqrt(np.mean(ref ** 2))


@pytest.mark.parametrize("k,n,groups,zp,bias", [(2048, 2048, 64, False, True), (16384, 2048, 512, False, False),
                                               (4096, 1536, 1, True, True), (512, 256, 16, True, False),
                                               (2048, 16384, 64, False, False), (100, 72, 1, False, True),
                                               (171 * 4, 536, 1, False, False), (8192, 2048, 64, False, True),
                                               (40000, 64, 1, False, False)])
def test_rows_kernel(oracle, k, n, groups, zp, bias):
    """One token on the row-interleaved kernel over weights packed in output groups of 2 slices:
    per-channel and group-wise scales, zero points, K shorter than a work-group's rows, K that needs
    several passes, K that is no multiple of the rows per pass."""
    case = W.make_fc_case(seed=k + n, m=1, k=k, n=n, weight_bits=4, tensor_dtype=np.float16, groups=groups,
                          with_bias=bias, with_zero_point=zp)
    print("rows kernel", k, n, groups, zp, bias, flush=True)
    dev = W.FcDevice(case, output_group=2)
    dev.run()
    got = dev.result()
    assert dev.op.kernel_name == "fc_w4_rows_kernel", dev.op.kernel_name
    dev.out.zero_()
    dev.run()
    assert np.array_equal(got, dev.result())
    ref = textbook(case)
    check_fp(got, ref, case, "textbook")
    if k * n <= 1 << 27:
        rest = oracle_fc(oracle, case).astype(np.float64)
        check_fp(got, rest, case, "kernel restatement")
        check_as_accurate_as(got, rest, ref, case, "fc_w4_rows_kernel")
    for waves in (1, 4, 16):
        with M.tuning(gemv_waves=waves):
            dev.out.zero_()
            dev.run()
            check_fp(dev.result(), ref, case, "waves %d" % waves)


@pytest.mark.parametrize("reference_layout", [False, True])
@pytest.mark.parametrize("m", [2, 3, 4])
@pytest.mark.parametrize("k,n,groups,bias", [(4096, 14336, 1, False), (2048, 16384, 64, True), (256, 8192, 1, True),
                                             (1024, 8192, 8, False), (512, 24576, 16, False)])
def test_strip_tokens_kernel(oracle, m, k, n, groups, bias, reference_layout):
    """2..4 tokens over at least 128 strips of 64 channels with one chunk per thread: the token form of the
    strip kernel (4x4x4 MFMAs, a lane's block holds 32 channels of one token), per-channel and group-wise
    scales, contiguous and strided strips; against the textbook product, the kernel restatement and the
    kernels that served these launches before."""
    case = W.make_fc_case(seed=k + n + m, m=m, k=k, n=n, weight_bits=4, tensor_dtype=np.float16, groups=groups,
                          with_bias=bias)
    got = run_case(oracle, case, "fc_w4_strip_tokens_kernel", layouts=[reference_layout])
    other = run_case(oracle, case, ("fc_w4_stream_kernel", "fc_w4_mfma_stream_kernel"), tune=dict(gemv_mfma=0),
                     layouts=[reference_layout])
    # (another order of the K sum: a result may land on the neighbouring fp16 value)
    assert np.abs(got.astype(np.float64) - other).max() <= 2.0 ** -9 * np.abs(other).max()


def test_strip_tokens_kernel_fused_launch(oracle):
    """Two matrices that read one source tensor of 2 tokens in one launch give the bytes of the single launches."""
    torch = torch_cuda()
    devs = []
    for i, (k, n, groups, bias) in enumerate([(1024, 8192, 32, True), (1024, 8256, 32, False)]):
        case = W.make_fc_case(seed=95 + i, m=2, k=k, n=n, weight_bits=4, tensor_dtype=np.float16, groups=groups, with_bias=bias)
        devs.append(W.FcDevice(case))
    d = devs[1]
    d.op.bind([devs[0].act, d.weights, d.scale], [d.out])
    d.case["act"] = devs[0].case["act"]
    single = []
    for d in devs:
        d.run()
        assert d.op.kernel_name == "fc_w4_strip_tokens_kernel", d.op.kernel_name
        single.append(d.result())
        check_fp(single[-1], textbook(d.case), d.case, "single launch")
        d.out.zero_()
    M.fc_launch_fused([d.op for d in devs], torch.cuda.current_stream().cuda_stream)
    for d, want in zip(devs, single):
        assert d.op.kernel_name == "fc_w4_strip_tokens_kernel", d.op.kernel_name
        assert np.array_equal(d.result(), want)


@pytest.mark.parametrize("m", [2, 3, 4])
@pytest.mark.parametrize("k,n,groups,zp,bias", [(2048, 2048, 64, False, False), (2048, 2560, 1, True, True),
                                               (16384, 2048, 512, False, True), (172, 536, 1, False, False),
                                               (40000, 64, 1, True, False), (4096, 1536, 32, True, True)])
def test_rows_kernel_tokens(oracle, m, k, n, groups, zp, bias):
    """2..4 tokens over weights packed in output groups of 2 slices: the token form of the row-interleaved
    kernel (a slot of 2 or 4 tokens, 3 tokens in a slot of 4), K that needs several passes and K that is no
    multiple of the rows per pass; every work-group size the launcher can pick."""
    case = W.make_fc_case(seed=k + n + m, m=m, k=k, n=n, weight_bits=4, tensor_dtype=np.float16, groups=groups,
                          with_bias=bias, with_zero_point=zp)
    print("rows kernel", m, "tokens", k, n, groups, zp, bias, flush=True)
    dev = W.FcDevice(case, output_group=2)
    dev.run()
    got = dev.result()
    assert dev.op.kernel_name == "fc_w4_rows_kernel", dev.op.kernel_name
    dev.out.zero_()
    dev.run()
    assert np.array_equal(got, dev.result())
    ref = textbook(case)
    check_fp(got, ref, case, "textbook")
    if m * k * n <= 1 << 27:
        rest = oracle_fc(oracle, case).astype(np.float64)
        check_fp(got, rest, case, "kernel restatement")
        check_as_accurate_as(got, rest, ref, case, "fc_w4_rows_kernel")
    for waves in (1, 2, 8):
        with M.tuning(gemv_waves=waves):
            dev.out.zero_()
            dev.run()
            check_fp(dev.result(), ref, case, "waves %d" % waves)
    # the streaming kernel that served these launches before agrees within the bar
    with M.tuning(gemv_fast=0):
        dev.out.zero_()
        dev.run()
        assert dev.op.kernel_name == "fc_w4_stream_kernel", dev.op.kernel_name
        check_fp(dev.result(), ref, case, "streaming kernel")


@pytest.mark.parametrize("td", [np.float32, np.float16])
@pytest.mark.parametrize("k,n,groups,zp,bias", [(2048, 2048, 1, False, False), (2048, 2048, 64, True, True),
                                               (171, 536, 1, True, True), (16384, 256, 512, False, False),
                                               (4096, 1536, 1, False, True), (40, 8, 1, False, False),
                                               (10000, 64, 1, True, False)])
def test_w8_rows_kernel(oracle, td, k, n, groups, zp, bias):
    """One token over uint8 weights packed in output groups of one slice (the layout FullyConnectedOI
    reads) on the row-interleaved kernel: fp32 and fp16 tensors, per-channel and group-wise scales,
    zero points, ragged K, K shorter than a work-group's rows and K that needs several passes."""
    case = W.make_fc_case(seed=k + n + 1, m=1, k=k, n=n, weight_bits=8, tensor_dtype=td, groups=groups,
                          with_bias=bias, with_zero_point=zp)
    print("w8 rows kernel", td.__name__, k, n, groups, zp, bias, flush=True)
    dev = W.FcDevice(case, decode_layout=True)
    assert dev.desc.output_group_size == 1
    dev.run()
    got = dev.result()
    assert dev.op.kernel_name == "fc_w8_rows_kernel", dev.op.kernel_name
    dev.out.zero_()
    dev.run()
    assert np.array_equal(got, dev.result())
    ref = textbook(case)
    check_fp(got, ref, case, "textbook")
    if k * n <= 1 << 24:
        rest = oracle_fc(oracle, case).astype(np.float64)
        check_fp(got, rest, case, "kernel restatement")
    for waves in (1, 2, 8):
        with M.tuning(gemv_waves=waves):
            dev.out.zero_()
            dev.run()
            check_fp(dev.result(), ref, case, "waves %d" % waves)


@pytest.mark.parametrize("td", [np.float32, np.float16])
@pytest.mark.parametrize("m", [2, 3, 4])
@pytest.mark.parametrize("k,n,groups,zp,bias", [(2048, 2048, 1, False, False), (2048, 2048, 64, True, True),
                                               (171, 536, 1, True, True), (16384, 256, 512, False, False),
                                               (4096, 1536, 1, False, True), (40, 8, 1, False, False),
                                               (10000, 64, 1, True, False)])
def test_w8_rows_kernel_tokens(oracle, td, m, k, n, groups, zp, bias):
    """2..4 tokens over uint8 weights packed in output groups of one slice: the token form of the
    row-interleaved kernel (slots of 2 or 4 tokens, 3 tokens in a slot of 4), both tensor types, every
    work-group size, ragged K and K that needs several passes."""
    case = W.make_fc_case(seed=k + n + m, m=m, k=k, n=n, weight_bits=8, tensor_dtype=td, groups=groups,
                          with_bias=bias, with_zero_point=zp)
    print("w8 rows kernel", m, "tokens", td.__name__, k, n, groups, zp, bias, flush=True)
    dev = W.FcDevice(case, decode_layout=True)
    assert dev.desc.output_group_size == 1
    dev.run()
    got = dev.result()
    assert dev.op.kernel_name == "fc_w8_rows_tokens_kernel", dev.op.kernel_name
    dev.out.zero_()
    dev.run()
    assert np.array_equal(got, dev.result())
    ref = textbook(case)
    check_fp(got, ref, case, "textbook")
    if m * k * n <= 1 << 25:
        rest = oracle_fc(oracle, case).astype(np.float64)
        check_fp(got, rest, case, "kernel restatement")
    for waves in (1, 2, 8):
        with M.tuning(gemv_waves=waves):
            dev.out.zero_()
            dev.run()
            check_fp(dev.result(), ref, case, "waves %d" % waves)
    # the unspecialised kernel agrees within the bar
    with M.tuning(force_generic=1):
        dev.out.zero_()
        dev.run()
        assert dev.op.kernel_name == "fc_generic_kernel", dev.op.kernel_name
        check_fp(dev.result(), ref, case, "unspecialised kernel")


@pytest.mark.parametrize("m", [2, 3, 4])
@pytest.mark.parametrize("groups", [1, 32])
def test_w8_stream_kernel_tokens_long_k(oracle, m, groups):
    """2..4 tokens over uint8 weights in the library layout with a K long enough for the large
    work-group of the streaming kernel (8 waves at these token counts)."""
    case = W.make_fc_case(seed=61 + m, m=m, k=4096, n=2048, weight_bits=8, tensor_dtype=np.float16,
                          groups=groups, with_bias=True, with_zero_point=groups > 1)
    run_case(oracle, case, "fc_w8_stream_kernel")


def test_config1_decode_layout(oracle):
    """c1 over the layout mldhip_fc_int8_weights_desc_decode asks for, as the bench runs it."""
    case = W.make_fc_case(**W.CONFIGS["c1"])
    dev = W.FcDevice(case, decode_layout=True)
    dev.run()
    got = dev.result()
    assert dev.op.kernel_name == "fc_w8_rows_kernel", dev.op.kernel_name
    check_fp(got, textbook(case), case, "textbook")
    check_fp(got, oracle_fc(oracle, case).astype(np.float64), case, "kernel restatement")
