"""GPU parity of the prefill-side MFMA kernels, through the C-ABI.

int4 GEMM (fp16 out): max|err| <= 2e-2 * RMS(reference output) against the textbook reference
over dequantised weights and, at sizes the oracle finishes quickly, against the restatement
of the reference's generated kernel.
int8 x int8: int32 accumulators bit-exact against the closed-form integer product; the
rescaled fp16 output is compared with the oracle's epilogue applied to the same accumulators."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

import mldhip as M
import workloads as W
from test_gpu_fc import check_as_accurate_as, check_fp, oracle_fc, restatement_affordable, textbook

FP16_TOL = 2e-2


def check_restatement(oracle, got, case, label):
    """Against the oracle's restatement of the reference kernel: the stated tolerance, and no less
    accurate (against float64) than that kernel itself."""
    rest = oracle_fc(oracle, case).astype(np.float64)
    check_fp(got, rest, case, label)
    check_as_accurate_as(got, rest, textbook(case), case, label)


def run_w4(case, reference_layout=None):
    """Runs the case on the matrix-core GEMM.  int4 cases whose library layout (output groups of 16
    slices) differs from the reference's run in both, and the two results must agree bit for bit:
    the layout moves the blocks in memory, not the order of the arithmetic."""
    print("w%d gemm" % case["weight_bits"], {k: case[k] for k in ("m", "k", "n", "groups")}, reference_layout, flush=True)
    from test_gpu_fc import native_layout_differs
    layouts = [reference_layout] if reference_layout is not None else ([False, True] if native_layout_differs(case) else [True])
    results = []
    for ref_layout in layouts:
        dev = W.FcDevice(case, reference_layout=ref_layout)
        dev.run()
        got = dev.result()
        assert dev.op.kernel_name == "fc_w%d_mfma_gemm_kernel" % case["weight_bits"], dev.op.kernel_name
        dev.run()
        assert np.array_equal(got, dev.result())
        results.append(got)
    if len(results) == 2:
        assert np.array_equal(results[0], results[1]), "the two weight layouts give different sums"
    return results[0]


@pytest.mark.parametrize("m,k,n,groups", [(16, 256, 128, 8), (5, 64, 8, 1), (128, 2048, 2048, 64),
                                          (77, 352, 200, 11), (130, 96, 260, 1), (64, 4096, 256, 128),
                                          (300, 1024, 1024, 8)])
def test_w4_gemm_shapes(oracle, m, k, n, groups):
    case = W.make_fc_case(seed=m + n, m=m, k=k, n=n, weight_bits=4, tensor_dtype=np.float16, groups=groups,
                          with_bias=(m % 2 == 1))
    got = run_w4(case)
    check_fp(got, textbook(case), case, "textbook")
    if restatement_affordable(case):
        check_restatement(oracle, got, case, "kernel restatement")


@pytest.mark.parametrize("m,k,n,groups", [(16, 256, 128, 8), (77, 1024, 200, 1), (128, 2048, 2048, 64)])
def test_w4_gemm_zero_points(oracle, m, k, n, groups):
    """Asymmetric int4 weights (a zero-point tensor shaped like the scales) on the MFMA kernel."""
    case = W.make_fc_case(seed=m + 3 * n, m=m, k=k, n=n, weight_bits=4, tensor_dtype=np.float16, groups=groups,
                          with_bias=True, with_zero_point=True)
    got = run_w4(case)
    check_fp(got, textbook(case), case, "textbook")
    if restatement_affordable(case):
        check_restatement(oracle, got, case, "kernel restatement")


@pytest.mark.parametrize("m,k,n,groups,zp", [(2048, 64, 4096, 2, False), (2050, 96, 4000, 1, False),
                                             (4096, 128, 2048, 4, True)])
def test_w4_gemm_wide_token_tile(oracle, m, k, n, groups, zp):
    """Launches big enough for the 128-token tile (one wave per SIMD, four MFMAs per dequantized
    operand), with ragged token / channel edges and K ranges that end inside a wave's share."""
    case = W.make_fc_case(seed=m + n, m=m, k=k, n=n, weight_bits=4, tensor_dtype=np.float16, groups=groups,
                          with_bias=True, with_zero_point=zp)
    got = run_w4(case)
    check_fp(got, textbook(case), case, "textbook")
    sub = dict(case, m=64, act=case["act"][:64])
    check_restatement(oracle, got[:64], sub, "kernel restatement (first 64 tokens)")


@pytest.mark.parametrize("m,k,n,groups,zp", [(16, 256, 128, 8, False), (5, 64, 8, 1, True), (128, 2048, 2048, 64, False),
                                             (77, 352, 200, 11, True), (130, 96, 260, 1, False),
                                             (64, 4096, 256, 128, True), (300, 1024, 1024, 8, False),
                                             (2048, 64, 4096, 2, True), (2050, 96, 4000, 1, False)])
def test_w8_gemm_shapes(oracle, m, k, n, groups, zp):
    """uint8 weights (16-byte blocks, u = w + 128) through the same matrix-core kernel: every token
    tile (32, 64, paired 64, 128), ragged edges, per-channel and group-wise scales, zero points."""
    case = W.make_fc_case(seed=2 * m + n, m=m, k=k, n=n, weight_bits=8, tensor_dtype=np.float16, groups=groups,
                          with_bias=(m % 2 == 1), with_zero_point=zp)
    got = run_w4(case)
    check_fp(got, textbook(case), case, "textbook")
    small = m if restatement_affordable(case) else min(m, 64)
    sub = dict(case, m=small, act=case["act"][:small])
    if restatement_affordable(sub):
        check_restatement(oracle, got[:small], sub, "kernel restatement")


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("m,k,n,groups", [(33, 512, 260, 4), (256, 1024, 512, 1)])
def test_gemm_fractional_zero_points(oracle, bits, m, k, n, groups):
    """Zero points that are not whole numbers (what `file / scale` of a checkpoint can give): the
    kernel applies them as -(zp * s) inside a fused multiply-add, not by moving the integer centre."""
    case = W.make_fc_case(seed=7 * m + bits, m=m, k=k, n=n, weight_bits=bits, tensor_dtype=np.float16, groups=groups,
                          with_bias=True, with_zero_point=True)
    rng = np.random.default_rng(m + bits)
    spread = 3.0 if bits == 4 else 40.0
    case["zero_point"] = rng.uniform(-spread, spread, size=(n, groups)).astype(np.float16).astype(np.float32)
    # activations with a mean, so that an error in the centre does not average out
    case["act"] = (case["act"].astype(np.float32) + 0.5).astype(np.float16)
    got = run_w4(case)
    check_fp(got, textbook(case), case, "textbook")
    small = min(m, 64)
    sub = dict(case, m=small, act=case["act"][:small])
    check_restatement(oracle, got[:small], sub, "kernel restatement")


@pytest.mark.parametrize("m,k,n,groups,zp,bias", [(256, 64, 256, 1, False, False),     # one tile, two stages
                                                  (300, 352, 1000, 11, True, True),    # ragged edges, 11 stages of one group each
                                                  (1026, 96, 260, 1, False, True),     # 5 token tiles, the last of 2 tokens
                                                  (512, 4096, 512, 128, False, False),
                                                  (2048, 64, 4096, 2, True, True),
                                                  (130, 1024, 640, 8, False, True),
                                                  (258, 160, 516, 1, True, False)])
def test_w4_gemm_tiled_kernel(oracle, m, k, n, groups, zp, bias):
    """The LDS-tiled int4 GEMM (256 x 256 tiles, weights dequantized once per work-group), forced on
    shapes of test size: ragged token and channel edges, stage counts that are no multiple of the
    four the loop is unrolled by, group-wise scales down to one stage per group, zero points, bias,
    both weight layouts (which must agree bit for bit)."""
    case = W.make_fc_case(seed=m + n + k, m=m, k=k, n=n, weight_bits=4, tensor_dtype=np.float16, groups=groups,
                          with_bias=bias, with_zero_point=zp)
    print("tiled gemm", m, k, n, groups, zp, bias, flush=True)
    from test_gpu_fc import native_layout_differs
    results = []
    with M.tuning(gemm_tiled=1):
        for ref_layout in ([False, True] if native_layout_differs(case) else [True]):
            dev = W.FcDevice(case, reference_layout=ref_layout)
            dev.run()
            got = dev.result()
            assert dev.op.kernel_name == "fc_w4_mfma_tiled_kernel", dev.op.kernel_name
            dev.out.zero_()
            dev.run()
            assert np.array_equal(got, dev.result())
            results.append(got)
    if len(results) == 2:
        assert np.array_equal(results[0], results[1]), "the two weight layouts give different sums"
    got = results[0]
    check_fp(got, textbook(case), case, "textbook")
    small = min(m, 64)
    sub = dict(case, m=small, act=case["act"][:small])
    if restatement_affordable(sub):
        check_restatement(oracle, got[:small], sub, "kernel restatement")
    # the last tokens too (the ragged token tile)
    tail = dict(case, m=min(m, 32), act=case["act"][-min(m, 32):])
    if restatement_affordable(tail):
        check_restatement(oracle, got[-min(m, 32):], tail, "kernel restatement (last tokens)")


def test_w4_gemm_tiled_kernel_chosen_for_one_round_of_large_tiles(oracle):
    """1024 tokens x 14336 channels are 224 tiles of 256 x 256 (one round of the 256 CUs) and 896 of
    128 x 128 (three and a half): the launcher takes the LDS-tiled kernel by itself; a forced direct
    launch agrees within the bar."""
    case = W.make_fc_case(seed=77, m=1024, k=256, n=14336, weight_bits=4, tensor_dtype=np.float16, groups=8, with_bias=True)
    dev = W.FcDevice(case)
    dev.run()
    got = dev.result()
    assert dev.op.kernel_name == "fc_w4_mfma_tiled_kernel", dev.op.kernel_name
    ref = textbook(case)
    check_fp(got, ref, case, "textbook")
    with M.tuning(gemm_tiled=0):
        dev.out.zero_()
        dev.run()
        assert dev.op.kernel_name == "fc_w4_mfma_gemm_kernel", dev.op.kernel_name
        check_fp(dev.result(), ref, case, "direct kernel")
    sub = dict(case, m=64, act=case["act"][:64])
    check_restatement(oracle, got[:64], sub, "kernel restatement (first 64 tokens)")


def test_w4_gemm_tiled_kernel_full_size(oracle):
    """The LDS-tiled kernel at the size its launcher picks it for (1024 tokens x 4096 x 14336, scale groups of
    32 channels: 128 stages per tile): every output against the textbook reference, the first and the last 32
    tokens against the restatement of the reference's kernel."""
    case = W.make_fc_case(seed=5, m=1024, k=4096, n=14336, weight_bits=4, tensor_dtype=np.float16, groups=128)
    dev = W.FcDevice(case)
    dev.run()
    got = dev.result()
    assert dev.op.kernel_name == "fc_w4_mfma_tiled_kernel", dev.op.kernel_name
    check_fp(got, textbook(case), case, "textbook")
    for name, rows in (("first", slice(0, 32)), ("last", slice(-32, None))):
        sub = dict(case, m=32, act=case["act"][rows])
        check_restatement(oracle, got[rows], sub, "kernel restatement (%s 32 tokens)" % name)


@pytest.mark.parametrize("bits,m,k,n,groups,zp", [(4, 64, 512, 384, 4, False),    # 3 channel tiles: the last pair holds one
                                                  (4, 130, 352, 1000, 11, True),   # ragged channels and tokens, 64-token tile
                                                  (4, 256, 96, 260, 1, False),
                                                  (8, 128, 1024, 640, 8, True),
                                                  (4, 4096, 64, 2048, 2, True),    # 128-token tile
                                                  (8, 2050, 96, 1100, 1, False)])
def test_gemm_two_tiles_per_work_group(oracle, bits, m, k, n, groups, zp):
    """The two-tile mode (half of a work-group's waves per channel tile), forced on shapes of test
    size: odd tile counts, ragged edges, zero points, both weight types, both token tiles; and
    the same bytes as the one-tile mode where the K shares coincide is not required - the bar is
    the FullyConnected one."""
    case = W.make_fc_case(seed=m + n + bits, m=m, k=k, n=n, weight_bits=bits, tensor_dtype=np.float16, groups=groups,
                          with_bias=True, with_zero_point=zp)
    with M.tuning(gemm_dual=1):
        got = run_w4(case)
    check_fp(got, textbook(case), case, "textbook")
    small = m if restatement_affordable(case) else min(m, 64)
    sub = dict(case, m=small, act=case["act"][:small])
    if restatement_affordable(sub):
        check_restatement(oracle, got[:small], sub, "kernel restatement")


def test_gemm_modes_random_sweep():
    """Seeded sweep over shapes with the two-tile mode forced on and off and every token tile
    forced in turn: all against the textbook reference at the fp16 bar."""
    rng = np.random.default_rng(31)
    for it in range(24):
        bits = int(rng.choice([4, 8]))
        m = int(rng.choice([6, 33, 64, 66, 128, 130, 258, 300]))
        k = int(rng.choice([64, 96, 352, 512, 1024]))
        n = int(rng.choice([8, 100, 128, 260, 384, 1000]))
        groups = 1
        gs = int(rng.choice([32, 64]))
        if k % gs == 0 and rng.random() < 0.6:
            groups = k // gs
        zp = bool(rng.random() < 0.4)
        case = W.make_fc_case(seed=900 + it, m=m, k=k, n=n, weight_bits=bits, tensor_dtype=np.float16, groups=groups,
                              with_bias=bool(it % 2), with_zero_point=zp)
        with M.tuning(gemm_dual=it % 2, gemm_fm=[1, 2, 4][it % 3]):
            got = run_w4(case, reference_layout=bool((it // 6) % 2))
        check_fp(got, textbook(case), case, "sweep %d" % it)


def test_gemm_two_tiles_fused_launch():
    """Three matrices in one two-tile launch: pairs of tiles that straddle two matrices (3 + 1 + 2
    channel tiles) against the single one-tile launches."""
    import torch
    m, k = 128, 512
    cases = [W.make_fc_case(seed=60 + i, m=m, k=k, n=n, weight_bits=4, tensor_dtype=np.float16, groups=4, with_bias=True)
             for i, n in enumerate((384, 100, 256))]
    for c in cases[1:]:
        c["act"] = cases[0]["act"]
    devs = [W.FcDevice(c) for c in cases]
    for d in devs[1:]:
        d.op.set_src(0, devs[0].act)
    single = []
    with M.tuning(gemm_dual=0):
        for d in devs:
            d.run()
            single.append(d.result())
            d.out.zero_()
    with M.tuning(gemm_dual=1):
        M.fc_launch_fused([d.op for d in devs], torch.cuda.current_stream().cuda_stream)
    for d, c, ref in zip(devs, cases, single):
        got = d.result()
        check_fp(got, textbook(c), c, "two-tile fused")
        rms = np.sqrt(np.mean(textbook(c) ** 2))
        assert np.abs(got - ref).max() <= 2e-3 * rms  # another K split among the waves: fp32 summation order


def test_fused_prefill_2048_tokens_default_modes():
    """q / k / v of the decoder stack (2048 -> 2048, 256, 256, group 32) at 2048 tokens in one launch with
    the dispatcher's own choices (128-token tiles, two channel tiles per work-group, pairs that
    straddle matrices): every output against the textbook reference."""
    import torch
    m, k = 2048, 2048
    cases = [W.make_fc_case(seed=70 + i, m=m, k=k, n=n, weight_bits=4, tensor_dtype=np.float16, groups=64)
             for i, n in enumerate((2048, 256, 256))]
    for c in cases[1:]:
        c["act"] = cases[0]["act"]
    devs = [W.FcDevice(c) for c in cases]
    for d in devs[1:]:
        d.op.set_src(0, devs[0].act)
    M.fc_launch_fused([d.op for d in devs], torch.cuda.current_stream().cuda_stream)
    for d, c in zip(devs, cases):
        check_fp(d.result(), textbook(c), c, "fused prefill n=%d" % c["n"])


def test_gemm_two_tiles_chosen_for_large_launches():
    """4096 x 4096 x 4096 (1024 tiles) runs in the two-tile mode by default and meets the bar."""
    case = W.make_fc_case(seed=5, m=4096, k=4096, n=4096, weight_bits=4, tensor_dtype=np.float16, groups=1)
    got = run_w4(case)
    check_fp(got, textbook(case), case, "textbook")


def test_w8_gemm_fused_launch():
    """Three uint8 matrices over one activation tensor in one launch give the bytes of the three
    single launches; a uint4 op cannot join them."""
    import torch
    m, k = 96, 512
    cases = [W.make_fc_case(seed=40 + i, m=m, k=k, n=n, weight_bits=8, tensor_dtype=np.float16, groups=4, with_bias=True)
             for i, n in enumerate((384, 128, 200))]
    for c in cases[1:]:
        c["act"] = cases[0]["act"]
    devs = [W.FcDevice(c) for c in cases]
    for d in devs[1:]:
        d.op.set_src(0, devs[0].act)
    single = []
    for d in devs:
        d.run()
        single.append(d.result())
        assert d.op.kernel_name == "fc_w8_mfma_gemm_kernel"
        d.out.zero_()
    M.fc_launch_fused([d.op for d in devs], torch.cuda.current_stream().cuda_stream)
    for d, c, ref in zip(devs, cases, single):
        got = d.result()
        check_fp(got, textbook(c), c, "fused uint8")
        assert np.array_equal(got, ref)
    other = W.make_fc_case(seed=50, m=m, k=k, n=128, weight_bits=4, tensor_dtype=np.float16, groups=4)
    other["act"] = cases[0]["act"]
    d4 = W.FcDevice(other)
    d4.op.set_src(0, devs[0].act)
    with pytest.raises(M.MldhipError) as err:
        M.fc_launch_fused([devs[0].op, d4.op])
    assert err.value.code == M.FAILED_PRECONDITION


def test_config3_prefill_gemm(oracle):
    case = W.make_fc_case(**W.CONFIGS["c3"])
    got = run_w4(case)
    rel = check_fp(got, textbook(case), case, "textbook")
    print("c3 max|err|/rms = %.3e" % rel)
    # every output of every tile against the restatement of the generated kernel (8.6e9 multiply-adds:
    # a few seconds on the oracle's eight-channel path), to the stated tolerance and to the bar "no less
    # accurate than the reference's kernel"
    check_restatement(oracle, got, case, "kernel restatement, all 512 x 4096 outputs")


def test_config5_prefill_shapes(oracle):
    for name, k, n in W.C5_LAYER:
        case = W.make_fc_case(seed=9, m=128, k=k, n=n, weight_bits=4, tensor_dtype=np.float16, groups=k // 32)
        got = run_w4(case)
        check_fp(got, textbook(case), case, name)


def make_int8_case(seed, m, k, n, with_zp=False, with_bias=False):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((m, k)).astype(np.float16)
    w = rng.integers(-127, 128, size=(n, k), dtype=np.int8)
    ws = (np.abs(rng.normal(0, 0.02, size=n)) / 127).astype(np.float32)
    wzp = rng.integers(-4, 5, size=n).astype(np.float32) if with_zp else None
    bias = (rng.uniform(-1, 1, size=n) * 0.1).astype(np.float16) if with_bias else None
    return dict(m=m, k=k, n=n, x=x, w=w, ws=ws, wzp=wzp, bias=bias)


def pad4(a, dtype):
    a = np.asarray(a, dtype).ravel()
    out = np.zeros((a.size + 3) // 4 * 4, dtype)
    out[:a.size] = a
    return out


def run_int8_pipeline(oracle, c, symmetric):
    """quantize (GPU) -> int8 MFMA conv (GPU): returns codes, params, int32 acc, fp16 out."""
    import torch
    m, k, n = c["m"], c["k"], c["n"]
    print("int8 pipeline", m, k, n, symmetric, flush=True)
    stream = torch.cuda.current_stream().cuda_stream
    src = torch.from_numpy(W.to_slices(c["x"])).cuda()
    k16 = (k + 15) // 16
    codes = torch.zeros((k16, m, 16), dtype=torch.int8, device="cuda")
    params = torch.zeros((m, 4), dtype=torch.float32, device="cuda")
    q = M.quantization_create(M.FLOAT16, M.PACKED_INT8C16, k, calculate_sum=True, symmetric=symmetric, max_tokens=m)
    q.bind([src], [codes, params])
    q.set_shape(1, 1, m)
    q.launch(stream)
    wd = M.conv_int8_weights_desc(n, k)
    wt = torch.from_numpy(M.rearrange_int8(c["w"], wd)).cuda()
    ns = (n + 3) // 4
    acc = torch.zeros((ns, m, 4), dtype=torch.int32, device="cuda")
    conv_raw = M.conv_int8_create(M.INT32, n, k, wd, max_tokens=m)
    conv_raw.bind([codes, wt], [acc])
    conv_raw.set_shape(1, 1, m)
    conv_raw.launch(stream)
    wsum = torch.from_numpy(pad4(M.weights_sum_i(c["w"]), np.int32)).cuda()
    wscale = torch.from_numpy(pad4(c["ws"], np.float32)).cuda()
    srcs = [codes, wt, params, wsum, wscale]
    if c["wzp"] is not None:
        srcs.append(torch.from_numpy(pad4(c["wzp"], np.float32)).cuda())
    if c["bias"] is not None:
        srcs.append(torch.from_numpy(pad4(c["bias"], np.float16)).cuda())
    out = torch.zeros((ns, m, 4), dtype=torch.float16, device="cuda")
    conv = M.conv_int8_create(M.FLOAT16, n, k, wd, has_zero_point=c["wzp"] is not None,
                              has_bias=c["bias"] is not None, max_tokens=m)
    conv.bind(srcs, [out])
    conv.set_shape(1, 1, m)
    conv.launch(stream)
    torch.cuda.synchronize()
    assert conv.kernel_name == "conv_int8_mfma_kernel"
    return codes.cpu().numpy(), params.cpu().numpy(), acc.cpu().numpy(), out.cpu().numpy()


def check_int8(oracle, c, symmetric):
    o = oracle
    m, k, n = c["m"], c["k"], c["n"]
    codes, params, acc, out = run_int8_pipeline(o, c, symmetric)
    # activation codes and params: bit-exact
    src_bits = o.f32_to_f16_bits(W.to_slices(c["x"]).astype(np.float32))
    rcodes, rparams = o.quantize(src_bits, m, k, o.PACKED_INT8C16, symmetric, True)
    assert np.array_equal(codes, rcodes)
    assert np.array_equal(params.view(np.uint32), rparams.view(np.uint32))
    # int32 accumulators: exact integer product
    q = rcodes.transpose(1, 0, 2).reshape(m, -1)[:, :k]
    ref_acc = q.astype(np.int64) @ c["w"].astype(np.int64).T
    assert np.array_equal(W.from_slices(acc, n).astype(np.int64), ref_acc)
    if m * k * n <= 1 << 24:
        assert np.array_equal(ref_acc, o.fc_reference_i8(q, c["w"]))
    # rescaled output: the oracle's epilogue on the same accumulators
    ref_out = o.dequantize(W.to_slices(ref_acc.astype(np.int32)), rparams, o.weights_sum_i(c["w"]), c["ws"], n, k,
                           weights_zero_point=c["wzp"],
                           bias=None if c["bias"] is None else c["bias"].view(np.uint16), dst_f16=True)
    ref_f = W.from_slices(o.f16_bits_to_f32(ref_out), n)
    got_f = W.from_slices(out.astype(np.float32), n)
    rms = np.sqrt(np.mean(ref_f.astype(np.float64) ** 2))
    assert np.abs(got_f - ref_f).max() <= FP16_TOL * rms
    mismatch = np.count_nonzero(out.view(np.uint16).ravel()[: ref_out.size] != ref_out.ravel())
    print("fp16 outputs differing from the oracle bit pattern: %d of %d" % (mismatch, ref_out.size))
    # and against the float product of the de-quantised operands (what the epilogue stands for)
    a_deq = q.astype(np.float64) * rparams[:, 0:1] + rparams[:, 1:2]
    w_deq = c["w"].astype(np.float64) * c["ws"][:, None] + (0 if c["wzp"] is None else c["wzp"][:, None])
    exact = a_deq @ w_deq.T + (0 if c["bias"] is None else c["bias"].astype(np.float64))
    assert np.abs(got_f - exact).max() <= FP16_TOL * np.sqrt(np.mean(exact ** 2))
    return mismatch


@pytest.mark.parametrize("m,k,n", [(32, 64, 32), (7, 48, 20), (128, 512, 384), (200, 1000, 300), (300, 2048, 512)])
@pytest.mark.parametrize("symmetric", [True, False])
def test_int8_conv_shapes(oracle, m, k, n, symmetric):
    c = make_int8_case(m + n, m, k, n, with_zp=(m % 2 == 1), with_bias=(n % 3 == 0))
    check_int8(oracle, c, symmetric)


@pytest.mark.parametrize("symmetric", [True, False])
def test_config4_int8_gemm(oracle, symmetric):
    c = make_int8_case(0, 2048, 2048, 8192)
    check_int8(oracle, c, symmetric)


def test_int8_pipeline_random_sweep(oracle):
    """Seeded sweep of the quantize -> int8 MFMA pipeline over ragged token / channel counts, all
    three token-tile sizes, both quantization modes, zero points and biases: codes, params and
    int32 accumulators bit-exact, rescaled output at the fp16 bar (check_int8)."""
    rng = np.random.default_rng(77)
    for it in range(16):
        m = int(rng.choice([1, 5, 33, 64, 65, 130, 257, 600, 1100]))
        k = int(rng.choice([16, 40, 100, 256, 1000, 2048]))
        n = int(rng.choice([4, 20, 100, 256, 260, 1000, 2100, 4096]))
        if m * k * n > 1 << 29:
            k = 256
        c = make_int8_case(500 + it, m, k, n, with_zp=bool(rng.random() < 0.4), with_bias=bool(rng.random() < 0.5))
        check_int8(oracle, c, symmetric=bool(rng.random() < 0.5))
