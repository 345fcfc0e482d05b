"""GPU parity of the FullyConnected over weights with the output slice outermost, the layout
FullyConnectedOI reads (kOSpatialIOGroupI4O4 with output_group_size = 1: linear_i4o4 =
dst_s * src_slices + src_s, common/kernels/fully_connected_oi.cc:122-133), and over any other
whole number of output groups: the reference's own test cases
(common/kernels/tests/fully_connected_oi_test_util.cc:340-412) and wider shapes, through the C-ABI,
against the float64 product and the oracle's kernel restatement (the arithmetic does not depend on
where a block lies in the buffer)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

import mldhip as M
import workloads as W
from refmath import textbook
from test_gpu_fc import check_as_accurate_as, check_fp, oracle_fc, restatement_affordable


def synthetic(shape, index_offset=0):
    """MakeSyntheticTensor of the reference's tests: sin of the linear index."""
    n = int(np.prod(shape))
    return np.sin(np.arange(index_offset, index_offset + n, dtype=np.float64)).astype(np.float32).reshape(shape)


def run_grouped(oracle, case, group, expect_kernel=None):
    import torch
    print("output group", group, {k: case[k] for k in ("m", "k", "n", "weight_bits", "groups")}, flush=True)
    dev = W.FcDevice(case, output_group=group)
    assert dev.desc.output_group_size == group
    # the packed bytes are the oracle's for this group size
    pack = oracle.int8_as_uint4 if case["weight_bits"] == 4 else oracle.int8_as_uint8
    assert np.array_equal(dev.packed_host, pack(case["w"], oracle.LAYOUT_I4O4, group))
    dev.run()
    got = dev.result()
    if expect_kernel:
        assert dev.op.kernel_name in expect_kernel, dev.op.kernel_name
    dev.run()
    assert np.array_equal(got, dev.result())
    ref = textbook(case)
    check_fp(got, ref, case, "textbook")
    if restatement_affordable(case):
        rest = oracle_fc(oracle, case).astype(np.float64)
        check_fp(got, rest, case, "kernel restatement")
        check_as_accurate_as(got, rest, ref, case, dev.op.kernel_name)
    return got, dev.op.kernel_name


@pytest.mark.parametrize("bits", [8, 4])
@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_reference_oi_cases(oracle, bits, dtype):
    """FullyConnectedOIWi8 / Wi4: 256 -> 256, one token, synthetic weights clamped to the code range,
    per-channel scales / 128 (/ 8), zero bias."""
    n = k = 256
    wf = synthetic((n, k))
    if bits == 8:
        w = (np.clip(((wf + 1.0) * 256.0).astype(np.int32), 0, 255) - 128).astype(np.int8)
        scale = synthetic((n, 1)) / 128.0
    else:
        w = (np.clip(((wf + 1.0) * 16.0).astype(np.int32), 0, 15) - 8).astype(np.int8)
        scale = synthetic((n, 1)) / 8.0
    case = W.make_fc_case(seed=0, m=1, k=k, n=n, weight_bits=bits, tensor_dtype=dtype, groups=1, with_bias=True)
    case["w"] = w
    case["scale"] = scale.astype(dtype).astype(np.float32)
    case["bias"] = np.zeros(n, np.float32)
    case["act"] = synthetic((1, k)).astype(dtype).astype(np.float32)
    run_grouped(oracle, case, 1)


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("m,k,n,groups,zp", [(1, 4096, 2048, 1, False), (1, 2048, 8192, 64, False), (3, 1024, 516, 1, True),
                                             (16, 4096, 8192, 1, False), (64, 512, 384, 4, True), (300, 1024, 1024, 8, False),
                                             (1, 171, 533, 1, False)])
def test_oi_layout_shapes(oracle, bits, m, k, n, groups, zp):
    """Output groups of one slice: decode, a few tokens (matrix-core GEMV where the layer is wide), GEMM
    tiles, ragged K and N on the unspecialised kernel."""
    case = W.make_fc_case(seed=m + k + n, m=m, k=k, n=n, weight_bits=bits, tensor_dtype=np.float16, groups=groups,
                          with_bias=True, with_zero_point=zp)
    _, kernel = run_grouped(oracle, case, 1)
    if m > 16 and k % 16 == 0:
        assert kernel == "fc_w%d_mfma_gemm_kernel" % bits, kernel


@pytest.mark.parametrize("group", [2, 3, 6, 32, 64])
@pytest.mark.parametrize("bits,m", [(4, 1), (4, 5), (8, 1), (4, 130), (8, 70)])
def test_other_group_sizes(oracle, group, bits, m):
    """Any whole number of output groups is addressed alike: 768 channels = 192 slices in groups of
    2, 3, 6, 32 and 64 slices."""
    case = W.make_fc_case(seed=group + m, m=m, k=512, n=768, weight_bits=bits, tensor_dtype=np.float16, groups=4,
                          with_bias=True)
    run_grouped(oracle, case, group)


@pytest.mark.parametrize("bits", [4, 8])
@pytest.mark.parametrize("m", [1, 4, 40])
def test_oi_int8_math_bit_exact(oracle, bits, m):
    """The integer-math variant over the same layout: int32 results equal the closed form."""
    import torch
    rng = np.random.default_rng(bits + m)
    k, n = 512, 260
    lim = 127 if bits == 8 else 7
    w = rng.integers(-lim - 1, lim + 1, size=(n, k), dtype=np.int8)
    act = rng.integers(-128, 128, size=(m, k), dtype=np.int8)
    desc = M.fc_int4_weights_desc(n, k, reference=True) if bits == 4 else M.fc_int8_weights_desc(n, k)
    desc.output_group_size = 1
    packed = (M.rearrange_int8_as_uint4 if bits == 4 else M.rearrange_int8_as_uint8)(w, desc)
    ns = (n + 3) // 4
    op = M.fc_create(M.PRECISION_F32, M.INT8, M.INT32, n, k, desc, scale_shape=(1, 1), max_tokens=m)
    out = torch.zeros((ns, m, 4), dtype=torch.int32, device="cuda")
    op.bind([torch.from_numpy(W.to_slices(act)).cuda(), torch.from_numpy(packed).cuda()], [out])
    op.set_shape(1, 1, m)
    print("int8 math, output groups of one slice", bits, m, flush=True)
    op.launch(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    got = W.from_slices(out.cpu().numpy(), n)
    assert np.array_equal(got, act.astype(np.int64) @ w.astype(np.int64).T)


def test_groups_that_do_not_divide_the_slices_are_refused():
    desc = M.fc_int4_weights_desc(768, 512, reference=True)
    desc.output_group_size = 5
    with pytest.raises(M.MldhipError) as e:
        M.fc_create(M.PRECISION_F32_F16, M.FLOAT16, M.FLOAT16, 768, 512, desc, scale_shape=(768, 1))
    assert e.value.code == M.INVALID_ARGUMENT and "output_group_size" in e.value.message
