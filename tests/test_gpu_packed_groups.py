"""GPU parity of the FullyConnected with packed groups (ConvRuntimeCheckDesc::PackedGroups: the
tokens of the source row sorted by weight matrix, group sizes and offsets read on the device - the
grouped FullyConnected of a mixture-of-experts prefill, MakeConvWithPackedGroups,
common/gpu_model_builder_moe_util.cc:119-230), through the C-ABI: the reference test's own flow
(common/kernels/tests/fully_connected_test_util.cc:2487-2597) against the per-token float64 products,
and against the oracle's restatement of the kernel."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

import mldhip as M
import workloads as W
from test_oracle_fc import (make_packed_groups_case, packed_groups_expected, run_packed_groups_oracle, unpack_groups)

FP16_TOL = 2e-2


def run_device(c, td, sizes=None, offsets=None, max_group_size=None, params_offset=0, fill=None, group=None):
    import torch
    tt = torch.float16 if td == np.float16 else torch.float32
    mt = M.FLOAT16 if td == np.float16 else M.FLOAT32
    n, k, batch = c["n"], c["k"], c["batch"]
    ns = W.div_up(n, 4)
    tokens = c["packed_src"].shape[0]
    desc = M.fc_int8_weights_desc(n, k) if c["bits"] == 8 else M.fc_int4_weights_desc(n, k, reference=True)
    if group is not None:  # output groups of `group` slices: the matrices of a group one after the other
        desc.output_group_size = group
    packed = (M.rearrange_int8_as_uint8 if c["bits"] == 8 else M.rearrange_int8_as_uint4)(c["w"], desc)

    def tensor(v):
        t = M.scale_to_tensor_batched(v, mt)
        return torch.from_numpy(t.view(td) if td == np.float16 else t).cuda()
    sizes = c["sizes"] if sizes is None else sizes
    offsets = c["offsets"] if offsets is None else offsets
    params = np.concatenate([np.full(params_offset, -12345, np.int32), sizes, offsets]).astype(np.int32)
    srcs = [torch.from_numpy(W.to_slices(c["packed_src"]).astype(td)).cuda(), torch.from_numpy(packed).cuda(),
            tensor(c["scale"])]
    if c["zp"] is not None:
        srcs.append(tensor(c["zp"]))
    srcs.append(torch.from_numpy(params).cuda())
    out = torch.full((ns, tokens, 4), 0.0 if fill is None else fill, dtype=tt, device="cuda")
    op = M.fc_create(M.PRECISION_F32 if td == np.float32 else M.PRECISION_F32_F16, mt, mt, n, k, desc,
                     scale_shape=(n, c["groups"]), has_zero_point_tensor=c["zp"] is not None, max_tokens=tokens,
                     packed_groups=(params_offset, batch, max_group_size or tokens))
    assert op.src_names[-1] == "params" and op.src_names[1] == "weights"
    op.bind(srcs, [out])
    op.set_shape(1, 1, tokens)
    print("packed groups", c["bits"], tokens, k, n, batch, c["groups"], td.__name__, flush=True)
    op.launch(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    # fp16 tensors run on the matrix cores (one launch plane per matrix), fp32 on the unspecialised kernel
    want = "fc_generic_kernel" if td == np.float32 or M.get_tuning_forced_generic() else "fc_w%d_mfma_gemm_kernel" % c["bits"]
    assert op.kernel_name == want, op.kernel_name
    first = out.clone()
    op.launch(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert torch.equal(first, out)
    return W.from_slices(out.cpu().numpy().astype(np.float32), n)


def check(got, ref, td, k):
    err = np.abs(got - ref).max()
    if td == np.float16:
        rms = np.sqrt(np.mean(ref ** 2))
        assert err <= FP16_TOL * rms, (err, rms)
    else:
        tol = 1.1920929e-7 * (k + 1) * max(1.0, np.abs(ref).max())
        assert err <= tol, (err, tol)


@pytest.mark.parametrize("td", [np.float32, np.float16])
@pytest.mark.parametrize("bits,groups,zp", [(8, 1, False), (4, 2, True)])
def test_reference_test_flow(oracle, td, bits, groups, zp):
    c = make_packed_groups_case(3 + bits, 64, 4, 64, 32, 16, bits, groups, zp)
    got = unpack_groups(c, run_device(c, td))
    assert not np.isnan(got).any()
    check(got, packed_groups_expected(oracle, c, td), td, c["k"])


@pytest.mark.parametrize("bits,width,per_item,k,n,batch,groups,zp,td", [
    (4, 512, 8, 2048, 768, 128, 64, False, np.float16),   # a mixture layer's prefill: 4096 routed tokens, 128 experts
    (4, 96, 2, 768, 2048, 8, 24, False, np.float16),      # its down projections
    (8, 33, 3, 171, 533, 5, 1, True, np.float32),         # the reference's odd sizes
    (4, 7, 1, 64, 20, 4, 2, True, np.float16),            # fewer tokens than a token block, ragged channels
])
def test_mixture_prefill_shapes(oracle, bits, width, per_item, k, n, batch, groups, zp, td):
    c = make_packed_groups_case(width + n, width, per_item, k, n, batch, bits, groups, zp)
    rows = run_device(c, td, params_offset=3)
    got = unpack_groups(c, rows)
    check(got, packed_groups_expected(oracle, c, td), td, k)
    if width * per_item * k * n <= 1 << 28:
        rest = run_packed_groups_oracle(oracle, c, oracle.PREC_F32 if td == np.float32 else oracle.PREC_F32F16)
        check(rows, rest.astype(np.float64), td, k)
    if td == np.float16:  # the same op on the unspecialised kernel
        with M.tuning(force_generic=1):
            slow = unpack_groups(c, run_device(c, td, params_offset=3))
        check(slow, packed_groups_expected(oracle, c, td), td, k)


@pytest.mark.parametrize("bits,width,per_item,k,n,batch,groups,zp,td,group", [
    (4, 512, 8, 2048, 768, 128, 64, False, np.float16, 16),  # the mixture layer's prefill over groups of 16 slices
    (4, 96, 2, 768, 2048, 8, 24, True, np.float16, 16),      # its down projections, zero points
    (8, 40, 3, 256, 536, 5, 1, False, np.float16, 2),        # uint8 weights in groups of 2 slices
    (4, 33, 3, 171, 536, 5, 1, True, np.float32, 67),        # fp32 tensors (unspecialised kernel), odd group
    (4, 7, 1, 64, 20, 4, 2, True, np.float16, 1),            # groups of one slice
])
def test_mixture_prefill_shapes_in_output_groups(oracle, bits, width, per_item, k, n, batch, groups, zp, td, group):
    """The batched weights packed in output groups (the layout the batch-ids op of the same layer
    streams fastest): same results."""
    c = make_packed_groups_case(width + n + group, width, per_item, k, n, batch, bits, groups, zp)
    rows = run_device(c, td, params_offset=2, group=group)
    check(unpack_groups(c, rows), packed_groups_expected(oracle, c, td), td, k)
    if width * per_item * k * n <= 1 << 28:
        rest = run_packed_groups_oracle(oracle, c, oracle.PREC_F32 if td == np.float32 else oracle.PREC_F32F16)
        check(rows, rest.astype(np.float64), td, k)


@pytest.mark.parametrize("fm", [1, 2, 4])
def test_groups_of_every_size_on_the_matrix_cores(oracle, fm):
    """Group sizes 0, 1, odd, one token tile exactly, several tiles, beyond max_group_size; offsets that
    are odd and that leave gaps; every token tile (32, 64 and 128 tokens).  fp16, against the restatement."""
    c = make_packed_groups_case(21, 300, 1, 256, 136, 8, 4, 8, True)
    sizes = np.array([0, 1, 33, 64, 65, 100, 7, 40], np.int32)
    # (runs that do not overlap; the last one is cut at the end of the tensor)
    offsets = np.array([0, 1, 3, 40, 110, 177, 258, 266], np.int32)
    with M.tuning(gemm_fm=fm):
        got = run_device(c, np.float16, sizes=sizes, offsets=offsets, max_group_size=80, fill=7.0)
    before = oracle.f32_to_f16_bits(np.full(((136 + 3) // 4, 300, 4), 7.0, np.float32))
    ref = run_packed_groups_oracle(oracle, c, oracle.PREC_F32F16, max_group_size=80, dst_before=before, sizes=sizes, offsets=offsets)
    assert np.array_equal(got == 7.0, ref == 7.0)
    written = ref != 7.0
    rms = np.sqrt(np.mean(ref[written] ** 2))
    assert np.abs(got - ref)[written].max() <= FP16_TOL * rms


def test_groups_of_hundreds_of_tokens(oracle):
    """Groups large enough for the 128-token tiles (max_group_size >= 256): sizes around the tile
    edges, odd offsets, zero points; against the restatement."""
    c = make_packed_groups_case(31, 900, 1, 128, 264, 3, 4, 4, True)
    sizes = np.array([257, 128, 385], np.int32)
    offsets = np.array([1, 260, 391], np.int32)
    got = run_device(c, np.float16, sizes=sizes, offsets=offsets, max_group_size=400, fill=7.0, group=2)
    before = oracle.f32_to_f16_bits(np.full(((264 + 3) // 4, 900, 4), 7.0, np.float32))
    ref = run_packed_groups_oracle(oracle, c, oracle.PREC_F32F16, max_group_size=400, dst_before=before, sizes=sizes,
                                   offsets=offsets)
    assert np.array_equal(got == 7.0, ref == 7.0)
    written = ref != 7.0
    assert written.sum() >= 0.999 * (257 + 128 + 385) * 264  # (a result may be 7.0 itself)
    rms = np.sqrt(np.mean(ref[written] ** 2))
    assert np.abs(got - ref)[written].max() <= FP16_TOL * rms


def test_tokens_outside_every_group_are_not_written(oracle):
    c = make_packed_groups_case(11, 16, 2, 32, 8, 4)
    sizes = np.array([5, 0, 9, 40], np.int32)
    offsets = np.array([2, 7, 10, 28], np.int32)
    got = run_device(c, np.float32, sizes=sizes, offsets=offsets, max_group_size=6, fill=7.0)
    before = np.full((2, 32, 4), 7.0, np.float32)
    ref = run_packed_groups_oracle(oracle, c, oracle.PREC_F32, max_group_size=6, dst_before=before, sizes=sizes, offsets=offsets)
    assert np.array_equal(got == 7.0, ref == 7.0)
    assert np.abs(got - ref).max() <= 1e-5


def test_packed_groups_arguments():
    d = M.fc_int4_weights_desc(64, 64, reference=True)
    with pytest.raises(M.MldhipError) as e:
        M.fc_create(M.PRECISION_F32_F16, M.FLOAT16, M.FLOAT16, 64, 64, d, scale_shape=(64, 1), packed_groups=(0, 4, 0))
    assert e.value.code == M.INVALID_ARGUMENT
    op = M.fc_create(M.PRECISION_F32, M.INT8, M.INT32, 64, 64, d, packed_groups=(0, 4, 8))
    assert op.src_names == ["src_tensor", "weights", "params"]


@pytest.mark.parametrize("bits,width,per_item,k,n,batch,group", [
    (8, 64, 4, 64, 32, 16, None), (4, 40, 3, 112, 152, 5, None), (4, 96, 2, 768, 512, 8, 16), (8, 7, 1, 64, 20, 4, 1)])
def test_integer_math_variant(bits, width, per_item, k, n, batch, group):
    """Packed groups on the integer-math FullyConnected (int8 sources -> int32; the reference's kernel has
    the group parameters in both variants, common/kernels/fully_connected.cc:706-710, 810-816): every token
    of a group against its matrix, bit for bit against the integer product; tokens outside every group
    keep what the tensor held."""
    import torch
    c = make_packed_groups_case(width + n, width, per_item, k, n, batch, bits)
    rng = np.random.default_rng(width)
    tokens = c["packed_src"].shape[0]
    src = rng.integers(-128, 128, size=(tokens, k), dtype=np.int8)
    desc = M.fc_int8_weights_desc(n, k) if bits == 8 else M.fc_int4_weights_desc(n, k, reference=True)
    if group is not None:
        desc.output_group_size = group
    packed = (M.rearrange_int8_as_uint8 if bits == 8 else M.rearrange_int8_as_uint4)(c["w"], desc)
    sizes, offsets = c["sizes"].copy(), c["offsets"].copy()
    sizes[0] = max(0, sizes[0] - 1)  # the last token of the first group belongs to no group
    params = np.concatenate([[77], sizes, offsets]).astype(np.int32)
    ns = W.div_up(n, 4)
    out = torch.full((ns, tokens, 4), -5, dtype=torch.int32, device="cuda")
    op = M.fc_create(M.PRECISION_F32, M.INT8, M.INT32, n, k, desc, max_tokens=tokens, packed_groups=(1, batch, tokens))
    op.bind([torch.from_numpy(W.to_slices(src)).cuda(), torch.from_numpy(packed).cuda(), torch.from_numpy(params).cuda()], [out])
    op.set_shape(1, 1, tokens)
    print("packed groups int8 math", bits, tokens, k, n, batch, group, flush=True)
    op.launch(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert op.kernel_name == "fc_int8_math_kernel", op.kernel_name
    got = W.from_slices(out.cpu().numpy(), n)
    ref = np.full((tokens, n), -5, np.int64)
    for g in range(batch):
        for t in range(int(offsets[g]), int(offsets[g]) + int(sizes[g])):
            ref[t] = c["w"][:, g, 0, :].astype(np.int64) @ src[t].astype(np.int64)
    assert np.array_equal(got, ref)
