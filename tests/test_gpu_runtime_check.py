"""GPU parity of the FullyConnected with runtime channel bounds (ConvRuntimeCheckDesc: src_end_ch /
dst_end_ch read at launch from the int32 "params" object), through the C-ABI, against the oracle's
restatement of the bounded kernel; the reference's own test shape and runtime channels
(common/kernels/tests/fully_connected_test_util.cc:1260-1300) and larger layers.  Up to 4 tokens the
bounded op runs on the streaming GEMVs (fc_w4_stream_kernel / fc_w8_stream_kernel), beyond on the
unspecialised kernel; every case also runs with the unspecialised kernel forced."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

import mldhip as M
import workloads as W
from test_gpu_fc import check_fp


def streaming_kernel_for(case):
    """The kernel a bounded op of this case takes (None: the unspecialised one)."""
    ks, ns, groups = (case["k"] + 3) // 4, (case["n"] + 3) // 4, case["groups"]
    if case["m"] > 4 or (groups > 1 and (ks % groups != 0 or (ks // groups) % 8 != 0)):
        return None
    if case["weight_bits"] == 8:
        return "fc_w8_stream_kernel"
    return "fc_w4_stream_kernel" if case["tensor_dtype"] == np.float16 and ns % 2 == 0 else None


def run_bounded(oracle, case, src_end_ch, dst_end_ch, params_values=None):
    got = run_bounded_once(oracle, case, src_end_ch, dst_end_ch, streaming_kernel_for(case) or "fc_generic_kernel")
    if streaming_kernel_for(case):
        with M.tuning(force_generic=1):
            run_bounded_once(oracle, case, src_end_ch, dst_end_ch, "fc_generic_kernel")
        if case["weight_bits"] == 4:
            # the same op over the layouts the library asks for (output groups of 16 slices; of 2 for a decode op)
            for layout in ("library", "decode"):
                other = run_bounded_once(oracle, case, src_end_ch, dst_end_ch, None, layout=layout)
                assert np.array_equal(other, got), layout
    return got


def run_bounded_once(oracle, case, src_end_ch, dst_end_ch, expect_kernel, layout="reference"):
    import torch
    o = oracle
    m, k, n, bits, groups = case["m"], case["k"], case["n"], case["weight_bits"], case["groups"]
    f16 = case["tensor_dtype"] == np.float16
    td = case["tensor_dtype"]
    tt = torch.float16 if f16 else torch.float32
    mt = M.FLOAT16 if f16 else M.FLOAT32
    ns = (n + 3) // 4
    desc, packed_dev = W.pack_fc_weights(case, reference_layout=layout == "reference", decode_layout=layout == "decode")
    packed = (o.int8_as_uint4 if bits == 4 else o.int8_as_uint8)(case["w"], o.LAYOUT_I4O4, ns)  # what the restatement reads
    # params: 4 int32 values as the reference's tests lay them out (src start, src end, dst start, dst end)
    params = np.full(4, -1, np.int32)
    kwargs = {}
    if src_end_ch is not None:
        params[1] = src_end_ch
        kwargs["src_end_ch_index"] = 1
    if dst_end_ch is not None:
        params[3] = dst_end_ch
        kwargs["dst_end_ch_index"] = 3
    scale_dev = torch.from_numpy(M.scale_to_tensor(case["scale"], mt).view(td) if f16 else M.scale_to_tensor(case["scale"], mt)).cuda()
    srcs = [torch.from_numpy(W.to_slices(case["act"]).astype(td)).cuda(), torch.from_numpy(packed_dev).cuda(), scale_dev]
    bias = None
    if case["bias"] is not None:
        bias = np.zeros(ns * 4, td)
        bias[:n] = case["bias"]
        srcs.append(torch.from_numpy(bias).cuda())
    srcs.append(torch.from_numpy(params).cuda())
    out = torch.full((ns, m, 4), 7.0, dtype=tt, device="cuda")
    op = M.fc_create(M.PRECISION_F32_F16 if f16 else M.PRECISION_F32, mt, mt, n, k, desc, scale_shape=(n, groups),
                     has_bias=case["bias"] is not None, max_tokens=m, **kwargs)
    assert op.src_names[-1] == "params"
    op.bind(srcs, [out])
    op.set_shape(1, 1, m)
    print("runtime check", m, k, n, bits, groups, src_end_ch, dst_end_ch, layout, expect_kernel, flush=True)
    op.launch(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    if expect_kernel is None:  # another layout of the same weights: the streaming kernel where it reads that layout
        assert op.kernel_name in ("fc_w4_stream_kernel", "fc_generic_kernel"), op.kernel_name
    else:
        assert op.kernel_name == expect_kernel, op.kernel_name
    got = out.cpu().numpy().astype(np.float32)
    # oracle: the bounded kernel restatement over the reference's layout
    prec = o.PREC_F32F16 if f16 else o.PREC_F32
    conv = (lambda a: o.f32_to_f16_bits(np.asarray(a, np.float32))) if f16 else (lambda a: np.asarray(a, np.float32))
    if groups == 1:
        sc = np.zeros(ns * 4, np.float32); sc[:n] = case["scale"][:, 0]
        kind = o.SCALE_LINEAR
    else:
        sc = o.scale_to_hoio4(case["scale"]); kind = o.SCALE_BLOCK
    ref = o.fc_kernel_runtime_check(conv(o.to_slices(case["act"])), packed, m, k, n, prec, bits, kind, conv(sc), None,
                                    None if bias is None else conv(bias.astype(np.float32)), groups,
                                    src_end_ch=src_end_ch, dst_end_ch=dst_end_ch,
                                    dst_before=conv(np.full((ns, m, 4), 7.0, np.float32)))
    ref = o.f16_bits_to_f32(ref) if f16 else ref
    ks_end, ns_end = o.runtime_end_slices(src_end_ch, dst_end_ch, k, n, groups > 1)
    # untouched slices are bit-identical (the fill), written ones meet the FullyConnected bar
    assert np.array_equal(got[ns_end:], ref[ns_end:]) and np.all(got[ns_end:] == 7.0)
    if ns_end:
        sub = dict(case, n=ns_end * 4)
        check_fp(W.from_slices(got[:ns_end], ns_end * 4), W.from_slices(ref[:ns_end], ns_end * 4).astype(np.float64), sub,
                 "bounded kernel restatement")
    return got


@pytest.mark.parametrize("dtype", [np.float32, np.float16])
@pytest.mark.parametrize("rc", [dict(src_end_ch=4, dst_end_ch=8), dict(src_end_ch=8), dict(src_end_ch=175), dict(dst_end_ch=14)])
def test_reference_runtime_channel_cases(oracle, dtype, rc):
    case = W.make_fc_case(seed=9, m=1, k=171, n=533, weight_bits=8, tensor_dtype=dtype, groups=1, with_bias=True,
                          act_uniform=True)
    run_bounded(oracle, case, rc.get("src_end_ch"), rc.get("dst_end_ch"))


@pytest.mark.parametrize("bits,m,k,n,groups,src_end,dst_end", [
    (4, 1, 4096, 2048, 1, 1000, 300), (4, 3, 2048, 1024, 64, 77, 1000), (8, 5, 1024, 516, 1, 0, 33),
    (4, 1, 512, 256, 1, 512, 0), (4, 2, 256, 8192, 1, 129, 4097), (8, 1, 96, 64, 3, 5, 64),
    (4, 1, 16384, 2048, 1, 5000, 2048), (4, 4, 4096, 14336, 1, 4096, 14000), (8, 2, 4096, 4096, 1, 37, 4096),
    (4, 1, 2048, 2048, 1, 0, 40), (8, 3, 2048, 1024, 64, 100, 500)])
def test_runtime_bounds_sweep(oracle, bits, m, k, n, groups, src_end, dst_end):
    """Bounds inside the tensors, at and beyond their ends, zero, unaligned to 4 and to 32; group-wise
    scales ignore the source bound (the reference's group loop runs over all groups)."""
    case = W.make_fc_case(seed=k + n, m=m, k=k, n=n, weight_bits=bits, tensor_dtype=np.float16, groups=groups, with_bias=True)
    run_bounded(oracle, case, src_end, dst_end)


def test_bounds_are_read_at_launch(oracle):
    """The same op, the bound rewritten on the device between two launches."""
    import torch
    case = W.make_fc_case(seed=4, m=1, k=1024, n=1024, weight_bits=4, tensor_dtype=np.float16, groups=1)
    a = run_bounded(oracle, case, 1024, 64)
    b = run_bounded(oracle, case, 1024, 1024)
    assert np.array_equal(a[:16], b[:16]) and np.all(a[16:] == 7.0) and not np.any(b == 7.0)


@pytest.mark.parametrize("bits,td", [(8, np.float32), (4, np.float16), (8, np.int8), (4, np.int8)])
def test_runtime_bounds_with_batched_weights(oracle, bits, td):
    """ConvRuntimeCheckDesc is independent of batched weights in the reference (common/kernels/
    fully_connected.cc:1123-1128: conv_params.runtime_check beside batched_weights): every dst row runs the
    bounded kernel with the matrix its id selects.  Floating-point variant against the oracle's bounded
    restatement per row; integer-math variant (np.int8) bit for bit against the integer product over the
    bounded K range."""
    import torch
    o = oracle
    rows, k, n, batch, src_end, dst_end = 5, 172, 536, 4, 61, 200
    rng = np.random.default_rng(bits)
    lim = 127 if bits == 8 else 7
    w = rng.integers(-lim, lim + 1, size=(n, batch, 1, k), dtype=np.int8)
    ids = np.array([2, 0, 3, 3, 1], np.int32)
    int8_math = td == np.int8
    f16 = td == np.float16
    desc = M.fc_int8_weights_desc(n, k) if bits == 8 else M.fc_int4_weights_desc(n, k, reference=True)
    packed = (M.rearrange_int8_as_uint8 if bits == 8 else M.rearrange_int8_as_uint4)(w, desc)
    ks, ns = (k + 3) // 4, (n + 3) // 4
    ks_end, ns_end = o.runtime_end_slices(src_end, dst_end, k, n, False)
    params = torch.tensor([-1, src_end, -1, dst_end], dtype=torch.int32, device="cuda")
    if int8_math:
        src = rng.integers(-128, 128, size=(rows, k), dtype=np.int8)
        out = torch.full((ns, rows, 4), -5, dtype=torch.int32, device="cuda")
        op = M.fc_create(M.PRECISION_F32, M.INT8, M.INT32, n, k, desc, max_tokens=rows, weights_batch=batch,
                         src_end_ch_index=1, dst_end_ch_index=3)
        assert op.src_names == ["src_tensor", "batch_ids", "weights", "params"]
        op.bind([torch.from_numpy(W.to_slices(src)).cuda(), torch.from_numpy(ids).cuda(), torch.from_numpy(packed).cuda(), params], [out])
    else:
        mt = M.FLOAT16 if f16 else M.FLOAT32
        src = rng.uniform(-1, 1, size=(rows, k)).astype(td).astype(np.float32)
        scale = (np.abs(rng.normal(0.0, 1.0, size=(n, batch, 1))) / 128.0 + 1e-3).astype(td).astype(np.float32)
        st = M.scale_to_tensor_batched(scale, mt)
        out = torch.full((ns, rows, 4), 7.0, dtype=torch.float16 if f16 else torch.float32, device="cuda")
        op = M.fc_create(M.PRECISION_F32_F16 if f16 else M.PRECISION_F32, mt, mt, n, k, desc, scale_shape=(n, 1),
                         max_tokens=rows, weights_batch=batch, src_end_ch_index=1, dst_end_ch_index=3)
        assert op.src_names == ["src_tensor", "batch_ids", "weights", "weights_scale", "params"]
        op.bind([torch.from_numpy(W.to_slices(src).astype(td)).cuda(), torch.from_numpy(ids).cuda(), torch.from_numpy(packed).cuda(),
                 torch.from_numpy(st.view(td) if f16 else st).cuda(), params], [out])
    op.set_shape(1, rows, 1)
    print("runtime bounds x batched weights", bits, td.__name__, flush=True)
    op.launch(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    want = "fc_int8_math_kernel" if int8_math else ("fc_w8_stream_kernel" if bits == 8 else ("fc_w4_stream_kernel" if f16 else "fc_generic_kernel"))
    assert op.kernel_name == want, op.kernel_name
    got = out.cpu().numpy()
    if int8_math:
        assert np.all(got[ns_end:] == -5)
        a = src.astype(np.int64).copy()
        a[:, ks_end * 4:] = 0
        for y in range(rows):
            ref = (w[:, ids[y], 0, :].astype(np.int64) @ a[y])[:ns_end * 4]
            assert np.array_equal(W.from_slices(got[:ns_end, y:y + 1], min(n, ns_end * 4))[0], ref[:min(n, ns_end * 4)])
        return
    got = got.astype(np.float32)
    assert np.all(got[ns_end:] == 7.0)
    conv = (lambda a: o.f32_to_f16_bits(np.asarray(a, np.float32))) if f16 else (lambda a: np.asarray(a, np.float32))
    prec = o.PREC_F32F16 if f16 else o.PREC_F32
    pack_o = o.int8_as_uint8 if bits == 8 else o.int8_as_uint4
    for y in range(rows):
        e = int(ids[y])
        sc = np.zeros(ns * 4, np.float32); sc[:n] = scale[:, e, 0]
        ref = o.fc_kernel_runtime_check(conv(o.to_slices(src[y:y + 1])), pack_o(w[:, e, 0, :], o.LAYOUT_I4O4, ns), 1, k, n, prec, bits,
                                        o.SCALE_LINEAR, conv(sc), None, None, 1, src_end_ch=src_end, dst_end_ch=dst_end)
        ref = o.f16_bits_to_f32(ref) if f16 else ref
        sub = dict(tensor_dtype=np.float16 if f16 else np.float32, k=k)
        check_fp(W.from_slices(got[:ns_end, y:y + 1], ns_end * 4), W.from_slices(ref[:ns_end], ns_end * 4).astype(np.float64), sub,
                 "bounded kernel restatement, row %d" % y)
