"""GPU parity of the FullyConnected with batched weights selected by runtime ids (the
mixture-of-experts projection, CreateFullyConnectedWeightsBatchIds), through the C-ABI: against
the oracle's restatement of the generated kernel and against the reference's float reference
over dequantized weights.  fp32 tensors: 1.2e-7 * (K + 1) relative; fp16: 2e-2 of the output RMS."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

import mldhip as M
import workloads as W
from test_oracle_fc import (batch_ids_float_weights, batch_ids_int8_exact, make_batch_ids_case,
                            make_batch_ids_int8_case, run_batch_ids_int8_oracle, run_batch_ids_oracle)

FP16_TOL = 2e-2


def run_device(c, td, bias=None, max_tokens=None, group=None):
    import torch
    tt = torch.float16 if td == np.float16 else torch.float32
    mt = M.FLOAT16 if td == np.float16 else M.FLOAT32
    n, k, batch = c["n"], c["k"], c["batch"]
    ns = W.div_up(n, 4)
    # batched weights come in the reference's layout (one output group, the batch outermost) or, with
    # `group`, in output groups of that many slices (the matrices of a group one after the other)
    desc = M.fc_int8_weights_desc(n, k) if c["bits"] == 8 else M.fc_int4_weights_desc(n, k, reference=True)
    if group is not None:
        desc.output_group_size = group
    packed = (M.rearrange_int8_as_uint8 if c["bits"] == 8 else M.rearrange_int8_as_uint4)(c["w"], desc)
    src2 = c["src"].reshape(c["src_rows"] * c["row_tokens"], k)
    act = torch.from_numpy(W.to_slices(src2).astype(td)).cuda()
    ids = torch.from_numpy(c["ids"]).cuda()
    weights = torch.from_numpy(packed).cuda()

    def tensor(v):
        t = M.scale_to_tensor_batched(v, mt)
        return torch.from_numpy(t.view(td) if td == np.float16 else t).cuda()
    srcs = [act, ids, weights, tensor(c["scale"])]
    if c["zp"] is not None:
        srcs.append(tensor(c["zp"]))
    if bias is not None:
        b = np.zeros(ns * 4, td)
        b[:n] = bias
        srcs.append(torch.from_numpy(b).cuda())
    out = torch.zeros((ns, c["rows"] * c["row_tokens"], 4), dtype=tt, device="cuda")
    precision = M.PRECISION_F32 if td == np.float32 else M.PRECISION_F32_F16
    op = M.fc_create(precision, mt, mt, n, k, desc, scale_shape=(n, c["groups"]),
                     has_zero_point_tensor=c["zp"] is not None, has_bias=bias is not None,
                     max_tokens=max_tokens or c["rows"] * c["row_tokens"], weights_batch=batch,
                     shared_src=c["src_rows"] == 1 and c["rows"] > 1)
    op.bind(srcs, [out])
    op.set_shape(1, c["rows"], c["row_tokens"])
    op.launch(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    got = W.from_slices(out.cpu().numpy().astype(np.float32), n).reshape(c["rows"], c["row_tokens"], n)
    return got, op.kernel_name


def check(c, td, got, oracle, bias=None):
    # FullyConnectedWeightsBatchIdsReference (common/task/testing_ref_ops.cc:1042-1067) in float64, vectorised:
    # the oracle's loop form of it is pinned in tests/test_oracle_fc.py and is too slow for these sizes
    src = c["src"].astype(td).astype(np.float64)
    wf = batch_ids_float_weights(oracle, c).astype(np.float64)
    ref = np.stack([src[0 if src.shape[0] == 1 else y] @ wf[:, int(c["ids"][y]), :].T for y in range(c["rows"])])
    if bias is not None:
        ref = ref + np.asarray(bias, np.float64)
    err = np.abs(got - ref).max()
    if td == np.float16:
        rms = np.sqrt(np.mean(ref ** 2))
        assert err <= FP16_TOL * rms, (err, rms)
    else:
        tol = 1.1920929e-7 * (c["k"] + 1) * max(1.0, np.abs(ref).max())
        assert err <= tol, (err, tol)


@pytest.mark.parametrize("src_shape,ids_count", [((1, 1, 32), 1), ((8, 1, 32), 8), ((128, 1, 64), 128),
                                                 ((1, 1, 32), 4)])
@pytest.mark.parametrize("td", [np.float32, np.float16])
def test_reference_test_shapes(oracle, src_shape, ids_count, td):
    """fully_connected_test.cc:227-250 (32 channels, 16 int8 matrices; the last case broadcasts
    one source row to 4 ids)."""
    src_rows, row_tokens, k = src_shape
    c = make_batch_ids_case(ids_count + k, ids_count, row_tokens, src_rows, k, 32, 16)
    print("batch ids", src_shape, ids_count, td.__name__, flush=True)
    got, name = run_device(c, td)
    check(c, td, got, oracle)
    if td == np.float32:  # and against the kernel restatement
        ref = run_batch_ids_oracle(oracle, c, 0)
        assert np.abs(got - ref).max() <= 1.1920929e-7 * (k + 1) * max(1.0, np.abs(ref).max())


@pytest.mark.parametrize("bits,rows,row_tokens,src_rows,k,n,batch,groups,zp", [
    (4, 8, 1, 1, 2048, 768, 8, 64, False),     # decode step of a mixture layer: one token, 8 of 8 experts, shared input
    (4, 8, 1, 8, 768, 2048, 8, 24, False),     # its down projections: one input row per expert
    (4, 5, 3, 5, 64, 20, 4, 2, True),          # several tokens per row, zero points, ragged channels
    (8, 6, 2, 1, 171, 533, 3, 1, True),        # the reference's odd sizes
    (4, 4, 7, 4, 352, 200, 128, 11, False),    # many matrices, few used
    (4, 3, 4, 3, 1000, 1032, 5, 1, True),      # per-channel scales + zero points, 4 tokens per row, ragged K
    (4, 16, 2, 1, 512, 72, 6, 16, True),       # narrow matrices (64-byte row segments), group-wise zero points
    (8, 8, 1, 1, 2048, 768, 16, 64, True),     # int8 matrices, group-wise, shared input
    (8, 4, 3, 4, 1000, 2048, 5, 1, False),     # int8 per-channel, 3 tokens per row, ragged K
])
@pytest.mark.parametrize("td", [np.float16, np.float32])
def test_mixture_shapes(oracle, bits, rows, row_tokens, src_rows, k, n, batch, groups, zp, td):
    c = make_batch_ids_case(rows * 7 + n, rows, row_tokens, src_rows, k, n, batch, bits, groups, zp)
    rng = np.random.default_rng(n)
    bias = (rng.uniform(-1, 1, size=n) * 0.1).astype(td).astype(np.float32)
    print("batch ids", bits, rows, row_tokens, src_rows, k, n, batch, groups, zp, td.__name__, flush=True)
    got, name = run_device(c, td, bias=bias)
    check(c, td, got, oracle, bias=bias)
    # rows of up to 4 tokens with whole 32-channel chunks per scale group stream through the GEMV
    # kernels (int4: fp16 tensors and an even slice count); everything else takes the
    # unspecialised kernel
    chunks_ok = groups == 1 or (k // 4 // groups) % 8 == 0
    expect = "fc_generic_kernel"
    if row_tokens <= 4 and chunks_ok:
        if bits == 4 and td == np.float16 and (n + 3) // 4 % 2 == 0:
            expect = "fc_w4_stream_kernel"
        elif bits == 8:
            expect = "fc_w8_stream_kernel"
    assert name == expect, (name, expect)


@pytest.mark.parametrize("bits,rows,row_tokens,src_rows,k,n,batch,groups,zp,group,td", [
    (4, 8, 1, 1, 2048, 768, 8, 64, False, 16, np.float16),    # mixture decode over the library's groups of 16 slices
    (4, 8, 1, 8, 768, 2048, 8, 24, False, 16, np.float16),    # its down projections: one input row per matrix
    (4, 2, 1, 1, 4096, 1024, 8, 1, False, 16, np.float16),    # per-channel scales
    (4, 4, 1, 1, 1024, 4096, 6, 1, True, 16, np.float16),     # 256 strips: per-channel scales and zero points, shared input
    (4, 7, 1, 7, 512, 2048, 5, 16, True, 16, np.float16),     # 224 strips: group-wise zero points, one input row per matrix
    (4, 2, 1, 1, 4096, 14336, 3, 1, False, 16, np.float16),   # two matrices of the c2 shape
    (4, 3, 4, 3, 1000, 1032, 5, 1, True, 6, np.float16),      # 4 tokens per row, zero points, groups of 6 of 258 slices
    (4, 4, 7, 4, 352, 200, 128, 11, False, 25, np.float16),   # many tokens per row, odd group (unspecialised kernel)
    (4, 5, 3, 5, 64, 20, 4, 2, True, 1, np.float32),          # groups of one slice, fp32
    (8, 6, 2, 1, 171, 536, 3, 1, True, 2, np.float32),        # uint8 weights in groups
    (8, 8, 1, 1, 2048, 768, 16, 64, True, 16, np.float16),    # uint8 group-wise, shared input
])
def test_mixture_shapes_in_output_groups(oracle, bits, rows, row_tokens, src_rows, k, n, batch, groups, zp, group, td):
    """Batched weights packed in output groups (the packers put the matrices of a group one after the
    other): same results as the float reference over the same weights."""
    c = make_batch_ids_case(rows * 5 + n + group, rows, row_tokens, src_rows, k, n, batch, bits, groups, zp)
    print("batch ids in groups", bits, rows, row_tokens, src_rows, k, n, batch, groups, zp, group, td.__name__, flush=True)
    got, name = run_device(c, td, group=group)
    check(c, td, got, oracle)
    if bits == 4 and td == np.float16 and row_tokens <= 4 and group % 2 == 0:
        # one token per row over at least 192 strips of 64 channels: the contiguous-strip kernel
        strip = row_tokens == 1 and group == 16 and k % 32 == 0 and (n // 64) * rows >= 192
        assert name == ("fc_w4_strip_kernel" if strip else "fc_w4_stream_kernel"), name


def test_repeated_and_out_of_range_ids(oracle):
    """The same matrix for several rows; an id outside the batch is clamped into it."""
    c = make_batch_ids_case(1, rows=6, row_tokens=2, src_rows=6, k=64, n=32, batch=4)
    c["ids"] = np.array([2, 2, 0, 3, 2, 0], np.int32)
    got, _ = run_device(c, np.float32)
    check(c, np.float32, got, oracle)
    bad = dict(c, ids=np.array([7, -1, 0, 3, 2, 0], np.int32))
    got_bad, _ = run_device(bad, np.float32)
    clamped = dict(c, ids=np.array([3, 0, 0, 3, 2, 0], np.int32))
    check(clamped, np.float32, got_bad, oracle)


def test_bindings_are_checked():
    import torch
    c = make_batch_ids_case(2, rows=4, row_tokens=1, src_rows=4, k=64, n=32, batch=4)
    desc = M.fc_int8_weights_desc(32, 64)
    op = M.fc_create(M.PRECISION_F32, M.FLOAT32, M.FLOAT32, 32, 64, desc, scale_shape=(32, 1), max_tokens=8,
                     weights_batch=4)
    op.set_shape(1, 4, 1)
    small = torch.zeros(16, dtype=torch.uint8, device="cuda")
    big = torch.zeros(1 << 16, dtype=torch.uint8, device="cuda")
    op.bind([big, big, small, big], [big])   # weights of one matrix only
    with pytest.raises(M.MldhipError) as e:
        op.launch(torch.cuda.current_stream().cuda_stream)
    assert e.value.code == M.INVALID_ARGUMENT and "weights" in str(e.value)
    with pytest.raises(M.MldhipError) as e:
        M.fc_launch_fused([op])
    assert e.value.code == M.FAILED_PRECONDITION


def test_random_sweep(oracle):
    """Seeded sweep over rows, tokens per row, shared / per-row sources, weight types, ragged K / N
    and scale groupings, whatever kernel the dispatcher picks."""
    rng = np.random.default_rng(77)
    seen = {}
    for it in range(30):
        bits = int(rng.choice([4, 8]))
        rows = int(rng.choice([1, 2, 3, 8, 17]))
        row_tokens = int(rng.choice([1, 1, 2, 4, 5]))
        shared = bool(rng.random() < 0.5)
        k = int(rng.choice([64, 96, 171, 256, 1000, 2048]))
        n = int(rng.choice([8, 20, 64, 152, 533, 1024, 2056]))
        batch = int(rng.choice([1, 2, 5, 32]))
        groups = 1
        gs = int(rng.choice([32, 64]))
        if k % gs == 0 and rng.random() < 0.6:
            groups = k // gs
        zp = bool(rng.random() < 0.3)
        td = np.float16 if rng.random() < 0.7 else np.float32
        c = make_batch_ids_case(500 + it, rows, row_tokens, 1 if shared else rows, k, n, batch, bits, groups, zp)
        print("sweep", it, dict(bits=bits, rows=rows, tok=row_tokens, shared=shared, k=k, n=n, batch=batch, groups=groups,
                                zp=zp, td=td.__name__), flush=True)
        got, name = run_device(c, td)
        seen[name] = seen.get(name, 0) + 1
        check(c, td, got, oracle)
    print("kernels exercised:", seen)
    assert len(seen) >= 3


@pytest.mark.parametrize("bits,rows,row_tokens,src_rows,k,n,batch", [
    (8, 8, 1, 8, 32, 32, 16), (8, 4, 1, 1, 32, 32, 16),      # the reference's batch-ids shapes, int8 sources
    (4, 8, 1, 1, 2048, 768, 16), (4, 8, 1, 8, 768, 2048, 16),  # mixture decode shapes (streaming kernel)
    (8, 3, 4, 3, 1000, 1032, 5), (4, 5, 3, 5, 171, 20, 3),     # ragged K, odd uint4 slice count (tiled kernel)
    (8, 2, 9, 1, 256, 64, 4),                                   # more than 4 tokens per row (tiled kernel)
])
@pytest.mark.parametrize("group", [None, 2])
def test_int8_math_bit_exact(oracle, bits, rows, row_tokens, src_rows, k, n, batch, group):
    """The integer-math FullyConnected over batched weights: int32 results bit for bit against the
    closed form and the oracle's kernel restatement."""
    import torch
    c = make_batch_ids_int8_case(rows + n + bits, rows, row_tokens, src_rows, k, n, batch, bits)
    print("batch ids int8", bits, rows, row_tokens, src_rows, k, n, batch, flush=True)
    ns = W.div_up(n, 4)
    desc = M.fc_int8_weights_desc(n, k) if bits == 8 else M.fc_int4_weights_desc(n, k, reference=True)
    if group is not None:  # output groups: the matrices of a group one after the other
        desc.output_group_size = group if ns % group == 0 else 1  # (an odd slice count: groups of one slice)
    packed = (M.rearrange_int8_as_uint8 if bits == 8 else M.rearrange_int8_as_uint4)(c["w"], desc)
    act = torch.from_numpy(W.to_slices(c["src"].reshape(-1, k))).cuda()
    ids = torch.from_numpy(c["ids"]).cuda()
    weights = torch.from_numpy(packed).cuda()
    out = torch.zeros((ns, rows * row_tokens, 4), dtype=torch.int32, device="cuda")
    op = M.fc_create(M.PRECISION_F32, M.INT8, M.INT32, n, k, desc, max_tokens=rows * row_tokens, weights_batch=batch,
                     shared_src=src_rows == 1 and rows > 1)
    op.bind([act, ids, weights], [out])
    op.set_shape(1, rows, row_tokens)
    op.launch(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    got = W.from_slices(out.cpu().numpy(), n).reshape(rows, row_tokens, n)
    assert np.array_equal(got, batch_ids_int8_exact(c))
    assert np.array_equal(got, run_batch_ids_int8_oracle(oracle, c))
    stream_ok = row_tokens <= 4 and (bits == 8 or ns % 2 == 0)
    assert op.kernel_name == ("fc_i8math_stream_kernel" if stream_ok else "fc_int8_math_kernel"), op.kernel_name
