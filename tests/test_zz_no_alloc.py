"""The allocation-free entry point (mldhip_fc_int4_decode_noalloc) against mldhip_op_launch on the same
inputs: two calls in a row, the second with a smaller input; results must agree bit for bit (the same
kernels run, the split-K sums only live elsewhere)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

import mldhip as M
import workloads as W


def run_pair(case, reference_layout, output_group=None):
    import torch
    dev = W.FcDevice(case, reference_layout=reference_layout, output_group=output_group)
    dev.run()
    ref = dev.result()
    kernel = dev.op.kernel_name
    out = torch.zeros_like(dev.out)
    bias = dev.bias if case["bias"] is not None else None
    M.fc_int4_decode_noalloc(dev.act, dev.weights, dev.scale, bias, out, case["n"], case["k"], case["groups"],
                             dev.desc.output_group_size, case["m"], torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    got = W.from_slices(out.cpu().numpy().astype(np.float32), case["n"])
    assert np.array_equal(got, ref), (kernel, np.abs(got - ref).max())
    return kernel


@pytest.mark.parametrize("reference_layout", [False, True])
def test_no_alloc_matches_op_launch(reference_layout):
    # first call: 16 MB matrix whose K is split across work-groups (the sums go through the scratch array)
    big = W.make_fc_case(seed=71, m=1, k=16384, n=2048, weight_bits=4, tensor_dtype=np.float16, groups=512, with_bias=True)
    print("no-alloc", big["k"], big["n"], reference_layout, flush=True)
    assert run_pair(big, reference_layout) in ("fc_w4_strip_kernel", "fc_w4_stream_kernel")
    # second call, smaller input, split as well; then two tokens
    small = W.make_fc_case(seed=72, m=1, k=16384, n=1024, weight_bits=4, tensor_dtype=np.float16, groups=1)
    print("no-alloc", small["k"], small["n"], reference_layout, flush=True)
    run_pair(small, reference_layout)
    two = W.make_fc_case(seed=73, m=2, k=4096, n=1536, weight_bits=4, tensor_dtype=np.float16, groups=1, with_bias=True)
    print("no-alloc", two["k"], two["n"], reference_layout, flush=True)
    run_pair(two, reference_layout)


def test_no_alloc_decode_layout():
    """Weights in output groups of 2 slices (the decode ops' layout) through the same entry point: the
    row-interleaved kernel, which needs no scratch; 8 slices per group on the streaming kernel."""
    case = W.make_fc_case(seed=74, m=1, k=16384, n=2048, weight_bits=4, tensor_dtype=np.float16, groups=512, with_bias=True)
    print("no-alloc, groups of 2 slices", flush=True)
    assert run_pair(case, False, output_group=2) == "fc_w4_rows_kernel"
    three = W.make_fc_case(seed=75, m=3, k=2048, n=1024, weight_bits=4, tensor_dtype=np.float16, groups=64)
    run_pair(three, False, output_group=2)
    run_pair(three, False, output_group=8)


def test_no_alloc_where_op_launch_takes_another_kernel(oracle):
    """2 and 4 tokens on a per-channel layer of 8192 channels and 1056 input channels: mldhip_op_launch runs the matrix-core
    GEMV there, this entry point the streaming one, so the result is held to the oracle, not to the op."""
    import torch
    from test_gpu_fc import check_as_accurate_as, check_fp, oracle_fc, textbook
    for m in (2, 4):
        # (K = 1056: 33 chunks, so the one-chunk token form of the strip kernel does not serve the launch either)
        case = W.make_fc_case(seed=76 + m, m=m, k=1056, n=8192, weight_bits=4, tensor_dtype=np.float16, groups=1, with_bias=True)
        dev = W.FcDevice(case)
        dev.run()
        assert dev.op.kernel_name == "fc_w4_mfma_stream_kernel", dev.op.kernel_name
        out = torch.zeros_like(dev.out)
        print("no-alloc", m, "tokens, 8192 channels", flush=True)
        M.fc_int4_decode_noalloc(dev.act, dev.weights, dev.scale, dev.bias, out, case["n"], case["k"], 1,
                                 dev.desc.output_group_size, m, torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        got = W.from_slices(out.cpu().numpy().astype(np.float32), case["n"])
        exact = textbook(case)
        check_fp(got, exact, case, "no-alloc")
        check_as_accurate_as(got, oracle_fc(oracle, case), exact, case, "no-alloc")


def test_no_alloc_rejects():
    import torch
    t = torch.zeros(4096, dtype=torch.float16, device="cuda")
    with pytest.raises(M.MldhipError) as e:
        M.fc_int4_decode_noalloc(t, t, t, None, t, 65540, 64, 1, 16385, 1)
    assert e.value.code == M.OUT_OF_RANGE
    with pytest.raises(M.MldhipError) as e:
        M.fc_int4_decode_noalloc(t, t, t, None, t, 64, 64, 1, 16, 5)
    assert e.value.code == M.OUT_OF_RANGE
    with pytest.raises(M.MldhipError) as e:
        M.fc_int4_decode_noalloc(t, t, t, None, t, 128, 64, 1, 7, 1)
    assert e.value.code == M.INVALID_ARGUMENT
