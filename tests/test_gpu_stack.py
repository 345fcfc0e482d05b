"""GPU parity of the decoder-stack FullyConnected sequence (18 layers x {q,k,v,o,gate,up,down},
int4 group-32, fp16), through the C-ABI: every FC of every layer against the textbook
reference over dequantised weights, max|err| <= 2e-2 * RMS(reference output), for a batch-1
decode step and a 128-token prefill; and launch-to-launch determinism."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

import workloads as W
from decoder_stack import DecoderStack
from test_gpu_fc import check_fp, textbook

LAYERS = 3  # distinct device copies; every layer is checked


@pytest.fixture(scope="module")
def stack():
    return DecoderStack(layers=LAYERS, max_tokens=128)


@pytest.fixture(scope="module")
def decode_stack():
    """The same stack with the weights packed as the ops of a decode graph ask for them."""
    return DecoderStack(layers=LAYERS, max_tokens=128, decode_layout=True)


@pytest.mark.parametrize("tokens", [1, 128, 7])
def test_stack_parity(stack, tokens):
    print("decoder stack, tokens =", tokens, flush=True)
    stack.set_tokens(tokens)
    stack.launch()
    first = {}
    for layer in range(LAYERS):
        for idx, case in enumerate(stack.cases):
            got = stack.result(layer, idx)
            ref = textbook(stack.case(idx, layer=layer))
            check_fp(got, ref, stack.case(idx, layer=layer), "layer %d %s" % (layer, case["name"]))
            first[(layer, idx)] = got
    names = set(stack.kernel_names())
    assert names <= {"fc_w4_stream_kernel", "fc_w4_strip_kernel", "fc_w4_mfma_gemm_kernel"}, names
    stack.launch()
    for (layer, idx), got in first.items():
        assert np.array_equal(got, stack.result(layer, idx))


@pytest.mark.parametrize("tokens", [1, 3, 128])
def test_decode_layout_stack_parity(decode_stack, tokens):
    """The decode layout: the 2048- and 256-channel layers in output groups of 2 slices (the
    row-interleaved kernel at one token), the 16384-channel ones in groups of 16 (the strip kernel);
    more tokens run on the general kernels over the same buffers."""
    import mldhip as M
    st = decode_stack
    assert [M.fc_int4_weights_desc(n, k, decode=True).output_group_size for _, k, n in W.C5_LAYER] == [2, 2, 2, 2, 16, 16, 2]
    st.set_tokens(tokens)
    for fused in (True, False):
        for out in st.outs:
            out.zero_()
        st.launch(fused=fused)
        for layer in range(LAYERS):
            for idx, case in enumerate(st.cases):
                got = st.result(layer, idx)
                check_fp(got, textbook(st.case(idx, layer=layer)), st.case(idx, layer=layer),
                         "decode layout layer %d %s" % (layer, case["name"]))
        if tokens == 1:
            names = st.kernel_names()[:7]
            assert names == ["fc_w4_rows_kernel"] * 4 + ["fc_w4_strip_kernel"] * 2 + ["fc_w4_rows_kernel"], names
    first = [st.result(layer, idx) for layer in range(LAYERS) for idx in range(len(st.cases))]
    st.launch(fused=False)
    again = [st.result(layer, idx) for layer in range(LAYERS) for idx in range(len(st.cases))]
    for a, b in zip(first, again):
        assert np.array_equal(a, b)


def test_stack_accounting(stack):
    per_layer = sum(c["k"] * c["n"] // 2 + (c["k"] // 32) * c["n"] * 2 for c in stack.cases)
    assert stack.weight_bytes() == LAYERS * per_layer
    assert per_layer == 61931520  # one layer of config 5


def test_fused_launch_matches_single_launches(stack):
    """q/k/v and gate/up as one launch each give the bytes of the one-by-one launches."""
    import mldhip as M
    stack.set_tokens(1)
    stack.launch(fused=False)
    single = [stack.result(layer, idx) for layer in range(LAYERS) for idx in range(len(stack.cases))]
    for out in stack.outs:
        out.zero_()
    stack.launch(fused=True)
    fused = [stack.result(layer, idx) for layer in range(LAYERS) for idx in range(len(stack.cases))]
    for a, b in zip(single, fused):
        assert np.array_equal(a, b)
    # ops over different inputs (o reads width 2048, down reads 16384) cannot share a launch
    names = [c["name"] for c in stack.cases]
    o_op = stack.nodes[names.index("o")][2]
    down_op = stack.nodes[names.index("down")][2]
    with pytest.raises(M.MldhipError) as err:
        M.fc_launch_fused([o_op, down_op])
    assert err.value.code == M.FAILED_PRECONDITION
    # prefill token counts: the MFMA kernel takes the fused launches; a fused launch may split K
    # across work-groups differently, so the comparison is the parity bar, plus closeness
    for tokens in (128, 7):
        stack.set_tokens(tokens)
        stack.launch(fused=False)
        single = [stack.result(layer, idx) for layer in range(LAYERS) for idx in range(len(stack.cases))]
        for out in stack.outs:
            out.zero_()
        stack.launch(fused=True)
        pos = 0
        for layer in range(LAYERS):
            for idx, case in enumerate(stack.cases):
                got = stack.result(layer, idx)
                ref = textbook(stack.case(idx, layer=layer))
                check_fp(got, ref, stack.case(idx, layer=layer), "fused layer %d %s" % (layer, case["name"]))
                rms = np.sqrt(np.mean(ref ** 2))
                worst = np.abs(got - single[pos]).max()
                print("tokens", tokens, case["name"], "fused vs single max|diff|/rms = %.2e" % (worst / rms), flush=True)
                assert worst <= 2e-3 * rms
                pos += 1


@pytest.mark.parametrize("decode_layout", [False, True])
def test_graph_replays_match_eager(decode_layout):
    """A decode step and a prefill step captured into a graph: several replays, with eager work
    and synchronisations in between, must reproduce the eager results bit for bit (launches
    allocate nothing and record no memset nodes); in the layout for both graphs and in the decode
    ops' layout."""
    import torch
    from decoder_stack import DecoderStack
    st = DecoderStack(layers=2, max_tokens=128, decode_layout=decode_layout)
    for tokens in (1, 128):
        st.set_tokens(tokens)
        st.launch()
        torch.cuda.synchronize()
        eager = [o.clone() for o in st.outs]
        stream = torch.cuda.Stream()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.stream(stream):
            with torch.cuda.graph(graph, stream=stream):
                st.launch(torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        for rep in range(3):
            for o in st.outs:
                o.zero_()
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            for idx, (a, b) in enumerate(zip(eager, st.outs)):
                assert torch.equal(a, b), (tokens, rep, idx)
            # eager work between replays
            st.launch()
            torch.cuda.synchronize()


@pytest.mark.timeout(900)
@pytest.mark.parametrize("decode_layout", [False, True])
def test_stack_chain_18_layers_decode(decode_layout):
    """The whole 18-layer stack at one token with the values flowing through it: every FC has its
    own weights (seed layer * 7 + index) and reads the re-normalised output of the FC before it in
    the layer's graph (q, k, v read the layer input; o reads q's output; gate and up read o's; down
    reads gate's; the next layer reads down's), N(0,1) after re-normalisation as the synthetic
    inputs are.  Each FC goes through the C-ABI on the kernel the bench uses (`decode_layout`: the weights
    as a decode graph's ops ask for them, the bench's default for the decode step; else the one layout
    that serves both graphs) and is held to the FullyConnected bar against float64 arithmetic over its
    dequantised weights."""
    import torch
    rng = np.random.default_rng(1234)
    x = rng.standard_normal(2048).astype(np.float16).astype(np.float32)

    def renorm(v):
        v = v.astype(np.float64)
        return ((v - v.mean()) / v.std()).astype(np.float16).astype(np.float32)

    def reference(case):
        q = case["w"].astype(np.float32)
        gs = case["k"] // case["groups"]
        prod = (q * case["act"][0][None, :]).reshape(case["n"], case["groups"], gs).sum(axis=2, dtype=np.float64)
        return (prod * case["scale"].astype(np.float64)).sum(axis=1)[None, :]

    worst = 0.0
    for layer in range(W.C5_LAYERS):
        outs = {}
        for idx, (name, k, n) in enumerate(W.C5_LAYER):
            src = {"q": x, "k": x, "v": x, "o": outs.get("q"), "gate": outs.get("o"), "up": outs.get("o"),
                   "down": outs.get("gate")}[name]
            case = W.make_fc_case(seed=layer * 7 + idx, m=1, k=k, n=n, weight_bits=4, tensor_dtype=np.float16,
                                  groups=k // 32)
            case["act"] = src[None, :].astype(np.float32)
            dev = W.FcDevice(case, decode_layout=decode_layout)
            dev.run()
            got = dev.result()
            want = "fc_w4_rows_kernel" if decode_layout and n < 8192 else "fc_w4_strip_kernel"
            assert dev.op.kernel_name == want, dev.op.kernel_name
            worst = max(worst, check_fp(got, reference(case), case, "layer %d %s" % (layer, name)))
            outs[name] = renorm(got[0])
            del dev
        x = outs["down"]
        print("layer", layer, "worst so far", worst, flush=True)
    torch.cuda.synchronize()
