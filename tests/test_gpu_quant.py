"""GPU parity of per-token quantization: codes and params bit-exact against the oracle."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

import mldhip as M
import workloads as W


def run_quant(src_slices_np, tokens, channels, packed_type, symmetric, calc_sum, batch=1):
    import torch
    f16 = src_slices_np.dtype == np.float16
    src = torch.from_numpy(src_slices_np).cuda()
    slices = (channels + 3) // 4
    c16 = packed_type in (M.PACKED_INT8C16, M.PACKED_UINT8C16)
    shape = ((slices + 3) // 4, tokens, 16) if c16 else (slices, tokens, 4)
    signed = packed_type in (M.PACKED_INT8C4, M.PACKED_INT8C16)
    codes = torch.zeros(shape, dtype=torch.int8 if signed else torch.uint8, device="cuda")
    params = torch.zeros((tokens, 4), dtype=torch.float32, device="cuda")
    op = M.quantization_create(M.FLOAT16 if f16 else M.FLOAT32, packed_type, channels, calc_sum,
                               symmetric, max_tokens=tokens)
    op.bind([src], [codes, params])
    op.set_shape(batch, 1, tokens // batch)
    print("quant", tokens, channels, packed_type, symmetric, calc_sum, flush=True)
    op.launch(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert op.kernel_name == "quantize_kernel"
    return codes.cpu().numpy(), params.cpu().numpy()


def edge_tensor(rng, tokens, channels):
    """Rows in the spirit of tests/quantize_and_dequantize_test_util.cc:554-585: an all-zero
    row, a +-65504 row, a constant row, shifted ranges, exact .5 ties."""
    x = rng.standard_normal((tokens, channels)).astype(np.float32) * 4
    if tokens > 1:
        x[0] = 0
        x[1] = rng.uniform(-1, 1, channels) * 65504
        x[1, 0], x[1, 1] = 65504, -65504
    if tokens > 2:
        x[2] = 3.25
    for t in range(3, tokens):
        x[t] += -4 if t % 2 else 4
    if tokens > 4:
        x[4, :16] = np.arange(16) * (127.0 / 254) * (8 / 127)  # multiples of half a step for absmax 8
        x[4, 16] = 8.0
        x[4, 17:] = np.clip(x[4, 17:], -8, 8)
    return x.astype(np.float16).astype(np.float32)


@pytest.mark.parametrize("tokens,channels", [(13 * 15, 237), (35, 64), (5, 2048), (1, 16)])
@pytest.mark.parametrize("dtype", [np.float16, np.float32])
@pytest.mark.parametrize("packed_type", [M.PACKED_INT8C4, M.PACKED_UINT8C4, M.PACKED_INT8C16, M.PACKED_UINT8C16])
@pytest.mark.parametrize("symmetric", [True, False])
def test_quantize_bit_exact(oracle, tokens, channels, dtype, packed_type, symmetric):
    rng = np.random.default_rng(tokens + channels)
    x = edge_tensor(rng, tokens, channels)
    src = W.to_slices(x).astype(dtype)
    for calc_sum in (False, True):
        codes, params = run_quant(src, tokens, channels, packed_type, symmetric, calc_sum)
        osrc = oracle.f32_to_f16_bits(src.astype(np.float32)) if dtype == np.float16 else src
        rcodes, rparams = oracle.quantize(osrc, tokens, channels, packed_type, symmetric, calc_sum)
        bad = np.nonzero((params.view(np.uint32) != rparams.view(np.uint32)).any(axis=1))[0]
        assert bad.size == 0, (bad[:5], params[bad[:5]], rparams[bad[:5]], x[bad[:3], :8])
        assert np.array_equal(codes, rcodes), np.argwhere(codes != rcodes)[:5]


def test_config4_activation_quantization(oracle):
    """c4's front half at full size: 2048 tokens x 2048 channels fp16 -> kInt8C16, symmetric
    (the config) and asymmetric (the reference's default)."""
    rng = np.random.default_rng(0)
    tokens = channels = 2048
    x = rng.standard_normal((tokens, channels)).astype(np.float16)
    src = W.to_slices(x)
    for symmetric in (True, False):
        codes, params = run_quant(src, tokens, channels, M.PACKED_INT8C16, symmetric, True)
        rcodes, rparams = oracle.quantize(oracle.f32_to_f16_bits(src.astype(np.float32)), tokens, channels,
                                          oracle.PACKED_INT8C16, symmetric, True)
        assert np.array_equal(params.view(np.uint32), rparams.view(np.uint32))
        assert np.array_equal(codes, rcodes)
        # size-independent property: x ~= q*inv_scale + offset within 0.51 of a step
        q = codes.transpose(1, 0, 2).reshape(tokens, -1)[:, :channels].astype(np.float32)
        deq = q * params[:, 0:1] + params[:, 1:2]
        assert np.all(np.abs(deq - x.astype(np.float32)) <= 0.51 * params[:, 0:1] + 1e-6)


def test_batched_seed_element(oracle):
    # tokens = (y*W+x)*B+b: the asymmetric search of token t starts from element (b = t % B, 0, 0, 0)
    rng = np.random.default_rng(3)
    tokens, channels, batch = 12, 40, 3
    x = rng.standard_normal((tokens, channels)).astype(np.float32)
    x[0, 0], x[1, 0], x[2, 0] = 50.0, -60.0, 70.0
    src = W.to_slices(x)
    codes, params = run_quant(src, tokens, channels, M.PACKED_INT8C4, False, False, batch=batch)
    rcodes, rparams = oracle.quantize(src, tokens, channels, oracle.PACKED_INT8C4, False, False, batch=batch)
    assert np.array_equal(params.view(np.uint32), rparams.view(np.uint32))
    assert np.array_equal(codes, rcodes)


@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_symmetric_literal_tie_vector_on_gpu(dtype):
    """The hand-worked half-up case of tests/test_oracle_quant.py, on the GPU: absmax 127 gives
    scale 1, and 0.5 -> 1, -0.5 -> 0, 1.5 -> 2, -1.5 -> -1."""
    from test_oracle_quant import LITERAL_TIE_CODES, LITERAL_TIE_ROW
    src = W.to_slices(LITERAL_TIE_ROW[None]).astype(dtype)
    codes, params = run_quant(src, 1, 8, M.PACKED_INT8C4, True, True)
    assert params[0, 0] == 1.0 and params[0, 1] == 0.0 and params[0, 2] == LITERAL_TIE_CODES.sum()
    assert np.array_equal(W.from_slices(codes, 8).astype(np.int32)[0], LITERAL_TIE_CODES)
