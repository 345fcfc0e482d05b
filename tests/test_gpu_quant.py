"""GPU parity of per-token quantization: codes and params bit-exact against the oracle."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

import mldhip as M
import workloads as W


def run_quant(src_slices_np, tokens, channels, packed_type, symmetric, calc_sum, batch=1, height=1, nearest_even=False):
    import torch
    f16 = src_slices_np.dtype == np.float16
    src = torch.from_numpy(src_slices_np).cuda()
    slices = (channels + 3) // 4
    width = tokens // (batch * height)
    signed = packed_type in (M.PACKED_INT8C4, M.PACKED_INT8C16, M.PACKED_INT8W4C4)
    if packed_type in (M.PACKED_INT8C16, M.PACKED_UINT8C16):
        shape = ((slices + 3) // 4, tokens, 16)
    elif packed_type in (M.PACKED_INT4C32, M.PACKED_UINT4C32):
        shape = ((slices + 7) // 8, tokens, 16)
    elif packed_type in (M.PACKED_INT8W4C4, M.PACKED_UINT8W4C4):
        shape = (slices, height, (width + 3) // 4, batch, 16)
    else:
        shape = (slices, tokens, 4)
    # a fill no code path leaves behind: every byte of the packed tensor must be written
    codes = torch.full(shape, 0x5A, dtype=torch.int8 if signed else torch.uint8, device="cuda")
    params = torch.zeros((tokens, 4), dtype=torch.float32, device="cuda")
    op = M.quantization_create(M.FLOAT16 if f16 else M.FLOAT32, packed_type, channels, calc_sum,
                               symmetric, max_tokens=tokens, round_to_nearest_even=nearest_even)
    op.bind([src], [codes, params])
    op.set_shape(batch, height, width)
    print("quant", tokens, channels, packed_type, symmetric, calc_sum, batch, height, flush=True)
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
@pytest.mark.parametrize("packed_type", [M.PACKED_INT8C4, M.PACKED_UINT8C4, M.PACKED_INT8C16, M.PACKED_UINT8C16,
                                         M.PACKED_INT4C32, M.PACKED_UINT4C32, M.PACKED_INT8W4C4, M.PACKED_UINT8W4C4])
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


@pytest.mark.parametrize("packed_type", [M.PACKED_INT8W4C4, M.PACKED_UINT8W4C4, M.PACKED_INT4C32, M.PACKED_INT8C16])
@pytest.mark.parametrize("b,h,w,c", [(1, 3, 7, 24), (3, 2, 5, 44), (2, 1, 1, 100), (1, 13, 15, 237), (4, 1, 64, 2048)])
def test_packed_outputs_with_height_width_batch(oracle, packed_type, b, h, w, c):
    """The packed tensors on BHWC shapes: W4C4 addresses by column (widths that are not multiples of 4
    repeat the last column), C16 / C32 groups that the channels do not fill repeat the last slice."""
    tokens = b * h * w
    rng = np.random.default_rng(b * 1000 + h * 100 + w + c)
    x = edge_tensor(rng, tokens, c)
    src = W.to_slices(x).astype(np.float16)
    osrc = oracle.f32_to_f16_bits(src.astype(np.float32))
    for symmetric in (True, False):
        codes, params = run_quant(src, tokens, c, packed_type, symmetric, True, batch=b, height=h)
        rcodes, rparams = oracle.quantize(osrc, tokens, c, packed_type, symmetric, True, batch=b, height=h)
        assert np.array_equal(params.view(np.uint32), rparams.view(np.uint32))
        assert codes.shape == rcodes.shape and np.array_equal(codes.view(np.uint8), rcodes.view(np.uint8))


def test_int4_literal_bytes_on_gpu():
    """The hand-computed 4-bit vector of the oracle's tests, straight through the C-ABI."""
    row = np.array([7.0, -7.0, 3.5, 0.5, -0.5, -3.5, 6.49, 0.0], np.float32)
    src = W.to_slices(row[None]).astype(np.float16)
    codes, params = run_quant(src, 1, 8, M.PACKED_INT4C32, True, True)
    assert codes.tobytes() == bytes([0x97, 0x14, 0xD0, 0x06] + [0xD0, 0x06] * 6)
    assert params[0].tolist() == [1.0, 0.0, 8.0, 0.0]
    codes, params = run_quant(src, 1, 8, M.PACKED_UINT4C32, True, False)
    assert codes.tobytes() == bytes([0x1F, 0x9C, 0x58, 0x8E] + [0x58, 0x8E] * 6)
    assert params[0].tolist() == [1.0, -8.0, 0.0, 0.0]


@pytest.mark.parametrize("symmetric", [True, False])
@pytest.mark.parametrize("dtype", [np.float16, np.float32])
def test_round_to_nearest_even_switch(oracle, symmetric, dtype):
    """The switch that is not the reference's rule: codes = rint(x * scale) + 128 (symmetric) or
    rint((x - min) * scale) (asymmetric), ties to even, with the params of the reference's rule.
    Against a numpy fp32 restatement of exactly that, bit for bit; and against the reference's rule:
    the two differ by one code, only where the scaled value lies half way between two codes (within
    the fp32 rounding of the reference's sum x * scale + 128.5), and the test prints how often."""
    rng = np.random.default_rng(17)
    tokens, channels = 64, 512
    x = edge_tensor(rng, tokens, channels)
    # a row of exact ties: multiples of half a step at scale 1 (symmetric: absmax 127; asymmetric: range 0 .. 255)
    x[5] = 0.0
    if symmetric:
        x[5, :255] = np.arange(-127, 128) * 0.5
        x[5, 255] = 127.0
    else:
        x[5, :511] = np.arange(511) * 0.5
        x[5, 511] = 255.0
    x = x.astype(dtype)
    src = W.to_slices(x)
    packed = M.PACKED_INT8C4
    ref_codes, ref_params = run_quant(src, tokens, channels, packed, symmetric, True)
    codes, params = run_quant(src, tokens, channels, packed, symmetric, True, nearest_even=True)
    assert np.array_equal(params[:, :2], ref_params[:, :2])  # inv_scale and offset do not depend on the rounding
    # numpy restatement of the switch, in fp32 like the kernel (the scale is the kernel's: 1 / inv_scale, or
    # 255 / range for the asymmetric rule, recomputed here from the oracle's params of the same rows)
    rc, rp = oracle.quantize(oracle.f32_to_f16_bits(src.astype(np.float32)) if dtype == np.float16 else src,
                             tokens, channels, oracle.PACKED_INT8C4, symmetric, True)
    assert np.array_equal(ref_codes, rc) and np.array_equal(ref_params, rp)
    xf = x.astype(np.float32)
    inv = rp[:, 0].astype(np.float32)
    want = np.zeros((tokens, channels), np.int32)
    for t in range(tokens):
        if symmetric:
            scale = np.float32(0.0) if inv[t] == 0 else np.float32(1.0) / inv[t]
            v = np.rint(xf[t] * scale).astype(np.float32) + np.float32(128.0)
        else:
            # (the reference's search starts from element (b, 0, 0, 0): the first channel of the batch
            # element's first token takes part in every token's range)
            mn, mx = min(xf[t].min(), xf[0, 0]), max(xf[t].max(), xf[0, 0])
            with np.errstate(over="ignore"):
                rng_t = np.float32(dtype(mx) - dtype(mn))  # in the source type: +-65504 in fp16 gives inf
            with np.errstate(divide="ignore", invalid="ignore"):
                scale = np.float32(255.0) / rng_t
                v = np.rint((xf[t] - mn) * scale)
            v = np.where(np.isnan(v), 0.0, v)
        want[t] = np.clip(v, 0, 255).astype(np.int32) - 128
    got = W.from_slices(codes.astype(np.int32), channels)
    assert np.array_equal(got, want)
    ref = W.from_slices(ref_codes.astype(np.int32), channels)
    diff = got != ref
    assert np.abs(got - ref).max() <= 1
    assert (got[5][diff[5]] % 2 == 0).all()  # in the row of exact ties the switch took the even code
    print("codes that differ between the two rules: %d of %d (%d of them in the row of exact ties)" % (
        diff.sum(), diff.size, diff[5].sum()))
    assert 0 < diff[5].sum() and diff.sum() - diff[5].sum() <= diff.size // 1000
