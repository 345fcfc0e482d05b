"""GPU parity of the FullyConnected over ringed uint8 weights (ConvRuntimeCheckDesc::ring_i_offset_index /
ring_o_offset_index read at launch from the int32 "params" object; common/kernels/fully_connected.cc:
411-471, 676-706), through the C-ABI, against the oracle's restatement and the float64 product over the
rolled weights.  Sizes and offsets are the reference's own (FullyConnectedRingedITest / RingedOTest,
common/kernels/tests/fully_connected_test_util.cc:628-900: 72 / 20 / 56 channels, offsets 0, 17, 20, 33, 49,
one and three weight matrices; the reference runs float weights there, this path uint8 ones), plus larger
rings."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

import mldhip as M
import workloads as W
from test_oracle_ring import make, rolled_product

OFFSETS = [0, 17, 20, 33, 49]


def run_ring(o, axis, src_c, dst_c, ring, batch, offsets, f16, seed, src_end_ch=None, tokens=1, dst_end_ch=None):
    """One op, its ring offset rewritten on the device between launches.  batch > 1: the batch-ids op with
    one dst row per matrix (the reference's test puts matrix y on row y)."""
    import torch
    q, act, scale, zp, bias = make(seed, src_c, dst_c, ring, axis, batch)
    if tokens > 1:
        rng = np.random.default_rng(seed + 100)
        act = rng.uniform(-1, 1, size=(batch * tokens, src_c)).astype(np.float32)
    td = np.float16 if f16 else np.float32
    mt = M.FLOAT16 if f16 else M.FLOAT32
    tt = torch.float16 if f16 else torch.float32
    act = act.astype(td).astype(np.float32)
    scale, bias = scale.astype(td).astype(np.float32), bias.astype(td).astype(np.float32)
    w_o, w_i = q.shape[0], q.shape[3]
    desc = M.make_desc(M.UINT8, M.LAYOUT_I4O4 if axis == "i" else M.LAYOUT_O4I4, (w_o + 3) // 4)
    packed = M.rearrange_int8_as_uint8(q, desc)
    assert np.array_equal(packed, o.int8_as_uint8(q, o.LAYOUT_I4O4 if axis == "i" else o.LAYOUT_O4I4, (w_o + 3) // 4))
    ks, ns = (src_c + 3) // 4, (dst_c + 3) // 4
    pad = lambda v: np.pad(v, (0, ns * 4 - dst_c)).astype(np.float32)
    tens = lambda v: torch.from_numpy(M.scale_to_tensor(v, mt).view(td) if f16 else M.scale_to_tensor(v, mt)).cuda()
    params = np.array([0, -1 if src_end_ch is None else src_end_ch, -1 if dst_end_ch is None else dst_end_ch], np.int32)
    kw = dict(ring_size=ring, has_bias=True, has_zero_point_tensor=True, scale_shape=(dst_c, 1), max_tokens=batch * tokens)
    kw["ring_i_offset_index" if axis == "i" else "ring_o_offset_index"] = 0
    if axis == "i":
        kw["src_channels"] = src_c
    else:
        kw["dst_channels"] = dst_c
    if src_end_ch is not None:
        kw["src_end_ch_index"] = 1
    if dst_end_ch is not None:
        kw["dst_end_ch_index"] = 2
    if batch > 1:
        kw["weights_batch"] = batch
    op = M.fc_create(M.PRECISION_F32_F16 if f16 else M.PRECISION_F32, mt, mt, w_o, w_i, desc, **kw)
    # rows of `tokens` tokens: tensors [slices][batch * tokens][4]
    d_act = torch.from_numpy(W.to_slices(act).astype(td)).cuda()
    d_params = torch.from_numpy(params).cuda()
    srcs = [d_act]
    if batch > 1:
        srcs.append(torch.arange(batch, dtype=torch.int32, device="cuda"))
        scale_t = torch.from_numpy(np.tile(pad(scale), batch).astype(td)).cuda()  # [1][batch][ns][4]
        zp_t = torch.from_numpy(np.tile(pad(zp), batch).astype(td)).cuda()
    else:
        scale_t, zp_t = tens(scale), tens(zp)
    srcs += [torch.from_numpy(packed).cuda(), scale_t, zp_t, torch.from_numpy(pad(bias).astype(td)).cuda(), d_params]
    out = torch.zeros((ns, batch * tokens, 4), dtype=tt, device="cuda")
    assert op.src_names[-1] == "params"
    op.bind(srcs, [out])
    op.set_shape(1, batch, tokens) if batch > 1 else op.set_shape(1, 1, tokens)
    conv = (lambda a: o.f32_to_f16_bits(np.asarray(a, np.float32))) if f16 else (lambda a: np.asarray(a, np.float32))
    # a ring over the input channels, a multiple of 4 long, with the window inside one turn, at up to 4
    # tokens per row and 16 per launch, runs on the kernel that walks the ring's rows; every case also
    # runs on the unspecialised kernel
    fast = axis == "i" and ring % 4 == 0 and src_c <= ring and tokens <= 4 and batch * tokens <= 16
    for forced, off in [(f, x) for f in (False, True) for x in offsets]:
        params[0] = off
        d_params.copy_(torch.from_numpy(params))
        out.fill_(7.0)
        print("ring", axis, src_c, dst_c, ring, "batch", batch, "tokens", tokens, "offset", off, "f16", f16, "src_end", src_end_ch,
              "unspecialised" if forced else "", flush=True)
        with M.tuning(**(dict(force_generic=1) if forced else {})):
            op.launch(torch.cuda.current_stream().cuda_stream)
        torch.cuda.synchronize()
        assert op.kernel_name == ("fc_w8_ring_i_kernel" if fast and not forced else "fc_generic_kernel"), op.kernel_name
        got = W.from_slices(out.cpu().numpy().astype(np.float32), dst_c)
        # dst slices from the bound (rounded up to 32 channels) on are not written
        n_written = dst_c if dst_end_ch is None else min((dst_end_ch + 31) // 32 * 32, ns * 4)
        if n_written < dst_c:
            assert np.all(got[:, n_written:] == 7.0), "dst slices beyond the bound were written"
        active = None if src_end_ch is None else (min(src_end_ch, src_c) + 3) // 4 * 4
        for b in range(batch):
            rows = slice(b * tokens, (b + 1) * tokens)
            a_rows = act[rows]
            rest = o.fc_ringed_kernel(conv(o.to_slices(a_rows)), packed, tokens, src_c, dst_c, axis, ring, off,
                                      o.PREC_F32F16 if f16 else o.PREC_F32, o.SCALE_LINEAR, conv(pad(scale)), conv(pad(zp)),
                                      conv(pad(bias)), 1, src_end_ch=src_end_ch, batch_id=b)
            rest = o.from_slices(o.f16_bits_to_f32(rest) if f16 else rest, dst_c)
            for t in range(tokens):
                exact = rolled_product(q, a_rows[t], scale, zp, bias, axis, ring, off, b, src_c, dst_c, active=active)
                exact = exact[:n_written]
                rms = np.sqrt(np.mean(exact ** 2))
                err = np.abs(got[rows][t][:n_written] - exact).max()
                err_rest = np.abs(rest[t][:n_written] - exact).max()
                if f16:
                    assert err <= 2e-2 * rms, (b, off, err, rms)
                else:
                    assert err <= 1.1920929e-7 * (src_c + 1) * max(1.0, np.abs(exact).max()), (b, off, err)
                # no less accurate than the reference kernel's restatement (floor: a quarter ulp of the output at the RMS)
                assert err <= 1.5 * err_rest + (2.0 ** -12 if f16 else 2.0 ** -25) * max(rms, np.abs(exact).max()), (b, off, err, err_rest)


@pytest.mark.parametrize("f16", [False, True])
@pytest.mark.parametrize("batch", [1, 3])
def test_reference_ringed_i_cases(oracle, f16, batch):
    run_ring(oracle, "i", 20, 72, 56, batch, OFFSETS, f16, seed=3 + batch)


@pytest.mark.parametrize("f16", [False, True])
@pytest.mark.parametrize("batch", [1, 3])
def test_reference_ringed_o_cases(oracle, f16, batch):
    run_ring(oracle, "o", 72, 20, 56, batch, OFFSETS, f16, seed=11 + batch)


@pytest.mark.parametrize("src_end_ch", [13, 24])
def test_ringed_i_with_src_end_ch(oracle, src_end_ch):
    """ring_i_offset_index beside src_end_ch_index, as the reference's ringed test binds them
    (params = {ring_offset, src_end_ch})."""
    run_ring(oracle, "i", 20, 72, 56, 1, [17, 49], False, seed=21, src_end_ch=src_end_ch)


@pytest.mark.parametrize("f16", [False, True])
def test_ring_i_window_shapes(oracle, f16):
    """The ring-walking kernel: windows that fill the ring (the window wraps onto its first row), windows of one
    and of a few channels, every offset modulo 4, dst widths below and above 64 slices, 2 and 4 tokens per
    row, rows with batched weights, a source bound inside the window."""
    run_ring(oracle, "i", 1024, 64, 1024, 1, [0, 1, 2, 3, 1021, 517], f16, seed=41)
    run_ring(oracle, "i", 1, 256, 64, 1, [0, 3, 62, 63], f16, seed=42)
    run_ring(oracle, "i", 6, 520, 128, 1, [0, 125, 127], f16, seed=43, tokens=2)
    run_ring(oracle, "i", 2048, 128, 2048, 4, [5, 2047], f16, seed=44, tokens=4)
    run_ring(oracle, "i", 4096, 256, 8192, 1, [0, 4095, 6001], f16, seed=45, src_end_ch=1001)
    run_ring(oracle, "i", 512, 320, 512, 2, [0, 258], f16, seed=46, dst_end_ch=70, tokens=2)


def test_larger_rings_and_odd_offsets(oracle):
    """A key cache of 1024 positions read through a window of 300 (ring over I), a value cache of 512
    rows of which 128 are taken (ring over O); negative offsets and offsets beyond the ring; 3 tokens."""
    run_ring(oracle, "i", 300, 128, 1024, 1, [0, 1, 725, 1023, -7, 5000], True, seed=31, tokens=3)
    run_ring(oracle, "o", 256, 128, 512, 1, [0, 3, 385, 511, -1, 1025], True, seed=32, tokens=3)
