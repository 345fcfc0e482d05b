"""The oracle's restatement of the FullyConnected over ringed uint8 weights
(ConvRuntimeCheckDesc::ring_i_offset_index / ring_o_offset_index, common/kernels/fully_connected.cc:
411-471, 676-706), pinned by what the mathematics fixes: a ring offset r is the plain FullyConnected
over the weights rolled by r along the ringed axis, computed here in float64 straight from the
unpacked values.  Sizes and offsets are those of the reference's own tests
(common/kernels/tests/fully_connected_test_util.cc:628-900: 72 / 20 / 56 channels, offsets
0, 17, 20, 33, 49, one and three weight matrices); the reference runs them with float weights, the
quantized path here with uint8 weights, per-channel scales and zero points.  CPU only."""
import numpy as np
import pytest

OFFSETS = [0, 17, 20, 33, 49]


def make(seed, src_c, dst_c, ring, axis, batch, with_zp=True):
    rng = np.random.default_rng(seed)
    # weights: the ring runs along I (shape OHWI(dst, batch, 1, ring)) or along O (OHWI(ring, batch, 1, src))
    shape = (dst_c, batch, 1, ring) if axis == "i" else (ring, batch, 1, src_c)
    q = rng.integers(-127, 128, size=shape, dtype=np.int8)
    act = rng.uniform(-1, 1, size=(batch, src_c)).astype(np.float32)  # one token per matrix row
    scale = (np.abs(rng.normal(0.0, 0.02, size=dst_c)) / 127.0 + 1e-5).astype(np.float32)
    zp = rng.integers(-3, 4, size=dst_c).astype(np.float32) if with_zp else None
    bias = (rng.uniform(-1, 1, size=dst_c) * 0.1).astype(np.float32)
    return q, act, scale, zp, bias


def rolled_product(q, act_row, scale, zp, bias, axis, ring, off, b, src_c, dst_c, active=None):
    """float64: out[o] = bias[o] + scale[o] * sum_i act[i] * (q_rolled[o, i] - zp[o])."""
    off = off % ring
    k = src_c if active is None else active
    a = np.zeros(k, np.float64)
    a[:min(k, src_c)] = act_row[:min(k, src_c)]
    if axis == "i":
        wi = (np.arange(k) + off) % ring
        w = q[:, b, 0, :][:, wi].astype(np.float64)  # [dst][k]
    else:
        wo = (np.arange(dst_c) + off) % ring
        w = q[wo, b, 0, :k].astype(np.float64)
    z = 0.0 if zp is None else zp.astype(np.float64)[:, None]
    return bias.astype(np.float64) + scale.astype(np.float64) * ((w - z) @ a)


def run_oracle(o, q, act, scale, zp, bias, axis, ring, off, src_c, dst_c, batch, f16, src_end_ch=None):
    layout = o.LAYOUT_I4O4 if axis == "i" else o.LAYOUT_O4I4
    packed = o.int8_as_uint8(q, layout, (q.shape[0] + 3) // 4)
    conv = (lambda a: o.f32_to_f16_bits(np.asarray(a, np.float32))) if f16 else (lambda a: np.asarray(a, np.float32))
    ns = (dst_c + 3) // 4
    pad = lambda v: np.pad(v, (0, ns * 4 - dst_c))
    outs = []
    for b in range(batch):
        r = o.fc_ringed_kernel(conv(o.to_slices(act[b:b + 1])), packed, 1, src_c, dst_c, axis, ring, off,
                               o.PREC_F32F16 if f16 else o.PREC_F32, o.SCALE_LINEAR, conv(pad(scale)),
                               None if zp is None else conv(pad(zp)), conv(pad(bias)), 1, src_end_ch=src_end_ch, batch_id=b)
        r = o.f16_bits_to_f32(r) if f16 else r
        outs.append(o.from_slices(r, dst_c)[0])
    return np.stack(outs)


@pytest.mark.parametrize("batch", [1, 3])
@pytest.mark.parametrize("off", OFFSETS + [-5, 56, 123])
def test_ring_i_equals_rolled_weights(oracle, batch, off):
    """FullyConnectedRingedITest: 20 src channels against a ring of 56 input rows, 72 dst channels."""
    o = oracle
    src_c, dst_c, ring = 20, 72, 56
    q, act, scale, zp, bias = make(3 + batch, src_c, dst_c, ring, "i", batch)
    got = run_oracle(o, q, act, scale, zp, bias, "i", ring, off, src_c, dst_c, batch, f16=False)
    for b in range(batch):
        ref = rolled_product(q, act[b], scale, zp, bias, "i", ring, off, b, src_c, dst_c)
        assert np.abs(got[b] - ref).max() <= 1.2e-7 * (src_c + 1) * max(1.0, np.abs(ref).max()), (b, off)


@pytest.mark.parametrize("batch", [1, 3])
@pytest.mark.parametrize("off", OFFSETS + [-1, 56, 200])
def test_ring_o_equals_rolled_weights(oracle, batch, off):
    """FullyConnectedRingedOTest: 20 dst channels out of a ring of 56 output rows, 72 src channels; scale,
    zero point and bias stay with the dst channel."""
    o = oracle
    src_c, dst_c, ring = 72, 20, 56
    q, act, scale, zp, bias = make(11 + batch, src_c, dst_c, ring, "o", batch)
    got = run_oracle(o, q, act, scale, zp, bias, "o", ring, off, src_c, dst_c, batch, f16=False)
    for b in range(batch):
        ref = rolled_product(q, act[b], scale, zp, bias, "o", ring, off, b, src_c, dst_c)
        assert np.abs(got[b] - ref).max() <= 1.2e-7 * (src_c + 1) * max(1.0, np.abs(ref).max()), (b, off)


@pytest.mark.parametrize("src_end_ch", [13, 20, 24, 0])
@pytest.mark.parametrize("off", [17, 49])
def test_ring_i_with_src_end_ch(oracle, src_end_ch, off):
    """The composition the reference's ringed test exercises (runtime_check.src_end_ch_index = 1 beside
    ring_i_offset_index = 0): the K loop stops after ceil(min(src_end_ch, src channels) / 4) slices."""
    o = oracle
    src_c, dst_c, ring = 20, 72, 56
    q, act, scale, zp, bias = make(21, src_c, dst_c, ring, "i", 1)
    got = run_oracle(o, q, act, scale, zp, bias, "i", ring, off, src_c, dst_c, 1, f16=False, src_end_ch=src_end_ch)
    active = (min(src_end_ch, src_c) + 3) // 4 * 4
    ref = rolled_product(q, act[0], scale, zp, bias, "i", ring, off, 0, src_c, dst_c, active=active)
    assert np.abs(got[0] - ref).max() <= 1.2e-7 * (src_c + 1) * max(1.0, np.abs(ref).max())


def test_zero_offset_is_the_plain_kernel(oracle):
    """With offset 0 and src channels = ring the gathered blocks are the packed buffer itself, and the
    result is the plain kernel's bit for bit (fp16 tensors)."""
    o = oracle
    q, act, scale, zp, bias = make(5, 56, 72, 56, "i", 1, with_zp=False)
    packed = o.int8_as_uint8(q, o.LAYOUT_I4O4, 18)
    assert np.array_equal(o.ringed_gather(packed, "i", 56, 0, 14, 18).reshape(-1), packed)
    h = lambda a: o.f32_to_f16_bits(np.asarray(a, np.float32))
    a = h(o.to_slices(act))
    ring = o.fc_ringed_kernel(a, packed, 1, 56, 72, "i", 56, 0, o.PREC_F32F16, o.SCALE_LINEAR, h(scale), None, h(bias), 1)
    plain = o.fc_kernel(a, packed, 1, 56, 72, o.PREC_F32F16, 8, o.SCALE_LINEAR, h(scale), None, h(bias), 1)
    assert np.array_equal(ring, plain)
    # the O4I4 buffer at offset 0 gathers to the same I4O4 blocks
    packed_o = o.int8_as_uint8(q, o.LAYOUT_O4I4, 18)
    assert np.array_equal(o.ringed_gather(packed_o, "o", 72, 0, 14, 18).reshape(-1), packed)
