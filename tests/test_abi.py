"""CPU-side checks of the product library: it loads, exports every symbol include/mldhip.h
declares, validates arguments like the reference factories do, and lists src/dst objects in
the reference's registration order.  No kernel is launched here."""
import os
import re

import pytest

import mldhip as M

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "mldhip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(mldhip_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    lib = M.lib()
    names = declared_symbols()
    assert len(names) >= 25
    for name in names:
        assert hasattr(lib, name), name
    assert sorted(M.SYMBOLS) == names
    assert b"gfx950" in lib.mldhip_version()


def test_fc_weights_desc_matches_reference_factories():
    # common/kernels/fully_connected.cc:1218-1246
    d = M.fc_int4_weights_desc(14336, 4096, reference=True)
    assert (d.type, d.layout, d.output_group_size) == (M.UINT4, M.LAYOUT_I4O4, 3584)
    # this device's choice: the same layout enum in output groups of 16 slices (64-channel strips),
    # one group where the channel count does not divide; groups of 8 and 4 slices are read as well
    d = M.fc_int4_weights_desc(14336, 4096)
    assert (d.type, d.layout, d.output_group_size) == (M.UINT4, M.LAYOUT_I4O4, 16)
    assert M.fc_int4_weights_desc(256, 2048).output_group_size == 16
    assert M.fc_int4_weights_desc(533, 171).output_group_size == 134
    assert M.fc_int4_weights_desc(1032, 64).output_group_size == 258
    with M.tuning(fc_group=4):
        assert M.fc_int4_weights_desc(2048, 16384).output_group_size == 4
        assert M.fc_int4_weights_desc(1032, 64).output_group_size == 258  # 258 slices do not divide
    for g in (4, 8, 16):
        M.fc_create(M.PRECISION_F32_F16, M.FLOAT16, M.FLOAT16, 128, 64, M.make_desc(M.UINT4, M.LAYOUT_I4O4, g),
                    scale_shape=(128, 1))
    d = M.fc_int8_weights_desc(533, 171)
    assert (d.type, d.layout, d.output_group_size) == (M.UINT8, M.LAYOUT_I4O4, 134)
    assert M.packed_bytes(M.fc_int4_weights_desc(14336, 4096), 14336, 1, 1, 4096) == 29360128
    assert M.packed_bytes(M.fc_int8_weights_desc(2048, 2048), 2048, 1, 1, 2048) == 4194304


def test_fc_object_order():
    # fully_connected.cc:359-360, 1160-1170; fully_connected_util.cc:409-487
    wd = M.fc_int4_weights_desc(64, 64)
    op = M.fc_create(M.PRECISION_F32_F16, M.FLOAT16, M.FLOAT16, 64, 64, wd, scale_shape=(64, 2),
                     has_zero_point_tensor=True, has_bias=True, max_tokens=4)
    assert op.src_names == ["src_tensor", "weights", "weights_scale", "weights_zero_point", "biases"]
    assert op.dst_names == ["dst_tensor"]
    op = M.fc_create(M.PRECISION_F32, M.FLOAT32, M.FLOAT32, 64, 64, M.fc_int8_weights_desc(64, 64),
                     scalar_scale=0.5, has_bias=True)
    assert op.src_names == ["src_tensor", "weights", "biases"]
    op = M.fc_create(M.PRECISION_F32, M.INT8, M.INT32, 64, 64, M.fc_int8_weights_desc(64, 64))
    assert op.src_names == ["src_tensor", "weights"]


def test_quantization_and_conv_object_order():
    # quantize_and_dequantize.cc:754-756; gpu_model_builder.cc:1414-1424
    q = M.quantization_create(M.FLOAT16, M.PACKED_INT8C16, 2048, max_tokens=8)
    assert q.src_names == ["src_tensor"] and q.dst_names == ["dst_tensor", "dst_params"]
    wd = M.conv_int8_weights_desc(128, 64)
    c = M.conv_int8_create(M.FLOAT16, 128, 64, wd, has_zero_point=True, has_bias=True)
    assert c.src_names == ["src_tensor", "weights", "params_tensor", "weights_sum", "weights_scale",
                           "weights_zero_point", "biases"]
    c = M.conv_int8_create(M.INT32, 128, 64, wd)
    assert c.src_names == ["src_tensor", "weights"]
    assert M.lib().mldhip_conv_int8_src_type() == M.PACKED_INT8C16


def expect_error(code, fn, *a, **k):
    with pytest.raises(M.MldhipError) as e:
        fn(*a, **k)
    assert e.value.code == code, e.value
    return e.value.message


def test_fc_create_rejects_what_the_reference_rejects():
    wd = M.fc_int4_weights_desc(64, 64)
    bad_group = M.make_desc(M.UINT4, M.LAYOUT_I4O4, 3)
    msg = expect_error(M.INVALID_ARGUMENT, M.fc_create, M.PRECISION_F16, M.FLOAT16, M.FLOAT16, 64, 64, bad_group)
    assert "output_group_size" in msg  # fully_connected.cc:1107-1110
    bad_layout = M.make_desc(M.UINT4, M.LAYOUT_O4I4, 16)
    # the reference reads kOSpatialIOGroupO4I4 as a linear layout; this library serves it for ringed weights only
    msg = expect_error(M.UNIMPLEMENTED, M.fc_create, M.PRECISION_F16, M.FLOAT16, M.FLOAT16, 64, 64, bad_layout)
    assert "kOSpatialIOGroupO4I4" in msg
    bad_type = M.make_desc(M.INT32, M.LAYOUT_I4O4, 16)
    expect_error(M.INVALID_ARGUMENT, M.fc_create, M.PRECISION_F16, M.FLOAT16, M.FLOAT16, 64, 64, bad_type)
    # precision / tensor type mismatch (fully_connected.cc:1098-1102 for the weights; same rule for tensors)
    expect_error(M.INVALID_ARGUMENT, M.fc_create, M.PRECISION_F32, M.FLOAT16, M.FLOAT16, 64, 64, wd)
    # texture layouts and float weights are declared out of scope
    tex = M.make_desc(M.UINT4, M.LAYOUT_2D_I4O4, 16)
    expect_error(M.UNIMPLEMENTED, M.fc_create, M.PRECISION_F16, M.FLOAT16, M.FLOAT16, 64, 64, tex)
    flt = M.make_desc(M.FLOAT16, M.LAYOUT_I4O4, 16)
    expect_error(M.UNIMPLEMENTED, M.fc_create, M.PRECISION_F16, M.FLOAT16, M.FLOAT16, 64, 64, flt)
    # scale groups must split K into whole slices
    expect_error(M.INVALID_ARGUMENT, M.fc_create, M.PRECISION_F16, M.FLOAT16, M.FLOAT16, 64, 64, wd,
                 scale_shape=(64, 3))
    expect_error(M.INVALID_ARGUMENT, M.fc_create, M.PRECISION_F16, M.INT8, M.FLOAT16, 64, 64, wd)


def test_op_binding_errors():
    wd = M.fc_int4_weights_desc(64, 64)
    op = M.fc_create(M.PRECISION_F32_F16, M.FLOAT16, M.FLOAT16, 64, 64, wd, scale_shape=(64, 1),
                     max_tokens=2)
    expect_error(M.OUT_OF_RANGE, op.set_shape, 1, 1, 3)
    expect_error(M.INVALID_ARGUMENT, op.set_shape, 0, 1, 1)
    expect_error(M.OUT_OF_RANGE, op.set_src_raw, 7, 4096, 16)
    expect_error(M.INVALID_ARGUMENT, op.set_src_raw, 0, 0, 16)
    msg = expect_error(M.FAILED_PRECONDITION, op.launch)  # nothing bound: refused before any GPU call
    assert "src_tensor" in msg
    # too-small buffers are refused at launch, before any GPU call
    op.set_src_raw(0, 4096, 16)
    op.set_src_raw(1, 4096, 10)
    op.set_src_raw(2, 4096, 10)
    op.set_dst_raw(0, 4096, 10)
    msg = expect_error(M.INVALID_ARGUMENT, op.launch)
    assert "smaller" in msg


def test_conv_int8_requires_its_layout():
    fc_layout = M.fc_int8_weights_desc(128, 64)
    msg = expect_error(M.INVALID_ARGUMENT, M.conv_int8_create, M.FLOAT16, 128, 64, fc_layout)
    assert "convert" in msg
    wd = M.conv_int8_weights_desc(128, 64)
    expect_error(M.UNIMPLEMENTED, M.conv_int8_create, M.FLOAT16, 128, 64, wd,
                 src_packed_type=M.PACKED_INT8C4)


def test_unsupported_pack_layout_is_unimplemented():
    import numpy as np
    d = M.make_desc(M.UINT4, M.LAYOUT_O4I4, 1)
    with pytest.raises(M.MldhipError) as e:  # weights_conversion.cc:1617
        M.rearrange_uint4_packed(np.zeros(8, np.uint8), (4, 1, 1, 4), d)
    assert e.value.code == M.UNIMPLEMENTED and "Unsupported layout" in e.value.message


def test_header_is_plain_c(tmp_path):
    """The boundary is a C ABI: the header must compile as C99 on its own (what a cgo / JNI / ctypes
    binding includes), with no C++ in it."""
    import shutil
    import subprocess
    gcc = shutil.which("gcc")
    if gcc is None:
        pytest.skip("no gcc")
    src = tmp_path / "use_header.c"
    src.write_text('#include "mldhip.h"\n'
                   "int main(void) { mldhip_checkpoint_fc c; (void)c; return MLDHIP_GATE_SILU == 2 ? 0 : 1; }\n")
    r = subprocess.run([gcc, "-std=c99", "-Wall", "-Wextra", "-pedantic", "-Werror", "-fsyntax-only",
                        "-I", os.path.join(ROOT, "include"), str(src)], capture_output=True, text=True)
    assert r.returncode == 0, r.stderr


def test_fc_batch_ids_object_order_and_validation():
    # fully_connected.cc:1203-1213: batch_ids is registered before the weights objects
    wd = M.fc_int8_weights_desc(32, 64)
    op = M.fc_create(M.PRECISION_F32_F16, M.FLOAT16, M.FLOAT16, 32, 64, wd, scale_shape=(32, 1), has_bias=True,
                     max_tokens=128, weights_batch=16)
    assert op.src_names == ["src_tensor", "batch_ids", "weights", "weights_scale", "biases"]
    assert op.dst_names == ["dst_tensor"]
    op.set_shape(1, 8, 2)
    # cost: 8 of the 16 matrices are read (gpu_model_builder_moe_util.cc:268-283), fp16 tensors
    nbytes, flops = op.cost()
    assert flops == 2 * 16 * 64 * 32
    assert nbytes == 16 * 64 * 2 + 8 * 4 + 8 * (64 * 32 + 32 * 2) + 32 * 2 + 16 * 32 * 2
    with pytest.raises(M.MldhipError) as e:   # tensors of a batch-ids op have batch 1
        op.set_shape(2, 4, 1)
    assert e.value.code == M.UNIMPLEMENTED
    with pytest.raises(M.MldhipError) as e:
        M.fc_create(M.PRECISION_F32_F16, M.FLOAT16, M.FLOAT16, 32, 64, wd, scale_shape=(32, 1), weights_batch=0)
    assert e.value.code == M.INVALID_ARGUMENT
    op8 = M.fc_create(M.PRECISION_F32, M.INT8, M.INT32, 32, 64, wd, max_tokens=8, weights_batch=4)
    assert op8.src_names == ["src_tensor", "batch_ids", "weights"]


def test_scale_to_tensor_batched_matches_oracle(oracle):
    import numpy as np
    rng = np.random.default_rng(1)
    s = rng.normal(size=(10, 3, 2)).astype(np.float32)
    got = M.scale_to_tensor_batched(s, M.FLOAT32)
    assert np.array_equal(got, oracle.scale_to_hoio4_batched(s).reshape(-1))
    got16 = M.scale_to_tensor_batched(s, M.FLOAT16)
    assert np.array_equal(got16, oracle.f32_to_f16_bits(oracle.scale_to_hoio4_batched(s).reshape(-1)))
    # one matrix: the unbatched conversion
    assert np.array_equal(M.scale_to_tensor_batched(s[:, :1, :], M.FLOAT32), M.scale_to_tensor(s[:, 0, :], M.FLOAT32))


def test_runtime_check_objects_and_ringed_weights():
    """Runtime channel bounds and ring offsets add a last src object "params".  Ringed weights are refused
    where the reference refuses them, with its messages (common/kernels/fully_connected.cc:1087-1097:
    types under 8 bits; layouts that are not linear, i.e. the 2D texture layouts,
    common/task/weights_layout.cc:167-171); uint8 weights in the two buffer layouts are served."""
    d4 = M.fc_int4_weights_desc(64, 64)
    op = M.fc_create(M.PRECISION_F32_F16, M.FLOAT16, M.FLOAT16, 64, 64, d4, scale_shape=(64, 1), has_bias=True,
                     src_end_ch_index=1, dst_end_ch_index=3)
    assert op.src_names == ["src_tensor", "weights", "weights_scale", "biases", "params"]
    msg = expect_error(M.INVALID_ARGUMENT, M.fc_create, M.PRECISION_F32_F16, M.FLOAT16, M.FLOAT16, 64, 64, d4,
                       scale_shape=(64, 1), ring_o_offset_index=0, ring_size=64)
    assert "type for ringed weights" in msg
    d2d = M.make_desc(M.UINT8, M.LAYOUT_2D_I4O4, 16)
    msg = expect_error(M.INVALID_ARGUMENT, M.fc_create, M.PRECISION_F32_F16, M.FLOAT16, M.FLOAT16, 64, 64, d2d,
                       scale_shape=(64, 1), ring_i_offset_index=0, ring_size=64)
    assert "layout for ringed weights" in msg
    # uint8, kOSpatialIOGroupI4O4: a ring over the input channels (20 src channels against 56 ring rows)
    d8 = M.fc_int8_weights_desc(72, 56)
    op = M.fc_create(M.PRECISION_F32_F16, M.FLOAT16, M.FLOAT16, 72, 56, d8, scale_shape=(72, 1), has_bias=True,
                     ring_i_offset_index=0, src_end_ch_index=1, ring_size=56, src_channels=20)
    assert op.src_names == ["src_tensor", "weights", "weights_scale", "biases", "params"]
    # uint8, kOSpatialIOGroupO4I4: a ring over the output channels (20 dst channels out of 56 ring rows)
    do = M.make_desc(M.UINT8, M.LAYOUT_O4I4, 14)
    op = M.fc_create(M.PRECISION_F32, M.FLOAT32, M.FLOAT32, 56, 72, do, scale_shape=(20, 1),
                     ring_o_offset_index=0, ring_size=56, dst_channels=20)
    assert op.src_names == ["src_tensor", "weights", "weights_scale", "params"]
    # what this library adds to the reference's refusals carries messages of its own
    expect_error(M.UNIMPLEMENTED, M.fc_create, M.PRECISION_F32, M.FLOAT32, M.FLOAT32, 56, 72, do, scale_shape=(56, 1))
    expect_error(M.UNIMPLEMENTED, M.fc_create, M.PRECISION_F32, M.FLOAT32, M.FLOAT32, 56, 72, d8, scale_shape=(56, 1),
                 ring_o_offset_index=0, ring_size=56)
    expect_error(M.UNIMPLEMENTED, M.fc_create, M.PRECISION_F32, M.INT8, M.INT32, 72, 56, d8, ring_i_offset_index=0, ring_size=56)
    expect_error(M.INVALID_ARGUMENT, M.fc_create, M.PRECISION_F32, M.FLOAT32, M.FLOAT32, 72, 56, d8, scale_shape=(72, 1),
                 ring_i_offset_index=0, ring_size=0)
    expect_error(M.INVALID_ARGUMENT, M.fc_create, M.PRECISION_F32, M.FLOAT32, M.FLOAT32, 72, 56, d8, scale_shape=(72, 1),
                 ring_i_offset_index=0, ring_size=64)
    expect_error(M.INVALID_ARGUMENT, M.fc_create, M.PRECISION_F32, M.FLOAT32, M.FLOAT32, 72, 56, d8, scale_shape=(72, 1),
                 src_channels=20)
