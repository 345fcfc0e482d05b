"""Synthetic workloads of the quantized fully-connected path and their device-side setup.

Generates seeded inputs in the shapes and value ranges of the benchmark configurations,
packs weights with the library's host packers and uploads everything as torch tensors in the
physical layouts the kernels read.  Nothing here computes a result.
"""
import numpy as np

import mldhip as M


def div_up(a, b):
    return (a + b - 1) // b


def to_slices(x):
    """[tokens][channels] -> slice-major [ceil(C/4)][tokens][4], zero padded."""
    x = np.asarray(x)
    t, c = x.shape
    s = div_up(c, 4)
    full = np.zeros((t, s * 4), x.dtype)
    full[:, :c] = x
    return np.ascontiguousarray(full.reshape(t, s, 4).transpose(1, 0, 2))


def from_slices(x, channels):
    x = np.asarray(x)
    s, t, _ = x.shape
    return np.ascontiguousarray(x.transpose(1, 0, 2).reshape(t, s * 4)[:, :channels])


def round_to(x, dtype):
    """Values as the tensor of `dtype` (np.float16 / np.float32) holds them, in float32."""
    return np.asarray(x, np.float32).astype(dtype).astype(np.float32)


def make_fc_case(seed, m, k, n, weight_bits, tensor_dtype, groups=1, with_bias=False,
                 with_zero_point=False, act_uniform=False):
    """Weights uniform over the full signed range of the bit width (int8: [-127,127]),
    scales |N(0,0.02)|/qmax, activations N(0,1) (or U(-1,1))."""
    rng = np.random.default_rng(seed)
    if weight_bits == 4:
        w = rng.integers(-8, 8, size=(n, k), dtype=np.int8)
        qmax = 7.0
    else:
        w = rng.integers(-127, 128, size=(n, k), dtype=np.int8)
        qmax = 127.0
    act = rng.uniform(-1, 1, size=(m, k)) if act_uniform else rng.standard_normal((m, k))
    act = round_to(act, tensor_dtype)
    scale = round_to(np.abs(rng.normal(0.0, 0.02, size=(n, groups))) / qmax, tensor_dtype)
    case = dict(m=m, k=k, n=n, weight_bits=weight_bits, tensor_dtype=tensor_dtype, groups=groups,
                act=act, w=w, scale=scale, bias=None, zero_point=None)
    if with_bias:
        case["bias"] = round_to(rng.uniform(-1, 1, size=n) * 0.1, tensor_dtype)
    if with_zero_point:
        case["zero_point"] = rng.integers(-3, 4, size=(n, groups)).astype(np.float32)
    return case


def pack_fc_weights(case, reference_layout=False, output_group=None, decode_layout=False):
    """Packs the case's weights for the FullyConnected op: in the layout the library asks for, or
    with `reference_layout` in the reference's own FullyConnected layout (one output group), or
    in output groups of `output_group` slices (1: the layout FullyConnectedOI reads)."""
    n, k = case["n"], case["k"]
    if case["weight_bits"] == 4:
        desc = M.fc_int4_weights_desc(n, k, reference=reference_layout or output_group is not None, decode=decode_layout)
        if output_group is not None:
            desc.output_group_size = output_group
        return desc, M.rearrange_int8_as_uint4(case["w"], desc)
    desc = M.fc_int8_weights_desc(n, k, decode=decode_layout)
    if output_group is not None:
        desc.output_group_size = output_group
    return desc, M.rearrange_int8_as_uint8(case["w"], desc)


def mld_type(np_dtype):
    return M.FLOAT16 if np_dtype == np.float16 else M.FLOAT32


class FcDevice:
    """An FC op with its device buffers (torch tensors) for one synthetic case."""

    def __init__(self, case, device="cuda", max_tokens=None, scalar_scale=None, reference_layout=False,
                 output_group=None, precision=None, decode_layout=False):
        import torch
        self.torch = torch
        self.case = case
        m, k, n = case["m"], case["k"], case["n"]
        td = case["tensor_dtype"]
        tt = torch.float16 if td == np.float16 else torch.float32
        self.desc, packed = pack_fc_weights(case, reference_layout, output_group, decode_layout)
        self.packed_host = packed
        self.weights = torch.from_numpy(packed).to(device)
        self.act = torch.from_numpy(to_slices(case["act"]).astype(td)).to(device)
        groups = case["groups"]
        mt = mld_type(td)
        srcs = [self.act, self.weights]
        scale_shape = (1, 1)
        if scalar_scale is None:
            scale_shape = (n, groups)
            sc = M.scale_to_tensor(case["scale"], mt)
            self.scale = torch.from_numpy(sc.view(td) if td == np.float16 else sc).to(device)
            srcs.append(self.scale)
            if case["zero_point"] is not None:
                zp = M.scale_to_tensor(case["zero_point"], mt)
                self.zero_point = torch.from_numpy(zp.view(td) if td == np.float16 else zp).to(device)
                srcs.append(self.zero_point)
        if case["bias"] is not None:
            b = np.zeros(div_up(n, 4) * 4, td)
            b[:n] = case["bias"]
            self.bias = torch.from_numpy(b).to(device)
            srcs.append(self.bias)
        self.out = torch.zeros((div_up(n, 4), m, 4), dtype=tt, device=device)
        if precision is None:
            precision = M.PRECISION_F32 if td == np.float32 else M.PRECISION_F32_F16
        self.op = M.fc_create(precision, mt, mt, n, k, self.desc, scale_shape=scale_shape,
                              scalar_scale=1.0 if scalar_scale is None else scalar_scale,
                              has_zero_point_tensor=scalar_scale is None and case["zero_point"] is not None,
                              has_bias=case["bias"] is not None,
                              max_tokens=max_tokens or m)
        self.op.bind(srcs, [self.out])
        self.op.set_shape(1, 1, m)

    def run(self, stream=None):
        s = self.torch.cuda.current_stream().cuda_stream if stream is None else stream
        self.op.launch(s)

    def result(self):
        self.torch.cuda.synchronize()
        return from_slices(self.out.cpu().numpy().astype(np.float32), self.case["n"])


# The benchmark configurations 1-4 as make_fc_case arguments.
CONFIGS = {
    "c1": dict(seed=0, m=1, k=2048, n=2048, weight_bits=8, tensor_dtype=np.float32, groups=1),
    "c2": dict(seed=0, m=1, k=4096, n=14336, weight_bits=4, tensor_dtype=np.float16, groups=1),
    "c3": dict(seed=0, m=512, k=4096, n=4096, weight_bits=4, tensor_dtype=np.float16, groups=128),
    "c4": dict(seed=0, m=2048, k=2048, n=8192, weight_bits=8, tensor_dtype=np.float16, groups=1),
}

# Config 5: one decoder layer's FullyConnected sequence (name, k, n), hidden 2048, MQA k/v 256,
# gated MLP 16384; 18 layers; all int4 group-32.
C5_LAYER = [("q", 2048, 2048), ("k", 2048, 256), ("v", 2048, 256), ("o", 2048, 2048),
            ("gate", 2048, 16384), ("up", 2048, 16384), ("down", 16384, 2048)]
C5_LAYERS = 18
