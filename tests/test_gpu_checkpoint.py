"""Checkpoint files -> C-ABI loader -> FullyConnected on the GPU, against the dequantized float
weights the files stand for.  fp16 tensors: max|err| <= 2e-2 * RMS(reference output)."""
import os

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

import mldhip as M
import workloads as W
from oracle import checkpoint as CK

FP16_TOL = 2e-2


@pytest.mark.parametrize("o,i,bits,block,zp,tokens", [
    (2048, 1024, 4, 32, False, 1),
    (2048, 1024, 4, 32, True, 3),
    (1000, 512, 4, 0, False, 1),
    (512, 2048, 4, 32, False, 64),
    (768, 1024, 8, 0, False, 1),
    (768, 1024, 8, 0, True, 2),
])
def test_fc_from_checkpoint_files(oracle, tmp_path, o, i, bits, block, zp, tokens):
    import torch
    rng = np.random.default_rng(o + i + bits)
    w = (rng.standard_normal((o, i)) * 0.05).astype(np.float32)
    q, s = (CK.quantize_int4_sym(w, block) if bits == 4 else CK.quantize_int8_sym(w))
    s = s.reshape(o, -1)
    z_int = rng.integers(-2, 3, size=s.shape).astype(np.float32) if zp else None
    d = str(tmp_path) + os.sep
    CK.write_fc_files(d, "blk.mlp.up", q, s, bits, zero_point=None if z_int is None else z_int * s)
    info = M.checkpoint_fc_probe(d, "blk.mlp.up.weight", "blk.mlp.up", o, i, bits)
    assert info.group_size == (block if block else i)
    host = M.checkpoint_fc_read(d, "blk.mlp.up.weight", "blk.mlp.up", info, M.FLOAT16)

    x = rng.standard_normal((tokens, i)).astype(np.float16)
    act = torch.from_numpy(W.to_slices(x)).cuda()
    wt = torch.from_numpy(host["weights"]).cuda()
    sc = torch.from_numpy(host["scale"].view(np.float16)).cuda()
    srcs = [act, wt, sc]
    if zp:
        srcs.append(torch.from_numpy(host["zero_point"].view(np.float16)).cuda())
    out = torch.zeros(((o + 3) // 4, tokens, 4), dtype=torch.float16, device="cuda")
    op = M.fc_create(M.PRECISION_F32_F16, M.FLOAT16, M.FLOAT16, o, i, info.weights,
                     scale_shape=(o, info.scale_i), has_zero_point_tensor=zp, max_tokens=tokens)
    op.bind(srcs, [out])
    op.set_shape(1, 1, tokens)
    print("checkpoint fc", o, i, bits, block, zp, tokens, flush=True)
    op.launch(torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    got = W.from_slices(out.cpu().numpy().astype(np.float32), o)

    # the float weights the files stand for: (q - zp) * s per group, with the fp16 scale the op reads
    s16 = s.astype(np.float16).astype(np.float64)
    rep = i // s.shape[1]
    deq = (q.astype(np.float64) - (0.0 if z_int is None else np.repeat(z_int, rep, axis=1))) * np.repeat(s16, rep, axis=1)
    ref = x.astype(np.float64) @ deq.T
    rms = np.sqrt(np.mean(ref ** 2))
    assert np.abs(got - ref).max() <= FP16_TOL * rms
    assert op.kernel_name in ("fc_w4_stream_kernel", "fc_w4_strip_kernel", "fc_w4_mfma_gemm_kernel", "fc_w8_stream_kernel"), op.kernel_name
