"""The measurement yardsticks of the C ABI (no counterpart in vecops): the matrix-instruction streams on both
instruction shapes and the read-only stream.  They compute nothing a caller uses; what is checked is what can be:
integer streams on known operands have a closed form, the read stream folds its input with xor, and bad arguments
are refused."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("shape", [0, 1])
def test_int8_matrix_stream_closed_form(device, shape):
    """All-ones int8 operands: every accumulator element of a 32x32x32 (16x16x64) instruction grows by 32 (64) per
    instruction; a lane folds its 16 tiles x 16 (4) elements into one word."""
    import torch
    from vecops_amd import capi
    workgroups, iters = 3, 5
    operands = torch.ones(4096, dtype=torch.int8, device=device)
    out = torch.zeros(workgroups * 256, dtype=torch.int32, device=device)
    ops = capi.mfma_stream(operands, workgroups, iters, out, shape=shape)
    torch.cuda.synchronize()
    k, elems, per_tile = ((32, 16, 2), (64, 4, 2))[shape]    # every tile is hit twice per trip (two fragment sets)
    assert ops == 2 * (32 * 32 * 32 if shape == 0 else 16 * 16 * 64) * 32 * iters * 4 * workgroups
    want = 16 * elems * per_tile * iters * k
    assert torch.equal(out, torch.full_like(out, want))


@pytest.mark.parametrize("shape", [0, 1])
def test_bf16_matrix_stream_runs_on_both_shapes(device, shape):
    import torch
    from vecops_amd import capi
    operands = torch.zeros(4096, dtype=torch.bfloat16, device=device)
    out = torch.full((256,), -1, dtype=torch.int32, device=device)
    ops = capi.mfma_stream(operands, 1, 2, out, shape=shape)
    torch.cuda.synchronize()
    assert ops == 2 * (32 * 32 * 16 if shape == 0 else 16 * 16 * 32) * 32 * 2 * 4
    assert torch.equal(out, torch.zeros_like(out))          # sums of zeros, folded as bit patterns


@pytest.mark.parametrize("nbytes,workgroups", [(16, 1), (4096 * 16 + 48, 2), (1 << 20, 7), ((1 << 20) + 16 * 37, 64)])
def test_read_stream_folds_every_piece_once(device, nbytes, workgroups):
    import torch
    from vecops_amd import capi
    rng = np.random.default_rng(5)
    host = rng.integers(0, 2 ** 32, size=nbytes // 4, dtype=np.uint32)
    src = torch.from_numpy(host.view(np.int32)).to(device)
    out = torch.zeros(workgroups * 256, dtype=torch.int32, device=device)
    assert capi.read_stream(src, workgroups, out) == nbytes
    torch.cuda.synchronize()
    got = np.bitwise_xor.reduce(out.cpu().numpy().view(np.uint32))
    assert got == np.bitwise_xor.reduce(host)


def test_yardsticks_refuse_bad_arguments(device):
    import torch
    from vecops_amd import capi
    src = torch.zeros(64, dtype=torch.int32, device=device)
    out = torch.zeros(256, dtype=torch.int32, device=device)
    lib = capi.lib()
    assert lib.vecops_hip_read_stream(src.data_ptr() + 4, 64, 1, out.data_ptr(), None) == 1    # misaligned
    assert lib.vecops_hip_read_stream(src.data_ptr(), 8, 1, out.data_ptr(), None) == 1         # less than one piece
    assert lib.vecops_hip_read_stream(src.data_ptr(), 64, 0, out.data_ptr(), None) == 1
    assert lib.vecops_hip_read_stream(None, 64, 1, out.data_ptr(), None) == 1
    assert lib.vecops_hip_mfma_stream_shape(capi.I8, 2, src.data_ptr(), 256, 1, 1, out.data_ptr(), None) == 1   # no such shape
    assert lib.vecops_hip_mfma_stream_shape(capi.F32, 1, src.data_ptr(), 256, 1, 1, out.data_ptr(), None) == 1   # fp32: no stream
