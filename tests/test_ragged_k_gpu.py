"""Seeded sweep over K extents that leave a partial last K tile - the tile the kernels stage through their
bounds-checked routine - for every operand class: K shorter than one 16-byte chunk, K one element past a chunk or a
tile, rows at every alignment, edge tiles in M and N, pitched rows, batches and K splits (few tiles, long ragged K).
Integer classes against exact int64 arithmetic (wrapped to int32), floating ones against float64 within the
summation-order bound used everywhere else."""
import numpy as np
import pytest

from conftest import rel_err
from vecops_amd import synth

pytestmark = pytest.mark.gpu

KINDS = ("bf16", "f16", "i8", "u8a", "u8b", "f32_as_bf16", "f32")


def _cases():
    rng = np.random.default_rng(20250117)
    cases = []
    for i in range(70):
        kind = KINDS[i % len(KINDS)]
        m = int(rng.choice([1, 5, 63, 64, 100, 129, 255, 300]))
        n = int(rng.choice([3, 40, 64, 77, 128, 200, 257]))
        k = int(rng.choice([1, 2, 3, 7, 9, 15, 17, 31, 33, 63, 65, 100, 127, 129, 191, 257, 520, 1001, 4099]))
        pitch = int(rng.choice([0, 0, 1, 3, 8]))          # extra elements between rows
        batch = int(rng.choice([0, 0, 0, 2]))
        cases.append((kind, m, n, k, pitch, batch))
    return cases


CASES = _cases()


def _host(kind, side, seed, shape):
    if kind in ("i8", "u8a", "u8b"):
        x = synth.int8_sym(seed, shape)
        unsigned = (kind == "u8a" and side == "a") or (kind == "u8b" and side == "b")
        return (x.astype(np.int16) + 128).astype(np.uint8) if unsigned else x
    x = synth.uniform_pm1(seed, shape)
    if kind == "bf16":
        return synth.bf16_round(x)          # bf16 bit patterns (uint16)
    if kind == "f16":
        return x.astype(np.float16)
    return x.astype(np.float32)


def _values(kind, x):
    """What the kernel multiplies, as float64 / int64."""
    if kind == "bf16":
        return synth.bf16_to_f32(x).astype(np.float64)
    if kind == "f32_as_bf16":
        return synth.bf16_to_f32(synth.bf16_round(x)).astype(np.float64)
    if kind in ("i8", "u8a", "u8b"):
        return x.astype(np.int64)
    return x.astype(np.float64)


def _dev(kind, x, pitch, device):
    """Device copy of x[..., rows, k] whose rows lie k + pitch elements apart."""
    import torch
    raw = x.view(np.int16) if x.dtype == np.uint16 else x
    t = torch.from_numpy(np.ascontiguousarray(raw))
    rows, k = raw.shape[-2], raw.shape[-1]
    store = torch.zeros(raw.shape[:-1] + (k + pitch,), dtype=t.dtype, device=device)
    store[..., :k].copy_(t)
    view = store[..., :k]
    assert view.stride(-2) == k + pitch and rows == view.shape[-2]
    return view.view(torch.bfloat16) if x.dtype == np.uint16 else view


@pytest.mark.parametrize("kind,m,n,k,pitch,batch", CASES, ids=[f"{c[0]}-{c[1]}x{c[2]}x{c[3]}-p{c[4]}-b{c[5]}" for c in CASES])
def test_partial_k_tiles_of_every_operand_class(device, kind, m, n, k, pitch, batch):
    import torch
    from vecops_amd import capi
    lead = (batch,) if batch else ()
    a, b = _host(kind, "a", 3, lead + (m, k)), _host(kind, "b", 4, lead + (n, k))
    ta, tb = _dev(kind, a, pitch, device), _dev(kind, b, pitch, device)
    integer = kind in ("i8", "u8a", "u8b")
    c = (torch.full(lead + (m, n), -7, dtype=torch.int32, device=device) if integer
         else torch.full(lead + (m, n), float("nan"), dtype=torch.float32, device=device))
    compute = capi.COMPUTE_F32 if kind == "f32" else capi.COMPUTE_BF16
    capi.matmul(ta, tb, c, compute=compute)
    torch.cuda.synchronize()
    want = np.einsum("...mk,...nk->...mn", _values(kind, a), _values(kind, b))
    got = c.cpu().numpy()
    if integer:
        assert np.array_equal(got, (want & 0xffffffff).astype(np.uint32).view(np.int32))
    else:
        assert rel_err(got, want) <= 2e-6 * max(1.0, k / 32)


@pytest.mark.parametrize("kind", ["bf16", "i8", "u8a", "f16", "f32"])
@pytest.mark.parametrize("k", [4099, 8191, 12289])
def test_partial_k_tile_under_a_k_split(device, kind, k):
    """Few output tiles and a long ragged K: the rule table splits K, and the last part owns the partial tile."""
    import torch
    from vecops_amd import capi
    m, n = 100, 40
    a, b = _host(kind, "a", 5, (m, k)), _host(kind, "b", 6, (n, k))
    ta, tb = _dev(kind, a, 0, device), _dev(kind, b, 0, device)
    integer = kind in ("i8", "u8a")
    c = torch.zeros((m, n), dtype=torch.int32 if integer else torch.float32, device=device)
    compute = capi.COMPUTE_F32 if kind == "f32" else capi.COMPUTE_BF16
    assert capi.plan_matmul(ta, tb, c, compute=compute).split_k > 1
    capi.matmul(ta, tb, c, compute=compute)
    torch.cuda.synchronize()
    want = _values(kind, a) @ _values(kind, b).T
    if integer:
        assert np.array_equal(c.cpu().numpy(), (want & 0xffffffff).astype(np.uint32).view(np.int32))
    else:
        assert rel_err(c.cpu().numpy(), want) <= 2e-6 * max(1.0, k / 32)
