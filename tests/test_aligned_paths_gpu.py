"""Seeded sweep over shapes whose operands are 16-byte aligned - the ones that take the kernels whose loads
write LDS themselves - for bf16, f16 and int8, B K-contiguous and B as [K,N], with K tails, edge tiles, batches
and offsets into larger buffers, against the oracle (int8 bit for bit, floating sums within the summation-order
bound used everywhere else).  The same shapes shifted off alignment take the register-staged kernels and must
give the same values."""
import numpy as np
import pytest

from conftest import rel_err
from oracle import oracle as O
from vecops_amd import synth

pytestmark = pytest.mark.gpu


def _cases():
    rng = np.random.default_rng(20240611)
    cases = []
    for i in range(36):
        kind = ("bf16", "i8", "f16")[i % 3]
        m = int(rng.choice([64, 128, 200, 256, 333, 512, 777, 1024]))
        n = int(rng.choice([128, 136, 256, 264, 512, 520, 1000, 1024]))       # multiples of 8: [K,N] layout allowed
        unit = 16 if kind == "i8" else 8
        k = int(rng.choice([4, 8, 9, 16, 33, 64, 65])) * unit                  # whole and partial K tiles
        layout = "kn" if (kind != "i8" and i % 2 == 0) else "nk"
        batch = int(rng.choice([0, 0, 2, 3]))
        cases.append((kind, m, n, k, layout, batch))
    return cases


CASES = _cases()


def _make(kind, seed, shape):
    if kind == "i8":
        return synth.int8_sym(seed, shape)
    x = synth.uniform_pm1(seed, shape)
    return synth.bf16_round(x) if kind == "bf16" else x.astype(np.float16)


def _dev(kind, x, device, offset_elems=0):
    """Device copy of x; with offset_elems the data starts that many elements into its buffer."""
    import torch
    host = np.ascontiguousarray(x)
    raw = host.view(np.int16) if kind != "i8" else host
    flat = torch.empty(raw.size + offset_elems, dtype=torch.int16 if kind != "i8" else torch.int8, device=device)
    view = flat[offset_elems:].view(raw.shape)
    view.copy_(torch.from_numpy(raw))
    if kind == "bf16":
        return view.view(torch.bfloat16)
    if kind == "f16":
        return view.view(torch.float16)
    return view


@pytest.mark.parametrize("kind,m,n,k,layout,batch", CASES, ids=[f"{c[0]}-{c[1]}x{c[2]}x{c[3]}-{c[4]}-b{c[5]}" for c in CASES])
def test_aligned_and_shifted_operands_agree_with_the_oracle(device, oracle, kind, m, n, k, layout, batch):
    import torch
    from vecops_amd import capi
    lead = (batch,) if batch else ()
    a, b = _make(kind, 1, lead + (m, k)), _make(kind, 2, lead + (n, k))
    integer = kind == "i8"
    want = np.zeros(lead + (m, n), np.int32 if integer else np.float32)
    atom = O.ATOM_I8I32 if integer else (O.ATOM_BF16F32 if kind == "bf16" else O.ATOM_F16F32)
    a_o = a if kind != "bf16" else a            # bf16 bits are uint16 arrays, which the oracle reads as bf16
    oracle.matmul(a_o, b, want, atom=atom, acc_f64=True, c_bf16=False)
    results = []
    for shift in (0, 1):                         # 0: aligned bases; 1: one element in (bases off by 1 or 2 bytes)
        ta, tb = _dev(kind, a, device, shift), _dev(kind, b, device, shift)
        if layout == "kn":
            tb = tb.transpose(-1, -2).contiguous().transpose(-1, -2)           # [.., N, K] view of [.., K, N] memory
            if shift:
                continue                         # the contiguous copy is aligned again: nothing new to see
        c = torch.full(lead + (m, n), -7 if integer else float("nan"), dtype=torch.int32 if integer else torch.float32,
                       device=device)
        capi.matmul(ta, tb, c)
        torch.cuda.synchronize()
        results.append(c.cpu().numpy())
    for got in results:
        if integer:
            assert np.array_equal(got, want)
        else:
            assert rel_err(got, want) <= 2e-6 * max(1.0, k / 32)
    if integer and len(results) == 2:
        assert np.array_equal(results[0], results[1])
