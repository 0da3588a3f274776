"""One-wave known-answer tests of the MFMA lane layouts the kernels are built on: one
instruction per launch, expectation computed on the host and placed by the layout the
kernels assume (after the reference's single-instruction test,
csrc/tests/fp8_mma_test.cu:81-145: asymmetric operands, exact products)."""

import pytest
import torch

pytestmark = pytest.mark.gpu
DEV = "cuda"

# kind -> (rows, K elements, element kind)
KINDS = {0: (16, 64, "i8"), 1: (16, 128, "e4m3"), 2: (16, 128, "e5m2"), 3: (32, 32, "i8"),
         4: (32, 64, "e4m3"), 5: (32, 64, "e5m2"), 6: (16, 32, "bf16"), 7: (32, 16, "bf16")}
# values both fp8 formats and bf16 hold exactly; products and sums stay exact in fp32
EXACT = torch.tensor([0.0, 0.5, -0.5, 1.0, -1.0, 1.5, -1.5, 2.0, -2.0, 3.0, -3.0, 4.0, 6.0, -8.0])


@pytest.fixture(scope="module")
def C():
    from astrai_amd.extension import _cabi
    assert _cabi.load() is not None, _cabi.load_error()
    return _cabi


def _operands(kind, seed):
    rows, k, elt = KINDS[kind]
    g = torch.Generator().manual_seed(seed)
    if elt == "i8":
        a = torch.randint(-127, 128, (rows, k), generator=g, dtype=torch.int8)
        b = torch.randint(-127, 128, (rows, k), generator=g, dtype=torch.int8)
        return a, b, a.long() @ b.long().t()
    a = EXACT[torch.randint(0, len(EXACT), (rows, k), generator=g)]
    b = EXACT[torch.randint(0, len(EXACT), (rows, k), generator=g)]
    dt = {"e4m3": torch.float8_e4m3fn, "e5m2": torch.float8_e5m2, "bf16": torch.bfloat16}[elt]
    aq, bq = a.to(dt), b.to(dt)
    assert torch.equal(aq.float(), a) and torch.equal(bq.float(), b)
    return aq, bq, a.double() @ b.double().t()


def _place(d, rows):
    """D [rows, rows] -> what lane l, register r should hold"""
    lane = torch.arange(64)
    if rows == 16:
        reg = torch.arange(4)
        i = 4 * (lane[:, None] // 16) + reg[None, :]
        j = (lane % 16)[:, None].expand(64, 4)
    else:
        reg = torch.arange(16)
        i = 8 * (reg[None, :] // 4) + 4 * (lane[:, None] // 32) + reg[None, :] % 4
        j = (lane % 32)[:, None].expand(64, 16)
    return d[i, j]


@pytest.mark.parametrize("kind", sorted(KINDS))
def test_mfma_lane_layout(C, kind):
    rows, _, elt = KINDS[kind]
    for seed in (1, 2):
        print(f"case kind={kind} seed={seed}", flush=True)
        a, b, d = _operands(kind, 100 * kind + seed)
        raw = C.mfma_probe(kind, a.to(DEV), b.to(DEV)).cpu()
        want = _place(d, rows)
        got = raw.long() if elt == "i8" else raw.view(torch.float32).double()
        assert torch.equal(got, want.to(got.dtype)), (kind, (got != want).nonzero()[:4])
        # the operands are asymmetric: the transposed product is a different matrix
        assert not torch.equal(want, _place(d.t(), rows))


def test_mfma_probe_single_entries(C):
    """a = e_i (row i, K position p), b = e_j (row j, same K position): exactly D[i][j] = 1 --
    K bytes of the two operands meet each other at every position, whatever lane holds them."""
    for kind in sorted(KINDS):
        rows, k, elt = KINDS[kind]
        dt = {"i8": torch.int8, "e4m3": torch.float8_e4m3fn, "e5m2": torch.float8_e5m2, "bf16": torch.bfloat16}[elt]
        for (i, j, p) in [(0, rows - 1, 0), (rows - 1, 3, k - 1), (5, 5, k // 2 + 1), (rows // 2, 1, 17 % k)]:
            print(f"case kind={kind} i={i} j={j} p={p}", flush=True)
            a = torch.zeros(rows, k)
            b = torch.zeros(rows, k)
            a[i, p] = 1
            b[j, p] = 1
            raw = C.mfma_probe(kind, a.to(dt).to(DEV), b.to(dt).to(DEV)).cpu()
            got = raw.long() if elt == "i8" else raw.view(torch.float32).long()
            d = torch.zeros(rows, rows, dtype=torch.long)
            d[i, j] = 1
            assert torch.equal(got, _place(d, rows)), (kind, i, j, p)
