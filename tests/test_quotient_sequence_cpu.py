"""The fp8 quantizer forms RN32(f / step) without a division per element:

    q0 = f * inv, e0 = fma(-q0, step, f), q1 = fma(e0, inv, q0), e1 = fma(-q1, step, f), q = fma(e1, inv, q1)

with inv = RN32(1 / step) (astrai_amd/csrc/quantize.hip, quant8_fp8). Its claim -- q is the
correctly rounded quotient for every bf16 input wherever the kernel takes this path (finite
quotient, step in [2^-60, 2^60] whose significand is not all ones, |f| >= 2^-102; smaller |f|
give a zero code either way) -- is checked here by emulating the five operations in extended
precision against numpy's float32 division, on every finite bf16 value under random steps,
steps next to powers of two and steps of the amax / 448 kind."""

import numpy as np

L = np.longdouble


def _f32(x):
    return x.astype(np.float32)


def _fma(a, b, c):
    # a * b is exact in 64-bit significands (24 x 24 bits); the sum is rounded twice only when
    # it falls within 2^-40 ulp of a float32 midpoint, which no case below does
    return _f32(a.astype(L) * b.astype(L) + c.astype(L))


def _sequence(f, step):
    inv = np.float32(1) / step
    s, i = np.full_like(f, step), np.full_like(f, inv)
    q0 = _f32(f * i)
    q1 = _fma(_fma(-q0, s, f), i, q0)
    q = _fma(_fma(-q1, s, f), i, q1)
    # the kernel gives the quotient the sign bit of f (it matters for a zero quotient only)
    return (q.view(np.uint32) | (f.view(np.uint32) & np.uint32(0x80000000))).view(np.float32)


def test_five_operation_quotient_is_the_ieee_quotient():
    assert np.finfo(L).nmant >= 63, "needs the x87 extended type"
    rng = np.random.default_rng(1)
    allf = (np.arange(65536, dtype=np.uint32) << 16).view(np.float32)
    allf = allf[np.isfinite(allf)]
    steps = list(np.exp2(rng.uniform(-40, 40, 40)).astype(np.float32))
    steps += [np.float32(v) for v in (1.0, 0.5, 3.0, 448.0, 1 / 448.0, 2.0 ** -60, 2.0 ** 60)]
    steps += list(np.array([0x3f800001, 0x3f7ffffe, 0x40000001, 0x3efffffe, 0x3fc00000, 0x3ffffffe],
                           dtype=np.uint32).view(np.float32))
    amaxs = allf[(allf > 1e-3) & (allf < 1e3)]
    steps += list(_f32(rng.choice(amaxs, 40) / np.float32(448)))
    checked = 0
    for step in steps:
        step = np.float32(step)
        with np.errstate(all="ignore"):
            want = _f32(allf / step)
            got = _sequence(allf, step)
        sel = np.isfinite(got) & ((np.abs(allf) >= 2.0 ** -102) | (allf == 0))
        bad = got[sel].view(np.uint32) != want[sel].view(np.uint32)   # bit for bit, the sign of zero included
        assert not bad.any(), (step, allf[sel][bad][:4], got[sel][bad][:4], want[sel][bad][:4])
        # where the kernel keeps this path although |f| is tiny, both quotients give a zero code
        tiny = np.isfinite(got) & (np.abs(allf) < 2.0 ** -102)
        assert (np.abs(got[tiny]) < 2.0 ** -18).all() and (np.abs(want[tiny]) < 2.0 ** -18).all()
        checked += int(sel.sum())
    assert checked > 5_000_000
