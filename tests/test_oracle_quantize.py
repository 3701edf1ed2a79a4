"""Pins the quantiser of the CPU oracle (C and numpy restatements of
kernel.cu:128-154) with hand-derived answers, an exhaustive sweep, invariants
and naive-loop addressing.  No GPU."""
import json
import os

import numpy as np
import pytest

HERE = os.path.dirname(os.path.abspath(__file__))


def _bits(x):
    return np.asarray(x, dtype=np.float16).view(np.uint16)


def test_known_answers(oracle):
    with open(os.path.join(HERE, "golden", "quantize_known_answers.json")) as f:
        cases = json.load(f)["cases"]
    assert len(cases) >= 5
    for c in cases:
        x = np.array(c["x"], dtype=np.float16)
        for fn in (oracle.quantize_groups_numpy, oracle.quantize_groups_c):
            q, s = fn(x)
            assert int(_bits(s)) == int(c["scale_bits"], 16), (fn.__name__, c)
            assert q.tolist() == c["q"], (fn.__name__, c)


def test_eps_is_the_half_subnormal(oracle):
    # half(1e-5f) = 168 * 2^-24
    assert int(oracle.lib().pmx_oracle_float_to_half(1e-5)) == 0x00A8
    assert float(np.float16(np.float32(1e-5))) == 168 * 2.0 ** -24


def test_half_conversions_exhaustive(oracle):
    L = oracle.lib()
    allh = np.arange(65536, dtype=np.uint16)
    as_f32 = allh.view(np.float16).astype(np.float32)
    for i in range(65536):
        v = np.float32(L.pmx_oracle_half_to_float(int(allh[i])))
        if np.isnan(as_f32[i]):
            assert np.isnan(v)
        else:
            assert v == as_f32[i] and np.signbit(v) == np.signbit(as_f32[i])
    # float -> half: every half value, its neighbours' midpoints and just off them
    fin = as_f32[np.isfinite(as_f32)]
    fin = np.unique(fin)
    mids = ((fin[:-1].astype(np.float64) + fin[1:].astype(np.float64)) / 2).astype(np.float32)
    probes = np.concatenate([fin, mids, np.nextafter(mids, np.float32(np.inf)), np.nextafter(mids, np.float32(-np.inf)),
                             np.array([65519.996, 65520.0, 1e9, -1e9, 2.0 ** -25, 2.0 ** -26], dtype=np.float32)])
    with np.errstate(over="ignore"):
        want = probes.astype(np.float16).view(np.uint16)
    for x, w in zip(probes, want):
        assert L.pmx_oracle_float_to_half(float(x)) == w, (x, hex(w))


def test_c_equals_numpy_on_every_absmax(oracle):
    """All 31743 positive finite halves as the group's absmax, with the other seven
    channels covering ratios that hit ties and near-ties."""
    pos = np.arange(1, 0x7C00, dtype=np.uint16).view(np.float16)
    fr = np.array([1.0, -1.0, 0.5, -0.25, 0.00390625, 0.9921875, -0.503937, 0.0118], dtype=np.float32)
    x = (pos.astype(np.float32)[:, None] * fr[None, :]).astype(np.float16)
    qn, sn = oracle.quantize_groups_numpy(x)
    # C path, vectorised through the batch entry point: one "token" per group
    n = x.shape[0]
    cache = np.zeros((1, 2, n, 1, 8), dtype=np.int8)
    scale = np.zeros((1, 2, n, 1, 1), dtype=np.float16)
    oracle.kv_cache_quantize(x.reshape(n, 1, 8), x.reshape(n, 1, 8)[::-1].copy(), np.array([0, n]), np.array([0]),
                             np.array([0]), 0, 1, 8, 0, cache_stride_s=8, cache_stride_l=2 * n * 8, cache_stride_h=8,
                             cache_stride_kv=n * 8, cachestarts_stride_b=1, cache=cache, scale=scale)
    assert np.array_equal(cache[0, 0, :, 0], qn)
    assert np.array_equal(_bits(scale[0, 0, :, 0, 0]), _bits(sn))
    assert np.array_equal(cache[0, 1, :, 0], qn[::-1])
    # facts that hold for every absmax
    assert np.abs(qn.astype(np.int32)).max() <= 127
    normal_scale = _bits(sn) >= 0x0400
    assert (np.abs(qn[normal_scale, 0]) == 127).all()  # absmax maps to +-127 when the scale is a normal half
    assert (qn[:, 0] == -qn[:, 1]).all()               # sign symmetry


def test_reciprocal_quotient_identity_over_every_pair(oracle):
    """The HIP quantiser divides once per group (rcp = 1/scale) and corrects each channel's x * rcp with a
    residual step; over every finite half x and every half scale >= eps the int8 result is that of the
    reference's half division (kernel.cu:144-148).  The half quotients differ in bits only for x = -0
    (one pair per scale), which quantises to 0 either way."""
    bad, half_differs = oracle.count_reciprocal_quotient_mismatches()
    assert bad == 0
    assert half_differs == 0x7C00 - 0x00A8


def test_scale_without_division_equals_the_division_for_every_absmax(oracle):
    """The HIP quantiser forms absmax / 127 as s0 = a * r, s = fma(fma(-s0, 127, a), r, s0) with r = fl(1 / 127)
    (binary32, every fma rounded once) and rounds s to half.  For every positive finite half a that half equals
    half(a / 127) with the binary32 division of the reference (kernel.cu:137-139).  The fmas are evaluated in
    exact rational arithmetic and rounded to binary32 here, so the check does not lean on the host's fma."""
    from fractions import Fraction

    def to_f32(fr):  # an exact rational rounded once to binary32, ties to even
        if fr == 0:
            return np.float32(0.0)
        sign, mag = (-1, -fr) if fr < 0 else (1, fr)
        e = mag.numerator.bit_length() - mag.denominator.bit_length() - 24
        while mag >= Fraction(2) ** (e + 24):
            e += 1
        while mag < Fraction(2) ** (e + 23):
            e -= 1
        e = max(e, -149)
        scaled = mag / Fraction(2) ** e
        n = scaled.numerator // scaled.denominator
        rem = scaled - n
        if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and n % 2 == 1):
            n += 1
        return np.float32(sign * float(Fraction(n) * Fraction(2) ** e))  # n < 2^24 + 1: exact in binary64

    r = np.float32(1.0) / np.float32(127.0)
    rf = Fraction(float(r))
    pos = np.arange(1, 0x7C00, dtype=np.uint16).view(np.float16)
    want = (pos.astype(np.float32) / np.float32(127.0)).astype(np.float16)
    got = np.empty_like(want)
    for i, a in enumerate(pos):
        af = Fraction(float(a))
        s0 = Fraction(float(to_f32(af * rf)))
        e = Fraction(float(to_f32(af - s0 * 127)))
        got[i] = np.float16(to_f32(e * rf + s0))
    assert np.array_equal(_bits(got), _bits(want))


def test_random_groups_c_equals_numpy_and_error_bound(oracle):
    rng = np.random.default_rng(5)
    x = (rng.standard_normal((20000, 8)) * 10.0 ** rng.integers(-6, 3, (20000, 1))).astype(np.float16)
    qn, sn = oracle.quantize_groups_numpy(x)
    n = x.shape[0]
    cache = np.zeros((1, 2, n, 1, 8), dtype=np.int8)
    scale = np.zeros((1, 2, n, 1, 1), dtype=np.float16)
    oracle.kv_cache_quantize(x.reshape(n, 1, 8), x.reshape(n, 1, 8), np.array([0, n]), np.array([0]),
                             np.array([0]), 0, 1, 8, 0, cache_stride_s=8, cache_stride_l=2 * n * 8, cache_stride_h=8,
                             cache_stride_kv=n * 8, cachestarts_stride_b=1, cache=cache, scale=scale)
    assert np.array_equal(cache[0, 0, :, 0], qn)
    assert np.array_equal(_bits(scale[0, 0, :, 0, 0]), _bits(sn))
    # |x - q*s| <= s/2 + one half ulp of the quotient's rounding (in units of s)
    s = sn.astype(np.float64)[:, None]
    err = np.abs(x.astype(np.float64) - qn.astype(np.float64) * s)
    assert (err <= s * (0.5 + 127 * 2.0 ** -11) + 1e-12).all()
    # permutation equivariance inside a group
    perm = rng.permutation(8)
    qp, sp = oracle.quantize_groups_numpy(x[:, perm])
    assert np.array_equal(qp, qn[:, perm]) and np.array_equal(_bits(sp), _bits(sn))


@pytest.mark.parametrize("cache_mode", [0, 1])
def test_addressing_against_naive_loops(oracle, pkg, cache_mode):
    """Token/head/group scatter (kernel.cu:97-126) against a triple loop, both cache modes,
    two layers, canary bytes everywhere else."""
    wl = pkg.workloads
    bt, rng = wl.custom_batch(11, num_heads=4, num_kv_heads=2, head_dim=16, cache_mode=cache_mode,
                              dec_kv_lens=[5, 130], prefill_q_lens=[7, 3], prefill_prior=[126, 0],
                              num_layer=2, layer_idx=1)
    lay = bt.layout
    cache = np.full(lay.cache_shape(), 0x5A, dtype=np.int8)
    scale = np.full(lay.scale_shape(), 1.5, dtype=np.float16)
    q, k, v = wl.step_inputs(bt, rng)
    oracle.kv_cache_quantize(k, v, bt.seqstarts, bt.cachestarts, bt.start_pos, bt.layer_idx, bt.num_kv_heads,
                             bt.head_dim, bt.page_size, cache_stride_s=lay.stride_s, cache_stride_l=lay.stride_l,
                             cache_stride_h=lay.stride_h, cache_stride_kv=lay.stride_kv,
                             cachestarts_stride_b=bt.cachestarts_stride_b, cache=cache, scale=scale)
    want_c = np.full(lay.cache_shape(), 0x5A, dtype=np.int8)
    want_s = np.full(lay.scale_shape(), 1.5, dtype=np.float16)
    for b in range(bt.batch):
        for i in range(int(bt.q_lens[b])):
            pos = int(bt.start_pos[b]) + i
            if cache_mode == 0:
                tok = int(bt.cachestarts[b]) + pos
            else:
                tok = int(bt.cachestarts[b, pos // 128]) + pos % 128
            row = int(bt.seqstarts[b]) + i
            for h in range(bt.num_kv_heads):
                for g in range(bt.head_dim // 8):
                    for plane, src in ((0, k), (1, v)):
                        qq, ss = oracle.quantize_groups_numpy(src[row, h, 8 * g:8 * g + 8])
                        want_c[1, plane, tok, h, 8 * g:8 * g + 8] = qq
                        want_s[1, plane, tok, h, g] = ss
    assert np.array_equal(cache, want_c)
    assert np.array_equal(_bits(scale), _bits(want_s))
    assert (cache[0] == 0x5A).all()  # the other layer is untouched
