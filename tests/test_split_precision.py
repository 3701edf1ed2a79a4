"""Why the MFMA kernels carry K^, V^ and p as hi + lo pairs of halves: a numpy emulation of their arithmetic
(fp16 operands, exact products, fp32-or-better accumulation) on data drawn like the benchmark workloads
(standard normal with 2 % of the channels scaled x10) against the fp64 attention over the exactly dequantised
cache, measured in units of the tolerance 2e-3 + 1e-2 |ref|.  CPU only; no library code is involved."""
import math

import numpy as np
import pytest


def _case(seed, prior, nq, heads=4, d=128):
    rng = np.random.default_rng(seed)
    length = prior + nq
    out_ch = rng.choice(d, size=math.ceil(0.02 * d), replace=False)

    def draw(n, h):
        x = rng.standard_normal((n, h, d), dtype=np.float32)
        x[:, :, out_ch] *= 10
        return x.astype(np.float16)

    q = draw(nq, heads).astype(np.float32)
    k, v = draw(length, 1)[:, 0], draw(length, 1)[:, 0]

    def quant(x):  # symmetric int8, groups of 8 channels, fp16 scale (kernel.cu:128-154)
        x32 = x.astype(np.float32).reshape(length, d // 8, 8)
        s = np.maximum((np.abs(x32).max(-1) / np.float32(127)).astype(np.float16), np.float16(1e-5))
        q8 = np.rint((x32 / s.astype(np.float32)[..., None]).astype(np.float16).astype(np.float32)).clip(-127, 127)
        return (q8 * s.astype(np.float32)[..., None]).reshape(length, d).astype(np.float32)  # exact in binary32

    kx, vx = quant(k), quant(v)
    mask = np.arange(length)[None, :] <= (prior + np.arange(nq))[:, None]
    return q, kx, vx, mask


def _f16(x):
    return x.astype(np.float16).astype(np.float32)


def _worst(q, kx, vx, mask, k_lo=True, p_lo=True, v_lo=True):
    scale = 1.0 / math.sqrt(q.shape[-1])
    s_ref = np.einsum("qhd,td->hqt", q.astype(np.float64), kx.astype(np.float64)) * scale
    s_ref = np.where(mask[None], s_ref, -np.inf)
    p_ref = np.exp(s_ref - s_ref.max(-1, keepdims=True))
    ref = np.einsum("hqt,td->qhd", p_ref / p_ref.sum(-1, keepdims=True), vx.astype(np.float64))

    k_hi = _f16(kx)
    s = np.einsum("qhd,td->hqt", q.astype(np.float64), k_hi.astype(np.float64))
    if k_lo:
        s += np.einsum("qhd,td->hqt", q.astype(np.float64), _f16(kx - k_hi).astype(np.float64))
    s = np.where(mask[None], (s * scale).astype(np.float32).astype(np.float64), -np.inf)
    p = np.exp(s - s.max(-1, keepdims=True)).astype(np.float32)
    denom = p.sum(-1, keepdims=True).astype(np.float64)
    p_hi, v_hi = _f16(p), _f16(vx)
    dot = lambda a, b: np.einsum("hqt,td->qhd", a.astype(np.float64), b.astype(np.float64))
    o = dot(p_hi, v_hi)
    if p_lo:
        o += dot(_f16(p - p_hi), v_hi)
    if v_lo:
        o += dot(p_hi, _f16(vx - v_hi))
    o = (o / np.transpose(denom, (1, 0, 2))).astype(np.float16).astype(np.float64)
    return float((np.abs(o - ref) / (2e-3 + 1e-2 * np.abs(ref))).max())


@pytest.mark.parametrize("seed,prior,nq", [(5, 300, 96), (6, 0, 160)])
def test_hi_lo_pairs_are_what_the_tolerance_costs(seed, prior, nq):
    """The five products of a tile: q.k_hi, q.k_lo, p_hi.v_hi, p_lo.v_hi, p_hi.v_lo.  With all five the worst element
    uses about a twentieth of the tolerance; without q.k_lo the result is outside it; each of the two small PV terms
    alone is worth several times the error of the full scheme (on 10^5 elements a third to two thirds of the
    tolerance, both together up to all of it), so none of the five can go at half precision -- but the small terms
    need only a few bits."""
    case = _case(seed, prior, nq)
    full = _worst(*case)
    assert full < 0.2
    assert _worst(*case, k_lo=False) > 1.0
    assert _worst(*case, p_lo=False) > 3 * full
    assert _worst(*case, v_lo=False) > 3 * full
    assert _worst(*case, p_lo=False, v_lo=False) > 5 * full
