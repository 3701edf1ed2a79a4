"""Pins the attention, prefill and combine functions of the CPU oracle with closed
forms, torch's scaled_dot_product_attention on the dequantised cache, naive
loops and log-sum-exp associativity.  No GPU."""
import numpy as np
import pytest
import torch

from conftest import (host_cache, make_prefill_mask, oracle_append_step, oracle_decode, oracle_fill_history,
                      oracle_layout_kwargs, oracle_prefill, oracle_prefill_ex)


def dequantised_sequence(bt, cache, scale, b, plane):
    """float32 [kvlen, KVH, D] of sequence b, gathered token by token (independent of the oracle's addressing)."""
    n = int(bt.kv_lens[b])
    out = np.zeros((n, bt.num_kv_heads, bt.head_dim), dtype=np.float32)
    for t in range(n):
        if bt.cache_mode == 0:
            tok = int(bt.cachestarts[b]) + t
        else:
            tok = int(bt.cachestarts[b, t // 128]) + t % 128
        q8 = cache[bt.layer_idx, plane, tok].astype(np.float32)
        s = scale[bt.layer_idx, plane, tok].astype(np.float32)
        out[t] = q8 * np.repeat(s, 8, axis=-1)
    return out


def build_case(oracle, pkg, seed, **kw):
    bt, rng = pkg.workloads.custom_batch(seed, **kw)
    cache, scale = host_cache(bt)
    oracle_fill_history(oracle, pkg, bt, rng, cache, scale)
    q, k, v = pkg.workloads.step_inputs(bt, rng)
    oracle_append_step(oracle, bt, k, v, cache, scale)
    return bt, q, k, v, cache, scale


@pytest.mark.parametrize("cache_mode", [0, 1])
@pytest.mark.parametrize("heads", [(4, 4), (8, 2)])
def test_decode_matches_torch_sdpa(oracle, pkg, cache_mode, heads):
    hq, hkv = heads
    bt, q, k, v, cache, scale = build_case(oracle, pkg, 21, num_heads=hq, num_kv_heads=hkv, head_dim=64,
                                           cache_mode=cache_mode, dec_kv_lens=[1, 9, 200, 131], outliers=True)
    got = oracle_decode(oracle, bt, q, cache, scale)
    rep = hq // hkv
    for b in range(bt.decoding_batches):
        kd = torch.from_numpy(dequantised_sequence(bt, cache, scale, b, 0)).double()
        vd = torch.from_numpy(dequantised_sequence(bt, cache, scale, b, 1)).double()
        kd = kd.repeat_interleave(rep, dim=1).permute(1, 0, 2)  # [Hq, T, D]
        vd = vd.repeat_interleave(rep, dim=1).permute(1, 0, 2)
        qq = torch.from_numpy(q[b].astype(np.float64))[:, None, :]  # [Hq, 1, D]
        ref = torch.nn.functional.scaled_dot_product_attention(qq, kd, vd, scale=bt.attn_scale)[:, 0]
        np.testing.assert_allclose(got[b], ref.numpy(), rtol=1e-5, atol=1e-6)


def test_decode_closed_forms(oracle, pkg):
    wl = pkg.workloads
    # kvlen = 1: output is the dequantised V row itself
    bt, q, k, v, cache, scale = build_case(oracle, pkg, 3, num_heads=4, num_kv_heads=2, head_dim=64, cache_mode=0,
                                           dec_kv_lens=[1, 1])
    got = oracle_decode(oracle, bt, q, cache, scale)
    for b in range(2):
        vd = dequantised_sequence(bt, cache, scale, b, 1)[0]
        np.testing.assert_array_equal(got[b], np.repeat(vd, 2, axis=0))
    # zero query: uniform weights -> mean of V
    bt, q, k, v, cache, scale = build_case(oracle, pkg, 4, num_heads=2, num_kv_heads=2, head_dim=64, cache_mode=1,
                                           dec_kv_lens=[150])
    got = oracle_decode(oracle, bt, np.zeros_like(q), cache, scale)
    vd = dequantised_sequence(bt, cache, scale, 0, 1)
    np.testing.assert_allclose(got[0], vd.mean(axis=0), rtol=1e-5, atol=1e-6)
    # q-heads of one kv group with identical queries give identical outputs
    bt, q, k, v, cache, scale = build_case(oracle, pkg, 5, num_heads=8, num_kv_heads=2, head_dim=64, cache_mode=0,
                                           dec_kv_lens=[77])
    q2 = q.copy()
    q2[:, 1:4] = q2[:, 0:1]
    got = oracle_decode(oracle, bt, q2, cache, scale)
    for g in range(1, 4):
        np.testing.assert_array_equal(got[0, g], got[0, 0])


def test_decode_dominant_key(oracle, pkg):
    """One key with a logit gap > 40 takes all the weight."""
    bt, rng = pkg.workloads.custom_batch(6, num_heads=1, num_kv_heads=1, head_dim=64, cache_mode=0, dec_kv_lens=[50])
    cache, scale = host_cache(bt)
    k = (rng.standard_normal((50, 1, 64)) * 0.01).astype(np.float16)
    v = rng.standard_normal((50, 1, 64)).astype(np.float16)
    k[17] = 8.0
    oracle.kv_cache_quantize(k, v, np.array([0, 50]), bt.cachestarts, np.array([0]), 0, 1, 64, 0,
                             cache=cache, scale=scale, **oracle_layout_kwargs(bt))
    q = np.ones((1, 1, 64), dtype=np.float16)
    got = oracle_decode(oracle, bt, q, cache, scale)
    vd = dequantised_sequence(bt, cache, scale, 0, 1)[17, 0]
    np.testing.assert_allclose(got[0, 0], vd, rtol=1e-6, atol=1e-7)


def test_decode_paged_equals_contiguous(oracle, pkg):
    wl = pkg.workloads
    outs = []
    for mode in (0, 1):
        bt, rng = wl.custom_batch(9, num_heads=4, num_kv_heads=2, head_dim=64, cache_mode=mode,
                                  dec_kv_lens=[260, 5, 128])
        # same values regardless of placement: draw from a dedicated generator
        vr = np.random.default_rng(99)
        cache, scale = host_cache(bt)
        for b in range(bt.batch):
            n = int(bt.kv_lens[b])
            kk = vr.standard_normal((n, 2, 64)).astype(np.float16)
            vv = vr.standard_normal((n, 2, 64)).astype(np.float16)
            oracle.kv_cache_quantize(kk, vv, np.array([0, n]), bt.cachestarts[b:b + 1], np.array([0]), 0, 2, 64,
                                     bt.page_size, cache=cache, scale=scale, **oracle_layout_kwargs(bt))
        q = vr.standard_normal((3, 4, 64)).astype(np.float16)
        outs.append(oracle_decode(oracle, bt, q, cache, scale))
    np.testing.assert_array_equal(outs[0], outs[1])


def test_decode_mask(oracle, pkg):
    bt, q, k, v, cache, scale = build_case(oracle, pkg, 12, num_heads=4, num_kv_heads=2, head_dim=64, cache_mode=0,
                                           dec_kv_lens=[40, 9])
    total = int(bt.kvstarts[-1])
    width = (total + 7) // 8 * 8
    rng = np.random.default_rng(1)
    mask = rng.standard_normal((bt.num_heads, bt.batch, width)).astype(np.float16)
    mask[:, 0, 3] = -np.inf
    got = oracle_decode(oracle, bt, q, cache, scale, attn_mask=mask, mask_stride_s=width, mask_stride_h=bt.batch * width)
    for b in range(2):
        kd = dequantised_sequence(bt, cache, scale, b, 0).astype(np.float64)
        vd = dequantised_sequence(bt, cache, scale, b, 1).astype(np.float64)
        for h in range(4):
            logits = (kd[:, h // 2] @ q[b, h].astype(np.float64)) * bt.attn_scale
            logits += mask[h, b, int(bt.kvstarts[b]):int(bt.kvstarts[b]) + len(logits)].astype(np.float64)
            p = np.exp(logits - logits.max())
            ref = (p[:, None] * vd[:, h // 2]).sum(0) / p.sum()
            np.testing.assert_allclose(got[b, h], ref, rtol=1e-5, atol=1e-6)


@pytest.mark.parametrize("cache_mode", [0, 1])
def test_prefill_matches_torch_sdpa_bottom_right_causal(oracle, pkg, cache_mode):
    bt, q, k, v, cache, scale = build_case(oracle, pkg, 31, num_heads=4, num_kv_heads=2, head_dim=64,
                                           cache_mode=cache_mode, dec_kv_lens=[33, 140],
                                           prefill_q_lens=[20, 7, 1], prefill_prior=[130, 0, 50])
    got = oracle_prefill(oracle, bt, q, cache, scale)
    dec = oracle_decode(oracle, bt, q, cache, scale)
    assert (got[:bt.decoding_batches] == 0).all()  # decode rows are not the prefill stage's
    for b in range(bt.decoding_batches, bt.batch):
        qlen, kvlen = int(bt.q_lens[b]), int(bt.kv_lens[b])
        kd = torch.from_numpy(dequantised_sequence(bt, cache, scale, b, 0)).double().repeat_interleave(2, 1).permute(1, 0, 2)
        vd = torch.from_numpy(dequantised_sequence(bt, cache, scale, b, 1)).double().repeat_interleave(2, 1).permute(1, 0, 2)
        rows = slice(int(bt.seqstarts[b]), int(bt.seqstarts[b + 1]))
        qq = torch.from_numpy(q[rows].astype(np.float64)).permute(1, 0, 2)
        i = torch.arange(qlen)[:, None]
        j = torch.arange(kvlen)[None, :]
        allowed = j <= i + (kvlen - qlen)  # bottom-right aligned
        ref = torch.nn.functional.scaled_dot_product_attention(qq, kd, vd, attn_mask=allowed, scale=bt.attn_scale)
        np.testing.assert_allclose(got[rows], ref.permute(1, 0, 2).numpy(), rtol=1e-5, atol=1e-6)
    # a prefill sequence with one query row is a decode step over the same cache
    b = bt.batch - 1
    single, _, _ = oracle.decode_partial(q[int(bt.seqstarts[b]):], cache, scale, bt.cachestarts[b:], 0, 1, 0,
                                         int(bt.kv_lens[b]), bt.num_heads, bt.num_kv_heads, bt.head_dim, bt.attn_scale,
                                         bt.layer_idx, bt.page_size, **oracle_layout_kwargs(bt))
    np.testing.assert_allclose(got[int(bt.seqstarts[b]), 1], single, rtol=1e-6, atol=1e-7)
    assert dec.shape[0] == bt.decoding_batches


def sdpa_reference(bt, b, q, kd, vd, bias):
    """float64 softmax(attn_scale q k^T + bias) v for prefill sequence b; bias [Hq, qlen, kvlen] with -inf where masked."""
    rep = bt.num_heads // bt.num_kv_heads
    rows = slice(int(bt.seqstarts[b]), int(bt.seqstarts[b + 1]))
    qq = torch.from_numpy(q[rows].astype(np.float64)).permute(1, 0, 2)
    kk = torch.from_numpy(kd).double().repeat_interleave(rep, 1).permute(1, 0, 2)
    vv = torch.from_numpy(vd).double().repeat_interleave(rep, 1).permute(1, 0, 2)
    ref = torch.nn.functional.scaled_dot_product_attention(qq, kk, vv, attn_mask=bias, scale=bt.attn_scale)
    return rows, ref.permute(1, 0, 2).numpy()


@pytest.mark.parametrize("is_causal", [True, False])
@pytest.mark.parametrize("per_head", [False, True])
def test_prefill_ex_mask_and_alibi_match_torch_sdpa(oracle, pkg, is_causal, per_head):
    bt, q, k, v, cache, scale = build_case(oracle, pkg, 37, num_heads=4, num_kv_heads=2, head_dim=64, cache_mode=1,
                                           dec_kv_lens=[33], prefill_q_lens=[20, 7, 1], prefill_prior=[130, 0, 50],
                                           is_causal=is_causal)
    rng = np.random.default_rng(5)
    mask, ms, mh = make_prefill_mask(bt, rng, per_head)
    slopes = np.array([0.5, 0.25, 0.125, 0.0625], dtype=np.float32)
    # without the optional inputs the extended function is the plain one
    np.testing.assert_array_equal(oracle_prefill_ex(oracle, bt, q, cache, scale), oracle_prefill(oracle, bt, q, cache, scale))
    got = oracle_prefill_ex(oracle, bt, q, cache, scale, attn_mask=mask, mask_stride_s=ms, mask_stride_h=mh,
                            alibi_slopes=slopes)
    for b in range(bt.decoding_batches, bt.batch):
        qlen, kvlen = int(bt.q_lens[b]), int(bt.kv_lens[b])
        i = torch.arange(qlen)[:, None]
        j = torch.arange(kvlen)[None, :]
        r0, c0 = int(bt.seqstarts[b]), int(bt.kvstarts[b])
        m = mask[:, r0:r0 + qlen, c0:c0 + kvlen] if per_head else np.broadcast_to(mask[r0:r0 + qlen, c0:c0 + kvlen], (4, qlen, kvlen))
        bias = torch.from_numpy(m.astype(np.float64)).clone()
        sl = torch.from_numpy(slopes.astype(np.float64))[:, None, None]
        if is_causal:
            bias += sl * j  # mask.h:191-193
            bias = bias.masked_fill(~(j <= i + (kvlen - qlen)), float("-inf"))
        else:
            bias -= sl * (i + kvlen - qlen - j).abs()  # mask.h:194-196
        rows, ref = sdpa_reference(bt, b, q, dequantised_sequence(bt, cache, scale, b, 0),
                                   dequantised_sequence(bt, cache, scale, b, 1), bias)
        np.testing.assert_allclose(got[rows], ref, rtol=1e-5, atol=1e-6)


def test_prefill_ex_from_current_key_value_matches_torch_sdpa(oracle, pkg):
    """enable_cache_prefill = false: the step's fp16 K/V rows only, kv length = query length."""
    bt, q, k, v, cache, scale = build_case(oracle, pkg, 41, num_heads=4, num_kv_heads=2, head_dim=64, cache_mode=0,
                                           dec_kv_lens=[9, 12], prefill_q_lens=[20, 7, 1], prefill_prior=[0, 0, 0])
    got = oracle_prefill_ex(oracle, bt, q, cache, scale, current_key=k, current_value=v)
    for b in range(bt.decoding_batches, bt.batch):
        qlen = int(bt.q_lens[b])
        rows = slice(int(bt.seqstarts[b]), int(bt.seqstarts[b + 1]))
        i = torch.arange(qlen)[:, None]
        j = torch.arange(qlen)[None, :]
        bias = torch.zeros(4, qlen, qlen, dtype=torch.float64).masked_fill(~(j <= i), float("-inf"))
        _, ref = sdpa_reference(bt, b, q, k[rows].astype(np.float32), v[rows].astype(np.float32), bias)
        np.testing.assert_allclose(got[rows], ref, rtol=1e-5, atol=1e-6)
    # with no prior context the cache holds exactly these rows, quantised: the two paths agree to quantisation error
    via_cache = oracle_prefill(oracle, bt, q, cache, scale)
    rows = slice(int(bt.seqstarts[bt.decoding_batches]), int(bt.seqstarts[-1]))
    assert np.abs(via_cache[rows] - got[rows]).max() < 0.1


def test_combine_is_split_invariant(oracle, pkg):
    bt, q, k, v, cache, scale = build_case(oracle, pkg, 41, num_heads=2, num_kv_heads=1, head_dim=64, cache_mode=1,
                                           dec_kv_lens=[37])
    full = oracle_decode(oracle, bt, q, cache, scale)[0, 1]
    n = 37
    kw = oracle_layout_kwargs(bt)
    rng = np.random.default_rng(0)
    for n_cuts in list(range(0, 6)) + [36]:
        cuts = sorted(rng.choice(np.arange(1, n), size=min(n_cuts, n - 1), replace=False).tolist())
        edges = [0] + cuts + [n]
        if n_cuts == 3:
            edges.insert(2, edges[2])  # an empty piece in the middle
        po, pm, ps = [], [], []
        for a, e in zip(edges[:-1], edges[1:]):
            o, m, s = oracle.decode_partial(q, cache, scale, bt.cachestarts, 0, 1, a, e, 2, 1, 64, bt.attn_scale, 0,
                                            bt.page_size, **kw)
            po.append(o), pm.append(m), ps.append(s)
        got = oracle.splitkv_combine(np.stack(po), np.array(pm), np.array(ps))
        np.testing.assert_allclose(got, full, rtol=1e-5, atol=1e-6)
    # no pieces at all -> zeros
    assert (oracle.splitkv_combine(np.zeros((1, 64)), np.array([0.0]), np.array([0.0])) == 0).all()
