"""Rotary position embedding: the CPU oracle is pinned by numpy complex arithmetic and closed forms; the HIP
kernel, alone and fused with the int8 append, is compared with the oracle (GPU tests)."""
import numpy as np
import pytest

from conftest import host_cache, oracle_layout_kwargs


def complex_reference(x, pos, theta, rotary_dim, scale=1.0):
    """float64: pairs (2i, 2i+1) as complex numbers times exp(i * angle); angle from the binary32 formula."""
    x = x.astype(np.float64)
    s, h, d = x.shape
    rd2 = rotary_dim // 2
    out = x.copy()
    i = np.arange(rd2)
    inv = (np.float32(1.0) / np.power(np.float64(theta), (i.astype(np.float32) / np.float32(rd2)).astype(np.float64)).astype(np.float32)).astype(np.float32)
    p = pos.astype(np.float32) if scale == 1.0 else (pos.astype(np.float32) / np.float32(scale)).astype(np.float32)
    ang = (inv[None, :] * p[:, None]).astype(np.float32).astype(np.float64)
    z = (x[:, :, 0:2 * rd2:2] + 1j * x[:, :, 1:2 * rd2:2]) * np.exp(1j * ang)[:, None, :]
    out[:, :, 0:2 * rd2:2] = z.real
    out[:, :, 1:2 * rd2:2] = z.imag
    return out


def make_inputs(seed, lens, starts, hq, hk, d):
    rng = np.random.default_rng(seed)
    seqstarts = np.concatenate([[0], np.cumsum(lens)]).astype(np.int64)
    start_pos = np.array(starts, dtype=np.int64)
    n = int(seqstarts[-1])
    q = rng.standard_normal((n, hq, d)).astype(np.float16)
    k = rng.standard_normal((n, hk, d)).astype(np.float16)
    v = rng.standard_normal((n, hk, d)).astype(np.float16)
    pos = np.concatenate([s + np.arange(l) for s, l in zip(starts, lens)]).astype(np.int64)
    return q, k, v, seqstarts, start_pos, pos


@pytest.mark.parametrize("rotary_dim", [64, 32])
def test_oracle_rope_matches_complex_rotation(oracle, rotary_dim):
    q, k, v, seqstarts, start_pos, pos = make_inputs(1, [5, 1, 9], [0, 4095, 100], 4, 2, 64)
    rq, rk = oracle.rotary_position_embedding(q, k, start_pos, seqstarts, 10000.0, rotary_dim)
    for got, x in ((rq, q), (rk, k)):
        ref = complex_reference(x, pos, 10000.0, rotary_dim)
        # one rounding to half of a binary32 result within a few binary32 ulps of the exact rotation
        assert np.abs(got.astype(np.float64) - ref).max() <= 2.0 ** -11 * np.abs(ref).max() * 1.01 + 1e-6
        np.testing.assert_array_equal(got[:, :, rotary_dim:], x[:, :, rotary_dim:])  # pass-through channels
    # position 0 is the identity; pair norms are preserved up to rounding
    np.testing.assert_array_equal(rq[0], q[0])
    n0 = np.hypot(q[:, :, 0::2].astype(np.float64), q[:, :, 1::2].astype(np.float64))
    n1 = np.hypot(rq[:, :, 0::2].astype(np.float64), rq[:, :, 1::2].astype(np.float64))
    assert np.abs(n1 - n0).max() < 4e-3
    # bypass_key copies the key
    _, rk2 = oracle.rotary_position_embedding(q, k, start_pos, seqstarts, 10000.0, rotary_dim, bypass_key=True)
    np.testing.assert_array_equal(rk2, k)


def test_oracle_rope_scaling_variants(oracle):
    q, k, v, seqstarts, start_pos, pos = make_inputs(2, [6, 3], [10, 5000], 2, 2, 32)
    # linear: the rotation at pos / factor
    rq, _ = oracle.rotary_position_embedding(q, k, start_pos, seqstarts, 10000.0, 32, scaling_type=1, scaling_factor=4.0)
    ref = complex_reference(q, pos, 10000.0, 32, scale=4.0)
    assert np.abs(rq.astype(np.float64) - ref).max() <= 2.0 ** -11 * np.abs(ref).max() * 1.01 + 1e-6
    # dynamic: sequences that stay inside max_position_embeddings keep theta; the long one gets
    # theta * (factor * end / max - (factor - 1)) ** (rd2 / (rd2 - 1))  (rotary_position_embedding.cu:78-85)
    rq, _ = oracle.rotary_position_embedding(q, k, start_pos, seqstarts, 10000.0, 32, max_position_embeddings=4096,
                                             scaling_type=2, scaling_factor=2.0)
    plain, _ = oracle.rotary_position_embedding(q, k, start_pos, seqstarts, 10000.0, 32)
    np.testing.assert_array_equal(rq[:6], plain[:6])
    base = np.float32(np.float32(2.0 * 5003) / np.float32(4096)) - np.float32(1.0)
    theta2 = float(np.float32(10000.0) * np.float32(np.power(np.float64(base), np.float64(np.float32(16) / np.float32(15)))))
    ref = complex_reference(q[6:], pos[6:], theta2, 32)
    assert np.abs(rq[6:].astype(np.float64) - ref).max() <= 2.0 ** -11 * np.abs(ref).max() * 1.01 + 1e-6


@pytest.mark.gpu
@pytest.mark.parametrize("shape,rotary_dim,scaling", [((8, 2, 128), 128, (0, 1.0)), ((4, 4, 64), 32, (1, 4.0)),
                                                       ((32, 8, 128), 128, (2, 2.0)), ((6, 2, 96), 96, (0, 1.0))])
def test_gpu_rope_and_fused_append_match_oracle(pkg, oracle, shape, rotary_dim, scaling):
    import torch
    hq, hk, d = shape
    bt, rng = pkg.workloads.custom_batch(900 + hq, num_heads=hq, num_kv_heads=hk, head_dim=d, cache_mode=1,
                                         dec_kv_lens=[300, 4099, 17], prefill_q_lens=[70, 129], prefill_prior=[130, 5000])
    dev = pkg.harness.DeviceBatch(bt)
    q, k, v = pkg.workloads.step_inputs(bt, rng)
    dev.set_step_inputs(q, k, v)
    kw = dict(theta=10000.0, rotary_dim=rotary_dim, batch=bt.batch, max_seqlen=bt.max_seqlen,
              max_position_embeddings=4096, scaling_type=scaling[0], scaling_factor=scaling[1])
    okw = dict(max_position_embeddings=4096, scaling_type=scaling[0], scaling_factor=scaling[1])
    rq_ref, rk_ref = oracle.rotary_position_embedding(q, k, bt.start_pos, bt.seqstarts, 10000.0, rotary_dim, **okw)
    d_rq = torch.empty_like(dev.query)
    d_rk = torch.empty_like(dev.new_key)
    pkg.ops.rotary_position_embedding(dev.query, dev.new_key, dev.start_pos, dev.seqstarts, d_rq, d_rk, **kw)
    torch.cuda.synchronize()
    rq, rk = d_rq.cpu().numpy(), d_rk.cpu().numpy()
    # the two sides share one definition of the angle; cos/sin are correctly rounded binary32 on both, so the
    # halves agree bit for bit (a disagreement needs a binary64 result within 1e-9 ulp of a rounding boundary)
    np.testing.assert_array_equal(rq.view(np.uint16), rq_ref.view(np.uint16))
    np.testing.assert_array_equal(rk.view(np.uint16), rk_ref.view(np.uint16))
    # fused with the append: cache bytes and scales equal oracle(rope) -> oracle(quantise), bit for bit
    cache_ref, scale_ref = host_cache(bt)
    oracle.kv_cache_quantize(rk_ref, v, bt.seqstarts, bt.cachestarts, bt.start_pos, bt.layer_idx, bt.num_kv_heads,
                             bt.head_dim, bt.page_size, cache=cache_ref, scale=scale_ref, **oracle_layout_kwargs(bt))
    d_rq2 = torch.empty_like(dev.query)
    lk = dev.layout_kwargs()
    pkg.ops.rope_key_value_cache(dev.query, dev.new_key, dev.new_value, dev.start_pos, dev.seqstarts, dev.cachestarts,
                                 d_rq2, None, dev.cache, dev.scale, num_layer=bt.num_layer, layer_idx=bt.layer_idx, **lk, **kw)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(d_rq2.cpu().numpy().view(np.uint16), rq_ref.view(np.uint16))
    np.testing.assert_array_equal(dev.cache.cpu().numpy(), cache_ref)
    np.testing.assert_array_equal(dev.scale.cpu().numpy().view(np.uint16), scale_ref.view(np.uint16))
    # and in place (rotated_query aliasing query)
    pkg.ops.rotary_position_embedding(dev.query, dev.new_key, dev.start_pos, dev.seqstarts, dev.query, dev.new_key, **kw)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(dev.query.cpu().numpy().view(np.uint16), rq_ref.view(np.uint16))


@pytest.mark.gpu
@pytest.mark.parametrize("shape", [(8, 2, 128), (4, 4, 64), (2, 1, 256), (6, 2, 96)])
@pytest.mark.parametrize("n_dec,n_prefill", [(100, 50), (0, 130), (1000, 100)])
def test_gpu_rope_many_sequences(pkg, oracle, shape, n_dec, n_prefill):
    """Batches of 130 to 1100 sequences, single-token and short multi-token ones mixed: a token's sequence is counted by
    the lanes of a wave (several entries per lane; one, two or four tokens per wave by head_dim) or, beyond 1024
    sequences, found by bisection.  RoPE alone and fused with the append, bit for bit against the oracle."""
    import torch
    hq, hk, d = shape
    r = np.random.default_rng(n_dec + n_prefill + d)
    bt, rng = pkg.workloads.custom_batch(77 + d, num_heads=hq, num_kv_heads=hk, head_dim=d, cache_mode=1,
                                         dec_kv_lens=r.integers(1, 200, n_dec).tolist(),
                                         prefill_q_lens=r.integers(1, 6, n_prefill).tolist(),
                                         prefill_prior=r.integers(0, 300, n_prefill).tolist())
    dev = pkg.harness.DeviceBatch(bt)
    q, k, v = pkg.workloads.step_inputs(bt, rng)
    dev.set_step_inputs(q, k, v)
    kw = dict(theta=10000.0, rotary_dim=d, batch=bt.batch, max_seqlen=bt.max_seqlen)
    rq_ref, rk_ref = oracle.rotary_position_embedding(q, k, bt.start_pos, bt.seqstarts, 10000.0, d)
    cache_ref, scale_ref = host_cache(bt)
    oracle.kv_cache_quantize(rk_ref, v, bt.seqstarts, bt.cachestarts, bt.start_pos, bt.layer_idx, bt.num_kv_heads,
                             bt.head_dim, bt.page_size, cache=cache_ref, scale=scale_ref, **oracle_layout_kwargs(bt))
    d_rq, d_rk = torch.empty_like(dev.query), torch.empty_like(dev.new_key)
    pkg.ops.rotary_position_embedding(dev.query, dev.new_key, dev.start_pos, dev.seqstarts, d_rq, d_rk, **kw)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(d_rq.cpu().numpy().view(np.uint16), rq_ref.view(np.uint16))
    np.testing.assert_array_equal(d_rk.cpu().numpy().view(np.uint16), rk_ref.view(np.uint16))
    d_rq.zero_()
    d_rk.zero_()
    pkg.ops.rope_key_value_cache(dev.query, dev.new_key, dev.new_value, dev.start_pos, dev.seqstarts, dev.cachestarts,
                                 d_rq, d_rk, dev.cache, dev.scale, num_layer=bt.num_layer, layer_idx=bt.layer_idx,
                                 **dev.layout_kwargs(), **kw)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(d_rq.cpu().numpy().view(np.uint16), rq_ref.view(np.uint16))
    np.testing.assert_array_equal(d_rk.cpu().numpy().view(np.uint16), rk_ref.view(np.uint16))
    np.testing.assert_array_equal(dev.cache.cpu().numpy(), cache_ref)
    np.testing.assert_array_equal(dev.scale.cpu().numpy().view(np.uint16), scale_ref.view(np.uint16))
