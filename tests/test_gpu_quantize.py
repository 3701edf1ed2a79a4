"""GPU parity of the quantise/append kernel against the CPU oracle: int8 bytes and
fp16 scales bit-exact, through the C ABI."""
import numpy as np
import pytest
import torch

from conftest import host_cache, oracle_append_step, oracle_layout_kwargs

pytestmark = pytest.mark.gpu


def _bits(a):
    return np.ascontiguousarray(a).view(np.uint16)


def run_append(pkg, bt, k, v, canary=(0x5A, 1.5)):
    dev = pkg.harness.DeviceBatch(bt)
    dev.fill_canary(*canary)
    kd = torch.from_numpy(k).cuda()
    vd = torch.from_numpy(v).cuda()
    pkg.ops.key_value_cache(kd, vd, dev.seqstarts, dev.cachestarts, dev.start_pos, dev.cache, dev.scale,
                            batch=bt.batch, max_seqlen=bt.max_seqlen, num_layer=bt.num_layer, layer_idx=bt.layer_idx,
                            num_kv_heads=bt.num_kv_heads, head_dim=bt.head_dim, **dev.layout_kwargs())
    torch.cuda.synchronize()
    return dev.cache.cpu().numpy(), dev.scale.cpu().numpy()


@pytest.mark.parametrize("cache_mode", [0, 1])
@pytest.mark.parametrize("shape", [(8, 8, 64), (32, 8, 128), (6, 3, 96), (4, 1, 256), (2, 2, 8)])
def test_append_bit_exact_ragged(pkg, oracle, cache_mode, shape):
    hq, hkv, d = shape
    bt, rng = pkg.workloads.custom_batch(100 + d + cache_mode, num_heads=hq, num_kv_heads=hkv, head_dim=d,
                                         cache_mode=cache_mode, dec_kv_lens=[5, 130, 1, 77],
                                         prefill_q_lens=[33, 1, 129], prefill_prior=[100, 0, 127],
                                         outliers=d >= 64, num_layer=2, layer_idx=1)
    q, k, v = pkg.workloads.step_inputs(bt, rng)
    # widen the dynamic range: tiny groups (eps clamp, subnormal scales) and large ones
    mag = 10.0 ** rng.integers(-6, 3, size=(k.shape[0], k.shape[1], d // 8, 1))
    k = (k.astype(np.float32).reshape(k.shape[0], k.shape[1], d // 8, 8) * mag).reshape(k.shape).astype(np.float16)
    v[::3] = 0
    got_c, got_s = run_append(pkg, bt, k, v)
    ref_c, ref_s = host_cache(bt, canary=(0x5A, 1.5))
    oracle_append_step(oracle, bt, k, v, ref_c, ref_s)
    assert np.array_equal(got_c, ref_c)
    assert np.array_equal(_bits(got_s), _bits(ref_s))
    assert (got_c[0] == 0x5A).all()  # other layer untouched


def test_append_exhaustive_numerators(pkg, oracle):
    """Every finite fp16 value as a numerator against scales that cover normal, subnormal and
    clamped cases: the group's absmax fixes the scale, the other channels sweep all halves."""
    fin = np.arange(65536, dtype=np.uint16).view(np.float16)
    fin = fin[np.isfinite(fin)]  # 63488 values
    absmaxes = np.array([65504.0, 30000.0, 1000.0, 127.0, 254.0, 100.0, 3.14159, 1.0, 0.7, 0.1, 0.0123, 7.75e-3,
                         5e-3, 2e-3, 1.3e-3, 1.298e-3, 1.27e-3, 1e-3, 1e-4, 6e-5, 6e-8, 0.0], dtype=np.float16)
    rows = []
    for am in absmaxes:
        vals = fin[np.abs(fin.astype(np.float32)) <= np.float32(am)] if am > 0 else np.zeros(7, np.float16)
        pad = (-len(vals)) % 7
        vals = np.concatenate([vals, np.zeros(pad, np.float16)]).reshape(-1, 7)
        grp = np.concatenate([np.full((vals.shape[0], 1), am, np.float16), vals], axis=1)
        rows.append(grp)
    groups = np.concatenate(rows)  # [n, 8]
    n = groups.shape[0]
    pad = (-n) % 16
    groups = np.concatenate([groups, np.zeros((pad, 8), np.float16)])
    tokens = groups.shape[0] // 16
    k = groups.reshape(tokens, 1, 128)
    v = (-groups[::-1]).copy().reshape(tokens, 1, 128)
    bt, _ = pkg.workloads.custom_batch(1, num_heads=1, num_kv_heads=1, head_dim=128, cache_mode=1,
                                       dec_kv_lens=[], prefill_q_lens=[tokens], prefill_prior=[0])
    got_c, got_s = run_append(pkg, bt, k, v)
    ref_c, ref_s = host_cache(bt, canary=(0x5A, 1.5))
    oracle_append_step(oracle, bt, k, v, ref_c, ref_s)
    assert np.array_equal(got_c, ref_c)
    assert np.array_equal(_bits(got_s), _bits(ref_s))
    # and against the independent numpy restatement
    qn, sn = oracle.quantize_groups_numpy(groups)
    tok = bt.cachestarts[0, np.arange(tokens) // 128] + np.arange(tokens) % 128
    assert np.array_equal(got_c[0, 0, tok, 0].reshape(-1, 8), qn)
    assert np.array_equal(_bits(got_s[0, 0, tok, 0].reshape(-1)), _bits(sn))


def test_append_every_absmax(pkg, oracle):
    """Every positive finite half once as a group's absmax (the scale's only input), the other seven channels at
    ratios that hit ties and near-ties: scales and bytes bit-exact against the C oracle and the numpy restatement."""
    pos = np.arange(1, 0x7C00, dtype=np.uint16).view(np.float16)
    fr = np.array([1.0, -1.0, 0.5, -0.25, 0.00390625, 0.9921875, -0.503937, 0.0118], dtype=np.float32)
    groups = (pos.astype(np.float32)[:, None] * fr[None, :]).astype(np.float16)
    pad = (-groups.shape[0]) % 16
    groups = np.concatenate([groups, np.zeros((pad, 8), np.float16)])
    tokens = groups.shape[0] // 16
    k = groups.reshape(tokens, 1, 128)
    v = (-groups[::-1]).copy().reshape(tokens, 1, 128)
    bt, _ = pkg.workloads.custom_batch(1, num_heads=1, num_kv_heads=1, head_dim=128, cache_mode=1,
                                       dec_kv_lens=[], prefill_q_lens=[tokens], prefill_prior=[0])
    got_c, got_s = run_append(pkg, bt, k, v)
    ref_c, ref_s = host_cache(bt, canary=(0x5A, 1.5))
    oracle_append_step(oracle, bt, k, v, ref_c, ref_s)
    assert np.array_equal(got_c, ref_c)
    assert np.array_equal(_bits(got_s), _bits(ref_s))
    qn, sn = oracle.quantize_groups_numpy(groups)
    tok = bt.cachestarts[0, np.arange(tokens) // 128] + np.arange(tokens) % 128
    assert np.array_equal(got_c[0, 0, tok, 0].reshape(-1, 8), qn)
    assert np.array_equal(_bits(got_s[0, 0, tok, 0].reshape(-1)), _bits(sn))


def test_append_empty_and_single(pkg, oracle):
    # sequences with zero new tokens in between, and a batch that appends nothing at all
    bt, rng = pkg.workloads.custom_batch(5, num_heads=4, num_kv_heads=4, head_dim=64, cache_mode=0,
                                         dec_kv_lens=[3, 9], prefill_q_lens=[4], prefill_prior=[2])
    bt.q_lens[1] = 0
    bt.kv_lens[1] = 8
    bt.seqstarts = np.concatenate([[0], np.cumsum(bt.q_lens)]).astype(np.int64)
    bt.start_pos = (bt.kv_lens - bt.q_lens).astype(np.int64)
    n = int(bt.q_lens.sum())
    k = rng.standard_normal((n, 4, 64)).astype(np.float16)
    v = rng.standard_normal((n, 4, 64)).astype(np.float16)
    got_c, got_s = run_append(pkg, bt, k, v)
    ref_c, ref_s = host_cache(bt, canary=(0x5A, 1.5))
    oracle_append_step(oracle, bt, k, v, ref_c, ref_s)
    assert np.array_equal(got_c, ref_c) and np.array_equal(_bits(got_s), _bits(ref_s))


@pytest.mark.parametrize("cache_mode", [0, 1])
@pytest.mark.parametrize("n_seq,hkv,d", [(300, 1, 8), (1500, 1, 8), (700, 2, 64)])
def test_append_many_short_sequences(pkg, oracle, cache_mode, n_seq, hkv, d):
    """Sequences of 0-5 new tokens behind a few decode sequences: a wave's lanes span many sequences (one 8-channel
    group per token at head_dim 8), empty ones among them; more than 1024 sequences take the bisected lookup."""
    rng0 = np.random.default_rng(n_seq + d)
    q_lens = rng0.integers(1, 6, size=n_seq).tolist()
    prior = rng0.integers(0, 200, size=n_seq).tolist()
    bt, rng = pkg.workloads.custom_batch(n_seq, num_heads=hkv, num_kv_heads=hkv, head_dim=d, cache_mode=cache_mode,
                                         dec_kv_lens=[7, 1, 300], prefill_q_lens=q_lens, prefill_prior=prior,
                                         outliers=False)
    empty = 3 + np.flatnonzero(rng0.random(n_seq) < 0.3)
    bt.kv_lens[empty] -= bt.q_lens[empty]
    bt.q_lens[empty] = 0
    bt.seqstarts = np.concatenate([[0], np.cumsum(bt.q_lens)]).astype(np.int64)
    bt.start_pos = (bt.kv_lens - bt.q_lens).astype(np.int64)
    n = int(bt.q_lens.sum())
    k = rng.standard_normal((n, hkv, d)).astype(np.float16)
    v = rng.standard_normal((n, hkv, d)).astype(np.float16)
    got_c, got_s = run_append(pkg, bt, k, v)
    ref_c, ref_s = host_cache(bt, canary=(0x5A, 1.5))
    oracle_append_step(oracle, bt, k, v, ref_c, ref_s)
    assert np.array_equal(got_c, ref_c) and np.array_equal(_bits(got_s), _bits(ref_s))


def test_key_value_cache_flat_entry_point(pkg, oracle):
    """pmxhip_key_value_cache (flattened argument list) writes the same bytes."""
    import ctypes
    bt, rng = pkg.workloads.custom_batch(8, num_heads=8, num_kv_heads=2, head_dim=128, cache_mode=1,
                                         dec_kv_lens=[200, 4], prefill_q_lens=[10], prefill_prior=[125])
    q, k, v = pkg.workloads.step_inputs(bt, rng)
    dev = pkg.harness.DeviceBatch(bt)
    dev.fill_canary()
    kd, vd = torch.from_numpy(k).cuda(), torch.from_numpy(v).cuda()
    lay = bt.layout
    rc = pkg._lib.lib().pmxhip_key_value_cache(
        ctypes.c_void_p(torch.cuda.current_stream().cuda_stream), kd.data_ptr(), vd.data_ptr(),
        dev.seqstarts.data_ptr(), dev.cachestarts.data_ptr(), dev.start_pos.data_ptr(),
        bt.batch, bt.max_seqlen, bt.num_layer, bt.layer_idx, bt.num_kv_heads, bt.head_dim, bt.cache_mode, 128,
        lay.stride_s, lay.stride_l, lay.stride_h, lay.stride_kv, bt.cachestarts_stride_b,
        dev.cache.data_ptr(), dev.scale.data_ptr())
    torch.cuda.synchronize()
    assert rc == 0
    ref_c, ref_s = host_cache(bt, canary=(0x5A, 1.5))
    oracle_append_step(oracle, bt, k, v, ref_c, ref_s)
    assert np.array_equal(dev.cache.cpu().numpy(), ref_c)
    assert np.array_equal(_bits(dev.scale.cpu().numpy()), _bits(ref_s))


def test_append_full_size_roundtrip_property(pkg):
    """C5-sized append (11104 new tokens): dequantised values stay within half a step of the
    input and the absmax element of every group maps to +-127 (size-independent properties)."""
    bt, rng = pkg.workloads.make_batch("C5")
    q, k, v = pkg.workloads.step_inputs(bt, rng)
    dev = pkg.harness.DeviceBatch(bt)
    kd, vd = torch.from_numpy(k).cuda(), torch.from_numpy(v).cuda()
    pkg.ops.key_value_cache(kd, vd, dev.seqstarts, dev.cachestarts, dev.start_pos, dev.cache, dev.scale,
                            batch=bt.batch, max_seqlen=bt.max_seqlen, num_layer=1, layer_idx=0,
                            num_kv_heads=bt.num_kv_heads, head_dim=bt.head_dim, **dev.layout_kwargs())
    torch.cuda.synchronize()
    # gather the rows that were written
    rows = []
    for b in range(bt.batch):
        pos = int(bt.start_pos[b]) + np.arange(int(bt.q_lens[b]))
        rows.append(bt.cachestarts[b, pos // 128] + pos % 128)
    rows = torch.from_numpy(np.concatenate(rows)).cuda()
    for plane, src in ((0, kd), (1, vd)):
        q8 = dev.cache[0, plane, rows].float()              # [n, KVH, D]
        s = dev.scale[0, plane, rows].float()               # [n, KVH, D/8]
        deq = q8 * s.repeat_interleave(8, dim=-1)
        err = (deq - src.float()).abs()
        bound = s.repeat_interleave(8, dim=-1) * (0.5 + 127 * 2.0 ** -11) + 1e-7
        assert bool((err <= bound).all())
        amax = q8.abs().reshape(q8.shape[0], q8.shape[1], -1, 8).amax(dim=-1)
        assert bool((amax[s >= 6.2e-5] == 127).all())
        assert int(q8.abs().max()) <= 127
