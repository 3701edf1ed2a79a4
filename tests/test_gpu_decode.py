"""GPU parity of decode attention (and its split-KV combine) against the CPU
oracle, through the C ABI.  Tolerance: |got - ref| <= 2e-3 + 1e-2 * |ref| against
the fp32 dequantised reference."""
import numpy as np
import pytest
import torch

from conftest import (assert_attention_close, host_cache, oracle_append_step, oracle_decode, oracle_fill_history,
                      oracle_layout_kwargs)

pytestmark = pytest.mark.gpu


def make_case(pkg, oracle, seed, **kw):
    """Cache quantised by the oracle on the host, uploaded as-is: decode parity is then
    independent of the append kernel."""
    bt, rng = pkg.workloads.custom_batch(seed, **kw)
    cache, scale = host_cache(bt)
    oracle_fill_history(oracle, pkg, bt, rng, cache, scale)
    q, k, v = pkg.workloads.step_inputs(bt, rng)
    oracle_append_step(oracle, bt, k, v, cache, scale)
    dev = pkg.harness.DeviceBatch(bt)
    dev.cache.copy_(torch.from_numpy(cache))
    dev.scale.copy_(torch.from_numpy(scale))
    dev.set_step_inputs(q, k, v)
    return bt, dev, q, cache, scale


def run_decode(dev, ranges=0, **kw):
    dev.output.fill_(float("nan"))
    plan, ws = dev.decode_only(num_token_ranges=ranges, **kw)
    torch.cuda.synchronize()
    return dev.output[:dev.bt.decoding_batches].float().cpu().numpy(), plan


SHAPES = [
    # (Hq, KVH, D)
    (8, 8, 64), (4, 4, 128), (32, 8, 128), (16, 2, 128), (12, 2, 128), (6, 2, 96), (4, 2, 256), (32, 2, 64),
    (3, 3, 128), (24, 8, 128), (2, 1, 128), (16, 8, 128), (8, 8, 128), (64, 16, 128), (64, 8, 128), (40, 8, 128),
    (28, 4, 128), (64, 4, 128), (128, 4, 128), (96, 8, 128),
    # the MFMA kernels with one or two kv heads (the share of one GPU under tensor parallelism)
    (8, 1, 128), (4, 1, 128), (40, 2, 128), (24, 1, 128), (12, 4, 128),
    # the quad kernel with four and two kv heads per workgroup
    (8, 2, 128), (6, 6, 128), (24, 12, 128), (16, 4, 128),
    # ... and with head_dim 256 (a wave per kv head)
    (16, 8, 256), (16, 16, 256), (3, 1, 256), (8, 2, 256), (5, 1, 256),
    # ... and with head_dim 64 (blocks of 32 tokens: the rows of a half-wave are two token groups)
    (32, 8, 64), (8, 4, 64), (6, 2, 64), (16, 16, 64), (18, 6, 64),
    # the 32-column MFMA kernel at head_dim 64, and with more than 32 query heads per kv head (passes of 32 columns:
    # multi-query models)
    (128, 8, 64), (14, 2, 64), (3, 1, 64), (71, 1, 64), (66, 2, 64), (48, 1, 128), (40, 1, 128), (132, 4, 128),
    # the quad kernel with an odd number of kv heads (the last half-wave has none)
    (5, 5, 128), (9, 3, 128), (14, 7, 128), (9, 9, 64), (12, 3, 64), (36, 9, 128),
    # head_dim 256 with five to eight query heads per kv head: two sets of waves
    (8, 1, 256), (32, 4, 256), (12, 2, 256), (40, 8, 256), (21, 3, 256),
]


@pytest.mark.parametrize("cache_mode", [0, 1])
@pytest.mark.parametrize("shape", SHAPES)
def test_decode_matches_oracle(pkg, oracle, shape, cache_mode):
    hq, hkv, d = shape
    bt, dev, q, cache, scale = make_case(pkg, oracle, 200 + hq + d, num_heads=hq, num_kv_heads=hkv, head_dim=d,
                                         cache_mode=cache_mode, dec_kv_lens=[1, 300, 17, 129, 640, 2, 128],
                                         outliers=True)
    ref = oracle_decode(oracle, bt, q, cache, scale)
    for ranges in (1, 0, 3, 11):
        got, plan = run_decode(dev, ranges)
        assert_attention_close(got, ref, "shape %s mode %d ranges %d" % (shape, cache_mode, plan.num_token_ranges))


KERNEL_NAMES = {1: "decode_attention_kernel", 2: "decode_attention_quad_kernel",
                3: "decode_attention_mfma16_kernel", 4: "decode_attention_mfma_kernel"}


@pytest.mark.parametrize("shape,kernels", [
    ((32, 8, 128), (1, 2, 3, 4)),   # Llama-3-8B: every kernel serves it
    ((64, 8, 128), (1, 2, 3, 4)),   # 8 query heads per kv head: the quad kernel runs two sets of waves
    ((8, 8, 128), (1, 2, 3)),
    ((12, 2, 128), (1, 3, 4)),
    ((96, 4, 128), (1, 4)),         # 24 per kv head: three passes of the general kernel, or 32 columns
    ((16, 8, 256), (1, 2)),
    ((6, 3, 128), (1, 2, 3)),
    ((5, 5, 128), (1, 2)),
    ((8, 1, 256), (1, 2)),
    ((32, 8, 64), (1, 2, 4)),
    ((4, 4, 64), (1, 2)),
    ((48, 1, 128), (1, 4)),         # multi-query: six passes of the general kernel, or two of 32 columns
    ((71, 1, 64), (1, 4)),
])
def test_decode_requested_kernel(pkg, oracle, shape, kernels):
    """Every token-range kernel that serves a shape, requested through the C ABI: the library reports that it
    runs, and the result is the oracle's whatever the split."""
    hq, hkv, d = shape
    bt, dev, q, cache, scale = make_case(pkg, oracle, 400 + hq + d, num_heads=hq, num_kv_heads=hkv, head_dim=d,
                                         cache_mode=1, dec_kv_lens=[1, 300, 17, 129, 640, 2, 128], outliers=True)
    ref = oracle_decode(oracle, bt, q, cache, scale)
    for k in kernels:
        assert dev.decode_only(kernel=k, name_only=True) == KERNEL_NAMES[k]
        for ranges in (1, 0, 5):
            got, plan = run_decode(dev, ranges, kernel=k)
            assert plan.kernel == k
            assert_attention_close(got, ref, "shape %s kernel %d ranges %d" % (shape, k, plan.num_token_ranges))


@pytest.mark.parametrize("shape", [(16, 4, 128), (8, 2, 128), (12, 6, 128), (8, 4, 256), (8, 4, 64)])
def test_decode_output_rows_aligned_to_8_bytes_only(pkg, oracle, shape):
    """The C ABI admits output rows that are 8-byte aligned; the quad kernel needs 16.  Such a call runs on the
    general kernel, and the token-range kernel and the combine kernel must then cut the ranges by the same unit
    (several ranges, so that sequences are split into pieces)."""
    hq, hkv, d = shape
    bt, dev, q, cache, scale = make_case(pkg, oracle, 450 + hq + d, num_heads=hq, num_kv_heads=hkv, head_dim=d,
                                         cache_mode=1, dec_kv_lens=[900, 300, 17, 129, 640, 2, 128], outliers=True)
    ref = oracle_decode(oracle, bt, q, cache, scale)
    assert dev.decode_only(name_only=True) == "decode_attention_quad_kernel"
    n = bt.decoding_batches * hq * d
    buf = torch.full((n + 8,), float("nan"), dtype=torch.float16, device="cuda")
    out = buf[4:4 + n].view(bt.decoding_batches, hq, d)
    assert out.data_ptr() % 16 == 8
    assert dev.decode_only(output=out, name_only=True) == "decode_attention_kernel"
    for ranges in (1, 0, 3, 11, 40):
        out.fill_(float("nan"))
        plan, _ = dev.decode_only(num_token_ranges=ranges, output=out)
        torch.cuda.synchronize()
        assert_attention_close(out.float().cpu().numpy(), ref, "shape %s ranges %d" % (shape, plan.num_token_ranges))
    assert torch.isnan(buf[:4]).all() and torch.isnan(buf[4 + n:]).all()
    # insisting on the quad kernel for these rows is refused, not silently served by another kernel
    with pytest.raises(pkg.ops.PmxError):
        dev.decode_only(output=out, kernel=2)


def test_decode_c1_golden_shape(pkg, oracle):
    """C1 against the frozen fixture (tests/golden/c1_decode_golden.npz), not against a live oracle: the append
    kernel's cache bytes and scales by digest and by the stored rows, the decode output within tolerance."""
    import hashlib
    import os
    want = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "c1_decode_golden.npz"),
                   allow_pickle=False)
    bt, rng = pkg.workloads.make_batch("C1")
    assert np.array_equal(bt.kv_lens, want["kv_lens"]) and np.array_equal(bt.cachestarts, want["cachestarts"])
    dev = pkg.harness.DeviceBatch(bt)
    dev.fill_history(rng)  # the history goes through the HIP append kernel
    q, k, v = pkg.workloads.step_inputs(bt, rng)
    dev.set_step_inputs(q, k, v)
    op = dev.make_operator()
    assert op.forward() == 0
    torch.cuda.synchronize()
    cache, scale = dev.cache.cpu().numpy(), dev.scale.cpu().numpy()
    rows = (bt.cachestarts + bt.start_pos).astype(np.int64)
    assert np.array_equal(cache[0, 0, rows], want["appended_k"]) and np.array_equal(cache[0, 1, rows], want["appended_v"])
    assert np.array_equal(scale[0, 0, rows].view(np.uint16), want["appended_k_scale"])
    assert hashlib.sha256(np.ascontiguousarray(cache).tobytes()).hexdigest() == str(want["sha_cache"])
    assert hashlib.sha256(np.ascontiguousarray(scale.view(np.uint16)).tobytes()).hexdigest() == str(want["sha_scale"])
    assert_attention_close(dev.output.float().cpu().numpy(), want["output"], "C1 through the operator")
    got, _ = run_decode(dev)
    assert_attention_close(got, want["output"], "C1")


def test_decode_empty_sequence_and_closed_forms(pkg, oracle):
    bt, dev, q, cache, scale = make_case(pkg, oracle, 77, num_heads=8, num_kv_heads=2, head_dim=128, cache_mode=1,
                                         dec_kv_lens=[1, 40, 1, 9])
    # make sequence 1 empty: kv length 0 -> zeros (the reference's 0/(0+1e-6))
    bt.kv_lens[1] = 0
    bt.kvstarts = np.concatenate([[0], np.cumsum(bt.kv_lens)]).astype(np.int64)
    dev.kvstarts.copy_(torch.from_numpy(bt.kvstarts))
    ref = oracle_decode(oracle, bt, q, cache, scale)
    assert (ref[1] == 0).all()
    for ranges in (1, 2):
        got, _ = run_decode(dev, ranges)
        assert_attention_close(got, ref, "empty seq")
        assert (got[1] == 0).all()
        # kvlen = 1: the output is the dequantised V row, exactly representable -> fp16 rounding only
        for b in (0, 2):
            tok = int(bt.cachestarts[b, 0])
            vrow = cache[0, 1, tok].astype(np.float32) * np.repeat(scale[0, 1, tok].astype(np.float32), 8, -1)
            want = np.repeat(vrow, 4, axis=0).astype(np.float16).astype(np.float32)
            np.testing.assert_allclose(got[b], want, rtol=2e-3, atol=1e-6)


@pytest.mark.parametrize("shape", [(8, 8, 64), (6, 2, 96), (32, 8, 128), (8, 2, 128), (4, 2, 256)])
def test_decode_many_pieces_per_sequence(pkg, oracle, shape):
    """Long sequences cut into many pieces: the combine kernel then shares the pieces of a row between
    two or four waves (chosen from ranges / sequences), for every row width."""
    hq, hkv, d = shape
    bt, dev, q, cache, scale = make_case(pkg, oracle, 300 + d, num_heads=hq, num_kv_heads=hkv, head_dim=d,
                                         cache_mode=1, dec_kv_lens=[5000, 700], outliers=True)
    ref = oracle_decode(oracle, bt, q, cache, scale)
    for ranges in (20, 40, 120):  # one, two and four waves per row
        got, plan = run_decode(dev, ranges)
        assert plan.num_token_ranges == ranges
        assert_attention_close(got, ref, "shape %s ranges %d" % (shape, ranges))


@pytest.mark.parametrize("shape", [(32, 8, 128), (8, 8, 64)])
def test_decode_more_sequences_than_the_counted_lookup(pkg, oracle, shape):
    """1500 short sequences (some empty): a range's first sequence is then found by bisection instead of the
    one-round count, and most ranges hold many whole sequences."""
    hq, hkv, d = shape
    lens = np.random.default_rng(9).integers(1, 40, 1500)
    bt, dev, q, cache, scale = make_case(pkg, oracle, 500 + d, num_heads=hq, num_kv_heads=hkv, head_dim=d,
                                         cache_mode=1, dec_kv_lens=lens.tolist())
    for b in (0, 7, 700, 1499):
        bt.kv_lens[b] = 0
    bt.kvstarts = np.concatenate([[0], np.cumsum(bt.kv_lens)]).astype(np.int64)
    dev.kvstarts.copy_(torch.from_numpy(bt.kvstarts))
    ref = oracle_decode(oracle, bt, q, cache, scale)
    for ranges in (0, 64, 1):
        got, plan = run_decode(dev, ranges)
        assert_attention_close(got, ref, "shape %s ranges %d" % (shape, plan.num_token_ranges))
        assert (got[[0, 7, 700, 1499]] == 0).all()


def test_decode_gqa_identical_queries_and_mha_equivalence(pkg, oracle):
    bt, dev, q, cache, scale = make_case(pkg, oracle, 78, num_heads=8, num_kv_heads=2, head_dim=128, cache_mode=0,
                                         dec_kv_lens=[333, 64])
    q2 = q.copy()
    q2[:, 1:4] = q2[:, 0:1]
    dev.query.copy_(torch.from_numpy(q2))
    got, _ = run_decode(dev, 2)
    for g in range(1, 4):
        assert np.array_equal(got[:, g], got[:, 0])


@pytest.mark.parametrize("heads", [(8, 4), (32, 4), (96, 4), (8, 8), (32, 8), (6, 2), (2, 1), (24, 8), (8, 4, 256), (2, 1, 256),
                                   # one query head per kv head: (heads, kv heads, head_dim, cache_mode)
                                   (16, 16, 128, 0), (4, 4, 256, 1), (2, 2, 256, 0),
                                   # passes of 32 columns, and head_dim 64 on the 32-column kernel
                                   (48, 1, 128, 1), (14, 2, 64, 1), (71, 1, 64, 0),
                                   # an odd number of kv heads on the quad kernel
                                   (5, 5, 128, 1), (12, 3, 128, 0)])
def test_decode_with_mask(pkg, oracle, heads):
    bt, dev, q, cache, scale = make_case(pkg, oracle, 79, num_heads=heads[0], num_kv_heads=heads[1],
                                         head_dim=heads[2] if len(heads) > 2 else 128,
                                         cache_mode=heads[3] if len(heads) > 3 else 1, dec_kv_lens=[70, 300, 5])
    total = int(bt.kvstarts[-1])
    width = (total + 7) // 8 * 8
    rng = np.random.default_rng(3)
    for per_head in (True, False):
        shape = (bt.num_heads, bt.batch, width) if per_head else (bt.batch, width)
        mask = rng.standard_normal(shape).astype(np.float16)
        mask[..., 1, 5:9] = -np.inf
        msh = bt.batch * width if per_head else 0
        ref = oracle_decode(oracle, bt, q, cache, scale, attn_mask=mask, mask_stride_s=width, mask_stride_h=msh)
        md = torch.from_numpy(mask).cuda()
        for ranges in (1, 4):
            got, _ = run_decode(dev, ranges, attn_mask=md, mask_stride_s=width, mask_stride_h=msh)
            assert_attention_close(got, ref, "mask per_head=%s ranges=%d" % (per_head, ranges))


def test_combine_entry_point_against_oracle_pieces(pkg, oracle):
    """pmxhip_splitkv_combine on pieces produced by the oracle: any cut of the kv range gives the single-pass result."""
    bt, dev, q, cache, scale = make_case(pkg, oracle, 80, num_heads=4, num_kv_heads=2, head_dim=128, cache_mode=1,
                                         dec_kv_lens=[97, 260])
    ref = oracle_decode(oracle, bt, q, cache, scale)
    kw = oracle_layout_kwargs(bt)
    log2e = 1.4426950408889634
    po, pml, begin, end = [], [], [], []
    rng = np.random.default_rng(4)
    for b in range(2):
        n = int(bt.kv_lens[b])
        for h in range(4):
            cuts = sorted(rng.choice(np.arange(1, n), size=int(rng.integers(0, 6)), replace=False).tolist())
            edges = [0] + cuts + [n]
            if h == 2:
                edges.insert(1, edges[1])  # an empty piece
            begin.append(len(po))
            for a, e in zip(edges[:-1], edges[1:]):
                o, m, s = oracle.decode_partial(q[b:], cache, scale, bt.cachestarts[b:], 0, h, a, e, 4, 2, 128,
                                                bt.attn_scale, 0, bt.page_size, **kw)
                po.append(o)
                # the kernel keeps the running max in log2 units; an empty piece carries sum 0
                pml.append([m * log2e if s > 0 else -1e30, s])
            end.append(len(po))
    out = torch.zeros(8, 128, dtype=torch.float16, device="cuda")
    pkg.ops.splitkv_combine(torch.tensor(np.stack(po), dtype=torch.float32, device="cuda"),
                            torch.tensor(pml, dtype=torch.float32, device="cuda"),
                            torch.tensor(begin, dtype=torch.int64, device="cuda"),
                            torch.tensor(end, dtype=torch.int64, device="cuda"), out, head_dim=128)
    torch.cuda.synchronize()
    assert_attention_close(out.float().cpu().numpy().reshape(2, 4, 128), ref, "combine")


@pytest.mark.parametrize("name", ["C2", "C3", "C4"])
def test_decode_full_size_properties(pkg, oracle, name):
    """At the benchmark's full sizes the oracle is too slow for every row, so: (1) the split count
    does not change the result (1 range vs the planned hundreds), (2) sampled rows match the oracle."""
    bt, rng = pkg.workloads.make_batch(name)
    dev = pkg.harness.DeviceBatch(bt)
    dev.fill_history_random_bytes(seed=bt.seed)
    q, k, v = pkg.workloads.step_inputs(bt, rng)
    dev.set_step_inputs(q, k, v)
    got_many, plan = run_decode(dev, 0)
    assert plan.num_token_ranges > 1
    got_few, _ = run_decode(dev, 7)
    assert not np.isnan(got_many).any()
    np.testing.assert_allclose(got_many, got_few, rtol=2e-2, atol=4e-3)
    # sampled rows against the oracle (host copy of the whole cache)
    cache = dev.cache.cpu().numpy()
    scale = dev.scale.cpu().numpy()
    kw = oracle_layout_kwargs(bt)
    pick = np.random.default_rng(0)
    for b in pick.choice(bt.decoding_batches, size=3, replace=False):
        for h in pick.choice(bt.num_heads, size=2, replace=False):
            o, _, _ = oracle.decode_partial(q[b:], cache, scale, bt.cachestarts[b:], 0, int(h), 0, int(bt.kv_lens[b]),
                                            bt.num_heads, bt.num_kv_heads, bt.head_dim, bt.attn_scale, 0,
                                            bt.page_size, **kw)
            assert_attention_close(got_many[b, h], o, "%s b=%d h=%d" % (name, b, h))
