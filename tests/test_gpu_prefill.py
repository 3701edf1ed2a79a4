"""GPU parity of the multi-query-token (chunked prefill) kernel against the CPU
oracle, through the C ABI.  Tolerance: |got - ref| <= 2e-3 + 1e-2 * |ref|."""
import numpy as np
import pytest
import torch

from conftest import (assert_attention_close, host_cache, make_prefill_mask, oracle_append_step, oracle_decode,
                      oracle_fill_history, oracle_prefill, oracle_prefill_ex)

pytestmark = pytest.mark.gpu


def make_case(pkg, oracle, seed, **kw):
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


def run_prefill(pkg, dev, is_causal=None, **extra):
    bt = dev.bt
    dev.output.fill_(float("nan"))
    pkg.ops.prefill_attention(dev.query, dev.output, dev.cache, dev.scale, dev.seqstarts, dev.kvstarts,
                              dev.cachestarts, attn_scale=bt.attn_scale,
                              is_causal=bt.is_causal if is_causal is None else is_causal, batch=bt.batch,
                              decoding_batches=bt.decoding_batches, max_seqlen=bt.max_seqlen, max_kvlen=bt.max_kvlen,
                              layer_idx=bt.layer_idx, num_heads=bt.num_heads, num_kv_heads=bt.num_kv_heads,
                              head_dim=bt.head_dim, **dev.layout_kwargs(), **extra)
    torch.cuda.synchronize()
    return dev.output.float().cpu().numpy()


@pytest.mark.parametrize("cache_mode", [0, 1])
@pytest.mark.parametrize("shape", [(8, 2, 128), (4, 4, 128), (12, 2, 128), (8, 8, 64), (16, 2, 64), (2, 1, 128), (16, 1, 128),
                                   (8, 2, 256), (4, 4, 256), (16, 1, 256), (8, 2, 96), (6, 6, 96), (12, 2, 96),
                                   # multi-query models: the query heads of one kv head fill most of a workgroup's columns
                                   (48, 1, 128), (71, 1, 64), (24, 1, 256)])
def test_prefill_matches_oracle(pkg, oracle, shape, cache_mode):
    hq, hkv, d = shape
    bt, dev, q, cache, scale = make_case(pkg, oracle, 300 + hq + d, num_heads=hq, num_kv_heads=hkv, head_dim=d,
                                         cache_mode=cache_mode, dec_kv_lens=[33, 140],
                                         prefill_q_lens=[70, 7, 1, 129, 200], prefill_prior=[130, 0, 50, 127, 0],
                                         outliers=True)
    ref = oracle_prefill(oracle, bt, q, cache, scale)
    got = run_prefill(pkg, dev)
    n_dec = bt.decoding_batches
    assert np.isnan(got[:n_dec]).all()  # the prefill stage leaves decode rows alone
    assert_attention_close(got[n_dec:], ref[n_dec:], "prefill %s mode %d" % (shape, cache_mode))


@pytest.mark.parametrize("shape", [(32, 8, 128), (8, 1, 128), (8, 8, 64), (64, 8, 128), (16, 8, 256), (8, 4, 96)])
def test_prefill_short_chunks_over_long_histories(pkg, oracle, shape):
    """A few query tokens per sequence over many kv tiles: most waves of a workgroup have no live column."""
    hq, hkv, d = shape
    bt, dev, q, cache, scale = make_case(pkg, oracle, 340 + hq + d, num_heads=hq, num_kv_heads=hkv, head_dim=d,
                                         cache_mode=1, dec_kv_lens=[],
                                         prefill_q_lens=[2, 4, 8, 16, 3, 1], prefill_prior=[1500, 700, 900, 33, 2047, 640],
                                         outliers=True)
    ref = oracle_prefill(oracle, bt, q, cache, scale)
    got = run_prefill(pkg, dev)
    assert_attention_close(got, ref, "short chunks %s" % (shape,))


@pytest.mark.parametrize("is_causal", [True, False])
@pytest.mark.parametrize("cache_mode", [0, 1])
@pytest.mark.parametrize("shape,q_lens", [((32, 8, 128), [4, 1, 8, 3, 2, 8, 5]), ((8, 8, 64), [16, 5, 32, 1, 31, 2, 9]),
                                          ((8, 1, 128), [4, 2, 1, 3, 4, 1, 2]), ((16, 2, 64), [3, 4, 1, 2, 4, 4, 1]),
                                          ((4, 4, 128), [32, 7, 20, 1, 2, 30, 16]), ((12, 3, 128), [8, 2, 1, 7, 3, 8, 4]),
                                          # up to 16 columns at head_dim 128: the 16-column form of the kernel
                                          ((32, 8, 128), [4, 1, 2, 3, 4, 4, 1]), ((8, 8, 128), [16, 3, 1, 9, 15, 2, 16]),
                                          ((16, 2, 128), [2, 1, 2, 2, 1, 2, 2])])
def test_prefill_short_chunks_on_the_decode_kernel(pkg, oracle, shape, q_lens, cache_mode, is_causal):
    """With the workspace of prefill_workspace_size() a batch whose (query position, query head) pairs per kv head fit
    32 columns runs on the decode step's MFMA kernel over token ranges: same results as the oracle and as the tile
    kernel, pieces in the workspace, rows of the decode sequences untouched."""
    hq, hkv, d = shape
    bt, dev, q, cache, scale = make_case(pkg, oracle, 360 + hq + d, num_heads=hq, num_kv_heads=hkv, head_dim=d,
                                         cache_mode=cache_mode, dec_kv_lens=[33, 140],
                                         prefill_q_lens=q_lens, prefill_prior=[1500, 0, 900, 33, 2047, 126, 640],
                                         outliers=True)
    bt.is_causal = is_causal
    ref = oracle_prefill(oracle, bt, q, cache, scale)
    ws_bytes = pkg.ops.prefill_workspace_size(bt.batch, bt.decoding_batches, bt.max_seqlen, bt.max_kvlen, hq, hkv, d)
    assert ws_bytes > 0
    ws = torch.full((ws_bytes // 4,), float("nan"), dtype=torch.float32, device="cuda")
    got = run_prefill(pkg, dev, is_causal=is_causal, workspace=ws)
    assert_attention_close(got[bt.decoding_batches:], ref[bt.decoding_batches:], "chunks on the decode kernel %s" % (shape,))
    assert np.isnan(got[:bt.decoding_batches]).all()       # the decode sequences' rows are not this stage's
    assert not torch.isnan(ws).all()                       # pieces were written: the decode kernel ran
    tile = run_prefill(pkg, dev, is_causal=is_causal)      # no workspace: the tile kernel
    assert_attention_close(tile[bt.decoding_batches:], ref[bt.decoding_batches:], "tile kernel %s" % (shape,))
    # a workspace that is too small is not an error: the tile kernel runs
    small = torch.full((16,), float("nan"), dtype=torch.float32, device="cuda")
    got2 = run_prefill(pkg, dev, is_causal=is_causal, workspace=small)
    assert_attention_close(got2[bt.decoding_batches:], ref[bt.decoding_batches:], "small workspace %s" % (shape,))
    assert torch.isnan(small).all()


def test_prefill_short_chunks_with_an_understated_max_seqlen(pkg, oracle):
    """The short-chunk route computes max_seqlen query positions per sequence.  A max_seqlen that the row count proves
    too small keeps the batch on the tile kernel (every row right, no piece written); one that the row count cannot
    expose leaves no row silently unwritten: the rows beyond it come back as NaN, every other row is right."""
    hq, hkv, d = 32, 8, 128

    def run(q_lens, claimed):
        bt, dev, q, cache, scale = make_case(pkg, oracle, 377, num_heads=hq, num_kv_heads=hkv, head_dim=d, cache_mode=1,
                                             dec_kv_lens=[33], prefill_q_lens=q_lens,
                                             prefill_prior=[1500, 0, 900, 33, 640][:len(q_lens)], outliers=True)
        ref = oracle_prefill(oracle, bt, q, cache, scale)
        ws_bytes = pkg.ops.prefill_workspace_size(bt.batch, 1, claimed, bt.max_kvlen, hq, hkv, d)
        assert ws_bytes > 0
        ws = torch.full((ws_bytes // 4,), float("nan"), dtype=torch.float32, device="cuda")
        dev.output.fill_(3.0)
        pkg.ops.prefill_attention(dev.query, dev.output, dev.cache, dev.scale, dev.seqstarts, dev.kvstarts, dev.cachestarts,
                                  attn_scale=bt.attn_scale, is_causal=True, batch=bt.batch, decoding_batches=1,
                                  max_seqlen=claimed, max_kvlen=bt.max_kvlen, layer_idx=0, num_heads=hq, num_kv_heads=hkv,
                                  head_dim=d, workspace=ws, **dev.layout_kwargs())
        torch.cuda.synchronize()
        return bt, dev.output.float().cpu().numpy(), ref, ws

    # 17 rows in 4 sequences: more than 4 * 4, so the hint cannot be right -> the tile kernel
    bt, got, ref, ws = run([4, 2, 8, 3], claimed=4)
    assert_attention_close(got[1:], ref[1:], "tile kernel on a provably wrong hint")
    assert torch.isnan(ws).all()
    # 16 rows in 5 sequences: 4 per sequence is possible, but the third has 8 -> its rows 4..7 are NaN
    bt, got, ref, ws = run([4, 2, 8, 1, 1], claimed=4)
    assert not torch.isnan(ws).all()
    first = int(bt.seqstarts[3])
    lost = np.zeros(got.shape[0], dtype=bool)
    lost[first + 4:first + 8] = True
    lost[0] = True  # the decode sequence's row is not this stage's
    assert np.isnan(got[first + 4:first + 8]).all()
    assert_attention_close(got[~lost], ref[~lost], "rows within the claimed max_seqlen")
    assert (got[0] == 3.0).all()


def test_prefill_workspace_size_is_zero_for_other_batches(pkg, hip_lib):
    f = pkg.ops.prefill_workspace_size
    assert f(8, 2, 8, 4096, 32, 8, 128, 256) > 0            # 8 positions x 4 query heads per kv head = 32 columns
    assert f(8, 2, 9, 4096, 32, 8, 128, 256) == 0           # 36 columns
    assert f(8, 8, 8, 4096, 32, 8, 128, 256) == 0           # no prefill sequence
    assert f(8, 2, 8, 4096, 32, 8, 96, 256) == 0 and f(8, 2, 8, 4096, 32, 8, 256, 256) == 0
    assert f(8, 2, 32, 4096, 8, 8, 64, 256) > 0


@pytest.mark.parametrize("n_seq,is_causal", [(150, True), (150, False), (1100, True)])
def test_prefill_many_sequences_every_tile_once(pkg, oracle, n_seq, is_causal):
    """The kernel numbers the batch's query tiles in the order of falling cost and every workgroup looks its own
    tile up: with more than 64 sequences a lane holds several of them, beyond 1024 the plain order applies.  Every
    output row must be written exactly once (rows left NaN or wrong show a tile that was skipped or mixed up);
    sequences with a short prior context and many rows sit next to long ones with one row."""
    rng0 = np.random.default_rng(n_seq)
    big = n_seq <= 200
    q_lens = rng0.integers(1, 150 if big else 4, size=n_seq)
    prior = rng0.integers(0, 300 if big else 40, size=n_seq)
    q_lens[::7] = 1
    prior[::7] = rng0.integers(200 if big else 30, 400 if big else 60, size=len(prior[::7]))
    bt, dev, q, cache, scale = make_case(pkg, oracle, 360 + n_seq, num_heads=4, num_kv_heads=2, head_dim=64,
                                         cache_mode=1, dec_kv_lens=[5], prefill_q_lens=q_lens.tolist(),
                                         prefill_prior=prior.tolist(), is_causal=is_causal)
    ref = oracle_prefill(oracle, bt, q, cache, scale)
    got = run_prefill(pkg, dev)
    assert np.isnan(got[:1]).all() and not np.isnan(got[1:]).any()
    assert_attention_close(got[1:], ref[1:], "many sequences %d" % n_seq)
    # the row count only sizes the launch: without it (0 = unknown) the rows are the same bit for bit
    got0 = run_prefill(pkg, dev, prefill_query_rows=0)
    assert np.array_equal(got0[1:].view(np.uint32), got[1:].view(np.uint32))


def test_prefill_non_causal_and_single_row_equals_decode(pkg, oracle):
    bt, dev, q, cache, scale = make_case(pkg, oracle, 320, num_heads=8, num_kv_heads=2, head_dim=128, cache_mode=1,
                                         dec_kv_lens=[], prefill_q_lens=[1, 65], prefill_prior=[300, 10],
                                         is_causal=False)
    ref = oracle_prefill(oracle, bt, q, cache, scale)
    got = run_prefill(pkg, dev)
    assert_attention_close(got, ref, "non-causal")
    # sequence 0 has one query row: the decode kernel over the same cache gives the same answer
    bt2, _ = pkg.workloads.custom_batch(320, num_heads=8, num_kv_heads=2, head_dim=128, cache_mode=1, dec_kv_lens=[301])
    dev2 = pkg.harness.DeviceBatch(bt2)
    dev2.cache = dev.cache
    dev2.scale = dev.scale
    dev2.cachestarts = dev.cachestarts[0:1].contiguous()
    bt2.cachestarts_stride_b = bt.cachestarts_stride_b
    bt2.layout = bt.layout
    dev2.set_step_inputs(q[0:1], q[0:1, :2], q[0:1, :2])
    dev2.decode_only(num_token_ranges=3)
    torch.cuda.synchronize()
    np.testing.assert_allclose(dev2.output.float().cpu().numpy()[0], got[0], rtol=1e-2, atol=2e-3)


def test_prefill_kv_shorter_than_query(pkg, oracle):
    """kvlen < qlen under the bottom-right mask: the first rows see no key and come out zero."""
    bt, dev, q, cache, scale = make_case(pkg, oracle, 330, num_heads=4, num_kv_heads=2, head_dim=128, cache_mode=0,
                                         dec_kv_lens=[], prefill_q_lens=[40], prefill_prior=[0])
    bt.kv_lens[0] = 25
    bt.kvstarts = np.array([0, 25], dtype=np.int64)
    dev.kvstarts.copy_(torch.from_numpy(bt.kvstarts))
    ref = oracle_prefill(oracle, bt, q, cache, scale)
    got = run_prefill(pkg, dev)
    assert (ref[:15] == 0).all() and (got[:15] == 0).all()
    assert_attention_close(got, ref, "kv shorter than q")


def test_prefill_full_size_c5(pkg, oracle):
    """The C5 prefill part at full size: sampled rows against the oracle."""
    bt, rng = pkg.workloads.make_batch("C5")
    dev = pkg.harness.DeviceBatch(bt)
    dev.fill_history_random_bytes(seed=5)
    q, k, v = pkg.workloads.step_inputs(bt, rng)
    dev.set_step_inputs(q, k, v)
    got = run_prefill(pkg, dev)
    n_dec = bt.decoding_batches
    assert not np.isnan(got[n_dec:]).any()
    cache = dev.cache.cpu().numpy()
    scale = dev.scale.cpu().numpy()
    from conftest import oracle_layout_kwargs
    kw = oracle_layout_kwargs(bt)
    pick = np.random.default_rng(1)
    for b in pick.choice(np.arange(n_dec, bt.batch), size=4, replace=False):
        qlen, kvlen = int(bt.q_lens[b]), int(bt.kv_lens[b])
        for i in (0, qlen // 2, qlen - 1):
            row = int(bt.seqstarts[b]) + i
            lim = i + 1 + kvlen - qlen
            for h in pick.choice(bt.num_heads, size=2, replace=False):
                o, _, _ = oracle.decode_partial(q[row:], cache, scale, bt.cachestarts[b:], 0, int(h), 0, lim,
                                                bt.num_heads, bt.num_kv_heads, bt.head_dim, bt.attn_scale, 0,
                                                bt.page_size, **kw)
                assert_attention_close(got[row, h], o, "C5 b=%d row=%d h=%d" % (b, i, h))


@pytest.mark.parametrize("is_causal", [True, False])
@pytest.mark.parametrize("shape,cache_mode,per_head", [((8, 2, 128), 1, True), ((4, 4, 64), 0, False), ((8, 8, 128), 1, False),
                                                       ((8, 2, 256), 1, True), ((6, 2, 96), 0, False)])
def test_prefill_mask_and_alibi_match_oracle(pkg, oracle, shape, cache_mode, per_head, is_causal):
    """The optional inputs of the prefill stage: additive attn_mask (2-d and per-head 3-d) and alibi slopes."""
    hq, hkv, d = shape
    bt, dev, q, cache, scale = make_case(pkg, oracle, 700 + hq + d, num_heads=hq, num_kv_heads=hkv, head_dim=d,
                                         cache_mode=cache_mode, dec_kv_lens=[33], prefill_q_lens=[70, 7, 1, 129],
                                         prefill_prior=[130, 0, 50, 127], is_causal=is_causal)
    rng = np.random.default_rng(11)
    mask, ms, mh = make_prefill_mask(bt, rng, per_head)
    slopes = (2.0 ** -np.arange(1, hq + 1)).astype(np.float32)
    d_mask = torch.from_numpy(mask).cuda()
    d_slopes = torch.from_numpy(slopes).cuda()
    n_dec = bt.decoding_batches
    for use_mask, use_alibi in ((True, False), (False, True), (True, True)):
        kw_o = dict(attn_mask=mask, mask_stride_s=ms, mask_stride_h=mh) if use_mask else {}
        kw_d = dict(attn_mask=d_mask, mask_stride_s=ms, mask_stride_h=mh) if use_mask else {}
        if use_alibi:
            kw_o["alibi_slopes"] = slopes
            kw_d["alibi_slopes"] = d_slopes
        ref = oracle_prefill_ex(oracle, bt, q, cache, scale, **kw_o)
        got = run_prefill(pkg, dev, **kw_d)
        assert_attention_close(got[n_dec:], ref[n_dec:], "prefill mask=%s alibi=%s %s" % (use_mask, use_alibi, shape))


@pytest.mark.parametrize("shape", [(8, 2, 128), (4, 4, 64), (32, 8, 128), (8, 2, 256), (6, 3, 96)])
def test_prefill_from_current_key_value(pkg, oracle, shape):
    """enable_cache_prefill = false: attention over the step's own fp16 K/V rows, no cache read."""
    hq, hkv, d = shape
    bt, rng = pkg.workloads.custom_batch(800 + hq, num_heads=hq, num_kv_heads=hkv, head_dim=d, cache_mode=0,
                                         dec_kv_lens=[5, 9], prefill_q_lens=[70, 7, 1, 129, 300], prefill_prior=[0] * 5,
                                         outliers=True)
    dev = pkg.harness.DeviceBatch(bt)
    q, k, v = pkg.workloads.step_inputs(bt, rng)
    dev.set_step_inputs(q, k, v)
    dev.cache.fill_(77)  # must not be read
    cache, scale = host_cache(bt)
    ref = oracle_prefill_ex(oracle, bt, q, cache, scale, current_key=k, current_value=v)
    got = run_prefill(pkg, dev, current_key=dev.new_key, current_value=dev.new_value)
    n_dec = bt.decoding_batches
    assert np.isnan(got[:n_dec]).all()
    assert_attention_close(got[n_dec:], ref[n_dec:], "prefill from current K/V %s" % (shape,))
    # the operator class with enable_cache_prefill = false takes the same path
    op = dev.make_operator(enable_cache_prefill=False)
    dev.output.fill_(float("nan"))
    assert op.forward_prefill() == 0
    torch.cuda.synchronize()
    assert_attention_close(dev.output.float().cpu().numpy()[n_dec:], ref[n_dec:], "operator, enable_cache_prefill=false")


def test_prefill_output_rows_aligned_to_8_bytes_only(pkg, oracle):
    """The C ABI admits output rows that are 8-byte aligned.  The tile kernel writes whole rows in 16-byte pieces where
    the rows allow it and in 8-byte pieces otherwise: same values, nothing written outside the rows."""
    bt, dev, q, cache, scale = make_case(pkg, oracle, 330, num_heads=8, num_kv_heads=2, head_dim=128, cache_mode=1,
                                         dec_kv_lens=[], prefill_q_lens=[70, 5, 129], prefill_prior=[130, 0, 300])
    ref = oracle_prefill(oracle, bt, q, cache, scale)
    got = run_prefill(pkg, dev)
    assert_attention_close(got, ref, "16-byte rows")
    n = dev.output.numel()
    buf = torch.full((n + 8,), float("nan"), dtype=torch.float16, device="cuda")
    out = buf[4:4 + n].view(dev.output.shape)
    assert out.data_ptr() % 16 == 8
    keep = dev.output
    dev.output = out
    try:
        got8 = run_prefill(pkg, dev)
    finally:
        dev.output = keep
    np.testing.assert_array_equal(got8, got)
    assert torch.isnan(buf[:4]).all() and torch.isnan(buf[4 + n:]).all()
