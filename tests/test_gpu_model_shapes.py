"""forward() of the operator on batches shaped like the models the reference serves (grouped-query, multi-query, odd
per-rank head counts, head_dim 64 / 128 / 256, short prefill chunks beside decode sequences): cache bytes bit-exact,
every output element within |got - ref| <= 2e-3 + 1e-2 |ref| of the oracle, at a few hundred to a few thousand kv
tokens per sequence so that every decode step is split into token ranges."""
import numpy as np
import pytest
import torch

from conftest import assert_attention_close, oracle_decode, oracle_prefill

pytestmark = pytest.mark.gpu

CASES = [
    # (query heads, kv heads, head_dim, cache_mode, decode sequences, prefill chunks (rows range), what)
    (32, 8, 128, 1, 24, None, "Llama-3-8B"),
    (64, 8, 128, 1, 12, None, "Llama-3-70B"),
    (8, 1, 128, 1, 24, None, "Llama-3-70B on eight ranks"),
    (32, 32, 128, 0, 16, None, "Llama-2-7B"),
    (5, 5, 128, 1, 16, None, "40 heads on eight ranks"),
    (48, 1, 128, 1, 12, None, "multi-query, 48 heads"),
    (71, 1, 64, 0, 12, None, "multi-query, 71 heads of 64"),
    (128, 8, 64, 1, 12, None, "16 query heads per kv head of 64"),
    (14, 2, 64, 1, 16, None, "7 query heads per kv head of 64"),
    (8, 1, 256, 1, 16, None, "multi-query, head_dim 256"),
    (16, 8, 256, 0, 12, None, "head_dim 256, two query heads per kv head"),
    (32, 8, 128, 1, 8, (1, 8), "speculative decoding beside decode sequences"),
    (8, 8, 64, 1, 0, (1, 32), "chunks of up to 32 rows, multi-head"),
    (32, 8, 128, 1, 8, (200, 600), "chunked prefill beside decode sequences"),
]


@pytest.mark.parametrize("case", CASES, ids=[c[-1] for c in CASES])
def test_operator_on_model_shaped_batches(pkg, oracle, case):
    hq, hkv, d, mode, n_dec, chunks, what = case
    r = np.random.default_rng(hq * 1000 + hkv * 10 + d)
    dec = r.integers(400, 3000, n_dec).tolist()
    pq, pp = [], []
    if chunks:
        n = 12 if chunks[1] <= 32 else 3
        pq = r.integers(chunks[0], chunks[1] + 1, n).tolist()
        pp = r.integers(0, 2500, n).tolist()
    bt, rng = pkg.workloads.custom_batch(77, num_heads=hq, num_kv_heads=hkv, head_dim=d, cache_mode=mode, dec_kv_lens=dec,
                                         prefill_q_lens=pq, prefill_prior=pp, outliers=True)
    dev = pkg.harness.DeviceBatch(bt)
    dev.fill_history(rng, max_rows=1 << 15)  # through the HIP append kernel; its bytes are checked elsewhere
    q, k, v = pkg.workloads.step_inputs(bt, rng)
    dev.set_step_inputs(q, k, v)
    dev.output.fill_(float("nan"))
    op = dev.make_operator()
    assert op.forward() == 0
    torch.cuda.synchronize()
    cache, scale = dev.cache.cpu().numpy(), dev.scale.cpu().numpy()
    ref = oracle_prefill(oracle, bt, q, cache, scale) if bt.batch > bt.decoding_batches else np.zeros(
        (q.shape[0], hq, d), np.float32)
    if bt.decoding_batches:
        ref[:bt.decoding_batches] = oracle_decode(oracle, bt, q, cache, scale)
    assert_attention_close(dev.output.float().cpu().numpy(), ref, what)
