#!/usr/bin/env python3
"""Writes the golden fixture of configuration C1 (batch 4, 8 q / 8 kv heads, head_dim 64, kv lengths uniform in
[128, 512], seed 1001, contiguous cache): tests/golden/c1_decode_golden.npz.

Everything is computed on the host by the CPU oracle (oracle/pmx_oracle.c): the history and the step's new token
go through its quantise/append, then its decode attention runs over the int8 cache.  The fixture holds
  * the index arrays and SHA-256 digests of the seeded inputs (query, new K/V) -- so that a change of the input
    recipe is told apart from a change of the arithmetic,
  * SHA-256 digests of the whole int8 cache and of the fp16 scales after the append,
  * the int8 bytes and scale bits of the four appended token rows (a readable sample of the digest),
  * the float32 attention output (4, 8, 64).
Run from the repository root:  python tests/golden/make_c1_golden.py
The reference repository holds no vectors for this path and cannot be built or imported here, so these are the
oracle's own results, frozen: a later change of the oracle or of the workload recipe that alters C1 fails
tests/test_golden_c1.py on the CPU, and the HIP path is compared with the frozen file, not with a live oracle."""
import hashlib
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, ROOT)
import __graft_entry__ as entry  # noqa: E402

PATH = os.path.join(HERE, "c1_decode_golden.npz")


def sha(a):
    return hashlib.sha256(np.ascontiguousarray(a).tobytes()).hexdigest()


def compute():
    """C1 through the oracle; returns the dictionary that the fixture stores."""
    pkg, oracle = entry.load_package(), entry.load_oracle()
    bt, rng = pkg.workloads.make_batch("C1")
    lay = bt.layout
    kw = dict(cache_stride_s=lay.stride_s, cache_stride_l=lay.stride_l, cache_stride_h=lay.stride_h,
              cache_stride_kv=lay.stride_kv, cachestarts_stride_b=bt.cachestarts_stride_b)
    cache = np.zeros(lay.cache_shape(), dtype=np.int8)
    scale = np.zeros(lay.scale_shape(), dtype=np.float16)
    for b, pos, k_rows, v_rows in pkg.workloads.history_chunks(bt, rng):
        oracle.kv_cache_quantize(k_rows, v_rows, np.array([0, len(k_rows)]), bt.cachestarts[b:b + 1], np.array([pos]),
                                 bt.layer_idx, bt.num_kv_heads, bt.head_dim, bt.page_size, cache=cache, scale=scale, **kw)
    q, k, v = pkg.workloads.step_inputs(bt, rng)
    oracle.kv_cache_quantize(k, v, bt.seqstarts, bt.cachestarts, bt.start_pos, bt.layer_idx, bt.num_kv_heads,
                             bt.head_dim, bt.page_size, cache=cache, scale=scale, **kw)
    out = oracle.decode_attention(q, cache, scale, bt.cachestarts, bt.kvstarts, bt.decoding_batches, bt.num_heads,
                                  bt.num_kv_heads, bt.head_dim, bt.attn_scale, bt.layer_idx, bt.page_size, **kw)
    rows = (bt.cachestarts + bt.start_pos).astype(np.int64)  # cache rows of the step's four new tokens
    return dict(
        kv_lens=bt.kv_lens.astype(np.int64), cachestarts=bt.cachestarts.astype(np.int64),
        sha_query=sha(q), sha_new_key=sha(k), sha_new_value=sha(v),
        sha_cache=sha(cache), sha_scale=sha(scale.view(np.uint16)),
        appended_k=cache[0, 0, rows].copy(), appended_v=cache[0, 1, rows].copy(),
        appended_k_scale=scale[0, 0, rows].view(np.uint16).copy(), appended_v_scale=scale[0, 1, rows].view(np.uint16).copy(),
        output=np.asarray(out, dtype=np.float32))


if __name__ == "__main__":
    d = compute()
    np.savez_compressed(PATH, **d)
    print("wrote %s (%d bytes): kv_lens %s, cache sha %s..." % (PATH, os.path.getsize(PATH), d["kv_lens"].tolist(), d["sha_cache"][:16]))
