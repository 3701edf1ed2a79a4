import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

import __graft_entry__ as entry  # noqa: E402


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(scope="session")
def pkg():
    return entry.load_package()


@pytest.fixture(scope="session")
def oracle():
    return entry.load_oracle()


@pytest.fixture(scope="session")
def hip_lib(pkg):
    """The built C-ABI library; built on demand only when nothing is there."""
    if not os.path.exists(pkg._lib.LIB_PATH):
        pkg.build.build(force=False)
    return pkg._lib.lib()


def oracle_layout_kwargs(bt):
    lay = bt.layout
    return dict(cache_stride_s=lay.stride_s, cache_stride_l=lay.stride_l, cache_stride_h=lay.stride_h,
                cache_stride_kv=lay.stride_kv, cachestarts_stride_b=bt.cachestarts_stride_b)


def host_cache(bt, canary=None):
    cache = np.zeros(bt.layout.cache_shape(), dtype=np.int8)
    scale = np.zeros(bt.layout.scale_shape(), dtype=np.float16)
    if canary is not None:
        cache[...] = canary[0]
        scale[...] = np.float16(canary[1])
    return cache, scale


def oracle_fill_history(oracle, pkg, bt, rng, cache, scale, chunks=None):
    """Quantise the prior context of every sequence into the host cache; returns the chunks."""
    out = []
    for b, pos, k_rows, v_rows in (chunks if chunks is not None else pkg.workloads.history_chunks(bt, rng)):
        oracle.kv_cache_quantize(k_rows, v_rows, np.array([0, len(k_rows)]), bt.cachestarts[b:b + 1],
                                 np.array([pos]), bt.layer_idx, bt.num_kv_heads, bt.head_dim, bt.page_size,
                                 cache=cache, scale=scale, **oracle_layout_kwargs(bt))
        out.append((b, pos, k_rows, v_rows))
    return out


def oracle_append_step(oracle, bt, k, v, cache, scale):
    oracle.kv_cache_quantize(k, v, bt.seqstarts, bt.cachestarts, bt.start_pos, bt.layer_idx, bt.num_kv_heads,
                             bt.head_dim, bt.page_size, cache=cache, scale=scale, **oracle_layout_kwargs(bt))


def oracle_decode(oracle, bt, q, cache, scale, **kw):
    return oracle.decode_attention(q, cache, scale, bt.cachestarts, bt.kvstarts, bt.decoding_batches, bt.num_heads,
                                   bt.num_kv_heads, bt.head_dim, bt.attn_scale, bt.layer_idx, bt.page_size,
                                   **oracle_layout_kwargs(bt), **kw)


def oracle_prefill(oracle, bt, q, cache, scale):
    return oracle.prefill_attention(q, cache, scale, bt.seqstarts, bt.kvstarts, bt.cachestarts, bt.batch,
                                    bt.decoding_batches, bt.is_causal, bt.num_heads, bt.num_kv_heads, bt.head_dim,
                                    bt.attn_scale, bt.layer_idx, bt.page_size, **oracle_layout_kwargs(bt))


def oracle_prefill_ex(oracle, bt, q, cache, scale, **extra):
    return oracle.prefill_attention_ex(q, cache, scale, bt.seqstarts, bt.kvstarts, bt.cachestarts, bt.batch,
                                       bt.decoding_batches, bt.is_causal, bt.num_heads, bt.num_kv_heads, bt.head_dim,
                                       bt.attn_scale, bt.layer_idx, bt.page_size, **oracle_layout_kwargs(bt), **extra)


def make_prefill_mask(bt, rng, per_head):
    """Additive fp16 attn_mask in the reference's dynamic-batch layout: (rows, aligned(kv columns, 8)) or
    (heads, rows, aligned(kv columns, 8)); columns are absolute kv-stream positions (kvstarts)."""
    rows = int(bt.seqstarts[-1])
    cols = (int(bt.kvstarts[-1]) + 7) // 8 * 8
    shape = (bt.num_heads, rows, cols) if per_head else (rows, cols)
    m = (rng.standard_normal(shape) * 2.0).astype(np.float16)
    m[rng.random(shape) < 0.1] = np.float16(-60000.0)  # some hard-masked entries
    return m, cols, (rows * cols if per_head else 0)


ATOL = 2e-3  # attention output tolerance against the fp32 dequantised reference:
RTOL = 1e-2  # |got - ref| <= ATOL + RTOL * |ref|


def assert_attention_close(got, ref, what=""):
    got = np.asarray(got, dtype=np.float32)
    ref = np.asarray(ref, dtype=np.float32)
    err = np.abs(got - ref)
    tol = ATOL + RTOL * np.abs(ref)
    bad = err > tol
    if bad.any():
        idx = np.unravel_index(np.argmax(err - tol), err.shape)
        raise AssertionError("%s: %d of %d outside tolerance; worst at %s: got %g ref %g (err %g, tol %g)" % (
            what, int(bad.sum()), bad.size, idx, got[idx], ref[idx], err[idx], tol[idx]))
    return float(err.max())
