"""Synthetic dynamic batches for the int8-KV attention path (numpy only).

Shapes and seeds of the five benchmark configurations, the cache layout
[layer, K/V, token, kv_head, head_dim] with its strides, and the index arrays
(seqstarts / kvstarts / cachestarts / start_pos) in both cache modes.  Values
are drawn with numpy.random.default_rng(seed): fp16 = standard_normal(float32)
cast to float16, with ceil(0.02 * D) "outlier" channels per kv head scaled x10
where a configuration asks for them.
"""
import math
from dataclasses import dataclass, field

import numpy as np

PAGE = 128


LAYOUTS = ("l2shd", "sl2hd", "lhs2d")


@dataclass
class CacheLayout:
    """int8 cache and fp16 scale (one scale per 8 channels: the same shape with D/8 last) in one of three orders
    of (layer L, K/V plane 2, token S, kv head H, channel D); the operator only sees the four strides.

    "l2shd"  [L, 2, S, H, D]  the order the benchmark configurations name
    "sl2hd"  [S, L, 2, H, D]  a token's rows of every layer together
    "lhs2d"  [L, H, S, 2, D]  a kv head's tokens together, K and V rows of a token side by side
    (the second and third are the two the reference's header documents, multi_head_cache_attention.h:145-146)."""
    num_layer: int
    pool_tokens: int
    num_kv_heads: int
    head_dim: int
    kind: str = "l2shd"

    def _dims(self):
        return dict(L=self.num_layer, K=2, S=self.pool_tokens, H=self.num_kv_heads, D=self.head_dim)

    def _order(self):
        return {"l2shd": "LKSHD", "sl2hd": "SLKHD", "lhs2d": "LHSKD"}[self.kind]

    def _stride(self, axis):
        dims, order = self._dims(), self._order()
        n = 1
        for ax in order[order.index(axis) + 1:]:
            n *= dims[ax]
        return n

    @property
    def stride_s(self):
        return self._stride("S")

    @property
    def stride_h(self):
        return self._stride("H")

    @property
    def stride_kv(self):
        return self._stride("K")

    @property
    def stride_l(self):
        return self._stride("L")

    @property
    def cache_elems(self):
        return self.num_layer * 2 * self.pool_tokens * self.num_kv_heads * self.head_dim

    def cache_shape(self):
        dims = self._dims()
        return tuple(dims[ax] for ax in self._order())

    def scale_shape(self):
        return self.cache_shape()[:-1] + (self.head_dim // 8,)

    def canonical(self, arr):
        """A view of a cache or scale array (numpy or torch) of this layout with its axes as [L, 2, S, H, D]."""
        order = self._order()
        axes = tuple(order.index(ax) for ax in "LKSHD")
        return np.transpose(arr, axes) if isinstance(arr, np.ndarray) else arr.permute(axes)


@dataclass
class Batch:
    name: str
    seed: int
    num_heads: int
    num_kv_heads: int
    head_dim: int
    cache_mode: int
    decoding_batches: int
    q_lens: np.ndarray   # new tokens per sequence (decode sequences first, 1 each)
    kv_lens: np.ndarray  # kv length per sequence after this step's append
    outliers: bool
    num_layer: int = 1
    layer_idx: int = 0
    is_causal: bool = True
    # filled by finalize()
    seqstarts: np.ndarray = field(default=None, repr=False)
    kvstarts: np.ndarray = field(default=None, repr=False)
    start_pos: np.ndarray = field(default=None, repr=False)
    cachestarts: np.ndarray = field(default=None, repr=False)
    cachestarts_stride_b: int = 0
    layout_kind: str = "l2shd"
    layout: CacheLayout = field(default=None, repr=False)
    outlier_channels: np.ndarray = field(default=None, repr=False)  # [KVH, n_out]

    @property
    def batch(self):
        return len(self.q_lens)

    @property
    def page_size(self):
        return PAGE if self.cache_mode == 1 else 0

    @property
    def max_seqlen(self):
        return int(self.q_lens.max()) if len(self.q_lens) else 0

    @property
    def max_kvlen(self):
        return int(self.kv_lens.max()) if len(self.kv_lens) else 0

    @property
    def attn_scale(self):
        return float(np.float32(1.0 / np.sqrt(np.float32(self.head_dim))))

    @property
    def decode_kv_tokens(self):
        return int(self.kv_lens[:self.decoding_batches].sum())

    def decode_algorithmic_bytes(self):
        """int8 K + int8 V + their fp16 group scales, plus fp16 Q read and O write."""
        d = self.head_dim
        per_token_head = 2 * d + 2 * (d // 8) * 2
        return (self.decode_kv_tokens * self.num_kv_heads * per_token_head
                + 2 * self.decoding_batches * self.num_heads * d * 2)

    def append_algorithmic_bytes(self):
        d = self.head_dim
        return int(self.q_lens.sum()) * self.num_kv_heads * (2 * d * 2 + 2 * d + 2 * (d // 8) * 2)

    def prefill_flops(self):
        tot = 0
        for b in range(self.decoding_batches, self.batch):
            q = int(self.q_lens[b])
            prior = int(self.kv_lens[b]) - q
            tot += q * prior + q * (q + 1) // 2
        return 4 * self.num_heads * self.head_dim * tot


def finalize(bt: Batch, rng: np.random.Generator, pool_tokens_at_least: int = 0):
    """Derives the index arrays and places the sequences in a token pool."""
    B = bt.batch
    bt.seqstarts = np.concatenate([[0], np.cumsum(bt.q_lens)]).astype(np.int64)
    bt.kvstarts = np.concatenate([[0], np.cumsum(bt.kv_lens)]).astype(np.int64)
    bt.start_pos = (bt.kv_lens - bt.q_lens).astype(np.int64)
    if bt.cache_mode == 1:
        pages = (bt.kv_lens + PAGE - 1) // PAGE
        n_pages = int(pages.sum())
        pool_pages = max(n_pages + 3, -(-pool_tokens_at_least // PAGE))  # a few pages nobody owns (canaries)
        perm = rng.permutation(pool_pages)[:n_pages]
        max_p = int(pages.max()) if B else 1
        table = np.zeros((B, max_p), dtype=np.int64)
        k = 0
        for b in range(B):
            n = int(pages[b])
            table[b, :n] = perm[k:k + n].astype(np.int64) * PAGE
            k += n
        bt.cachestarts = table
        bt.cachestarts_stride_b = max_p
        pool_tokens = pool_pages * PAGE
    else:
        # contiguous runs, sequences placed in shuffled order with small gaps
        order = rng.permutation(B)
        starts = np.zeros(B, dtype=np.int64)
        cur = 5
        for b in order:
            starts[b] = cur
            cur += int(bt.kv_lens[b]) + int(rng.integers(0, 4))
        bt.cachestarts = starts
        bt.cachestarts_stride_b = 1
        pool_tokens = max(cur + 3, pool_tokens_at_least)
    bt.layout = CacheLayout(bt.num_layer, int(pool_tokens), bt.num_kv_heads, bt.head_dim, bt.layout_kind)
    n_out = int(math.ceil(0.02 * bt.head_dim)) if bt.outliers else 0
    if n_out:
        bt.outlier_channels = np.stack(
            [rng.choice(bt.head_dim, size=n_out, replace=False) for _ in range(bt.num_kv_heads)])
    else:
        bt.outlier_channels = np.zeros((bt.num_kv_heads, 0), dtype=np.int64)
    return bt


def draw_fp16(bt: Batch, rng, n_rows, heads, for_query=False):
    """[n_rows, heads, D] float16; outlier channels (per kv head) scaled x10."""
    x = rng.standard_normal((n_rows, heads, bt.head_dim), dtype=np.float32)
    if bt.outlier_channels.shape[1]:
        rep = heads // bt.num_kv_heads
        for kvh in range(bt.num_kv_heads):
            ch = bt.outlier_channels[kvh]
            x[:, kvh * rep:(kvh + 1) * rep, ch] *= np.float32(10.0)
    return x.astype(np.float16)


def _loguniform_int(rng, lo, hi, n):
    return np.floor(np.exp(rng.uniform(np.log(lo), np.log(hi), n))).astype(np.int64)


def make_batch(name: str, scale: float = 1.0, layout: str = "l2shd", num_layer: int = 1) -> Batch:
    """The five benchmark configurations; `scale` < 1 shrinks sequence lengths
    (and keeps every other property) so that CPU checks finish quickly."""
    def sc(v):
        return np.maximum(1, np.floor(np.asarray(v, dtype=np.float64) * scale)).astype(np.int64)

    if name == "C1":
        seed = 1001
        rng = np.random.default_rng(seed)
        kv = sc(rng.integers(128, 513, 4))
        bt = Batch(name, seed, 8, 8, 64, 0, 4, np.ones(4, np.int64), kv, outliers=False)
    elif name == "C2":
        seed = 1002
        rng = np.random.default_rng(seed)
        kv = sc(rng.integers(512, 4097, 64))
        bt = Batch(name, seed, 32, 32, 128, 0, 64, np.ones(64, np.int64), kv, outliers=True)
    elif name in ("C3", "C3m0"):
        seed = 1003
        rng = np.random.default_rng(seed)
        kv = sc(_loguniform_int(rng, 1024, 8192, 128))
        bt = Batch(name, seed, 32, 8, 128, 1 if name == "C3" else 0, 128, np.ones(128, np.int64), kv, outliers=True)
    elif name == "C4":
        seed = 1004
        rng = np.random.default_rng(seed)
        kv = np.clip(np.floor(np.exp(rng.normal(np.log(16384.0), 0.5, 32))), 1024, 32768).astype(np.int64)
        bt = Batch(name, seed, 64, 8, 128, 1, 32, np.ones(32, np.int64), sc(kv), outliers=True)
    elif name == "C5":
        seed = 1005
        rng = np.random.default_rng(seed)
        # draw order: prefill query lengths, prefill prior context, decode kv lengths
        pq = sc(rng.integers(256, 1025, 16))
        prior = np.floor(rng.integers(0, 2049, 16) * scale).astype(np.int64)
        dec_kv = sc(rng.integers(512, 4097, 240))
        q_lens = np.concatenate([np.ones(240, np.int64), pq])
        kv_lens = np.concatenate([dec_kv, prior + pq])
        bt = Batch(name, seed, 32, 8, 128, 1, 240, q_lens, kv_lens, outliers=True)
    else:
        raise KeyError(name)
    bt.layout_kind = layout
    bt.num_layer = num_layer
    return finalize(bt, rng), rng


def custom_batch(seed, num_heads, num_kv_heads, head_dim, cache_mode, dec_kv_lens, prefill_q_lens=(),
                 prefill_prior=(), outliers=False, num_layer=1, layer_idx=0, is_causal=True, layout="l2shd",
                 pool_tokens_at_least=0):
    """Arbitrary ragged batch for tests."""
    rng = np.random.default_rng(seed)
    dec_kv = np.asarray(dec_kv_lens, dtype=np.int64)
    pq = np.asarray(prefill_q_lens, dtype=np.int64)
    pp = np.asarray(prefill_prior, dtype=np.int64)
    q_lens = np.concatenate([np.ones(len(dec_kv), np.int64), pq]).astype(np.int64)
    kv_lens = np.concatenate([dec_kv, pp + pq]).astype(np.int64)
    bt = Batch("custom", seed, num_heads, num_kv_heads, head_dim, cache_mode, len(dec_kv), q_lens, kv_lens,
               outliers=outliers, num_layer=num_layer, layer_idx=layer_idx, is_causal=is_causal, layout_kind=layout)
    return finalize(bt, rng, pool_tokens_at_least), rng


def history_chunks(bt: Batch, rng, max_rows=1 << 16):
    """Yields (seq index, first position, K rows, V rows) covering positions
    [0, start_pos[b]) of every sequence: the context already in the cache."""
    for b in range(bt.batch):
        n = int(bt.start_pos[b])
        pos = 0
        while pos < n:
            m = min(max_rows, n - pos)
            yield b, pos, draw_fp16(bt, rng, m, bt.num_kv_heads), draw_fp16(bt, rng, m, bt.num_kv_heads)
            pos += m


def step_inputs(bt: Batch, rng):
    """Q, new K, new V of this step: [sum(q_lens), heads, D] float16 each."""
    n = int(bt.q_lens.sum())
    q = draw_fp16(bt, rng, n, bt.num_heads, for_query=True)
    k = draw_fp16(bt, rng, n, bt.num_kv_heads)
    v = draw_fp16(bt, rng, n, bt.num_kv_heads)
    return q, k, v
