"""Device-side set-up of a synthetic batch and one step through the operator.

Everything that computes goes through ``ops`` (the C ABI); torch only allocates
and copies.  Used by the GPU tests, the smoke check and the benchmark.
"""
import numpy as np
import torch

from . import ops, workloads


class DeviceBatch:
    """Index arrays, cache pool and step inputs of a workloads.Batch on the GPU."""

    def __init__(self, bt: workloads.Batch, device="cuda"):
        self.bt = bt
        self.device = device
        lay = bt.layout
        self.seqstarts = torch.from_numpy(bt.seqstarts).to(device)
        self.kvstarts = torch.from_numpy(bt.kvstarts).to(device)
        self.start_pos = torch.from_numpy(bt.start_pos).to(device)
        self.cachestarts = torch.from_numpy(np.ascontiguousarray(bt.cachestarts)).to(device)
        self.cache = torch.zeros(lay.cache_shape(), dtype=torch.int8, device=device)
        self.scale = torch.zeros(lay.scale_shape(), dtype=torch.float16, device=device)
        self.query = None
        self.new_key = None
        self.new_value = None
        self.output = None

    # ---- common keyword sets -------------------------------------------------
    def layout_kwargs(self):
        bt, lay = self.bt, self.bt.layout
        return dict(cache_mode=bt.cache_mode, page_size=workloads.PAGE if bt.cache_mode == 1 else 0,
                    cache_stride_s=lay.stride_s, cache_stride_l=lay.stride_l, cache_stride_h=lay.stride_h,
                    cache_stride_kv=lay.stride_kv, cachestarts_stride_b=bt.cachestarts_stride_b)

    def fill_canary(self, q=0x5A, s=1.5):
        self.cache.fill_(q)
        self.scale.fill_(s)

    # ---- history: the context already in the cache before this step ----------
    def append_rows(self, b, first_pos, k_rows, v_rows, layer_idx=None):
        """Quantise/append fp16 rows of one sequence at positions first_pos.. (product path)."""
        bt = self.bt
        n = k_rows.shape[0]
        k = torch.from_numpy(k_rows).to(self.device)
        v = torch.from_numpy(v_rows).to(self.device)
        seqstarts = torch.tensor([0, n], dtype=torch.int64, device=self.device)
        start_pos = torch.tensor([first_pos], dtype=torch.int64, device=self.device)
        if bt.cache_mode == 1:
            cachestarts = self.cachestarts[b:b + 1].contiguous()
        else:
            cachestarts = self.cachestarts[b:b + 1].contiguous()
        ops.key_value_cache(k, v, seqstarts, cachestarts, start_pos, self.cache, self.scale,
                            batch=1, max_seqlen=n, num_layer=bt.num_layer,
                            layer_idx=bt.layer_idx if layer_idx is None else layer_idx,
                            num_kv_heads=bt.num_kv_heads, head_dim=bt.head_dim, **self.layout_kwargs())

    def fill_history(self, rng, max_rows=1 << 16):
        for b, pos, k_rows, v_rows in workloads.history_chunks(self.bt, rng, max_rows):
            self.append_rows(b, pos, k_rows, v_rows)
        torch.cuda.synchronize()

    def fill_history_random_bytes(self, seed=0):
        """Fast fill for timing runs: random int8 payload and plausible fp16 scales
        written directly (no fp16 source rows).  Not for parity checks."""
        g = torch.Generator(device=self.device)
        g.manual_seed(seed)
        n = self.cache.numel()
        flat = self.cache.view(-1)
        step = 1 << 28
        for i in range(0, n, step):
            m = min(step, n - i)
            flat[i:i + m] = torch.randint(-127, 128, (m,), dtype=torch.int8, device=self.device, generator=g)
        self.scale.copy_((torch.rand(self.scale.shape, device=self.device, generator=g) * 0.03 + 0.005).to(torch.float16))
        torch.cuda.synchronize()

    def copy_layer(self, src, dst):
        """Layer `dst` of the cache becomes a copy of layer `src` (timing runs over several layers)."""
        lay = self.bt.layout
        lay.canonical(self.cache)[dst].copy_(lay.canonical(self.cache)[src])
        lay.canonical(self.scale)[dst].copy_(lay.canonical(self.scale)[src])

    def set_step_inputs(self, q, k, v):
        self.query = torch.from_numpy(q).to(self.device)
        self.new_key = torch.from_numpy(k).to(self.device)
        self.new_value = torch.from_numpy(v).to(self.device)
        self.output = torch.zeros_like(self.query)

    # ---- the operator ----------------------------------------------------------
    def make_operator(self, specify_decoding_multi_block=1, attn_mask=None, attn_mask_shape=(), **overrides):
        bt = self.bt
        op = ops.DynamicBatchingMultiHeadCacheAttention()
        n_rows = int(bt.q_lens.sum())
        kw = dict(
            query=self.query, query_shape=(n_rows, bt.num_heads, bt.head_dim),
            current_key=self.new_key, current_key_shape=(n_rows, bt.num_kv_heads, bt.head_dim),
            current_value=self.new_value, current_value_shape=(n_rows, bt.num_kv_heads, bt.head_dim),
            attn_mask=attn_mask, attn_mask_shape=attn_mask_shape,
            seqstarts=self.seqstarts, kvstarts=self.kvstarts, cachestarts=self.cachestarts,
            start_pos=self.start_pos, is_causal=bt.is_causal,
            batch=bt.batch, decoding_batches=bt.decoding_batches, max_seqlen=bt.max_seqlen,
            max_kvlen=bt.max_kvlen, layer_idx=bt.layer_idx, num_layer=bt.num_layer,
            num_heads=bt.num_heads, num_kv_heads=bt.num_kv_heads, head_dim=bt.head_dim,
            specify_decoding_multi_block=specify_decoding_multi_block,
            cache=self.cache, scale=self.scale, output=self.output,
            output_shape=(n_rows, bt.num_heads, bt.head_dim))
        kw.update(self.layout_kwargs())
        kw.update(overrides)
        rc = op.heuristic_prepare(**kw)
        if rc != ops.RC_SUCCESS:
            raise ops.PmxError(rc, "heuristic_prepare")
        op.allocate_workspace(self.device)
        return op

    def decode_only(self, num_token_ranges=0, workspace=None, attn_mask=None, mask_stride_s=0, mask_stride_h=0,
                    output=None, stage=0, kernel=0, static_workspace=False, output_stride_s=None, name_only=False,
                    stream=None, layer_idx=None):
        """Decode attention through the flat C entry point (no operator object).  `kernel` requests a
        token-range kernel; `static_workspace` uses the entry point that allocates nothing; `name_only`
        launches nothing and returns the name of the kernel the call would run."""
        bt = self.bt
        plan = ops.decode_plan(bt.decoding_batches, bt.num_heads, bt.num_kv_heads, bt.head_dim, bt.max_kvlen,
                               ranges_hint=num_token_ranges, kernel=kernel)
        if workspace is None and plan.workspace_size > 0 and not static_workspace and not name_only:
            workspace = torch.empty(int(plan.workspace_size), dtype=torch.uint8, device=self.device)
        out = self.output if output is None else output
        r = ops.decode_attention(self.query, out, self.cache, self.scale, self.cachestarts, self.kvstarts,
                                 attn_scale=bt.attn_scale, layer_idx=bt.layer_idx if layer_idx is None else layer_idx,
                                 decoding_batches=bt.decoding_batches, num_heads=bt.num_heads,
                                 num_kv_heads=bt.num_kv_heads, head_dim=bt.head_dim,
                                 num_token_ranges=plan.num_token_ranges, workspace=workspace,
                                 attn_mask=attn_mask, mask_stride_s=mask_stride_s, mask_stride_h=mask_stride_h, stage=stage,
                                 kernel=kernel, static_workspace=static_workspace, output_stride_s=output_stride_s,
                                 name_only=name_only, stream=stream, **self.layout_kwargs())
        if name_only:
            return r
        return plan, workspace
