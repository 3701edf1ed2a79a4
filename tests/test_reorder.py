"""kv_cache_reorder / kv_cache_invert_reorder: the CPU oracle is pinned against numpy's own gather and
transpose on a concrete pair of layouts and by the round trip; the HIP path is compared with the oracle
byte for byte (GPU tests), on the 16-byte fast path and on the bytewise path."""
import numpy as np
import pytest


def layouts(L, H, NP, D, G, tp_size):
    """Cache side: int8 [L, 2, H, NP * D tokens, D] (a page = D tokens, as the reference's kernel assumes) and
    scales [L, 2, H, NP * D, D/G] halves.  Outer side per (slot, rank): cache bytes [T, H, 2, L, D], then scale
    bytes [T, H, 2, L, D/G*2].  Returns shapes, byte strides and per-page byte counts."""
    T = D
    SB = D // G * 2
    tok = NP * T
    src = [0, 2 * H * tok * D, H * tok * D, tok * D, D, 1,
           0, 2 * H * tok * SB, H * tok * SB, tok * SB, SB, 1]
    pcb, psb = T * H * 2 * L * D, T * H * 2 * L * SB
    dst = [0, D, L * D, 2 * L * D, H * 2 * L * D, 1,
           0, SB, L * SB, 2 * L * SB, H * 2 * L * SB, 1]
    src[0], src[6] = pcb, psb  # the reference reads the page byte counts from src_stride in both directions
    return dict(T=T, SB=SB, src=src, dst=dst, pcb=pcb, psb=psb, cache_shape=(L, 2, H, tok, D), scale_shape=(L, 2, H, tok, SB),
                outer_bytes=(pcb + psb) * tp_size)


def numpy_reorder(cache, scale, page_ids, lay, L, H, D, tp_rank, tp_size):
    """The gather written with numpy indexing only."""
    T, SB = lay["T"], lay["SB"]
    out = np.zeros((len(page_ids), lay["outer_bytes"]), dtype=np.uint8)
    for j, pg in enumerate(page_ids):
        c = cache[:, :, :, pg * T:(pg + 1) * T, :]             # [L, 2, H, T, D]
        s = scale[:, :, :, pg * T:(pg + 1) * T, :]
        out[j, tp_rank * lay["pcb"]:(tp_rank + 1) * lay["pcb"]] = np.transpose(c, (3, 2, 1, 0, 4)).reshape(-1)
        o = tp_size * lay["pcb"] + tp_rank * lay["psb"]
        out[j, o:o + lay["psb"]] = np.transpose(s, (3, 2, 1, 0, 4)).reshape(-1)
    return out.reshape(-1)


CASES = [dict(L=2, H=3, NP=5, D=32, G=8, tp_rank=1, tp_size=2, page_ids=[3, 0, 4]),
         dict(L=1, H=2, NP=4, D=16, G=8, tp_rank=0, tp_size=1, page_ids=[2, 2, 1])]


@pytest.mark.parametrize("case", CASES)
def test_oracle_reorder_is_numpy_gather_and_round_trips(oracle, case):
    L, H, NP, D, G = case["L"], case["H"], case["NP"], case["D"], case["G"]
    lay = layouts(L, H, NP, D, G, case["tp_size"])
    rng = np.random.default_rng(9)
    cache = rng.integers(0, 256, lay["cache_shape"], dtype=np.uint8)
    scale = rng.integers(0, 256, lay["scale_shape"], dtype=np.uint8)
    ids = np.array(case["page_ids"], dtype=np.int64)
    outer = np.full(len(ids) * lay["outer_bytes"], 0xEE, dtype=np.uint8)
    oracle.kv_cache_reorder(False, cache, scale, outer, ids, lay["src"], lay["dst"], L, H, lay["T"], D, G,
                            case["tp_rank"], case["tp_size"])
    ref = numpy_reorder(cache, scale, ids, lay, L, H, D, case["tp_rank"], case["tp_size"])
    # this rank's share equals the numpy gather; the other ranks' shares stay untouched
    other = np.ones_like(outer, dtype=bool).reshape(len(ids), -1)
    r = case["tp_rank"]
    other[:, r * lay["pcb"]:(r + 1) * lay["pcb"]] = False
    o = case["tp_size"] * lay["pcb"] + r * lay["psb"]
    other[:, o:o + lay["psb"]] = False
    assert (outer.reshape(len(ids), -1)[other] == 0xEE).all()
    np.testing.assert_array_equal(outer.reshape(len(ids), -1)[~other], ref.reshape(len(ids), -1)[~other])
    # the inverse scatters the same bytes back: only the selected pages change
    cache2 = np.zeros_like(cache)
    scale2 = np.zeros_like(scale)
    oracle.kv_cache_reorder(True, cache2, scale2, outer, ids, lay["dst"][:0] + [lay["pcb"]] + lay["dst"][1:6] + [lay["psb"]] + lay["dst"][7:],
                            lay["src"], L, H, lay["T"], D, G, case["tp_rank"], case["tp_size"])
    T = lay["T"]
    for pg in range(NP):
        sl = (slice(None), slice(None), slice(None), slice(pg * T, (pg + 1) * T))
        if pg in case["page_ids"]:
            np.testing.assert_array_equal(cache2[sl], cache[sl])
            np.testing.assert_array_equal(scale2[sl], scale[sl])
        else:
            assert not cache2[sl].any() and not scale2[sl].any()


@pytest.mark.gpu
@pytest.mark.parametrize("case", CASES + [dict(L=2, H=8, NP=6, D=128, G=8, tp_rank=1, tp_size=2, page_ids=[5, 1, 2, 0])])
@pytest.mark.parametrize("misalign", [0, 1])
def test_gpu_reorder_matches_oracle(pkg, oracle, case, misalign):
    import torch
    L, H, NP, D, G = case["L"], case["H"], case["NP"], case["D"], case["G"]
    lay = layouts(L, H, NP, D, G, case["tp_size"])
    rng = np.random.default_rng(10)
    cache = rng.integers(0, 256, lay["cache_shape"], dtype=np.uint8)
    scale = rng.integers(0, 256, lay["scale_shape"], dtype=np.uint8)
    ids = np.array(case["page_ids"], dtype=np.int64)
    n_outer = len(ids) * lay["outer_bytes"]
    outer_ref = np.full(n_outer, 0xEE, dtype=np.uint8)
    oracle.kv_cache_reorder(False, cache, scale, outer_ref, ids, lay["src"], lay["dst"], L, H, lay["T"], D, G,
                            case["tp_rank"], case["tp_size"])
    d_cache = torch.from_numpy(cache).cuda()
    d_scale = torch.from_numpy(scale).cuda()
    d_ids = torch.from_numpy(ids).cuda()
    # misalign = 1 shifts the outer buffer by one byte: the bytewise path instead of 16-byte moves
    buf = torch.full((n_outer + 16,), 0xEE, dtype=torch.uint8, device="cuda")
    d_outer = buf[misalign:misalign + n_outer]
    kw = dict(layers=L, kv_heads=H, tokens=lay["T"], head_dim=D, group_size=G, tp_rank=case["tp_rank"], tp_size=case["tp_size"])
    pkg.ops.kv_cache_reorder(d_cache, d_scale, d_ids, lay["src"], lay["dst"], outer_mem=d_outer.data_ptr(), **kw)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(d_outer.cpu().numpy(), outer_ref)
    # and back into an empty cache
    inv_src = [lay["pcb"]] + lay["dst"][1:6] + [lay["psb"]] + lay["dst"][7:]
    cache_ref = np.zeros_like(cache)
    scale_ref = np.zeros_like(scale)
    oracle.kv_cache_reorder(True, cache_ref, scale_ref, outer_ref, ids, inv_src, lay["src"], L, H, lay["T"], D, G,
                            case["tp_rank"], case["tp_size"])
    d_cache2 = torch.zeros_like(d_cache)
    d_scale2 = torch.zeros_like(d_scale)
    pkg.ops.kv_cache_invert_reorder(d_outer.data_ptr(), d_ids, inv_src, lay["src"], kv_cache=d_cache2, kv_scale=d_scale2, **kw)
    torch.cuda.synchronize()
    np.testing.assert_array_equal(d_cache2.cpu().numpy(), cache_ref)
    np.testing.assert_array_equal(d_scale2.cpu().numpy(), scale_ref)
