"""Configuration C1 against its frozen fixture (tests/golden/c1_decode_golden.npz, written by
tests/golden/make_c1_golden.py): the oracle recomputed on the CPU must reproduce the file -- cache and scale
digests exactly, outputs to float32 rounding -- so a change of the oracle or of the workload recipe that moves
C1 fails here, before any GPU test looks at the oracle."""
import importlib.util
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def load_generator():
    spec = importlib.util.spec_from_file_location("make_c1_golden", os.path.join(HERE, "golden", "make_c1_golden.py"))
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def test_oracle_reproduces_the_c1_fixture():
    gen = load_generator()
    want = np.load(gen.PATH, allow_pickle=False)
    got = gen.compute()
    assert int(want["kv_lens"].sum()) == 1415  # the token count the configuration is specified with
    for key in ("kv_lens", "cachestarts", "appended_k", "appended_v", "appended_k_scale", "appended_v_scale"):
        assert np.array_equal(want[key], got[key]), key
    for key in ("sha_query", "sha_new_key", "sha_new_value", "sha_cache", "sha_scale"):
        assert str(want[key]) == got[key], key
    assert want["output"].shape == (4, 8, 64) and want["output"].dtype == np.float32
    # float32 accumulation in a fixed order: identical up to the last bits of libm's exp
    np.testing.assert_allclose(got["output"], want["output"], rtol=1e-6, atol=1e-7)


def test_c1_fixture_against_an_independent_numpy_computation(pkg, oracle):
    """The frozen outputs and appended rows, recomputed without the C oracle: the numpy restatement of the
    quantiser (every half operation correctly rounded), plain row indexing of the contiguous cache, and a float64
    softmax(q K^T / sqrt(D)) V over the dequantised rows.  A wrong index, a transposed operand or a dropped scale in
    the oracle would have been frozen into the fixture; this would not follow it."""
    gen = load_generator()
    want = np.load(gen.PATH, allow_pickle=False)
    bt, rng = pkg.workloads.make_batch("C1")
    hist = {}
    for b, pos, k_rows, v_rows in pkg.workloads.history_chunks(bt, rng):
        hist.setdefault(b, []).append((k_rows, v_rows))
    q, k, v = pkg.workloads.step_inputs(bt, rng)
    out = np.zeros((4, 8, 64))
    for b in range(4):
        k_all = np.concatenate([c[0] for c in hist[b]] + [k[b:b + 1]])  # (kvlen, 8, 64) float16
        v_all = np.concatenate([c[1] for c in hist[b]] + [v[b:b + 1]])
        assert len(k_all) == int(bt.kv_lens[b])
        kq, ks = oracle.quantize_groups_numpy(k_all.reshape(-1, 8, 8, 8))
        vq, vs = oracle.quantize_groups_numpy(v_all.reshape(-1, 8, 8, 8))
        assert np.array_equal(kq[-1].reshape(8, 64), want["appended_k"][b])
        assert np.array_equal(vq[-1].reshape(8, 64), want["appended_v"][b])
        assert np.array_equal(ks[-1].view(np.uint16), want["appended_k_scale"][b])
        assert np.array_equal(vs[-1].view(np.uint16), want["appended_v_scale"][b])
        kd = (kq.astype(np.float64) * ks.astype(np.float64)[..., None]).reshape(-1, 8, 64)
        vd = (vq.astype(np.float64) * vs.astype(np.float64)[..., None]).reshape(-1, 8, 64)
        for h in range(8):
            logits = kd[:, h] @ q[b, h].astype(np.float64) * float(bt.attn_scale)
            p = np.exp(logits - logits.max())
            out[b, h] = (p / p.sum()) @ vd[:, h]
    np.testing.assert_allclose(want["output"], out, rtol=2e-5, atol=2e-6)
