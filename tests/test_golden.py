"""Golden fixtures (tests/golden/*.npz, written by tests/golden/make_fixtures.py from the pinned
oracle): the oracle must keep reproducing them on the CPU, and the HIP path must reproduce them
on the GPU through the C ABI."""
import os
import sys

import numpy as np
import pytest
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(HERE, "golden"))

import make_fixtures as mf  # noqa: E402
from oracle.attention import OracleCascadeAttention  # noqa: E402
from oracle.update import OracleCache  # noqa: E402

META = ("mask", "sink_mask", "pos", "og_pos", "sink_pos", "stored_tokens", "start_indices", "stored_sinks")


def load(name):
    return np.load(os.path.join(HERE, "golden", name), allow_pickle=False)


def same_bits(t, arr):
    got = t.detach().cpu()
    got = got.view(torch.int16).numpy() if got.dtype == torch.bfloat16 else got.numpy()
    return got.dtype == arr.dtype and np.array_equal(got, arr)


def test_oracle_reproduces_update_fixture():
    cfg, gold = mf.UPDATE_CFG, load("update_stream.npz")
    c = OracleCache(window_length=cfg["W"], num_sink_tokens=cfg["NS"], max_batch_size=cfg["B"], heads=cfg["H"],
                    dim=cfg["D"], max_seq_len=cfg["W"] * cfg["C"], dtype=torch.bfloat16, eager_fill=False)
    for k, v, s in mf.update_inputs(cfg):
        c.update(k, v, s)
    for name in mf.STATE:
        assert same_bits(getattr(c, name), gold[name]), name


def test_oracle_reproduces_attention_fixture():
    cfg, gold = mf.ATTN_CFG, load("attn_stream.npz")
    c = OracleCache(window_length=cfg["W"], num_sink_tokens=cfg["NS"], max_batch_size=cfg["B"], heads=cfg["KVH"],
                    dim=cfg["D"], max_seq_len=cfg["W"] * cfg["C"], dtype=torch.float32)
    layer = OracleCascadeAttention(cfg["H"], cfg["KVH"], cfg["D"], rope_theta=cfg["theta"])
    for i, (q, k, v) in enumerate(mf.attn_inputs(cfg)):
        out = layer.forward(q, k, v, c)
        assert np.allclose(out.numpy(), gold["outs"][i], atol=1e-6), f"chunk {i}"
    for name in META:
        assert same_bits(getattr(c, name), gold[name]), name


@pytest.mark.gpu
def test_hip_update_reproduces_fixture_bit_exactly():
    from cascading_kv_cache_amd.cascading_cache import CascadingKVCache

    cfg, gold = mf.UPDATE_CFG, load("update_stream.npz")
    c = CascadingKVCache(window_length=cfg["W"], num_sink_tokens=cfg["NS"], max_batch_size=cfg["B"], heads=cfg["H"],
                         dim=cfg["D"], max_seq_len=cfg["W"] * cfg["C"], device="cuda:0", dtype=torch.bfloat16,
                         layers=1, eager_fill=False, verbose=False)
    for k, v, s in mf.update_inputs(cfg):
        c.update(k.cuda(), v.cuda(), 0, s.cuda())
    torch.cuda.synchronize()
    for name in mf.STATE:
        assert same_bits(getattr(c, name)[0], gold[name]), name


@pytest.mark.gpu
def test_hip_attention_stream_reproduces_fixture():
    """Free-running float32 stream: outputs within 1e-4, every index/position/mask and the set of
    retained tokens bit-exact."""
    from cascading_kv_cache_amd.cascade_attention import cascade_attention, default_inv_freq
    from cascading_kv_cache_amd.cascading_cache import CascadingKVCache

    cfg, gold = mf.ATTN_CFG, load("attn_stream.npz")
    c = CascadingKVCache(window_length=cfg["W"], num_sink_tokens=cfg["NS"], max_batch_size=cfg["B"], heads=cfg["KVH"],
                         dim=cfg["D"], max_seq_len=cfg["W"] * cfg["C"], device="cuda:0", dtype=torch.float32,
                         layers=1, verbose=False)
    inv_freq = default_inv_freq(cfg["D"], cfg["theta"], "cuda:0")
    for i, (q, k, v) in enumerate(mf.attn_inputs(cfg)):
        out, new = cascade_attention(q.cuda(), k.cuda(), v.cuda(), c, 0, inv_freq)
        assert np.abs(out.cpu().numpy() - gold["outs"][i]).max() <= 1e-4, f"chunk {i}"
        ref = gold["new_scores"][i]
        assert np.abs(new.cpu().numpy() - ref).max() <= 1e-4 * np.abs(ref).max() + 1e-12
    torch.cuda.synchronize()
    for name in META:
        assert same_bits(getattr(c, name)[0], gold[name]), name
    assert np.abs(c.key_cache[0].cpu().numpy() - gold["key_cache"]).max() == 0.0
