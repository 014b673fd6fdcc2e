"""Stage timers of the library (``ckv_profile_enable`` / ``ckv_profile_read``), the counterpart of the
reference's ``BENCHMARK=True`` event timing (cascading_cache.py:986-1026)."""
import pytest
import torch

from cascading_kv_cache_amd import _abi
from cascading_kv_cache_amd.cascade_attention import cascade_attention, default_inv_freq
from cascading_kv_cache_amd.cascading_cache import CascadingKVCache

pytestmark = pytest.mark.gpu


def _run(level, steps_prefill=3, steps_decode=4):
    B, H, KVH, D, NS, W, C = 2, 8, 2, 128, 64, 256, 2
    dev, dtype = "cuda:0", torch.bfloat16
    cache = CascadingKVCache(window_length=W, num_sink_tokens=NS, max_batch_size=B, heads=KVH, dim=D,
                             max_seq_len=W * C, device=dev, dtype=dtype, layers=1, verbose=False)
    inv_freq = default_inv_freq(D, 5e5, dev)
    g = torch.Generator().manual_seed(11)
    _abi.profile_enable(level)
    _abi.profile_read()
    try:
        for q_len in [256] * steps_prefill + [1] * steps_decode:
            q = torch.randn(B, H, q_len, D, generator=g).to(dtype).to(dev)
            k = torch.randn(B, KVH, q_len, D, generator=g).to(dtype).to(dev)
            v = torch.randn(B, KVH, q_len, D, generator=g).to(dtype).to(dev)
            out, _ = cascade_attention(q, k, v, cache, 0, inv_freq)
        torch.cuda.synchronize()
        assert torch.isfinite(out.float()).all()
        return _abi.profile_read()
    finally:
        _abi.profile_enable(0)


def test_main_kernels_only():
    """Level 2: one span per launch of the prefill forward and the decode main kernel (timed by events on the
    kernels' own dispatch), nothing else."""
    st = _run(2)
    assert st["fwd"][1] == 3 and st["decode"][1] == 4
    assert 0.0 < st["fwd"][0] < 100.0 and 0.0 < st["decode"][0] < 100.0
    for name, (ms, n) in st.items():
        if name not in ("fwd", "decode"):
            assert n == 0 and ms == 0.0, name


def test_main_kernels_sampled():
    """Level 4: as level 2, but the first and then every fourth launch of each of the two kernels."""
    st = _run(4, steps_prefill=5, steps_decode=9)
    assert st["fwd"][1] == 2 and st["decode"][1] == 3   # launches 0 and 4 of 5; 0, 4 and 8 of 9
    assert 0.0 < st["fwd"][0] < 100.0 and 0.0 < st["decode"][0] < 100.0
    for name, (ms, n) in st.items():
        if name not in ("fwd", "decode"):
            assert n == 0 and ms == 0.0, name


def test_every_stage():
    st = _run(1)
    assert st["fwd"][1] == 3 and st["scores"][1] == 3 and st["finish"][1] == 3
    assert st["decode"][1] == 4 and st["decode_tail"][1] == 4
    # a chunk's update is planned by two launches (the steady-state kernel, then the general one for the units it
    # left), a single token's by one (with so few units)
    assert st["prep"][1] == 7 and st["plan"][1] == 3 * 2 + 4 and st["apply"][1] == 7
    assert all(ms > 0.0 for ms, n in st.values())


def test_update_kernels_only():
    """Level 3: the kernels of the cache update, each timed on its own dispatch, nothing else."""
    st = _run(3)
    assert st["plan"][1] == 3 * 2 + 4 and st["apply"][1] == 7
    assert 0.0 < st["plan"][0] < 100.0 and 0.0 < st["apply"][0] < 100.0
    for name, (ms, n) in st.items():
        if name not in ("plan", "apply"):
            assert n == 0 and ms == 0.0, name


def test_off_records_nothing():
    st = _run(0)
    assert all(n == 0 for _, n in st.values())
