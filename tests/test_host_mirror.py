"""CPU checks of the host-side mirror of the reference interface (no kernel launches)."""
import inspect

import pytest
import torch

from cascading_kv_cache_amd import _abi
from cascading_kv_cache_amd.cascade_attention import CascadeAttention, chunk_positions, default_inv_freq
from cascading_kv_cache_amd.cascading_cache import CascadingKVCache, acceptance_periods, sink_cache
from cascading_kv_cache_amd.flash_attention import attention
from oracle.update import CASCADE_FUNCS
from oracle.update import acceptance_periods as oracle_periods


def make(**kw):
    args = dict(window_length=4, num_sink_tokens=2, max_batch_size=2, heads=3, dim=8, max_seq_len=16, device="cpu",
                dtype=torch.float32, layers=2, verbose=False)
    args.update(kw)
    return CascadingKVCache(**args)


def test_constructor_signature_matches_the_reference():
    """cascade/models/cascading_cache.py:1032-1047."""
    names = list(inspect.signature(CascadingKVCache.__init__).parameters)[1:]
    assert names == ["window_length", "num_sink_tokens", "max_batch_size", "heads", "dim", "max_seq_len", "device",
                     "dtype", "cascade_func", "head_reduction", "layers", "eager_fill", "verbose"]
    d = inspect.signature(CascadingKVCache.__init__).parameters
    assert d["window_length"].default == 8 and d["num_sink_tokens"].default == 4 and d["max_seq_len"].default == 32
    assert d["dtype"].default == torch.float16 and d["cascade_func"].default == "pow2" and d["layers"].default == 32
    assert d["eager_fill"].default is True and d["head_reduction"].default == "mean"


def test_state_layout():
    """cascade/models/cascading_cache.py:1196-1276."""
    c = make()
    assert c.cascades == [4, 4] and len(c) == 2 and c.beta == 0.9999999
    assert c.key_cache[0].shape == (2, 3, 16, 8) and c.score_cache[1].shape == (2, 3, 16)
    assert c.sink_keys[0].shape == (2, 3, 2, 8) and c.pos[0].dtype == torch.long
    assert c.mask[0].dtype == torch.bool and c.mask[0].all() and c.sink_mask[1].all()
    assert c.stored_tokens[0].shape == (2, 3, 4) and c.stored_sinks[0].shape == (2, 3)
    assert c.do_cache_every_n[0].tolist() == [1, 2, 4, 8] and c.seen_tokens_by_layer.shape == (2,)
    assert c.get_max_length() == 16 and c.get_seq_length(0) == 0


def test_per_layer_window_lists():
    """cascade/models/test.py:325-377 builds caches whose layers differ in size."""
    c = make(window_length=[4, 8], max_seq_len=[16, 8])
    assert c.cascades == [4, 1] and c.key_cache[1].shape == (2, 3, 8, 8)
    with pytest.raises(ValueError):
        make(window_length=[4, 8], max_seq_len=16)
    with pytest.raises(ValueError):
        make(window_length=5)
    with pytest.raises(ValueError):
        make(cascade_func="nope")


def test_get_vals_applies_the_sink_shift_once_enough_tokens_were_seen():
    """cascade/models/cascading_cache.py:1278-1295."""
    c = make()
    c.pos[0][0, 0, :3] = torch.tensor([5, 6, 7])
    assert c.get_vals(0)[6][0, :3].tolist() == [5, 6, 7]
    c._seen_host[0] = 2
    assert c.get_vals(0)[6][0, :3].tolist() == [5, 6, 7]  # not MORE than the sink count yet
    c._seen_host[0] = 3
    vals = c.get_vals(0)
    assert vals[6][0, :3].tolist() == [7, 8, 9] and vals[6].shape == (1, 16) and vals[2].shape == (1, 2)
    assert len(vals) == 9 and vals[8] is c.og_pos[0]
    assert c[0][4] is c.key_cache[0] and len(list(iter(c))) == 2


def test_reset_and_unsupported_hf_methods():
    c = make()
    c.key_cache[0].fill_(3)
    c.mask[0].fill_(False)
    c.stored_tokens[1].fill_(2)
    c._seen_host[0] = 9
    c.reset(verbose=False)
    assert c.key_cache[0].abs().sum() == 0 and c.mask[0].all() and c.stored_tokens[1].sum() == 0
    assert c._seen_host == [0, 0]
    for call in (c.to_legacy_cache, lambda: c.crop(1), lambda: c.batch_split(1, 1), lambda: c.batch_repeat_interleave(2),
                 lambda: c.batch_select_indices(None), lambda: c.reorder_cache(None), lambda: c.seen_tokens,
                 lambda: CascadingKVCache.from_legacy_cache(None), lambda: CascadingKVCache.from_batch_splits([])):
        with pytest.raises(NotImplementedError):
            call()


def test_acceptance_schedules_agree_with_the_oracle_tables():
    for name in CASCADE_FUNCS:
        for c in (1, 2, 4, 8, 16):
            assert acceptance_periods(name, c) == oracle_periods(name, c), (name, c)


def test_chunk_positions_need_the_device():
    """cascade/models/cascade_attention.py:119-150 is one kernel of the library (checked against the rule on
    the GPU, tests/test_gpu_attention.py): on host tensors it refuses, like every other entry point."""
    c = make()
    with pytest.raises(_abi.CkvError):
        chunk_positions(c, 0, 3)


def test_no_cpu_fallback_anywhere():
    c = make()
    k = torch.zeros(2, 3, 1, 8)
    with pytest.raises(_abi.CkvError):
        c.update(k, k.clone(), 0)
    with pytest.raises(_abi.CkvError):
        attention(torch.zeros(1, 1, 16, 64), torch.zeros(1, 1, 16, 64), torch.zeros(1, 1, 16, 64), True, 1.0,
                  torch.zeros(0, dtype=torch.bool), 0.9)
    assert callable(sink_cache) and hasattr(CascadeAttention, "forward_cascade") and hasattr(CascadeAttention, "qkv")
    assert hasattr(CascadeAttention, "calc_scores")


def test_default_inv_freq_is_the_hf_formula():
    inv = default_inv_freq(128, 5e5, "cpu")
    assert inv.dtype == torch.float32 and inv.shape == (64,)
    assert inv[0].item() == 1.0
    assert abs(inv[32].item() - 5e5 ** -0.5) < 1e-9


def test_state_loaded_from_elsewhere_needs_a_counter_sync():
    """State copied into a cache behind ``update``'s back (a saved stream, the module-level operator plus a hand
    bump of ``seen_tokens_by_layer``, which the reference allows): the host mirror is stale until
    ``sync_host_counter`` re-reads the device counter; ``check_host_counter`` says so."""
    c = make()
    c.pos[0][0, 0, :3] = torch.tensor([0, 1, 2])
    c.seen_tokens_by_layer[0] = 5            # what a loader would restore
    c.seen_tokens_by_layer[1] = 5
    assert c.pos_shift(0) == 0               # stale mirror: no sink shift yet
    with pytest.raises(_abi.CkvError):
        c.check_host_counter(0)
    assert c.sync_host_counter() == [5, 5]
    c.check_host_counter(0)
    c.check_host_counter(1)
    assert c.pos_shift(0) == c.num_sink_tokens and c.get_vals(0)[6][0, :3].tolist() == [2, 3, 4]
    gen = c._generation
    c.reset(verbose=False)
    assert c._generation == gen + 1 and c.sync_host_counter() == [0, 0]


def test_reference_mixin_names_are_present():
    """cascade/models/cascade_attention.py:202-229, 250-340, 343-367."""
    from cascading_kv_cache_amd.cascade_attention import LlamaCascadeAttention, Qwen2CascadeAttention

    for cls in (CascadeAttention, LlamaCascadeAttention, Qwen2CascadeAttention):
        for name in ("forward", "qkv", "forward_cascade", "calc_scores", "cascade_attn_flash", "cascade_attn_eager", "rope"):
            assert callable(getattr(cls, name)), (cls.__name__, name)
    names = list(inspect.signature(CascadeAttention.cascade_attn_flash).parameters)[1:]
    assert names == ["query_states", "key_states", "value_states", "key_states_pos", "v_states", "sink_key_states",
                     "sink_value_states", "k_states", "sink_mask", "key_mask", "first_it", "past_key_value", "scale",
                     "q_len", "homogeneous_heads"]


def test_rope_flavours_agree_and_match_the_complex_rotation():
    """``rope`` on the CPU (plain torch): the table lookup of the Qwen2 flavour and the direct computation of the
    Llama flavour give the same rotation, and both equal multiplication by e^{i pos theta_j} on (x_j, x_{j+D/2})."""
    from types import SimpleNamespace

    from cascading_kv_cache_amd.cascade_attention import LlamaCascadeAttention, Qwen2CascadeAttention

    D = 16
    x = torch.randn(2, 3, 5, D, dtype=torch.float64, generator=torch.Generator().manual_seed(4))
    pos = torch.tensor([[0, 1, 7, 30, 63]])
    layers = []
    for cls in (LlamaCascadeAttention, Qwen2CascadeAttention):
        layer = cls()
        layer.head_dim, layer.rope_theta, layer.max_position_embeddings = D, 1e4, 64
        layer.config = SimpleNamespace()
        layers.append(layer)
    (a, cos_a, _), (b, cos_b, _) = layers[0].rope(x, pos), layers[1].rope(x, pos)
    assert cos_a.shape == (1, 5, D) and cos_b.shape == (64, D)      # per position / whole table
    assert torch.allclose(a, b, atol=1e-6)
    inv = 1.0 / (1e4 ** (torch.arange(0, D, 2, dtype=torch.float64) / D))
    z = torch.complex(x[..., :D // 2], x[..., D // 2:]) * torch.polar(torch.ones(5, D // 2, dtype=torch.float64),
                                                                        pos[0, :, None].double() * inv)
    want = torch.cat((z.real, z.imag), dim=-1)
    assert torch.allclose(a, want, atol=1e-5)   # the angles are fp32 products, as in the reference
    # tables handed back are reused
    again, _, _ = layers[1].rope(x, pos, cos=cos_b, sin=layers[1].rope(x, pos)[2])
    assert torch.equal(again, b)
