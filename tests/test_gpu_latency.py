"""The single-layer harness (cascade/main/jobs/latency.py:10-84): a concrete attention layer with
projections on top of the library, checked against the CPU oracle, and the latency job itself.

The projections are torch matmuls on the device; to keep BLAS rounding out of the comparison the oracle
is fed the q/k/v the device produced, and its output goes through the same device o_proj.  What is
checked is therefore everything between the projections: views and strides handed to the C ABI,
rotation, attention, scores and the cache update, within 2e-2 abs on the attention output (16-bit).
"""
import pytest
import torch

from oracle.attention import OracleCascadeAttention
from oracle.update import OracleCache

pytestmark = pytest.mark.gpu

STATE = ("key_cache", "value_cache", "score_cache", "sink_keys", "sink_values", "mask", "sink_mask", "pos",
         "og_pos", "sink_pos", "stored_tokens", "start_indices", "stored_sinks")
META = ("mask", "sink_mask", "pos", "sink_pos", "stored_tokens", "start_indices", "stored_sinks")


@pytest.mark.parametrize("dtype,reduction,bias", [(torch.bfloat16, "max", False), (torch.float16, "mean", True)])
def test_projected_layer_against_the_oracle(dtype, reduction, bias):
    from cascading_kv_cache_amd.cascading_cache import CascadingKVCache
    from cascading_kv_cache_amd.latency import ProjectedCascadeAttention

    hidden, H, KVH, D, NS, W, C = 256, 4, 2, 128, 4, 64, 2
    torch.manual_seed(11)
    layer = ProjectedCascadeAttention(hidden, H, KVH, D, rope_theta=5e5, qkv_bias=bias, head_reduction=reduction,
                                      dtype=dtype, device="cuda:0")
    gpu = CascadingKVCache(W, num_sink_tokens=NS, max_batch_size=1, heads=KVH, dim=D, max_seq_len=W * C,
                           device="cuda:0", dtype=dtype, head_reduction=reduction, layers=1, verbose=False)
    cpu = OracleCache(window_length=W, num_sink_tokens=NS, max_batch_size=1, heads=KVH, dim=D, max_seq_len=W * C,
                      dtype=dtype)
    oracle = OracleCascadeAttention(H, KVH, D, rope_theta=5e5, head_reduction=reduction)
    gen = torch.Generator().manual_seed(5)
    with torch.no_grad():
        for c, q_len in enumerate((48, 48, 48, 48, 1, 1, 20)):
            x = torch.randn(1, q_len, hidden, generator=gen).to(dtype).cuda()
            for name in STATE:  # teacher forcing: both sides start the chunk from the oracle's state
                getattr(gpu, name)[0].copy_(getattr(cpu, name))
            gpu.seen_tokens_by_layer[0] = int(cpu.seen_tokens)
            gpu._seen_host[0] = int(cpu.seen_tokens)
            out_g, _, same_cache = layer(x, use_cache=True, past_key_value=gpu)
            assert same_cache is gpu and out_g.shape == (1, q_len, hidden)
            q, k, v = layer.qkv(x, (1, q_len, H, D), (1, q_len, KVH, D))
            attn_c = oracle.forward(q.cpu(), k.cpu(), v.cpu(), cpu)            # (1, H, q, D)
            want = layer.o_proj(attn_c.to(dtype).cuda().transpose(1, 2).reshape(1, q_len, H * D))
            torch.cuda.synchronize()
            # o_proj sums H * D attention values with weights below 1 / sqrt(H * D) in magnitude
            err = (out_g.float() - want.float()).abs().max().item()
            assert err <= 2e-2 * 4, f"chunk {c}: layer output differs by {err:.3e}"
            for name in META:
                assert torch.equal(getattr(gpu, name)[0].cpu(), getattr(cpu, name)), f"chunk {c}: {name}"


def test_latency_job_runs_prefill_and_decode_strides():
    from cascading_kv_cache_amd.latency import job_latency

    kw = dict(hidden_size=256, num_heads=4, num_key_value_heads=2, head_dim=128, dtype=torch.float16, verbose=False)
    res = job_latency(window=256, cascades=2, cascade_stride=128, lengths=[512, 1024], **kw)
    assert [r["len"] for r in res] == [512, 1024] and all(r["seconds"] > 0 for r in res)
    res = job_latency(window=128, cascades=1, cascade_stride=1, lengths=[192], **kw)
    assert res[0]["tokens_per_s"] > 0
    res = job_latency(window=128, cascades=2, cascade_stride=256, lengths=[512], **kw)  # stride longer than a cascade
    assert res[0]["seconds"] > 0
