"""Single-layer latency harness: the "sink" arm of the reference's latency job
(cascade/main/jobs/latency.py:10-84, driven by test-latency.bash:5-40).

One attention layer with q/k/v/o projections takes a stream of random hidden states in strides of
``cascade_stride`` tokens against a :class:`CascadingKVCache` (sink 4, window ``window`` split into
``cascades``), once untimed, then, after ``reset()``, once timed up to a device synchronisation.
The projections are plain ``torch.nn.Linear`` (rocBLAS / hipBLASLt through PyTorch); rotation,
attention, score sums and the cache update are the library's kernels.  Weights are random: the
reference loads a checkpoint only to take one layer out of it, and latency does not depend on
their values.

    python -m cascading_kv_cache_amd.latency --window 16384 --cascades 4 --cascade-stride 4096 --max-len 65536
"""
import argparse
import json
import time
from types import SimpleNamespace

import torch
from torch import nn

from .cascade_attention import CascadeAttention
from .cascading_cache import CascadingKVCache


class ProjectedCascadeAttention(CascadeAttention):
    """A concrete layer for :class:`CascadeAttention`: the attributes the reference's mixin reads off
    a Llama / Qwen2 attention module (cascade_attention.py:103-112, llama_eval.py:142-152)."""

    def __init__(self, hidden_size=4096, num_heads=32, num_key_value_heads=8, head_dim=128, rope_theta=5e5,
                 qkv_bias=False, head_reduction="max", homogeneous_heads=False, do_og_pos=False, layer_idx=0,
                 dtype=torch.float16, device="cuda"):
        super().__init__()
        self.hidden_size, self.num_heads, self.num_key_value_heads = hidden_size, num_heads, num_key_value_heads
        self.head_dim, self.rope_theta, self.layer_idx = head_dim, rope_theta, layer_idx
        self.config = SimpleNamespace(_homogeneous_heads=homogeneous_heads, _do_og_pos=do_og_pos,
                                      _head_reduction=head_reduction)
        kw = dict(dtype=dtype, device=device)
        self.q_proj = nn.Linear(hidden_size, num_heads * head_dim, bias=qkv_bias, **kw)
        self.k_proj = nn.Linear(hidden_size, num_key_value_heads * head_dim, bias=qkv_bias, **kw)
        self.v_proj = nn.Linear(hidden_size, num_key_value_heads * head_dim, bias=qkv_bias, **kw)
        self.o_proj = nn.Linear(num_heads * head_dim, hidden_size, bias=False, **kw)
        self._w_qkv = self._b_qkv = None

    def fuse_projections(self):
        """Keep the three projection matrices in one buffer (``q_proj`` / ``k_proj`` / ``v_proj`` become views of
        it), so that ``qkv`` is one matrix product instead of three: per token the projections are launch- and
        bandwidth-bound, and the two small ones are the least efficient.  Same values, no extra memory."""
        with torch.no_grad():
            mods = (self.q_proj, self.k_proj, self.v_proj)
            w = torch.cat([m.weight for m in mods], dim=0)
            b = torch.cat([m.bias for m in mods], dim=0) if self.q_proj.bias is not None else None
            at = 0
            for m in mods:
                n = m.weight.size(0)
                m.weight.data = w[at:at + n]
                if b is not None:
                    m.bias.data = b[at:at + n]
                at += n
            self._w_qkv, self._b_qkv = w, b

    def qkv(self, x, size, kv_size):
        if self._w_qkv is None:
            return super().qkv(x, size, kv_size)
        n_q, n_kv = self.q_proj.weight.size(0), self.k_proj.weight.size(0)
        q, k, v = nn.functional.linear(x, self._w_qkv, self._b_qkv).split((n_q, n_kv, n_kv), dim=-1)
        return q.view(*size).transpose(1, 2), k.view(*kv_size).transpose(1, 2), v.view(*kv_size).transpose(1, 2)


def stream_through(layer, cache, hidden, stride):
    """One pass of ``hidden (B, L, hidden)`` through the layer in strides (latency.py:61-64)."""
    out = None
    for i in range(0, hidden.size(1), stride):
        out = layer(hidden[:, i:i + stride], use_cache=True, past_key_value=cache)
        cache = out[2]
    return out


def job_latency(window=16384, cascades=4, cascade_stride=4096, lengths=None, head_reduction="max",
                hidden_size=4096, num_heads=32, num_key_value_heads=8, head_dim=128, num_sink_tokens=4,
                dtype=torch.float16, device="cuda:0", seed=0, verbose=True):
    """Seconds to stream ``l`` tokens for every ``l`` in ``lengths`` (default 4K .. 1M in powers of two, 4K .. 32K
    for stride 1, as latency.py:14-19).  Returns ``[{"len": l, "seconds": t, "tokens_per_s": l / t}, ...]``."""
    if lengths is None:
        lengths = [2 ** i for i in (range(12, 16) if cascade_stride == 1 else range(12, 21))]
    torch.manual_seed(seed)
    layer = ProjectedCascadeAttention(hidden_size, num_heads, num_key_value_heads, head_dim,
                                      head_reduction=head_reduction, dtype=dtype, device=device)
    layer.fuse_projections()  # q, k, v as one product
    results = []
    with torch.no_grad():
        for length in lengths:
            # the reference repeats one block of 1024 random rows (latency.py:31)
            block = torch.randn(1, min(1024, length), hidden_size, dtype=dtype, device=device)
            hidden = block.repeat(1, max(1, length // block.size(1)), 1)
            cache = CascadingKVCache(window // cascades, num_sink_tokens=num_sink_tokens, max_batch_size=1,
                                     heads=num_key_value_heads, dim=head_dim, max_seq_len=window, dtype=dtype,
                                     device=device, cascade_func="pow2", head_reduction=head_reduction, layers=1,
                                     verbose=False)
            stream_through(layer, cache, hidden, cascade_stride)
            torch.cuda.synchronize(device)
            cache.reset(verbose=False)
            tic = time.perf_counter()
            stream_through(layer, cache, hidden, cascade_stride)
            torch.cuda.synchronize(device)
            t = time.perf_counter() - tic
            results.append({"len": length, "seconds": t, "tokens_per_s": length / t})
            if verbose:
                print(f"latency for sink: len: {length}: {t}", flush=True)
            del hidden, cache
    return results


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--window", type=int, default=16384)
    ap.add_argument("--cascades", type=int, default=4)
    ap.add_argument("--cascade-stride", type=int, default=4096)
    ap.add_argument("--head-reduction", default="max")
    ap.add_argument("--min-len", type=int, default=4096)
    ap.add_argument("--max-len", type=int, default=65536)
    ap.add_argument("--dtype", default="float16", choices=["float16", "bfloat16"])
    args = ap.parse_args(argv)
    lengths, length = [], args.min_len
    while length <= args.max_len:
        lengths.append(length)
        length *= 2
    res = job_latency(args.window, args.cascades, args.cascade_stride, lengths, args.head_reduction,
                      dtype=getattr(torch, args.dtype), verbose=False)
    print(json.dumps({"method": "sink", "window": args.window, "cascades": args.cascades,
                      "cascade_stride": args.cascade_stride, "dtype": args.dtype, "results": res}))


if __name__ == "__main__":
    main()
