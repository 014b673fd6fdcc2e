"""Minimal decoder around the library and the generation loop of the reference: chunked prefill in
strides, then greedy decoding one token at a time (cascade/models/cascade_attention.py:452-538,
``_sample_monkeypatch``).

The reference patches Hugging Face Llama / Qwen2 models; this module carries just enough of such a
decoder (embedding, RMSNorm, gated MLP, untied head; projections with optional bias) to run the
benchmark shapes end to end with random weights.  Everything outside attention is plain PyTorch;
attention, scores and the cache are the library's (:class:`ProjectedCascadeAttention`).

    python -m cascading_kv_cache_amd.decoder --preset llama3.1-8b --layers 4 --prompt 16384 --stride 4096 --new 32
"""
import argparse
import json
import time
from dataclasses import dataclass, replace

import torch
from torch import nn

from .cascading_cache import CascadingKVCache
from .latency import ProjectedCascadeAttention


@dataclass
class DecoderConfig:
    vocab_size: int
    hidden_size: int
    intermediate_size: int
    num_layers: int
    num_heads: int
    num_kv_heads: int
    head_dim: int = 128
    rope_theta: float = 5e5
    rms_eps: float = 1e-5
    qkv_bias: bool = False
    head_reduction: str = "max"


PRESETS = {
    # Llama-3.1-8B: 32 layers, hidden 4096, MLP 14336, 32q/8kv heads, vocab 128256, theta 5e5
    "llama3.1-8b": DecoderConfig(128256, 4096, 14336, 32, 32, 8, 128, 5e5, 1e-5, False),
    # Qwen2-7B: 28 layers, hidden 3584, MLP 18944, 28q/4kv heads (7 per kv head), QKV bias, theta 1e6
    "qwen2-7b": DecoderConfig(152064, 3584, 18944, 28, 28, 4, 128, 1e6, 1e-6, True),
    "tiny": DecoderConfig(512, 256, 512, 2, 4, 2, 128, 5e5, 1e-5, False),
}


class RMSNorm(nn.Module):
    def __init__(self, size, eps, dtype, device):
        super().__init__()
        self.weight = nn.Parameter(torch.ones(size, dtype=dtype, device=device))
        self.eps = eps
        self.fused = False

    def forward(self, x):
        if self.fused:  # one kernel; rounds once where the line below rounds twice
            return nn.functional.rms_norm(x, (x.size(-1),), self.weight, self.eps)
        xf = x.float()
        xf = xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + self.eps)
        return self.weight * xf.to(x.dtype)


class GatedMLP(nn.Module):
    def __init__(self, cfg, dtype, device):
        super().__init__()
        kw = dict(bias=False, dtype=dtype, device=device)
        self.gate_proj = nn.Linear(cfg.hidden_size, cfg.intermediate_size, **kw)
        self.up_proj = nn.Linear(cfg.hidden_size, cfg.intermediate_size, **kw)
        self.down_proj = nn.Linear(cfg.intermediate_size, cfg.hidden_size, **kw)

        self._w_gate_up = None

    def fuse_projections(self):
        """``gate_proj`` and ``up_proj`` as views of one buffer: one matrix product instead of two."""
        with torch.no_grad():
            w = torch.cat([self.gate_proj.weight, self.up_proj.weight], dim=0)
            n = self.gate_proj.weight.size(0)
            self.gate_proj.weight.data, self.up_proj.weight.data = w[:n], w[n:]
            self._w_gate_up = w

    def forward(self, x):
        if self._w_gate_up is None:
            return self.down_proj(nn.functional.silu(self.gate_proj(x)) * self.up_proj(x))
        gate, up = nn.functional.linear(x, self._w_gate_up).chunk(2, dim=-1)
        return self.down_proj(nn.functional.silu(gate) * up)


class DecoderLayer(nn.Module):
    def __init__(self, cfg, layer_idx, dtype, device):
        super().__init__()
        self.self_attn = ProjectedCascadeAttention(cfg.hidden_size, cfg.num_heads, cfg.num_kv_heads, cfg.head_dim,
                                                   rope_theta=cfg.rope_theta, qkv_bias=cfg.qkv_bias,
                                                   head_reduction=cfg.head_reduction, layer_idx=layer_idx, dtype=dtype,
                                                   device=device)
        self.mlp = GatedMLP(cfg, dtype, device)
        self.input_layernorm = RMSNorm(cfg.hidden_size, cfg.rms_eps, dtype, device)
        self.post_attention_layernorm = RMSNorm(cfg.hidden_size, cfg.rms_eps, dtype, device)

    def forward(self, x, cache):
        x = x + self.self_attn(self.input_layernorm(x), use_cache=True, past_key_value=cache)[0]
        return x + self.mlp(self.post_attention_layernorm(x))


class CascadeDecoder(nn.Module):
    """Decoder-only model whose every layer attends through one :class:`CascadingKVCache`."""

    def __init__(self, cfg: DecoderConfig, dtype=torch.bfloat16, device="cuda:0", seed=0, init_on_device=False):
        """Weights are N(0, 0.02) from ``seed``: drawn on the CPU (the same bits whatever the device, what the parity
        tests need) or, with ``init_on_device``, by the device's generator (seconds instead of minutes at 8B)."""
        super().__init__()
        self.cfg, self.dtype, self.device = cfg, dtype, device
        self.embed_tokens = nn.Embedding(cfg.vocab_size, cfg.hidden_size, dtype=dtype, device=device)
        self.layers = nn.ModuleList(DecoderLayer(cfg, i, dtype, device) for i in range(cfg.num_layers))
        self.norm = RMSNorm(cfg.hidden_size, cfg.rms_eps, dtype, device)
        self.lm_head = nn.Linear(cfg.hidden_size, cfg.vocab_size, bias=False, dtype=dtype, device=device)
        gen = torch.Generator(device=device if init_on_device else "cpu").manual_seed(seed)
        with torch.no_grad():
            for name, prm in self.named_parameters():
                if name.endswith("layernorm.weight") or name == "norm.weight":
                    continue
                if init_on_device:
                    prm.normal_(0.0, 0.02, generator=gen)
                else:
                    prm.copy_((torch.randn(prm.shape, generator=gen) * 0.02).to(dtype))

    def fuse_projections(self):
        """Fewer, larger launches outside attention (same weights, kept in shared buffers): q/k/v and gate/up
        projections as one matrix product each, the norms as one kernel.  Off by default: the parity tests compare
        the plain formulation with the CPU's."""
        for layer in self.layers:
            layer.self_attn.fuse_projections()
            layer.mlp.fuse_projections()
            layer.input_layernorm.fused = layer.post_attention_layernorm.fused = True
        self.norm.fused = True
        return self

    def new_cache(self, window, cascades, batch=1, num_sink_tokens=64, **kw):
        """One cache layer per decoder layer: ``window`` slots split into ``cascades`` rings.  Both may be lists
        with one entry per layer (the reference builds such caches, cascade/models/test.py:325-377)."""
        if isinstance(window, (list, tuple)):
            per_ring = [w // c for w, c in zip(window, cascades)]
            window = list(window)
        else:
            per_ring = window // cascades
        return CascadingKVCache(per_ring, num_sink_tokens=num_sink_tokens, max_batch_size=batch,
                                heads=self.cfg.num_kv_heads, dim=self.cfg.head_dim, max_seq_len=window,
                                dtype=self.dtype, device=self.device, head_reduction=self.cfg.head_reduction,
                                layers=self.cfg.num_layers, verbose=False, **kw)

    def forward(self, input_ids, cache, last_only=True):
        """``input_ids (B, q)`` -> logits ``(B, 1, vocab)`` (``last_only``) or ``(B, q, vocab)``."""
        x = self.embed_tokens(input_ids)
        for layer in self.layers:
            x = layer(x, cache)
        if last_only:
            x = x[:, -1:]
        return self.lm_head(self.norm(x))


@torch.no_grad()
def generate(model, input_ids, cache, stride, max_new_tokens):
    """Greedy generation as the reference runs it: the prompt goes through in strides of ``stride`` tokens,
    every later step feeds the last token only (cascade_attention.py:473-499, 527-538)."""
    logits = None
    for i in range(0, input_ids.size(1), stride):
        logits = model(input_ids[:, i:i + stride], cache)
    out = input_ids
    for step in range(max_new_tokens):
        nxt = torch.argmax(logits[:, -1, :], dim=-1)
        out = torch.cat([out, nxt[:, None]], dim=-1)
        if step + 1 < max_new_tokens:
            logits = model(out[:, -1:], cache)
    return out


def main(argv=None):
    ap = argparse.ArgumentParser(description=__doc__.split("\n")[0])
    ap.add_argument("--preset", default="llama3.1-8b", choices=sorted(PRESETS))
    ap.add_argument("--layers", type=int, default=None, help="override the number of layers")
    ap.add_argument("--batch", type=int, default=1)
    ap.add_argument("--prompt", type=int, default=16384)
    ap.add_argument("--stride", type=int, default=4096)
    ap.add_argument("--new", type=int, default=32)
    ap.add_argument("--window", type=int, default=65536)
    ap.add_argument("--cascades", type=int, default=8)
    args = ap.parse_args(argv)
    cfg = PRESETS[args.preset]
    if args.layers:
        cfg = replace(cfg, num_layers=args.layers)
    model = CascadeDecoder(cfg)
    ids = torch.randint(0, cfg.vocab_size, (args.batch, args.prompt), generator=torch.Generator().manual_seed(1)).cuda()
    res = {}
    for phase in ("warm", "timed"):
        cache = model.new_cache(args.window, args.cascades, batch=args.batch)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(0, ids.size(1), args.stride):
            logits = model(ids[:, i:i + args.stride], cache)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        out = ids[:, -1:]
        for _ in range(args.new):
            nxt = torch.argmax(logits[:, -1, :], dim=-1)
            logits = model(nxt[:, None], cache)
        torch.cuda.synchronize()
        t2 = time.perf_counter()
        res = {"prefill_tokens_per_s": args.batch * args.prompt / (t1 - t0),
               "decode_tokens_per_s": args.batch * args.new / max(t2 - t1, 1e-9)}
        del cache, out
    print(json.dumps({"preset": args.preset, "layers": cfg.num_layers, "batch": args.batch, "prompt": args.prompt,
                      "stride": args.stride, "new": args.new, "window": args.window, "cascades": args.cascades, **res}))


if __name__ == "__main__":
    main()
