"""Zutalix: a decoder whose layers are listed one by one in the checkpoint's
config. Two layer types: 'parallel' (block-local softmax attention beside
decayed linear attention, followed by a clamped-GLU feed-forward) and
'channel_delta' (gated delta rule with per-channel decay, no feed-forward
unless the config lists one). Every sublayer is normed before AND after:
    x <- x + norm_b(sublayer(norm_a(x)))
with the residual stream x kept in fp32. The embedding is normed once before
the first layer, and the final norm precedes the LM head.

The model runs "segment" batches only (ForwardBatch.seg_start etc.): prompt
portions, decoded tokens and mixes of both take the same path, attention
through the paged cache and recurrent state through per-sequence slots — so
logits do not depend on how a prompt was cut or batched.
"""

from __future__ import annotations

import hashlib
import math
from typing import Dict, Iterable, List, Optional, Tuple

import torch
import torch.nn as nn
import torch.nn.functional as F

from .. import ops
from ..engine.config import HybridArchConfig, HybridLayerSpec
from ..engine.kvcache import LayerCacheSpec, LayerState
from ..parallel.tp import ParallelContext
from .listed import ListedLayerLM
from .llama import ForwardBatch
from .mixers import ChannelDeltaMixer, ClampedGLU, ParallelMixer, _param


class HybridLayer(nn.Module):
    def __init__(self, spec: HybridLayerSpec, hidden: int, eps: float, dtype):
        super().__init__()
        self.eps = eps
        self.kind = spec.type
        self.norm1 = _param(hidden, dtype=torch.float32)
        self.norm1b = _param(hidden, dtype=torch.float32)
        if spec.type == "parallel":
            self.mix = ParallelMixer(spec.parallel, hidden, eps, dtype)
        else:
            self.mix = ChannelDeltaMixer(spec.channel_delta, hidden, eps, dtype)
        self.mlp: Optional[ClampedGLU] = None
        if spec.mlp is not None:
            self.norm2 = _param(hidden, dtype=torch.float32)
            self.norm2b = _param(hidden, dtype=torch.float32)
            self.mlp = ClampedGLU(spec.mlp, hidden, dtype)

    def forward(self, x: torch.Tensor, h: torch.Tensor, batch: ForwardBatch, st: LayerState,
                next_norm: torch.Tensor) -> torch.Tensor:
        """x: fp32 residual (updated in place); h = norm1(x) in the model
        dtype. Returns the next layer's normed input."""
        after_mix = self.norm2 if self.mlp is not None else next_norm
        if self.kind == "parallel":
            left, right = self.mix(h, batch, st)
            h = ops.sandwich_residual(x, left, self.norm1b, self.eps, b=right, wa=self.mix.left_out,
                                      wb=self.mix.right_out, w_next=after_mix, out_dtype=h.dtype)
        else:
            y = self.mix(h, batch, st)
            h = ops.sandwich_residual(x, y, self.norm1b, self.eps, w_next=after_mix, out_dtype=h.dtype)
        if self.mlp is not None:
            y = self.mlp(h)
            h = ops.sandwich_residual(x, y, self.norm2b, self.eps, w_next=next_norm, out_dtype=h.dtype)
        return h

    def checkpoint_map(self, pre: str) -> Dict[str, torch.Tensor]:
        m = {pre + "norm1": self.norm1, pre + "norm1b": self.norm1b}
        m.update(self.mix.checkpoint_map(pre + "mix."))
        if self.mlp is not None:
            m[pre + "norm2"] = self.norm2
            m[pre + "norm2b"] = self.norm2b
            m.update(self.mlp.checkpoint_map(pre + "mlp."))
        return m


class ZutalixForCausalLM(ListedLayerLM):
    def __init__(self, cfg: HybridArchConfig, ctx: Optional[ParallelContext] = None, dtype=torch.bfloat16):
        super().__init__()
        self.cfg = cfg
        self.ctx = ctx or ParallelContext()
        assert self.ctx.world_size == 1, "the Zutalix family runs unsharded (tp_size must be 1)"
        self.dtype = dtype
        self.eps = cfg.rms_norm_eps
        W = cfg.hidden_size
        self.embed_tokens = nn.Embedding(cfg.vocab_size, W, dtype=dtype)
        self.embed_tokens.weight.requires_grad_(False)
        self.embed_norm = _param(W, dtype=torch.float32)
        self.layers = nn.ModuleList([HybridLayer(sp, W, self.eps, dtype) for sp in cfg.layers])
        self.final_norm = _param(W, dtype=torch.float32)
        self.lm_head = nn.Linear(W, cfg.vocab_size, bias=False, dtype=dtype)
        self.lm_head.weight.requires_grad_(False)

    # --- cache layout ---------------------------------------------------------
    def cache_layout(self) -> List[LayerCacheSpec]:
        return [layer.mix.cache_spec() for layer in self.layers]

    # --- weights ----------------------------------------------------------------
    def checkpoint_map(self) -> Dict[str, torch.Tensor]:
        """Checkpoint tensor name -> the parameter (or the slice of a fused
        parameter) it fills."""
        m = {"embed": self.embed_tokens.weight, "embed.norm": self.embed_norm,
             "final.norm": self.final_norm, "head": self.lm_head.weight}
        for i, layer in enumerate(self.layers):
            m.update(layer.checkpoint_map(f"l{i}."))
        return m

    def _after_load(self) -> None:
        self._zero_unbiased()

    def _zero_unbiased(self) -> None:
        for layer in self.layers:
            inp = layer.mix.inp
            if inp.bias is not None:
                for name, (off, n) in inp.parts.items():
                    if name not in inp.bias_parts:
                        inp.bias[off:off + n].zero_()

    @torch.no_grad()
    def random_init_(self, seed: int = 0) -> None:
        """Deterministic random init, one generator per checkpoint name:
        matrices ~ N(0, 1/in), norm weights 1, recurrence constants small."""
        for name, dst in self.checkpoint_map().items():
            g = torch.Generator(device="cpu")
            g.manual_seed(int(hashlib.md5(f"{seed}/{name}".encode()).hexdigest()[:15], 16))
            leaf = name.split(".")[-1]
            if leaf in ("norm", "norm1", "norm2", "norm1b", "norm2b", "out"):
                t = torch.ones(dst.shape)
            elif leaf in ("A_log", "dt_bias", "b") and dst.dim() == 1:
                t = torch.randn(dst.shape, generator=g) * 0.1
            elif leaf == "conv":
                t = torch.randn(dst.shape, generator=g) * 0.5
            elif leaf == "embed":
                t = torch.randn(dst.shape, generator=g)
            else:
                t = torch.randn(dst.shape, generator=g) / math.sqrt(dst.shape[-1])
            dst.copy_(t.to(device=dst.device, dtype=dst.dtype))
        self._zero_unbiased()

    # --- forward ------------------------------------------------------------------
    def forward_hidden(self, input_ids: torch.Tensor, batch: ForwardBatch) -> torch.Tensor:
        assert batch.seg_start is not None, "this model takes segment batches"
        x = ops.embed_rmsnorm(input_ids, self.embed_tokens.weight, self.embed_norm, self.eps)
        h = ops.rmsnorm_cast(x, self.layers[0].norm1, self.eps, self.dtype)
        n = len(self.layers)
        for i, layer in enumerate(self.layers):
            nxt = self.layers[i + 1].norm1 if i + 1 < n else self.final_norm
            h = layer(x, h, batch, batch.kv_caches[i], nxt)
            if self.trace_layers is not None:
                self.trace_layers.append(x.clone())
        return h
