"""Medilix: a decoder of parallel layers
    x <- x + mixer(norm1(x)) + ff(norm2(x))
with the residual stream x in fp32. The config lists the layers one by one:
each has one of three mixers (windowed softmax attention with kept first
tokens and a sink, wkv time mixing, mlstm matrix memory) and a dense clamped
GLU, routed experts, or no feed-forward. The norm is an RMS norm over equal
groups of the row. The embedding is the scaled token row plus a row of a
bigram table addressed by a hash of (previous token, token). A range of layers
may repeat several times with the same weights; every pass has its own cache
and state, and starts by mixing the stream with the embedding output through
one [W, 2W] matrix.
"""

from __future__ import annotations

import hashlib
import math
from typing import Dict, List, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from .. import ops
from ..engine.config import MedilixArchConfig, MedilixLayerSpec
from ..engine.kvcache import LayerCacheSpec, LayerState
from ..parallel.tp import ParallelContext
from .listed import ListedLayerLM
from .llama import ForwardBatch
from .mixers import ClampedGLU, MlstmMixer, RoutedExperts, WindowSinkAttention, WkvMixer, _param


class MedilixLayer(nn.Module):
    def __init__(self, spec: MedilixLayerSpec, hidden: int, eps: float, dtype):
        super().__init__()
        self.kind = spec.type
        self.norm1 = _param(hidden, dtype=torch.float32)
        if spec.type == "attention":
            self.mix = WindowSinkAttention(spec.attention, hidden, eps, dtype)
        elif spec.type == "wkv":
            self.mix = WkvMixer(spec.wkv, hidden, eps, dtype)
        else:
            self.mix = MlstmMixer(spec.mlstm, hidden, eps, dtype)
        self.mlp = None
        self.norm2 = None
        if spec.mlp is not None:
            self.norm2 = _param(hidden, dtype=torch.float32)
            self.mlp = (ClampedGLU(spec.mlp, hidden, dtype) if spec.mlp.kind == "dense"
                        else RoutedExperts(spec.mlp, hidden, dtype))

    def checkpoint_map(self, pre: str) -> Dict[str, torch.Tensor]:
        m = {pre + "norm1": self.norm1}
        m.update(self.mix.checkpoint_map(pre + "mix."))
        if self.mlp is not None:
            m[pre + "norm2"] = self.norm2
            m.update(self.mlp.checkpoint_map(pre + "mlp."))
        return m


class MedilixForCausalLM(ListedLayerLM):
    def __init__(self, cfg: MedilixArchConfig, ctx: Optional[ParallelContext] = None, dtype=torch.bfloat16):
        super().__init__()
        self.cfg = cfg
        self.ctx = ctx or ParallelContext()
        assert self.ctx.world_size == 1, "the Medilix family runs unsharded (tp_size must be 1)"
        self.dtype = dtype
        self.eps = cfg.rms_norm_eps
        W = cfg.hidden_size
        assert W % cfg.norm_groups == 0
        self.embed_tokens = nn.Embedding(cfg.vocab_size, W, dtype=dtype)
        self.embed_tokens.weight.requires_grad_(False)
        self.bigram = _param(cfg.bigram.buckets + 1, W, dtype=dtype) if cfg.bigram is not None else None
        self.loop_in = _param(W, 2 * W, dtype=dtype) if cfg.loop is not None else None
        self.layers = nn.ModuleList([MedilixLayer(sp, W, self.eps, dtype) for sp in cfg.layers])
        self.runs = cfg.layer_runs()
        self.final_norm = _param(W, dtype=torch.float32)
        self.lm_head = nn.Linear(W, cfg.vocab_size, bias=False, dtype=dtype)
        self.lm_head.weight.requires_grad_(False)

    # --- cache layout ---------------------------------------------------------
    def cache_layout(self) -> List[LayerCacheSpec]:
        """One entry per layer RUN (a looped layer keeps separate cache and
        state for each pass), then one for the embedding's previous token."""
        specs = [self.layers[li].mix.cache_spec() for li, _ in self.runs]
        specs.append(LayerCacheSpec(tok=self.bigram is not None))
        return specs

    # --- weights ----------------------------------------------------------------
    def checkpoint_map(self) -> Dict[str, torch.Tensor]:
        m = {"embed": self.embed_tokens.weight, "final.norm": self.final_norm, "head": self.lm_head.weight}
        if self.bigram is not None:
            m["bigram"] = self.bigram
        if self.loop_in is not None:
            m["loop.in"] = self.loop_in
        for i, layer in enumerate(self.layers):
            m.update(layer.checkpoint_map(f"l{i}."))
        return m

    @torch.no_grad()
    def random_init_(self, seed: int = 0) -> None:
        """Deterministic random init, one generator per checkpoint name."""
        for name, dst in self.checkpoint_map().items():
            g = torch.Generator(device="cpu")
            g.manual_seed(int(hashlib.md5(f"{seed}/{name}".encode()).hexdigest()[:15], 16))
            parts = name.split(".")
            leaf = parts[-1]
            if leaf in ("norm", "norm1", "norm2"):
                t = torch.ones(dst.shape)
            elif len(parts) >= 2 and parts[-2] == "mu":
                t = torch.rand(dst.shape, generator=g)
            elif leaf == "w0":
                t = torch.randn(dst.shape, generator=g) * 0.5 - 1.0
            elif leaf == "u":
                t = torch.randn(dst.shape, generator=g) * 0.3
            elif leaf == "correction":
                t = torch.randn(dst.shape, generator=g) * 0.01
            elif leaf == "b":
                t = torch.randn(dst.shape, generator=g) * 0.1 + (3.0 if parts[-2] == "f" else 0.0)
            elif leaf in ("embed", "bigram"):
                t = torch.randn(dst.shape, generator=g) * (1.0 if leaf == "embed" else 0.3)
            elif leaf == "in" and parts[0] == "loop":
                W = dst.shape[0]
                t = torch.randn(dst.shape, generator=g) * 0.02
                t[:, :W] += torch.eye(W)
            else:
                t = torch.randn(dst.shape, generator=g) / math.sqrt(dst.shape[-1])
            dst.copy_(t.to(device=dst.device, dtype=dst.dtype))

    # --- forward ------------------------------------------------------------------
    def forward_hidden(self, input_ids: torch.Tensor, batch: ForwardBatch) -> torch.Tensor:
        assert batch.seg_start is not None, "this model takes segment batches"
        cfg = self.cfg
        states: List[LayerState] = batch.kv_caches
        bg = cfg.bigram
        x = ops.embed_bigram(input_ids, self.embed_tokens.weight, self.bigram, cfg.embed_scale,
                             bg.mul_prev if bg else 0, bg.mul_cur if bg else 0, bg.buckets if bg else 1,
                             states[len(self.runs)].tok, batch.state_slots, batch.cu_seqlens, batch.seg_start,
                             batch.token_seg)
        x0 = x.clone() if self.loop_in is not None else None
        a = b = None     # the previous layer's branch outputs, not yet added to x
        for run, (li, pass_start) in enumerate(self.runs):
            layer = self.layers[li]
            if pass_start:
                # x <- W_in [x; x0]: the pending branches are added on the way
                x = F.linear(ops.cast_concat(x, x0, a, b, self.dtype), self.loop_in).float()
                a = b = None
            h1, h2 = ops.group_norm_pair(x, a, b, layer.norm1, layer.norm2, cfg.norm_groups, self.eps, self.dtype)
            a = layer.mix(h1, batch, states[run])
            b = layer.mlp(h2) if layer.mlp is not None else None
            if self.trace_layers is not None:
                self.trace_layers.append(x + a.float() + (b.float() if b is not None else 0.0))
        h, _ = ops.group_norm_pair(x, a, b, self.final_norm, None, cfg.norm_groups, self.eps, self.dtype)
        return h
