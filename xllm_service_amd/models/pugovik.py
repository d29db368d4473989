"""Pugovik: a hybrid decoder on the paged-cache / state-slot engine.

Each layer picks its sequence mixer (latent attention, optionally reading
an earlier layer's latent cache, or decayed linear attention with a
recurrent state) and may have a routed-expert feed-forward. Around every
sublayer:

    h   = gnorm_a(x)
    y   = sublayer(h) * sigmoid(W_r h + b_r)          gated residual
    x  += mult * scale * gnorm_b(y)                   layer scale, residual

gnorm = RMS norm over equal consecutive groups of the width. The residual
stream x is fp32; norms, gates, scores, recurrent state and router are
fp32; GEMMs and their activations run in the model dtype (hipBLASLt).
Everything a mixer and the residual gate read from h comes out of ONE
merged projection per sublayer.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from xllm_service_amd.engine.metadata import AttnMetadata
from xllm_service_amd.models.config import PugovikConfig
from xllm_service_amd.models.mixers import (DecayLinearAttention,
                                            LatentAttention)
from xllm_service_amd.models.moe import RoutedExperts
from xllm_service_amd.ops import hybrid as hops


def _f32(n, fill=1.0):
    return nn.Parameter(torch.full((n,), fill, dtype=torch.float32))


class PugovikLayer(nn.Module):
    def __init__(self, cfg: PugovikConfig, index: int, dtype):
        super().__init__()
        lc = cfg.layers[index]
        W, eps = cfg.hidden_size, cfg.rms_eps
        self.eps, self.groups, self.mult = eps, cfg.norm_groups, \
            cfg.residual_mult
        self.dtype = dtype
        m = lc.mixer
        if lc.type == "latent_attention":
            self.mixer = LatentAttention(
                W, m["heads"], m["dim"], m["rot_dim"], m["vdim"],
                m["kv_rank"], m["scale"], m["rot"], eps, m.get("kv_from"),
                dtype)
        else:
            self.mixer = DecayLinearAttention(
                W, m["heads"], m["dim"], m["vdim"], m["decay"], eps, dtype)
        # merged projection of the mixer input: [mixer rows | residual gate]
        self.in_proj = nn.Parameter(torch.empty(self.mixer.in_width + W, W,
                                                dtype=dtype))
        self.norm1, self.norm1b, self.ls1 = _f32(W), _f32(W), _f32(W)
        self.rg1_b = _f32(W, 0.0)
        self.mlp = None
        if lc.mlp is not None:
            if lc.mlp.get("kind", "moe") != "moe":
                raise ValueError(f"layer {index}: unknown feed-forward kind")
            r = lc.mlp["router"]
            g = r.get("groups") or {}
            self.mlp = RoutedExperts(W, lc.mlp["expert"]["ff"], r["experts"],
                                     r["top"], g.get("count", 1),
                                     g.get("keep", 1), dtype)
            self.rg2 = nn.Parameter(torch.empty(W, W, dtype=dtype))
            self.norm2, self.norm2b, self.ls2 = _f32(W), _f32(W), _f32(W)
            self.rg2_b = _f32(W, 0.0)

    def forward(self, x, positions, cache, meta, aux):
        h = hops.group_rmsnorm(x, self.norm1, self.eps, self.groups,
                               self.dtype)
        proj = F.linear(h, self.in_proj)
        y = self.mixer(proj, positions, cache, meta, aux)
        hops.gated_norm_residual(x, y, proj[:, self.mixer.in_width:],
                                 self.rg1_b, self.norm1b, self.ls1, self.mult,
                                 self.eps, self.groups)
        if self.mlp is not None:
            h = hops.group_rmsnorm(x, self.norm2, self.eps, self.groups,
                                   self.dtype)
            y = self.mlp(h)
            hops.gated_norm_residual(x, y, F.linear(h, self.rg2), self.rg2_b,
                                     self.norm2b, self.ls2, self.mult,
                                     self.eps, self.groups)
        return x


class PugovikForCausalLM(nn.Module):
    def __init__(self, cfg: PugovikConfig, dtype=torch.bfloat16):
        super().__init__()
        self.cfg, self.dtype = cfg, dtype
        W = cfg.hidden_size
        self.embed = nn.Embedding(cfg.vocab_size, W, dtype=dtype)
        self.embed_norm, self.final_norm = _f32(W), _f32(W)
        self.layers = nn.ModuleList(
            [PugovikLayer(cfg, i, dtype) for i in range(cfg.num_layers)])
        self.lm_head = nn.Parameter(torch.empty(cfg.vocab_size, W,
                                                dtype=dtype))

    def cache_specs(self):
        return [l.mixer.cache_spec() for l in self.layers]

    # ---- weights -----------------------------------------------------------
    def load_weights(self, tensors: Dict[str, torch.Tensor]) -> None:
        """Checkpoint names: embed, embed.norm, final.norm, head, and per
        layer l<i>.{norm1,norm1b,norm2,norm2b,ls1,ls2,rg1,rg1.b,rg2,rg2.b},
        l<i>.mix.* and l<i>.mlp.{router,e<j>.{gate,up,down}}."""
        used = set()

        def take(name):
            if name not in tensors:
                raise KeyError(f"checkpoint lacks {name!r}")
            used.add(name)
            return tensors[name]

        def put(param, value):
            if tuple(param.shape) != tuple(value.shape):
                raise ValueError(f"shape mismatch: {tuple(value.shape)} "
                                 f"for {tuple(param.shape)}")
            with torch.no_grad():
                param.copy_(value.to(param.dtype))

        put(self.embed.weight, take("embed"))
        put(self.embed_norm, take("embed.norm"))
        put(self.final_norm, take("final.norm"))
        put(self.lm_head, take("head"))
        for i, layer in enumerate(self.layers):
            p = f"l{i}."
            mx = layer.mixer
            if isinstance(mx, LatentAttention):
                parts = [take(p + "mix.q")]
                if mx.kv_from is None:
                    parts.append(take(p + "mix.dkv"))
                    put(mx.dkv_norm, take(p + "mix.dkv.norm"))
                parts.append(take(p + "mix.g"))
                H, r = mx.heads, mx.kv_rank
                put(mx.w_uk, take(p + "mix.uk").view(H, mx.dim, r))
                put(mx.w_uv_t,
                    take(p + "mix.uv").view(H, mx.vdim, r).transpose(1, 2))
            else:
                parts = [take(p + "mix." + n) for n in "qkvg"]
                put(mx.out_norm, take(p + "mix.norm"))
            put(mx.o_proj, take(p + "mix.o"))
            parts.append(take(p + "rg1"))
            put(layer.in_proj, torch.cat(parts, 0))
            put(layer.rg1_b, take(p + "rg1.b"))
            for n in ("norm1", "norm1b", "ls1"):
                put(getattr(layer, n), take(p + n))
            if layer.mlp is not None:
                e = layer.mlp
                put(e.router, take(p + "mlp.router"))
                put(e.w_gate_up, torch.stack([
                    torch.cat([take(f"{p}mlp.e{j}.gate"),
                               take(f"{p}mlp.e{j}.up")], 0)
                    for j in range(e.experts)]))
                put(e.w_down, torch.stack([take(f"{p}mlp.e{j}.down")
                                           for j in range(e.experts)]))
                put(layer.rg2, take(p + "rg2"))
                put(layer.rg2_b, take(p + "rg2.b"))
                for n in ("norm2", "norm2b", "ls2"):
                    put(getattr(layer, n), take(p + n))
        extra = set(tensors) - used
        if extra:
            raise ValueError(f"unused checkpoint tensors: {sorted(extra)[:8]}")

    def random_init(self, seed: int = 0):
        dev = next(self.parameters()).device
        gen = torch.Generator(device=dev).manual_seed(seed)
        with torch.no_grad():
            for name, p in self.named_parameters():
                if p.dtype == torch.float32 and p.dim() == 1:
                    if name.endswith("_b"):
                        p.zero_()
                    else:
                        p.copy_(1.0 + 0.1 * torch.randn(
                            p.shape, generator=gen, device=dev))
                    continue
                std = 1.0 / math.sqrt(p.shape[-1])
                p.copy_((torch.randn(p.shape, generator=gen, device=dev,
                                     dtype=torch.float32) * std).to(p.dtype))

    # ---- forward -----------------------------------------------------------
    def forward(self, input_ids, positions, kv_caches: List,
                meta: AttnMetadata,
                inputs_embeds: Optional[torch.Tensor] = None):
        e = inputs_embeds if inputs_embeds is not None \
            else self.embed(input_ids)
        cfg = self.cfg
        x = hops.group_rmsnorm(e, self.embed_norm, cfg.rms_eps,
                               cfg.norm_groups, torch.float32)
        aux = {}
        if meta.num_decode_tokens:
            aux["decode_ctx_lens"] = meta.decode_seq_lens - 1
        for i, layer in enumerate(self.layers):
            x = layer(x, positions, kv_caches[i], meta, aux)
        return hops.group_rmsnorm(x, self.final_norm, cfg.rms_eps,
                                  cfg.norm_groups, self.dtype)

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        return F.linear(hidden, self.lm_head)
