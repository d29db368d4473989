"""Dunusun: a hybrid decoder on the paged-cache / state-slot engine.

Each layer has one sequence mixer — a selective state space mixer, or a
soft-capped softmax attention beside a gated linear attention — and an
optional dense squared-ReLU feed-forward. A token carries `streams` copies
of the residual (fp32); every sublayer reads one mixture of them through a
layer norm with bias and writes back into all of them:

    u   = sum_s in[s] x_s
    y   = sublayer(layernorm(u))
    x_j = sum_s mix[s, j] x_s + out[j] y          for all j at once

(one stream with in = mix = out = 1 is the plain pre-norm residual). A run
of consecutive layers may repeat with the same weights; every pass owns its
cache and state, so caches are laid out per layer RUN. The output is the
layer norm of the summed streams, the head, and a tanh soft cap.

fp32: streams, norms, rotary angles, scores and softmax, decays, recurrent
states, the soft caps. Model dtype: GEMMs, convolutions, gates. Everything a
mixer reads from its input comes out of ONE merged projection per layer.
"""
from __future__ import annotations

import math
from typing import Dict, List, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from xllm_service_amd.engine.metadata import AttnMetadata
from xllm_service_amd.models.config import DunusunConfig
from xllm_service_amd.models.mixers import (CappedAttention,
                                            GatedLinearAttention,
                                            ParallelMixer,
                                            SelectiveStateSpace)
from xllm_service_amd.ops import hybrid as hops


def _f32(*shape, fill=1.0):
    return nn.Parameter(torch.full(shape, fill, dtype=torch.float32))


class StreamPort(nn.Module):
    """How one sublayer reads from and writes to the residual streams, with
    the layer norm in front of it."""

    def __init__(self, width: int, streams: Optional[int], eps: float):
        super().__init__()
        self.eps = eps
        self.norm_w, self.norm_b = _f32(width), _f32(width, fill=0.0)
        self.mixed = streams is not None
        if self.mixed:
            self.w_in, self.w_out = _f32(streams), _f32(streams)
            self.mix = nn.Parameter(torch.eye(streams, dtype=torch.float32))

    def read(self, x, dtype):
        return hops.streams_mix_norm(x, self.w_in if self.mixed else None,
                                     self.norm_w, self.norm_b, self.eps, dtype)

    def write_then_read(self, x, nxt: "StreamPort", y1, a1=1.0, y2=None,
                        a2=0.0):
        """This sublayer's write and the next port's read in one pass over
        the streams; returns the next sublayer's normed input."""
        mix, w_out = (self.mix, self.w_out) if self.mixed else (None, None)
        return hops.streams_update_mix_norm_(
            x, mix, w_out, y1, a1, y2, a2, nxt.w_in if nxt.mixed else None,
            nxt.norm_w, nxt.norm_b, nxt.eps)


class DunusunLayer(nn.Module):
    def __init__(self, cfg: DunusunConfig, index: int, ranks: Dict[int, int],
                 dtype):
        super().__init__()
        lc = cfg.layers[index]
        W, eps = cfg.hidden_size, cfg.rms_eps
        self.dtype = dtype
        m = lc.mixer
        if lc.type == "mamba2":
            self.mixer = SelectiveStateSpace(
                W, m["heads"], m["vdim"], m["state"], m["groups"],
                m["norm_groups"], m["conv"], eps, dtype)
        else:
            L, R = m["left"], m["right"]
            left = CappedAttention(
                W, L["heads"], L["kv_heads"], L["dim"], L["vdim"], L["conv"],
                L.get("rot"), L["scale"], L.get("softcap"), dtype)
            right = GatedLinearAttention(
                W, R["heads"], R["dim"], R["vdim"], R["tau"],
                ranks.get(index, R.get("rank", 16)), eps, dtype)
            self.mixer = ParallelMixer(left, right, m["left_scale"],
                                       m["right_scale"])
        self.in_proj = nn.Parameter(torch.empty(self.mixer.in_width, W,
                                                dtype=dtype))
        self.port1 = StreamPort(W, cfg.streams, eps)
        self.ff = lc.mlp is not None
        if self.ff:
            self.up = nn.Parameter(torch.empty(lc.mlp["ff"], W, dtype=dtype))
            self.down = nn.Parameter(torch.empty(W, lc.mlp["ff"], dtype=dtype))
            self.port2 = StreamPort(W, cfg.streams, eps)

    def forward(self, x, h, positions, cache, meta, aux, next_port):
        """x: the streams (updated in place); h: this layer's normed mixer
        input, read by the previous layer's last write. Returns the streams
        and the normed input of whatever follows (`next_port`)."""
        y = self.mixer(F.linear(h, self.in_proj), positions, cache, meta, aux)
        after = self.port2 if self.ff else next_port
        if isinstance(y, tuple):
            a1, a2 = self.mixer.scales
            h = self.port1.write_then_read(x, after, y[0], a1, y[1], a2)
        else:
            h = self.port1.write_then_read(x, after, y)
        if self.ff:
            y = F.linear(hops.relu_sq_(F.linear(h, self.up)), self.down)
            h = self.port2.write_then_read(x, next_port, y)
        return x, h


class DunusunForCausalLM(nn.Module):
    def __init__(self, cfg: DunusunConfig, dtype=torch.bfloat16):
        super().__init__()
        self.cfg, self.dtype = cfg, dtype
        W = cfg.hidden_size
        self.n_streams = cfg.streams or 1
        if not 1 <= self.n_streams <= 8:
            raise ValueError("1..8 residual streams supported")
        self.embed = nn.Embedding(cfg.vocab_size, W, dtype=dtype)
        ranks = self._decay_ranks(cfg)
        self.layers = nn.ModuleList(
            [DunusunLayer(cfg, i, ranks, dtype)
             for i in range(cfg.num_layers)])
        # the read in front of the head: plain sum of the streams, normed
        self.final = StreamPort(W, None, cfg.rms_eps)
        self.lm_head = nn.Parameter(torch.empty(cfg.vocab_size, W,
                                                dtype=dtype))
        self.runs: List[int] = cfg.layer_runs

    @staticmethod
    def _decay_ranks(cfg: DunusunConfig) -> Dict[int, int]:
        """The low-rank size of the decay projection is a tensor shape, not a
        config entry: read it from the checkpoint header when there is one."""
        if not cfg.model_dir:
            return {}
        from xllm_service_amd.models.loader import safetensors_shapes
        shapes = safetensors_shapes(cfg.model_dir)
        out = {}
        for i, lc in enumerate(cfg.layers):
            sh = shapes.get(f"l{i}.mix.right.a1")
            if sh is not None:
                out[i] = int(sh[0])
        return out

    def cache_specs(self):
        """One entry per layer run: a looped layer has a cache per pass."""
        return [self.layers[li].mixer.cache_spec() for li in self.runs]

    # ---- weights -----------------------------------------------------------
    def load_weights(self, tensors: Dict[str, torch.Tensor]) -> None:
        """Checkpoint names: embed, final.norm(.b), head, and per layer
        l<i>.{norm1,norm2}(.b), l<i>.{hc1,hc2}.{in,out,mix},
        l<i>.mlp.{up,down} and l<i>.mix.* (mamba2: in, conv, conv.b,
        dt_bias, A_log, D, norm, o; parallel: left.{q,k,v}(.conv), left.{g,o},
        right.{q,k,v,g,o,norm,a1,a2,a2.b})."""
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

        def put_port(port, p, q):
            put(port.norm_w, take(f"{p}norm{q}"))
            put(port.norm_b, take(f"{p}norm{q}.b"))
            if port.mixed:
                put(port.w_in, take(f"{p}hc{q}.in"))
                put(port.w_out, take(f"{p}hc{q}.out"))
                put(port.mix, take(f"{p}hc{q}.mix"))

        put(self.embed.weight, take("embed"))
        put(self.final.norm_w, take("final.norm"))
        put(self.final.norm_b, take("final.norm.b"))
        put(self.lm_head, take("head"))
        for i, layer in enumerate(self.layers):
            p = f"l{i}."
            mx = layer.mixer
            if isinstance(mx, SelectiveStateSpace):
                put(layer.in_proj, take(p + "mix.in"))
                put(mx.conv_w, take(p + "mix.conv"))
                put(mx.conv_b, take(p + "mix.conv.b"))
                put(mx.dt_bias, take(p + "mix.dt_bias"))
                put(mx.A_log, take(p + "mix.A_log"))
                put(mx.D, take(p + "mix.D"))
                put(mx.out_norm, take(p + "mix.norm"))
                put(mx.o_proj, take(p + "mix.o"))
            else:
                lp, rp = p + "mix.left.", p + "mix.right."
                put(layer.in_proj, torch.cat(
                    [take(lp + n) for n in "qkvg"]
                    + [take(rp + n) for n in ("q", "k", "v", "g", "a1")], 0))
                put(mx.left.conv_w, torch.cat(
                    [take(f"{lp}{n}.conv") for n in "qkv"], 0))
                put(mx.left.o_proj, take(lp + "o"))
                put(mx.right.a2, take(rp + "a2"))
                put(mx.right.a2_b, take(rp + "a2.b"))
                put(mx.right.out_norm, take(rp + "norm"))
                put(mx.right.o_proj, take(rp + "o"))
            put_port(layer.port1, p, 1)
            if layer.ff:
                put(layer.up, take(p + "mlp.up"))
                put(layer.down, take(p + "mlp.down"))
                put_port(layer.port2, p, 2)
        extra = set(tensors) - used
        if extra:
            raise ValueError(f"unused checkpoint tensors: {sorted(extra)[:8]}")

    def random_init(self, seed: int = 0):
        dev = next(self.parameters()).device
        gen = torch.Generator(device=dev).manual_seed(seed)

        def randn(shape):
            return torch.randn(shape, generator=gen, device=dev,
                               dtype=torch.float32)
        with torch.no_grad():
            for name, p in self.named_parameters():
                leaf = name.rsplit(".", 1)[-1]
                if leaf == "mix":
                    p.copy_(0.8 * torch.eye(p.shape[0], device=dev)
                            + 0.1 * randn(p.shape))
                elif leaf == "w_in":
                    p.fill_(1.0 / p.shape[0])
                elif leaf in ("norm_b", "conv_b", "dt_bias"):
                    p.zero_()
                elif leaf == "A_log":
                    p.copy_(-1.0 + 0.5 * randn(p.shape))
                elif leaf == "a2_b":
                    p.fill_(3.0)
                elif leaf == "conv_w":
                    p.copy_((randn(p.shape) * 0.5).to(p.dtype))
                elif p.dtype == torch.float32 and p.dim() == 1:
                    p.copy_(1.0 + 0.1 * randn(p.shape))
                else:
                    std = 1.0 / math.sqrt(p.shape[-1])
                    p.copy_((randn(p.shape) * std).to(p.dtype))

    # ---- forward -----------------------------------------------------------
    def forward(self, input_ids, positions, kv_caches: List,
                meta: AttnMetadata,
                inputs_embeds: Optional[torch.Tensor] = None):
        e = inputs_embeds if inputs_embeds is not None \
            else self.embed(input_ids)
        T, W = e.shape
        x = e.float().unsqueeze(1).expand(T, self.n_streams, W).contiguous()
        aux = {}
        if meta.num_decode_tokens:
            aux["decode_ctx_lens"] = meta.decode_seq_lens - 1
        if not self.runs:
            return self.final.read(x, self.dtype)
        # every write to the streams is fused with the read that follows it
        h = self.layers[self.runs[0]].port1.read(x, self.dtype)
        for run, li in enumerate(self.runs):
            nxt = (self.layers[self.runs[run + 1]].port1
                   if run + 1 < len(self.runs) else self.final)
            x, h = self.layers[li](x, h, positions, kv_caches[run], meta, aux,
                                   nxt)
        return h

    def compute_logits(self, hidden: torch.Tensor) -> torch.Tensor:
        logits = F.linear(hidden, self.lm_head)
        if self.cfg.logit_softcap:
            return hops.softcap(logits, self.cfg.logit_softcap)
        return logits.float()
