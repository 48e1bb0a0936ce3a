"""Nositar: a decoder-only stack whose layers are listed one by one in the configuration.  A layer is a mixer --
sigmoid attention with head-mixed scores over a window plus kept first tokens (``attention``), or a gated delta
rule with per-channel decay (``channel_delta``, ``channel_delta_2``) -- and an optional ReLU-gated feed-forward,
each reading and writing fp32 residual streams through learned hyper-connection weights (or a plain fp32 residual
when the configuration names no streams).  Norms carry a single gain.  Logits are soft-capped.

Attention layers keep pages of the paged KV cache, delta-rule layers a state slot per request (the hybrid layout of
the other attention + recurrent stacks), so the scheduler, chunked prefill, batching and sampling are the common ones.

Configuration (``config.json``): ``architecture: "Nositar"``, ``vocab``, ``width``, ``layers`` (``type``, ``mixer``
sizes, ``mlp`` or null), ``norm.eps``, ``embedding.scale``, optional ``streams`` and ``logit_softcap``.  The ranks
of the low-rank decay / gate projections are read from the checkpoint's tensor shapes.
Checkpoint names: ``embed``, ``head``, ``final.norm``, ``l<i>.norm1|norm2``, ``l<i>.hc1|hc2.in|out|mix``,
``l<i>.mix.*``, ``l<i>.mlp.gate|up|down``.
"""
from __future__ import annotations

import os
import re
from typing import Iterable, Optional

import torch
import torch.nn as nn

from .. import ops
from ..config import VllmConfig
from ..layers.basic import LogitsProcessor, ParallelLMHead, VocabParallelEmbedding
from ..layers.delta_rule import GatedDeltaRule
from ..layers.hyper_connections import ScalarRMSNorm, StreamPort, read_streams, write_read_streams
from ..layers.sigmoid_attention import SigmoidWindowAttention
from ..layers.linear import default_weight_loader
from .llama import LlamaMLP

ARCHITECTURE = "NositarForCausalLM"
DELTA_KINDS = ("channel_delta", "channel_delta_2")
DEFAULT_CONTEXT = 131072          # nothing in the design depends on absolute position


def is_nositar_config(d: dict) -> bool:
    return d.get("architecture") == "Nositar" or ARCHITECTURE in (d.get("architectures") or [])


def normalise_config(d: dict, model_dir: Optional[str] = None) -> dict:
    """Give the engine the names it reads (hidden_size, vocab_size, heads ...) and complete the mixers' sizes with
    what only tensor shapes tell (ranks of the low-rank projections)."""
    d = dict(d)
    layers = [dict(l, mixer=dict(l["mixer"])) for l in d["layers"]]
    shapes = {}
    st = os.path.join(model_dir, "model.safetensors") if model_dir else None
    if st and os.path.isfile(st):
        from .loader import read_safetensors_header
        header, _ = read_safetensors_header(st)
        shapes = {k: v["shape"] for k, v in header.items() if k != "__metadata__"}
    for i, l in enumerate(layers):
        kind, m = l["type"], l["mixer"]
        if kind in DELTA_KINDS:
            for key, name in (("decay_rank", f"l{i}.mix.a1"), ("gate_rank", f"l{i}.mix.g1")):
                if name in shapes:
                    m[key] = int(shapes[name][0])
                elif key not in m:
                    raise ValueError(f"layer {i}: {key} is neither in the configuration nor readable from the "
                                     f"shape of {name}")
        elif kind != "attention":
            raise ValueError(f"layer {i}: unknown mixer type {kind!r}")
        if l.get("mlp") is not None and l["mlp"].get("kind", "dense") != "dense":
            raise ValueError(f"layer {i}: unknown feed-forward kind {l['mlp'].get('kind')!r}")
    att = [l["mixer"] for l in layers if l["type"] == "attention"]
    d.update(
        layers=layers, architectures=[ARCHITECTURE], model_type="nositar", hidden_size=int(d["width"]),
        vocab_size=int(d["vocab"]), num_hidden_layers=len(layers),
        num_attention_heads=max((int(m["heads"]) for m in att), default=1),
        num_key_value_heads=max((int(m["kv_heads"]) for m in att), default=1),
        head_dim=max((max(int(m["dim"]), int(m["vdim"])) for m in att), default=int(d["width"])),
        tie_word_embeddings=False)
    d.setdefault("max_position_embeddings", DEFAULT_CONTEXT)
    d.setdefault("torch_dtype", "bfloat16")
    return d


class NositarLayer(nn.Module):
    def __init__(self, spec: dict, width: int, eps: float, streams: int, learned: bool, quant_config, prefix: str):
        super().__init__()
        kind, m = spec["type"], spec["mixer"]
        self.kind = kind
        self.norm1 = ScalarRMSNorm(eps)
        self.port1 = StreamPort(streams, learned)
        if kind == "attention":
            mask = m.get("mask") or {}
            self.mixer = SigmoidWindowAttention(
                width, int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"]), float(m["scale"]),
                mask.get("size"), int(mask.get("keep_first", 0) or 0), eps, quant_config, f"{prefix}.mixer")
        else:
            self.mixer = GatedDeltaRule(width, int(m["heads"]), int(m["kv_heads"]), int(m["dim"]), int(m["vdim"]),
                                        int(m["conv"]), int(m["decay_rank"]), int(m["gate_rank"]), eps,
                                        quant_config, f"{prefix}.mixer")
        mlp = spec.get("mlp")
        self.has_mlp = mlp is not None
        if self.has_mlp:
            self.norm2 = ScalarRMSNorm(eps)
            self.port2 = StreamPort(streams, learned)
            self.mlp = LlamaMLP(width, int(mlp["ff"]), False, quant_config, f"{prefix}.mlp", act="relu")

    def forward(self, xs: torch.Tensor, h: torch.Tensor, nxt_port: StreamPort, nxt_norm: ScalarRMSNorm):
        """``h`` is this layer's first read of the streams; returns the next layer's."""
        y = self.mixer(h)
        if self.has_mlp:
            h = write_read_streams(xs, y, self.port1, self.port2, self.norm2)
            y = self.mlp(h)
            return write_read_streams(xs, y, self.port2, nxt_port, nxt_norm)
        return write_read_streams(xs, y, self.port1, nxt_port, nxt_norm)


class NositarForCausalLM(nn.Module):
    supports_pp = False
    supports_lora = False
    # delta-rule states live in per-row slots even when no layer is an attention layer
    row_state_slots = True
    # kernels outside the common set that this model launches (ops/build.py builds them on first use)
    native_sources = ("streams.hip", "sigmoid_attention.hip", "delta_rule.hip", "mamba.hip")

    def __init__(self, vllm_config: VllmConfig, prefix: str = ""):
        super().__init__()
        config = vllm_config.model_config.hf_config
        self.config = config
        quant_config = getattr(vllm_config, "quant_config", None)
        width, eps = int(config.width), float(config.norm["eps"])
        streams = config.get("streams")
        self.learned_streams = streams is not None
        self.streams = int(streams) if streams is not None else 1
        self.embed_scale = float((config.get("embedding") or {}).get("scale", 1.0))
        self.embed_tokens = VocabParallelEmbedding(int(config.vocab), width)
        self.layers = nn.ModuleList([
            NositarLayer(spec, width, eps, self.streams, self.learned_streams, quant_config, f"layers.{i}")
            for i, spec in enumerate(config.layers)])
        self.norm = ScalarRMSNorm(eps)
        self.out_port = StreamPort(self.streams, learned=False)       # the output is the plain sum of the streams
        self.lm_head = ParallelLMHead(int(config.vocab), width)
        cap = config.get("logit_softcap")
        self.soft_cap = float(cap) if cap else None
        self.logits_processor = LogitsProcessor(int(config.vocab))

    def get_input_embeddings(self, input_ids):
        return self.embed_tokens(input_ids) * self.embed_scale

    def forward(self, input_ids, positions, intermediate_tensors=None, inputs_embeds=None):
        dtype = self.embed_tokens.weight.dtype
        if inputs_embeds is not None:
            xs = inputs_embeds.float().unsqueeze(0).repeat(self.streams, 1, 1)
        else:
            xs = ops.stream_embed(input_ids, self.embed_tokens.weight, self.embed_scale, self.streams)
        n = len(self.layers)
        h = read_streams(xs, self.layers[0].port1, self.layers[0].norm1, dtype) if n else None
        for i, layer in enumerate(self.layers):
            nxt = self.layers[i + 1] if i + 1 < n else None
            h = layer(xs, h, nxt.port1 if nxt else self.out_port, nxt.norm1 if nxt else self.norm)
        return h if n else read_streams(xs, self.out_port, self.norm, dtype)

    def compute_logits(self, hidden_states):
        logits = self.logits_processor(self.lm_head, hidden_states).float()
        if self.soft_cap is not None:
            logits = torch.tanh(logits / self.soft_cap) * self.soft_cap
        return logits

    # checkpoint name -> (parameter name, shard id)
    _MIX_ATT = {"q": ("qkv_proj.weight", 0), "k": ("qkv_proj.weight", 1), "v": ("qkv_proj.weight", 2),
                "o": ("o_proj.weight", None), "talk": ("talk", None), "pb": ("score_bias", None)}
    _MIX_DELTA = {"q": ("in_proj.weight", 0), "k": ("in_proj.weight", 1), "v": ("in_proj.weight", 2),
                  "a1": ("in_proj.weight", 3), "g1": ("in_proj.weight", 4), "b": ("in_proj.weight", 5),
                  "a2": ("decay_up.weight", None), "g2": ("gate_up.weight", None), "o": ("o_proj.weight", None),
                  "q.conv": ("conv_weight", 0), "k.conv": ("conv_weight", 1), "v.conv": ("conv_weight", 2),
                  "A_log": ("A_log", None), "dt_bias": ("dt_bias", None), "norm": ("norm_weight", None)}
    _MLP = {"gate": ("gate_up_proj.weight", 0), "up": ("gate_up_proj.weight", 1), "down": ("down_proj.weight", None)}
    _PORT = {"in": "w_in", "out": "w_out", "mix": "mix"}
    _TOP = {"embed": "embed_tokens.weight", "head": "lm_head.weight", "final.norm": "norm.weight"}

    def _target(self, name: str):
        if name in self._TOP:
            return self._TOP[name], None
        m = re.fullmatch(r"l(\d+)\.(.+)", name)
        if not m or int(m.group(1)) >= len(self.layers):
            return None, None
        i, rest = int(m.group(1)), m.group(2)
        base = f"layers.{i}."
        if rest in ("norm1", "norm2"):
            return base + rest + ".weight", None
        part, _, leaf = rest.partition(".")
        if part in ("hc1", "hc2") and leaf in self._PORT:
            return f"{base}port{part[-1]}.{self._PORT[leaf]}", None
        if part == "mlp" and leaf in self._MLP:
            t, shard = self._MLP[leaf]
            return f"{base}mlp.{t}", shard
        if part == "mix":
            table = self._MIX_ATT if self.layers[i].kind == "attention" else self._MIX_DELTA
            if leaf in table:
                t, shard = table[leaf]
                return f"{base}mixer.{t}", shard
        return None, None

    def load_weights(self, weights: Iterable[tuple[str, torch.Tensor]]) -> set[str]:
        params = dict(self.named_parameters())
        loaded: set[str] = set()
        for name, t in weights:
            target, shard = self._target(name)
            if target is None or target not in params:
                raise ValueError(f"checkpoint tensor {name!r} has no place in this model")
            p = params[target]
            loader = getattr(p, "weight_loader", default_weight_loader)
            if shard is None:
                loader(p, t)
            else:
                loader(p, t, shard)
            loaded.add(target)
        return loaded
