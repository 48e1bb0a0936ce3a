"""Rapovik: a decoder-only stack whose layers are listed one by one in the configuration, part of which can run several
times in a row with the same weights.  A layer is a mixer -- latent attention over a sliding window
(``latent_attention``), a Mamba-2 state-space block (``mamba2``) or an mLSTM matrix memory (``mlstm``) -- and an optional
feed-forward: a dense gated one with biases, or a mixture of experts with sigmoid scores, a selection bias, group-limited
choice and a shared expert.  Every sub-layer sits between two norms, x <- x + norm_b(sublayer(norm_a(x))), with gains
stored around zero; the residual is kept in fp32.

Attention layers keep pages of the paged cache (latent rows), recurrent layers a state slot per request (the hybrid
layout of the other attention + recurrent stacks); a layer inside the loop owns one cache or state per pass.  The
scheduler, chunked prefill, batching and sampling are the common ones.

Configuration (``config.json``): ``architecture: "Rapovik"``, ``vocab``, ``width``, ``norm.eps``, ``layers`` (``type``,
``mixer`` sizes, ``mlp`` or null), optional ``loop`` (``start``, ``stop``, ``times``: layers start .. stop - 1 run
``times`` times in a row).
Checkpoint names: ``embed``, ``head``, ``final.norm``, ``l<i>.norm1|norm1b|norm2|norm2b``, ``l<i>.mix.*``,
``l<i>.mlp.gate|up|down[.b]`` (dense) or ``l<i>.mlp.router|correction|e<j>.gate|up|down|shared.gate|up|down``.
"""
from __future__ import annotations

import re
from types import SimpleNamespace
from typing import Iterable, Optional

import torch
import torch.nn as nn
import torch.nn.functional as F

from .. import ops
from ..config import VllmConfig
from ..layers.basic import LogitsProcessor, ParallelLMHead, VocabParallelEmbedding
from ..layers.hyper_connections import _fp32_param
from ..layers.latent_attention import WindowedLatentAttention
from ..layers.linear import ReplicatedLinear, default_weight_loader
from ..layers.mlstm import MLSTMMixer
from ..layers.moe import FusedMoE
from .llama import LlamaMLP
from .mamba import Mamba2Mixer

ARCHITECTURE = "RapovikForCausalLM"
MIXERS = ("latent_attention", "mamba2", "mlstm")
DEFAULT_CONTEXT = 131072
GATED_ACT = "clamped_swiglu"         # min(g, L) * sigmoid(1.702 min(g, L)) * (clamp(u, -L, L) + 1)


def is_rapovik_config(d: dict) -> bool:
    return d.get("architecture") == "Rapovik" or ARCHITECTURE in (d.get("architectures") or [])


def run_order(num_layers: int, loop: Optional[dict]) -> list[tuple[int, int]]:
    """(layer, pass) in the order the stack runs them."""
    if not loop:
        return [(i, 0) for i in range(num_layers)]
    a, b, times = int(loop["start"]), int(loop["stop"]), int(loop["times"])
    if not (0 <= a <= b <= num_layers) or times < 1:
        raise ValueError(f"loop {loop} does not fit {num_layers} layers")
    return [(i, 0) for i in range(a)] + [(i, p) for p in range(times) for i in range(a, b)] + \
        [(i, 0) for i in range(b, num_layers)]


def normalise_config(d: dict, model_dir: Optional[str] = None) -> dict:
    """Give the engine the names it reads (hidden_size, vocab_size, heads ...)."""
    d = dict(d)
    layers = d["layers"]
    for i, l in enumerate(layers):
        if l["type"] not in MIXERS:
            raise ValueError(f"layer {i}: unknown mixer type {l['type']!r}")
        if l.get("mlp") is not None and l["mlp"].get("kind", "dense") not in ("dense", "moe"):
            raise ValueError(f"layer {i}: unknown feed-forward kind {l['mlp'].get('kind')!r}")
    att = [l["mixer"] for l in layers if l["type"] == "latent_attention"]
    d.update(
        architectures=[ARCHITECTURE], model_type="rapovik", hidden_size=int(d["width"]), vocab_size=int(d["vocab"]),
        num_hidden_layers=len(layers), num_attention_heads=max((int(m["heads"]) for m in att), default=1),
        num_key_value_heads=1,
        head_dim=max((int(m["kv_rank"]) + int(m["rot_dim"]) for m in att), default=int(d["width"])),
        tie_word_embeddings=False)
    d.setdefault("max_position_embeddings", DEFAULT_CONTEXT)
    d.setdefault("torch_dtype", "bfloat16")
    return d


class GainAroundZero(nn.Module):
    """The gain of an RMS norm, stored as its offset from one (fp32); applied by ``ops.residual_norms``."""

    def __init__(self, width: int):
        super().__init__()
        self.weight = _fp32_param((width,), 0.0)


class RapovikMoE(nn.Module):
    """Experts chosen by sigmoid scores plus a selection bias, from the best groups of neighbouring experts only;
    weighted by the plain scores, not renormalised; plus a shared expert for every token."""

    def __init__(self, width: int, spec: dict, quant_config, prefix: str):
        super().__init__()
        r, ex = spec["router"], spec["expert"]
        E, top = int(r["experts"]), int(r["top"])
        groups = r.get("groups") or {}
        count, keep = int(groups.get("count", 1) or 1), int(groups.get("keep", 1) or 1)
        if E % count or keep > count or top > (E // count) * keep:
            raise ValueError(f"{prefix}: {E} experts, {count} groups (keep {keep}) and top {top} do not fit")
        self.router = ReplicatedLinear(width, E, bias=False, params_dtype=torch.float32, prefix=f"{prefix}.router")
        self.correction = _fp32_param((E,), 0.0)
        self.experts = FusedMoE(E, top, width, int(ex["ff"]), renormalize=False, use_grouped_topk=True,
                                num_expert_group=count, topk_group=keep, quant_config=quant_config,
                                prefix=f"{prefix}.experts", scoring_func="sigmoid",
                                e_score_correction_bias=self.correction, activation=GATED_ACT,
                                act_limit=float(ex["limit"]))
        sh = spec.get("shared")
        self.shared = LlamaMLP(width, int(sh["ff"]), False, quant_config, f"{prefix}.shared", act=GATED_ACT,
                               act_limit=float(sh["limit"])) if sh else None

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        logits = F.linear(x.float(), self.router.weight)                  # the router runs in fp32
        out = self.experts(x, logits)
        return out + self.shared(x) if self.shared is not None else out


class RapovikLayer(nn.Module):
    def __init__(self, spec: dict, width: int, eps: float, passes: int, quant_config, prefix: str):
        super().__init__()
        kind, m = spec["type"], spec["mixer"]
        self.kind, self.eps = kind, eps
        self.norm1, self.norm1b = GainAroundZero(width), GainAroundZero(width)
        if kind == "latent_attention":
            rot, mask = m.get("rot") or {}, m.get("mask") or {}
            self.mixer = WindowedLatentAttention(
                width, int(m["heads"]), int(m["dim"]), int(m["rot_dim"]), int(m["vdim"]), int(m["kv_rank"]),
                float(m["scale"]), mask.get("size"), rot.get("base"), int(rot.get("dims", m["rot_dim"])), eps,
                passes, quant_config, f"{prefix}.mixer")
        elif kind == "mamba2":
            cfg = SimpleNamespace(hidden_size=width, num_heads=int(m["heads"]), head_dim=int(m["vdim"]),
                                  intermediate_size=int(m["heads"]) * int(m["vdim"]), state_size=int(m["state"]),
                                  conv_kernel=int(m["conv"]), n_groups=int(m.get("groups", 1)), use_bias=False,
                                  use_conv_bias=True, gated_norm=True, layer_norm_epsilon=eps,
                                  gated_norm_groups=int(m.get("norm_groups", 1)), time_step_limit=None)
            self.mixer = Mamba2Mixer(cfg, f"{prefix}.mixer")
            self.mixer.add_passes(passes)
        else:
            self.mixer = MLSTMMixer(width, int(m["heads"]), int(m["dim"]), int(m["vdim"]), float(m["gate_cap"]), eps,
                                    quant_config, f"{prefix}.mixer")
            self.mixer.add_passes(passes)
        mlp = spec.get("mlp")
        self.has_mlp = mlp is not None
        if self.has_mlp:
            self.norm2, self.norm2b = GainAroundZero(width), GainAroundZero(width)
            if mlp.get("kind", "dense") == "dense":
                self.mlp = LlamaMLP(width, int(mlp["ff"]), True, quant_config, f"{prefix}.mlp", act=GATED_ACT,
                                    act_limit=float(mlp["limit"]))
            else:
                self.mlp = RapovikMoE(width, mlp, quant_config, f"{prefix}.mlp")

    def forward(self, x: torch.Tensor, h: torch.Tensor, positions: torch.Tensor, pass_index: int,
                next_gain: torch.Tensor) -> torch.Tensor:
        """``x``: the fp32 residual, updated in place; ``h``: this layer's normed input; returns the next layer's."""
        if self.kind == "latent_attention":
            y = self.mixer(h, positions, pass_index)
        else:
            self.mixer.select_pass(pass_index)
            y = self.mixer(h)
        if self.has_mlp:
            h = ops.residual_norms(x, y, self.norm1b.weight, self.norm2.weight, self.eps, y.dtype)
            y = self.mlp(h)
            return ops.residual_norms(x, y, self.norm2b.weight, next_gain, self.eps, y.dtype)
        return ops.residual_norms(x, y, self.norm1b.weight, next_gain, self.eps, y.dtype)


class RapovikForCausalLM(nn.Module):
    supports_pp = False
    supports_lora = False
    # recurrent states live in per-row slots even when no layer is an attention layer
    row_state_slots = True
    # kernels outside the common set that this model launches (ops/build.py builds them on first use)
    native_sources = ("latent_attention.hip", "mla.hip", "mlstm.hip", "mamba.hip", "moe.hip", "gemm_tile.hip")

    def __init__(self, vllm_config: VllmConfig, prefix: str = ""):
        super().__init__()
        config = vllm_config.model_config.hf_config
        self.config = config
        quant_config = getattr(vllm_config, "quant_config", None)
        width, self.eps = int(config.width), float(config.norm["eps"])
        self.runs = run_order(len(config.layers), config.get("loop"))
        passes = [0] * len(config.layers)
        for i, p in self.runs:
            passes[i] = max(passes[i], p + 1)
        self.embed_tokens = VocabParallelEmbedding(int(config.vocab), width)
        self.layers = nn.ModuleList([
            RapovikLayer(spec, width, self.eps, max(passes[i], 1), quant_config, f"layers.{i}")
            for i, spec in enumerate(config.layers)])
        self.norm = GainAroundZero(width)
        self.lm_head = ParallelLMHead(int(config.vocab), width)
        self.logits_processor = LogitsProcessor(int(config.vocab))

    def get_input_embeddings(self, input_ids):
        return self.embed_tokens(input_ids)

    def forward(self, input_ids, positions, intermediate_tensors=None, inputs_embeds=None):
        e = inputs_embeds if inputs_embeds is not None else self.embed_tokens(input_ids)
        dtype = self.embed_tokens.weight.dtype
        x = e.float().contiguous() if e.dtype != torch.float32 else e.clone()
        gains = [self.layers[i].norm1.weight for i, _ in self.runs] + [self.norm.weight]
        h = ops.residual_norms(x, None, None, gains[0], self.eps, dtype)
        for r, (i, p) in enumerate(self.runs):
            h = self.layers[i](x, h, positions, p, gains[r + 1])
        return h

    def compute_logits(self, hidden_states):
        return self.logits_processor(self.lm_head, hidden_states).float()

    # checkpoint name -> (parameter name, shard id)
    _MIX = {
        "latent_attention": {"q": ("q_proj.weight", None), "dkv": ("dkv_proj.weight", None),
                             "dkv.norm": ("c_norm", None), "uk": ("uk_proj.weight", None),
                             "uv": ("uv_proj.weight", None), "o": ("o_proj.weight", None)},
        "mamba2": {"in": ("in_proj.weight", None), "conv": ("conv_weight", None), "conv.b": ("conv_bias", None),
                   "dt_bias": ("dt_bias", None), "A_log": ("A", None), "D": ("D", None), "norm": ("norm_weight", None),
                   "o": ("out_proj.weight", None)},
        "mlstm": {"q": ("in_proj.weight", 0), "k": ("in_proj.weight", 1), "v": ("in_proj.weight", 2),
                  "g": ("in_proj.weight", 3), "i": ("in_proj.weight", 4), "f": ("in_proj.weight", 5),
                  "i.b": ("i_bias", None), "f.b": ("f_bias", None), "norm": ("norm_weight", None),
                  "o": ("o_proj.weight", None)},
    }
    _FF = {"gate": ("gate_up_proj.weight", 0), "up": ("gate_up_proj.weight", 1), "down": ("down_proj.weight", None),
           "gate.b": ("gate_up_proj.bias", 0), "up.b": ("gate_up_proj.bias", 1), "down.b": ("down_proj.bias", None)}
    _TOP = {"embed": "embed_tokens.weight", "head": "lm_head.weight", "final.norm": "norm.weight"}
    _EXPERT = {"gate": ("w13_weight", "w1"), "up": ("w13_weight", "w3"), "down": ("w2_weight", "w2")}

    def _target(self, name: str):
        """Returns (parameter name, shard id, expert id) or None."""
        if name in self._TOP:
            return self._TOP[name], None, None
        m = re.fullmatch(r"l(\d+)\.(.+)", name)
        if not m or int(m.group(1)) >= len(self.layers):
            return None
        i, rest = int(m.group(1)), m.group(2)
        layer, base = self.layers[i], f"layers.{i}."
        if rest in ("norm1", "norm1b", "norm2", "norm2b"):
            return base + rest + ".weight", None, None
        part, _, leaf = rest.partition(".")
        if part == "mix" and leaf in self._MIX[layer.kind]:
            t, shard = self._MIX[layer.kind][leaf]
            return f"{base}mixer.{t}", shard, None
        if part == "mlp" and layer.has_mlp:
            if isinstance(layer.mlp, LlamaMLP):
                if leaf in self._FF:
                    t, shard = self._FF[leaf]
                    return f"{base}mlp.{t}", shard, None
                return None
            if leaf == "router":
                return f"{base}mlp.router.weight", None, None
            if leaf == "correction":
                return f"{base}mlp.correction", None, None
            sub, _, w = leaf.partition(".")
            if sub == "shared" and layer.mlp.shared is not None and w in ("gate", "up", "down"):
                t, shard = self._FF[w]
                return f"{base}mlp.shared.{t}", shard, None
            em = re.fullmatch(r"e(\d+)", sub)
            if em and w in self._EXPERT and int(em.group(1)) < layer.mlp.experts.global_num_experts:
                t, shard = self._EXPERT[w]
                return f"{base}mlp.experts.{t}", shard, int(em.group(1))
        return None

    def load_weights(self, weights: Iterable[tuple[str, torch.Tensor]]) -> set[str]:
        params = dict(self.named_parameters())
        loaded: set[str] = set()
        for name, t in weights:
            tgt = self._target(name)
            if tgt is None or tgt[0] not in params:
                raise ValueError(f"checkpoint tensor {name!r} has no place in this model")
            target, shard, expert = tgt
            p = params[target]
            loader = getattr(p, "weight_loader", default_weight_loader)
            if expert is not None:
                loader(p, t, shard, expert)
            elif shard is None:
                loader(p, t)
            else:
                loader(p, t, shard)
            loaded.add(target)
        return loaded
