"""Attention whose weights are sigmoids of head-mixed scores, over a sliding window plus the sequence's first tokens.

    q, k per head divided by their root mean square (no learned weight), no rotation
    raw[g](i, j) = scale * q[i, g] . k[j, kv(g)]
    s[h](i, j)   = sum_g talk[h, g] raw[g](i, j) + bias[h]           (scores of all heads mixed before the weight)
    out[i, h]    = sum_j sigmoid(s[h](i, j)) v[j, kv(h)]              (no normalisation over keys)
    key j is visible to query i when j <= i and (i - j < window or j < keep_first); window None: all j <= i.

The layer owns pages of the ordinary paged KV cache (the scheduler and KV-cache manager treat it as a full-attention
layer: kept first tokens stay in their pages at their true positions, the kernel skips what the window hides).
Its cache keeps the NORMALISED keys; the layout is the framework's (K [blocks, kv_heads, block, dim], V [blocks,
kv_heads, vdim, block]) with key and value widths of their own.  Kernels: ops/csrc/sigmoid_attention.hip.
"""
from __future__ import annotations

from typing import Optional

import torch
import torch.nn as nn

from .. import ops
from ..forward_context import get_forward_context
from ..parallel.state import get_tensor_model_parallel_world_size
from ..sched.kv_cache_interface import FullAttentionSpec, KVCacheSpec
from .hyper_connections import _fp32_param
from .linear import MergedColumnParallelLinear, RowParallelLinear


class SigmoidWindowAttention(nn.Module):
    is_paged_kv_layer = True

    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, v_head_dim: int,
                 scale: float, window: Optional[int], keep_first: int, eps: float, quant_config=None,
                 prefix: str = ""):
        super().__init__()
        if get_tensor_model_parallel_world_size() > 1:
            raise NotImplementedError("head-mixing attention needs every head's score on one rank: "
                                      "tensor_parallel_size must be 1")
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} query heads do not divide into {num_kv_heads} key/value heads")
        self.num_heads, self.num_kv_heads, self.head_dim, self.v_head_dim = num_heads, num_kv_heads, head_dim, v_head_dim
        self.scale, self.eps = float(scale), float(eps)
        self.window, self.keep_first = int(window or 0), int(keep_first or 0)
        self.layer_name = prefix
        H, G, D, Dv = num_heads, num_kv_heads, head_dim, v_head_dim
        self.qkv_proj = MergedColumnParallelLinear(hidden_size, [H * D, G * D, G * Dv], bias=False,
                                                   quant_config=quant_config, prefix=f"{prefix}.qkv_proj")
        self.o_proj = RowParallelLinear(H * Dv, hidden_size, bias=False, quant_config=quant_config,
                                        prefix=f"{prefix}.o_proj")
        self.talk = _fp32_param((H, H), 0.0)
        self.score_bias = _fp32_param((H,), 0.0)
        self.k_cache: Optional[torch.Tensor] = None
        self.v_cache: Optional[torch.Tensor] = None

    def get_kv_cache_spec(self, block_size: int, dtype: torch.dtype) -> KVCacheSpec:
        return FullAttentionSpec(block_size=block_size, num_kv_heads=self.num_kv_heads, head_size=self.head_dim,
                                 dtype=dtype, v_head_size=self.v_head_dim)

    def bind_kv_cache(self, k_cache: torch.Tensor, v_cache: torch.Tensor) -> None:
        self.k_cache, self.v_cache = k_cache, v_cache

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        md = get_forward_context().attn_metadata
        H, G, D, Dv = self.num_heads, self.num_kv_heads, self.head_dim, self.v_head_dim
        qkv = self.qkv_proj(x)
        if md is None or self.k_cache is None:            # memory-profiling run: the projections carry the footprint
            return self.o_proj(qkv[:, : H * D].reshape(-1, H, D)[..., :1].expand(-1, H, Dv).reshape(-1, H * Dv)
                               .contiguous())
        T, n = qkv.shape[0], md.num_actual_tokens
        S = md.num_decode_seqs + md.num_prefill_seqs
        qn = ops.unit_rms_qk_and_cache(qkv[:n], H, G, D, Dv, self.eps, self.k_cache, self.v_cache,
                                       md.slot_mapping[:n])
        out = ops.sigmoid_window_attention(qn, self.k_cache, self.v_cache, md.block_table[:S], md.seq_lens[:S],
                                           md.query_start_loc[:S + 1], self.talk, self.score_bias, self.scale,
                                           self.window, self.keep_first, md.max_query_len, qkv.dtype,
                                           max_seq_len=md.max_seq_len)
        if n < T:
            out = torch.cat([out, out.new_zeros((T - n, out.shape[1]))], dim=0)
        return self.o_proj(out)
