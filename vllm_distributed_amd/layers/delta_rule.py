"""Gated delta-rule mixer with one decay per head and key channel (a linear-attention layer with a fixed-size
recurrent state per request).

    q, k, v = silu(short causal convolution over time of the projections), per channel
    q, k  <- unit vectors per head (q also times dim^-1/2);  head h reads q / k head h // (heads / kv_heads)
    beta   = sigmoid(W_b x);   decay = exp(-exp(A_log[h]) * softplus(W_a2 (W_a1 x) + dt_bias))   [heads, dim]
    S <- diag(decay) S;  u = beta (v - S^T k);  S <- S + k u^T;  o = S^T q      (S: [dim, vdim] per head, fp32)
    out = W_o (o / rms(o) * norm * sigmoid(W_g2 (W_g1 x)))

The state (S and the convolution's last taps - 1 inputs) lives in the runner's per-request state slots, the
mechanism of the other recurrent mixers; everything the recurrence consumes besides the projections is fp32.
Kernels: ops/csrc/delta_rule.hip (the recurrence, norms, decays, gates, output norm in one launch),
ops/csrc/mamba.hip (the convolution, shared with the state-space mixers).
"""
from __future__ import annotations

import torch
import torch.nn as nn

from .. import ops
from ..forward_context import get_forward_context
from ..models.mamba import StateSpaceLayer
from ..parallel.state import get_tensor_model_parallel_world_size
from .hyper_connections import _fp32_param
from .linear import MergedColumnParallelLinear, ReplicatedLinear, RowParallelLinear, set_weight_attrs


class GatedDeltaRule(StateSpaceLayer):
    def __init__(self, hidden_size: int, num_heads: int, num_kv_heads: int, head_dim: int, v_head_dim: int,
                 conv_taps: int, decay_rank: int, gate_rank: int, eps: float, quant_config=None, prefix: str = ""):
        super().__init__()
        if get_tensor_model_parallel_world_size() > 1:
            raise NotImplementedError("delta-rule layers run with tensor_parallel_size=1")
        if num_heads % num_kv_heads:
            raise ValueError(f"{num_heads} heads do not divide into {num_kv_heads} query/key heads")
        H, G, D, Dv = num_heads, num_kv_heads, head_dim, v_head_dim
        self.num_heads, self.num_kv_heads, self.head_dim, self.v_head_dim = H, G, D, Dv
        self.taps, self.eps = int(conv_taps), float(eps)
        self.decay_rank, self.gate_rank = int(decay_rank), int(gate_rank)
        self.layer_name = prefix
        dtype = torch.get_default_dtype()
        self.conv_dtype = dtype
        self.state_dtypes = (dtype, torch.float32)
        self.conv_dim = 2 * G * D + H * Dv
        # one GEMM for everything that reads x: q | k | v | decay low-rank | gate low-rank | beta
        self.sizes = [G * D, G * D, H * Dv, self.decay_rank, self.gate_rank, H]
        self.in_proj = MergedColumnParallelLinear(hidden_size, self.sizes, bias=False, quant_config=quant_config,
                                                  prefix=f"{prefix}.in_proj")
        self.decay_up = ReplicatedLinear(self.decay_rank, H * D, bias=False, prefix=f"{prefix}.decay_up")
        self.gate_up = ReplicatedLinear(self.gate_rank, H * Dv, bias=False, prefix=f"{prefix}.gate_up")
        self.o_proj = RowParallelLinear(H * Dv, hidden_size, bias=False, quant_config=quant_config,
                                        prefix=f"{prefix}.o_proj")
        self.conv_weight = nn.Parameter(torch.zeros((self.conv_dim, self.taps), dtype=dtype), requires_grad=False)
        offs = [0, G * D, 2 * G * D]

        def load_conv(param, t, shard_id=None):
            if shard_id is None:
                param.data.copy_(t.reshape(param.shape))
            else:
                t = t.reshape(t.shape[0], -1)
                param.data[offs[shard_id]: offs[shard_id] + t.shape[0]].copy_(t)
        set_weight_attrs(self.conv_weight, {"weight_loader": load_conv})
        self.A_log = _fp32_param((H,), 0.0)
        self.dt_bias = _fp32_param((H * D,), 0.0)
        self.norm_weight = _fp32_param((Dv,))

    def state_shapes(self) -> tuple:
        return ((self.conv_dim, self.taps - 1), (self.num_heads, self.v_head_dim, self.head_dim))

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        md = get_forward_context().attn_metadata
        H, G, D, Dv, C = self.num_heads, self.num_kv_heads, self.head_dim, self.v_head_dim, self.conv_dim
        p = self.in_proj(x)
        ra, rg = self.decay_rank, self.gate_rank
        a_raw = self.decay_up(p[:, C: C + ra])
        gate_raw = self.gate_up(p[:, C + ra: C + ra + rg])
        if md is None or self.conv_state is None:          # memory-profiling run
            return self.o_proj((gate_raw * p[:, 2 * G * D: C]).contiguous() + a_raw[:, :1])
        T, n = p.shape[0], md.num_actual_tokens
        S = md.num_decode_seqs + md.num_prefill_seqs
        tbl = self.slot_table(md)[:S]
        qsl, lens = md.query_start_loc[:S + 1], md.seq_lens[:S]
        xc = ops.causal_conv1d(p[:n, :C], self.conv_weight, None, self.conv_state, qsl, lens, tbl, md.max_query_len)
        out = ops.gated_delta_rule(xc, a_raw[:n], p[:n, C + ra + rg:], gate_raw[:n], self.A_log, self.dt_bias,
                                   self.norm_weight, self.ssm_state, qsl, lens, tbl, H, G, D, Dv, self.eps)
        if n < T:
            out = torch.cat([out, out.new_zeros((T - n, out.shape[1]))], dim=0)
        return self.o_proj(out)
