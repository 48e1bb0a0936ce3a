"""mLSTM mixer (the matrix memory of xLSTM): a linear-attention layer with exponential input / forget gates that are
kept in range by a running maximum, and a fixed-size recurrent state per request.

    q = W_q x * D^-1/2, k = W_k x (heads x D), v = W_v x (heads x Dv)
    i = cap tanh((W_i x + b_i) / cap)                    log input gate, per head
    f = logsigmoid(cap tanh((W_f x + b_f) / cap))        log forget gate, per head
    m' = max(f + m, i);  S' = e^(f + m - m') S + e^(i - m') k v^T;  n' = e^(f + m - m') n + e^(i - m') k
    o = S'^T q / (max(|n' . q|, e^-m') + 1e-6)           (m, S, n start at zero)
    out = W_o (o / rms(o) per head * norm * sigmoid(W_g x))

One GEMM produces everything that reads x.  The state (S, n and m, fp32) lives in the runner's per-request state
slots, the mechanism of the other recurrent mixers; gates, the recurrence and the output norm are fp32
(ops/csrc/mlstm.hip).
"""
from __future__ import annotations

import torch
import torch.nn as nn

from .. import ops
from ..forward_context import get_forward_context
from ..models.mamba import StateSpaceLayer
from ..parallel.state import get_tensor_model_parallel_world_size
from .hyper_connections import _fp32_param
from .linear import MergedColumnParallelLinear, RowParallelLinear


class MLSTMMixer(StateSpaceLayer):
    def __init__(self, hidden_size: int, num_heads: int, head_dim: int, v_head_dim: int, gate_cap: float, eps: float,
                 quant_config=None, prefix: str = ""):
        super().__init__()
        if get_tensor_model_parallel_world_size() > 1:
            raise NotImplementedError("mLSTM layers run with tensor_parallel_size=1")
        H, D, Dv = int(num_heads), int(head_dim), int(v_head_dim)
        self.num_heads, self.head_dim, self.v_head_dim = H, D, Dv
        self.gate_cap, self.eps = float(gate_cap), float(eps)
        self.layer_name = prefix
        self.conv_dtype = torch.float32
        self.state_dtypes = (torch.float32, torch.float32)
        # n and the running maximum share one row per head, padded to whole 16-byte groups
        self.nm_width = (D + 1 + 3) // 4 * 4
        # q | k | v | output gate | input gate | forget gate
        self.sizes = [H * D, H * D, H * Dv, H * Dv, H, H]
        self.in_proj = MergedColumnParallelLinear(hidden_size, self.sizes, bias=False, quant_config=quant_config,
                                                  prefix=f"{prefix}.in_proj")
        self.o_proj = RowParallelLinear(H * Dv, hidden_size, bias=False, quant_config=quant_config,
                                        prefix=f"{prefix}.o_proj")
        self.i_bias = _fp32_param((H,), 0.0)
        self.f_bias = _fp32_param((H,), 0.0)
        self.norm_weight = _fp32_param((H * Dv,))

    def state_shapes(self) -> tuple:
        return ((self.num_heads, self.nm_width), (self.num_heads, self.head_dim, self.v_head_dim))

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        md = get_forward_context().attn_metadata
        H, D, Dv = self.num_heads, self.head_dim, self.v_head_dim
        p = self.in_proj(x)
        if md is None or self.conv_state is None:          # memory-profiling run
            v0 = 2 * H * D
            return self.o_proj((p[:, v0: v0 + H * Dv] * p[:, v0 + H * Dv: v0 + 2 * H * Dv]).contiguous())
        T, n = p.shape[0], md.num_actual_tokens
        S = md.num_decode_seqs + md.num_prefill_seqs
        out = ops.mlstm(p[:n], self.i_bias, self.f_bias, self.norm_weight, self.conv_state, self.ssm_state,
                        md.query_start_loc[:S + 1], md.seq_lens[:S], self.slot_table(md)[:S], H, D, Dv, self.gate_cap,
                        self.eps)
        if n < T:
            out = torch.cat([out, out.new_zeros((T - n, out.shape[1]))], dim=0)
        return self.o_proj(out)
