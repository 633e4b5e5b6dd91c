from __future__ import annotations

import torch

from ..cache.specs import StateSpec
from ..kernels import ops
from ..registry import register_mixer
from ..weights.loader import ParamSpec
from .base import Part

_NAMES = {"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight", "g": "g_proj.weight", "o": "o_proj.weight",
          "norm": "norm.weight", "i": "igate.weight", "i_bias": "igate.bias", "f": "fgate.weight", "f_bias": "fgate.bias"}


@register_mixer("mlstm")
class MatrixLSTM(Part):
    """The matrix memory of the xLSTM family.  Per head, q = W_q h * d^(-1/2), k = W_k h (``head_dim`` d) and v = W_v h
    (``v_head_dim`` dv); two gates in logarithms, capped: i = cap tanh((W_i h + b_i) / cap), f = logsigmoid(cap tanh((W_f h
    + b_f) / cap)), cap = ``gate_cap``.  With a running maximum m that keeps the exponentials in range (it starts at
    0, as S and n do at zero):

        m_t = max(f + m_{t-1}, i);   S_t = exp(f + m_{t-1} - m_t) S_{t-1} + exp(i - m_t) k v^T;   n_t likewise with k
        y = S_t^T q / (max(|n_t . q|, exp(-m_t)) + 1e-6)

    Every head's y is divided by its root mean square (``norm_eps``); the heads side by side are multiplied by a
    weight [H dv] and by sigmoid(W_g h), and projected.  S [H, d, dv], n and m are float32 state of every sequence
    (two ``StateSpec``s: S, and n with m behind it), carried from step to step; gates, decays and the recurrence are
    float32 whatever the matrices' type.  With the maxima m_t known (one short chain per head) the recurrence of S and n is
    linear, and a 16-bit model walks a long prompt in segments side by side (each twice: for what it adds to the state, then
    from the state before it).  The six input projections are one product against [Wq; Wk; Wv; Wg; Wi; Wf].
    ``names``: local tensor names."""

    takes_lazy_norm = True

    def __init__(self, *, hidden_size, n_heads, head_dim, v_head_dim, gate_cap, norm_eps, names=None, position=None,
                 prefix, dtype, device):
        if not (1 <= head_dim <= 256 and v_head_dim >= 1 and n_heads >= 1):
            raise ValueError(f"mlstm: head sizes {head_dim} / {v_head_dim} (keys up to 256 wide)")
        if not gate_cap > 0:
            raise ValueError("mlstm: a positive gate cap")
        self.hidden_size, self.n_heads, self.head_dim, self.v_head_dim = hidden_size, n_heads, head_dim, v_head_dim
        self.gate_cap, self.norm_eps = float(gate_cap), float(norm_eps)
        self.names = {**_NAMES, **(names or {})}
        self.prefix, self.dtype, self.device = prefix, dtype, device
        self.w_in = self.wo = self.norm = self.i_bias = self.f_bias = None

    def params(self):
        H, d, dv, w, n = self.n_heads, self.head_dim, self.v_head_dim, self.hidden_size, self.names
        return {n["q"]: ParamSpec((H * d, w)), n["k"]: ParamSpec((H * d, w)), n["v"]: ParamSpec((H * dv, w)),
                n["g"]: ParamSpec((H * dv, w)), n["i"]: ParamSpec((H, w)), n["f"]: ParamSpec((H, w)),
                n["i_bias"]: ParamSpec((H,), "vector", "small"), n["f_bias"]: ParamSpec((H,), "vector", "ones"),
                n["norm"]: ParamSpec((H * dv,), "vector", "ones"), n["o"]: ParamSpec((w, H * dv))}

    def bind(self, tensors):
        n = self.names
        self.w_in = ops.prepare_weight(torch.cat([tensors[n[k]] for k in ("q", "k", "v", "g", "i", "f")], 0).contiguous())
        self.wo = ops.prepare_weight(tensors[n["o"]])
        self.norm, self.i_bias, self.f_bias = tensors[n["norm"]], tensors[n["i_bias"]], tensors[n["f_bias"]]

    def cache_specs(self):
        return [StateSpec((self.n_heads, self.head_dim, self.v_head_dim), "float32"),
                StateSpec((self.n_heads, self.head_dim + 1), "float32")]

    def forward(self, h, ctx, views, residual, owns_cache=True):
        if not owns_cache:
            raise ValueError("a matrix memory keeps a state of its own in every run")
        H, d, dv = self.n_heads, self.head_dim, self.v_head_dim
        proj = ops.linear(h, self.w_in, out_dtype=torch.float32)
        k_col, v_col = H * d, 2 * H * d
        g_col = v_col + H * dv
        i_col = g_col + H * dv
        # a 16-bit model walks long prompts in segments side by side; a float32 model (and every decode step) walks each
        # sequence in order, which gives the same bits however a prompt is cut
        segments = None
        if self.dtype != torch.float32 and not ctx.is_decode and getattr(ctx, "host_qlens", None):
            waves_a_token = H * ((dv + 63) // 64)
            length = max(16, min(ops.SSM_SEGMENT, 1 << max(0, (ctx.n_tokens * waves_a_token // ops.SSM_WAVES).bit_length() - 1)))
            if max(ctx.host_qlens) > length:
                segments = ops.ssm_segments(ctx, length)
        y = ops.mlstm_scan(proj, 0, k_col, v_col, i_col, i_col + H, self.i_bias, self.f_bias, self.gate_cap, float(d) ** -0.5,
                           views[0].state, views[1].state, ctx, H, d, dv, segments)
        a = ops.gated_head_norm(y, self.norm, proj, g_col, H, self.norm_eps, self.dtype)
        ops.linear(a, self.wo, ops.EPI_ADD, out=residual)
