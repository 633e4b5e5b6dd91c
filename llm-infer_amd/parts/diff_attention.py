from __future__ import annotations

import math

import torch

from ..cache.specs import KVSpec
from ..kernels import ops
from ..registry import register_mixer
from ..weights.loader import ParamSpec
from .base import Part

_NAMES = {"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight", "o": "o_proj.weight",
          "q_norm": "q_norm.weight", "k_norm": "k_norm.weight",
          "lq1": "lambda_q1", "lk1": "lambda_k1", "lq2": "lambda_q2", "lk2": "lambda_k2"}


@register_mixer("diff_attention")
class DifferentialAttention(Part):
    """Causal grouped-query attention made of ``maps`` softmax maps (2: differential attention; 1: plain) over
    the same values.  Wq has H * maps * d rows and Wk G * maps * d, head by head with a head's maps side by
    side; values are G * dv wide; query head h reads key/value head h // (H / G).  Per head

        a_m = softmax(q_m . k_m * scale) v   (m = 1, 2; the visible keys only)
        o   = a_1 - lambda a_2,   lambda = exp(lq1 . lk1) - exp(lq2 . lk2) + lambda_init

    with lq1, lk1, lq2, lk2 four tensors of size d, so lambda is one number of the layer.  ``qk_norm_eps`` not
    None: every map of every q and k head is first divided by its root mean square over d and multiplied by a
    weight of size d (one for q, one for k, shared by heads and maps).  ``out_norm_eps`` not None: o is divided
    by its root mean square over dv (no weight) and multiplied by ``out_scale``.  No rotation: positions enter
    only through what is visible.  ``block`` b: position i sees j <= i with j // b == i // b, blocks counted
    from position 0 of the sequence (None: every j <= i); ``window`` w: at most the last w positions.
    Scores, weights and all norms are float32 whatever the matrices' type.

    The three input projections are one product against [Wq; Wk; Wv].  The cache keeps, for every token, the
    normed keys of all maps side by side (each padded to a multiple of 16) and the values, in the matrix cores'
    operand order; pages behind the newest token's block are given back.  A 16-bit model runs prompts and decode
    steps through one matrix-core kernel, compiled for the pair of head sizes at first use; a float32 model runs
    one workgroup per (token, head).
    ``names``: local tensor names."""

    takes_lazy_norm = True

    def __init__(self, *, hidden_size, n_heads, n_kv_heads, head_dim, v_head_dim=None, scale, maps=2, lambda_init=0.0,
                 qk_norm_eps=None, out_norm_eps=None, out_scale=1.0, block=None, window=None, names=None, position=None,
                 prefix, dtype, device):
        if n_heads % n_kv_heads != 0:
            raise ValueError("n_heads must be a multiple of n_kv_heads")
        if maps not in (1, 2):
            raise ValueError(f"differential attention has one or two maps, not {maps}")
        v_head_dim = v_head_dim or head_dim
        if not 1 <= v_head_dim <= 256 or head_dim < 1:
            raise ValueError(f"head sizes {head_dim} / {v_head_dim}: values up to 256 wide")
        if block is not None and int(block) < 1:
            raise ValueError("block: a positive number of positions")
        self.hidden_size, self.n_heads, self.n_kv_heads = hidden_size, n_heads, n_kv_heads
        self.head_dim, self.v_head_dim, self.maps = head_dim, v_head_dim, maps
        self.scale, self.lambda_init = float(scale), float(lambda_init)
        self.qk_norm_eps = None if qk_norm_eps is None else float(qk_norm_eps)
        self.out_norm_eps = None if out_norm_eps is None else float(out_norm_eps)
        self.out_scale = float(out_scale)
        self.block = None if block is None else int(block)
        self.window = None if window is None else int(window)
        self.names = {**_NAMES, **(names or {})}
        self.prefix, self.dtype, self.device = prefix, dtype, device
        self.w_in = self.wo = self.q_norm = self.k_norm = None
        self.lam = 0.0

    def params(self):
        H, G, d, dv, w, n, m = (self.n_heads, self.n_kv_heads, self.head_dim, self.v_head_dim, self.hidden_size, self.names,
                                self.maps)
        out = {n["q"]: ParamSpec((H * m * d, w)), n["k"]: ParamSpec((G * m * d, w)), n["v"]: ParamSpec((G * dv, w)),
               n["o"]: ParamSpec((w, H * dv))}
        if self.qk_norm_eps is not None:
            out[n["q_norm"]] = ParamSpec((d,), "vector", "ones")
            out[n["k_norm"]] = ParamSpec((d,), "vector", "ones")
        if m == 2:
            for key in ("lq1", "lk1", "lq2", "lk2"):
                out[n[key]] = ParamSpec((d,), "vector", "small")
        return out

    def bind(self, tensors):
        n = self.names
        self.w_in = ops.prepare_weight(torch.cat([tensors[n["q"]], tensors[n["k"]], tensors[n["v"]]], 0).contiguous())
        self.wo = ops.prepare_weight(tensors[n["o"]])
        if self.qk_norm_eps is not None:
            self.q_norm, self.k_norm = tensors[n["q_norm"]], tensors[n["k_norm"]]
        if self.maps == 2:
            dot = lambda a, b: float((tensors[n[a]].float() * tensors[n[b]].float()).sum(dtype=torch.float32))
            f32 = lambda v: float(torch.tensor(v, dtype=torch.float32))
            self.lam = f32(f32(math.exp(dot("lq1", "lk1"))) - f32(math.exp(dot("lq2", "lk2"))) + self.lambda_init)

    def cache_spec(self):
        return KVSpec(self.n_kv_heads, self.maps * ops.padded_map_dim(self.head_dim), self.window, self.v_head_dim, self.block,
                      "maps")

    def _key_shares(self, ctx) -> int:
        """Workgroups that share a token's keys in a decode step of a 16-bit model (a block bounds what a token sees)."""
        if self.dtype == torch.float32 or not ctx.is_decode:
            return 1
        shares = ctx.decode_splits(self.n_kv_heads, self.n_heads)
        if self.block:
            shares = min(shares, max(1, self.block // 128))
        return shares

    def forward(self, h, ctx, view, residual, owns_cache=True):
        if not owns_cache:
            raise ValueError("differential attention writes its own keys and values in every run")
        H, G, d, dv, m = self.n_heads, self.n_kv_heads, self.head_dim, self.v_head_dim, self.maps
        proj = ops.linear(h, self.w_in, out_dtype=torch.float32)
        kv = view.as_tuple()
        q = ops.qk_norm_store(proj, 0, self.q_norm, self.k_norm, self.qk_norm_eps, ctx.pos, ctx.tok_slot, kv, H, G, m, d, dv)
        a = ops.diff_attention(q, kv, ctx.pos, ctx.tok_slot, H, G, m, d, dv, self.scale, self.block, self.window, self.lam,
                               self.out_norm_eps, self.out_scale, self.dtype,
                               ops.diff_tiles(ctx, self.block, self.window) if self.dtype != torch.float32 else None,
                               key_shares=self._key_shares(ctx))
        ops.linear(a, self.wo, ops.EPI_ADD, out=residual)
