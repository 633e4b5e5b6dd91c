from __future__ import annotations

import torch

from ..cache.specs import KVSpec
from ..kernels import ops
from ..registry import register_mixer
from ..weights.loader import ParamSpec
from .base import Part

_NAMES = {"q": "q_proj.weight", "dkv": "kv_down.weight", "kv_norm": "kv_norm.weight", "uk": "k_up.weight",
          "uv": "v_up.weight", "o": "o_proj.weight", "sink": "sink", "g": "g_proj.weight"}


@register_mixer("latent_attention")
class LatentAttention(Part):
    """Causal softmax attention whose keys and values are up-projections of one small latent per token.  With H
    heads, ``head_dim`` d unrotated and ``rot_dim`` rd rotated query/key dimensions a head, values ``v_head_dim`` dv
    wide and a latent of ``kv_rank`` r:

        q = W_q h  (per head [d | rd]);   W_dkv h = [c_raw (r) | k_rot (rd)];   c = N(c_raw) * w_c
        k_h = [W_uk,h c | rot(k_rot)],  v_h = W_uv,h c;   score = (q_h[:d] . W_uk,h c + rot(q_h[d:]) . rot(k_rot)) * scale

    N divides by the root mean square (``norm_eps``), k_rot is shared by all heads, and rot turns the rotated part by
    the layer's position part (its frequencies and rotated dimensions; adjacent pairs).  ``sink``: every head's
    softmax sum also counts exp(sink[h]), a learned score with no key and no value that is not scaled.
    ``gate``: the heads' outputs side by side are multiplied by sigmoid(W_g h) before the output product.

    Only c and k_rot are cached.  The key's up-projection is taken into the query, q'_h = W_uk,h^T q_h[:d], so that a
    score is q'_h . c + q_rot . k_rot, and the value's is taken out of the weighted sum, o_h = W_uv,h (sum_j p_j c_j):
    all heads read one key [c | k_rot] and one value c per token, which the pages hold in the matrix cores' operand
    order (the cache layout of ``diff_attention`` with one map and one key/value head).  The input products are one
    product against [W_q; W_dkv; W_g].  Scores, weights, the norm and the angles are float32 whatever the matrices'
    type.  ``names``: local tensor names."""

    takes_lazy_norm = True

    def __init__(self, *, hidden_size, n_heads, head_dim, rot_dim, v_head_dim, kv_rank, scale, norm_eps, sink=False,
                 gate=False, window=None, names=None, position=None, prefix, dtype, device):
        if min(n_heads, v_head_dim, kv_rank) < 1 or head_dim < 0 or rot_dim < 0 or head_dim + rot_dim < 1:
            raise ValueError("latent attention: positive sizes")
        if kv_rank > 512:
            raise ValueError(f"latent attention: a latent of {kv_rank} (the kernels take up to 512)")
        self.hidden_size, self.n_heads, self.head_dim, self.rot_dim = hidden_size, n_heads, head_dim, rot_dim
        self.v_head_dim, self.kv_rank = v_head_dim, kv_rank
        self.scale, self.norm_eps = float(scale), float(norm_eps)
        self.sink, self.gate = bool(sink), bool(gate)
        self.window = None if window is None else int(window)
        self.position = position
        self.names = {**_NAMES, **(names or {})}
        self.prefix, self.dtype, self.device = prefix, dtype, device
        rot = getattr(position, "rotary_dim", 0) if position is not None else 0
        if rot > rot_dim or rot % 2:
            raise ValueError(f"latent attention: {rot} rotated dimensions in a rotated part of {rot_dim}")
        if rot and getattr(position, "pairing", "adjacent") != "adjacent":
            raise ValueError("latent attention rotates adjacent pairs")
        self.rot = rot
        self.key_dim = kv_rank + rot_dim                          # of the one key that all heads read
        self.w_in = self.wo = self.w_uk = self.w_uv = self.kv_norm = self.sinks = None

    def params(self):
        H, d, rd, dv, r, w, n = self.n_heads, self.head_dim, self.rot_dim, self.v_head_dim, self.kv_rank, self.hidden_size, self.names
        out = {n["q"]: ParamSpec((H * (d + rd), w)), n["dkv"]: ParamSpec((r + rd, w)),
               n["kv_norm"]: ParamSpec((r,), "vector", "ones"), n["uk"]: ParamSpec((H * d, r)),
               n["uv"]: ParamSpec((H * dv, r)), n["o"]: ParamSpec((w, H * dv))}
        if self.sink:
            out[n["sink"]] = ParamSpec((H,), "vector", "small")
        if self.gate:
            out[n["g"]] = ParamSpec((H * dv, w))
        return out

    def bind(self, tensors):
        n, H, d, dv, r = self.names, self.n_heads, self.head_dim, self.v_head_dim, self.kv_rank
        rows = [tensors[n["q"]], tensors[n["dkv"]]] + ([tensors[n["g"]]] if self.gate else [])
        self.w_in = ops.prepare_weight(torch.cat(rows, 0).contiguous())
        self.wo = ops.prepare_weight(tensors[n["o"]])
        # the products per head keep their matrices [H, outputs, inputs]: W_uk turned (a head's d rows of r are its inputs), W_uv as stored
        # (in the model's type also where the file stores them wider: their products run beside 16-bit queries and sums)
        self.w_uk = tensors[n["uk"]].as_subclass(torch.Tensor).view(H, d, r).transpose(1, 2).to(self.dtype).contiguous() if d else None
        self.w_uv = tensors[n["uv"]].as_subclass(torch.Tensor).view(H, dv, r).to(self.dtype).contiguous()
        self.kv_norm = tensors[n["kv_norm"]]
        self.sinks = tensors[n["sink"]] if self.sink else None

    def cache_spec(self):
        return KVSpec(1, ops.padded_map_dim(self.key_dim), self.window, self.kv_rank, None, "maps")

    def forward(self, h, ctx, view, residual, owns_cache=True):
        if not owns_cache:
            raise ValueError("latent attention writes its own latents in every run")
        H, d, rd, dv, r = self.n_heads, self.head_dim, self.rot_dim, self.v_head_dim, self.kv_rank
        proj = ops.linear(h, self.w_in, out_dtype=torch.float32)
        kv = view.as_tuple()
        kv_col = H * (d + rd)
        q = ops.latent_store(proj, 0, kv_col, self.kv_norm, self.norm_eps, getattr(self.position, "inv_freq", None), self.rot,
                             ctx.pos, ctx.tok_slot, kv, H, d, rd, r)
        kw = q.shape[2]
        if d:
            ops.head_linear(proj, 0, d + rd, self.w_uk, q, 0, kw)              # q' into the first r columns of every head
        else:
            q[:, :, :r].zero_()
        sixteen = self.dtype != torch.float32 and ops.diff_attention_fits(self.key_dim, r)
        a = ops.diff_attention(q, kv, ctx.pos, ctx.tok_slot, H, 1, 1, self.key_dim, r, self.scale, None, self.window, 0.0, None,
                               1.0, self.dtype, ops.diff_tiles(ctx, None, self.window) if sixteen else None, sink=self.sinks,
                               key_shares=ctx.decode_splits(1, H) if sixteen and ctx.is_decode else 1)
        o = torch.empty((a.shape[0], H * dv), dtype=self.dtype, device=a.device)
        ops.head_linear(a, 0, r, self.w_uv, o, 0, dv, gate=proj if self.gate else None, gate_col=kv_col + r + rd)
        ops.linear(o, self.wo, ops.EPI_ADD, out=residual)
