from __future__ import annotations

import torch

from ..cache.specs import KVSpec, StateSpec
from ..kernels import ops
from ..registry import register_mixer
from ..weights.loader import ParamSpec
from .base import Part

_NAMES = {"q": "q_proj.weight", "k": "k_proj.weight", "v": "v_proj.weight", "o": "o_proj.weight", "g": "g_proj.weight",
          "sink": "sink", "q_bias": "q_proj.bias", "k_bias": "k_proj.bias", "v_bias": "v_proj.bias",
          "q_conv": "q_conv.weight", "k_conv": "k_conv.weight", "v_conv": "v_conv.weight"}


@register_mixer("gated_attention")
class GatedAttention(Part):
    """Causal grouped-query softmax attention with a learned sink in every head's sum, a sigmoid gate on every head's
    output and keys and values of sizes of their own.  With H query heads on G key/value heads (query head h reads
    key/value head h // (H / G)), keys ``head_dim`` d and values ``v_head_dim`` dv wide, per head

        p_j = exp(s_j) / (exp(sink_h) + sum over the visible j' of exp(s_j')),   s_j = q . k_j * scale - slope_h (i - j)
        o_h = sigmoid(W_g x)_h * sum_j p_j v_j,      out = W_o [o_1 .. o_H]

    The sink has no key and no value, is not scaled and gets no bias.  What is visible from position i: j <= i, with
    ``window`` w only i - j < w, with ``block`` b only the j of i's own block of b positions (counted from position 0).
    ``sink`` / ``gate`` False leave those out.  Variants, all parameters:

    * ``values`` "keys": there is no value projection; a token's values are its keys as projected, before any rotation.
    * the layer's position part (``rope_half``): q and k are turned in their first ``rotary_dim`` dimensions, i paired
      with i + rotary_dim / 2; values never are.
    * ``bias``: q, k and v have biases, added in the projection.
    * ``conv_taps`` n > 0: a causal convolution over time, channel by channel, directly behind the projection of q, k
      and v (weights [channels, n], the last column the current token's; zeros before a sequence's first token).  The
      last n - 1 projected rows of every sequence are state of the cache.
    * ``slope_exponent`` c: slope_h = 2^(-c (h + 1) / H) (None: no bias by distance).
    * ``reads_kv``: the layer has no key and value tensors and reads the cache of another run (its schedule entry's
      ``cache_from``), whose mixer has the same head counts; its own queries, mask, sink, gate and output.
    * ``keep_window`` / ``keep_block``: what the cache may give back (default: what this layer's own mask lets go of;
      a layer whose cache another layer reads with another mask keeps what both need).

    The input products are one product against [W_q; W_k; W_v; W_g].  The cache keeps keys (after rotation or
    convolution) and values in the matrix cores' operand order (one map of keys: the layout that the softmax decoder's
    kernels read too).  A 16-bit model whose keys and values have one size that is a multiple of 16 runs prompts
    through the softmax decoder's prompt kernel (``ops.attention_prefill``, which takes the sink, the slopes, the
    blocks and the gate); every other size, and every decode step, runs through the matrix-core kernel of
    ``diff_attention`` with one map; a float32 model runs one workgroup per (token, head).
    Scores, weights, angles, the sink and the gate are float32 whatever the matrices' type.  ``names``: local tensor
    names."""

    writes_rows = True          # forward_into overwrites the rows it is handed

    def __init__(self, *, hidden_size, n_heads, n_kv_heads, head_dim, v_head_dim=None, scale, window=None, block=None,
                 sink=True, gate=True, values="own", bias=False, conv_taps=0, slope_exponent=None, reads_kv=False,
                 keep_window="own", keep_block="own", names=None, position=None, prefix, dtype, device):
        if n_heads % n_kv_heads != 0:
            raise ValueError("n_heads must be a multiple of n_kv_heads")
        if values not in ("own", "keys"):
            raise ValueError("gated attention: values 'own' or 'keys'")
        v_head_dim = v_head_dim or head_dim
        if values == "keys" and v_head_dim != head_dim:
            raise ValueError("gated attention: values that are the keys have the keys' size")
        if not 1 <= v_head_dim <= 512 or head_dim < 1:
            raise ValueError(f"head sizes {head_dim} / {v_head_dim}: values up to 512 wide")
        if not 0 <= conv_taps <= 16:
            raise ValueError(f"gated attention: a convolution over {conv_taps} tokens (up to 16)")
        for name, v in (("window", window), ("block", block)):
            if v is not None and int(v) < 1:
                raise ValueError(f"{name}: a positive number of positions")
        self.hidden_size, self.n_heads, self.n_kv_heads = hidden_size, n_heads, n_kv_heads
        self.head_dim, self.v_head_dim, self.scale = head_dim, v_head_dim, float(scale)
        self.window = None if window is None else int(window)
        self.block = None if block is None else int(block)
        self.keep_window = self.window if keep_window == "own" else (None if keep_window is None else int(keep_window))
        self.keep_block = self.block if keep_block == "own" else (None if keep_block is None else int(keep_block))
        self.sink, self.gate, self.values_are_keys, self.bias = bool(sink), bool(gate), values == "keys", bool(bias)
        self.conv_taps, self.reads_kv = int(conv_taps), bool(reads_kv)
        self.slope_exponent = None if slope_exponent is None else float(slope_exponent)
        self.position = position
        self.rot = int(getattr(position, "rotary_dim", 0) or 0) if position is not None else 0
        if self.rot and (getattr(position, "pairing", None) != "half" or self.rot > head_dim or self.rot % 2):
            raise ValueError("gated attention turns an even number of half-paired dimensions within the head ('rope_half')")
        self.names = {**_NAMES, **(names or {})}
        self.prefix, self.dtype, self.device = prefix, dtype, device
        # the columns of the input product: q | k | v | g (k and v only where the layer has them)
        H, G, d, dv = n_heads, 0 if reads_kv else n_kv_heads, head_dim, v_head_dim
        self.q_col, self.k_col = 0, H * d
        self.v_col = self.k_col if self.values_are_keys else self.k_col + G * d
        self.channels = H * d + G * d + (0 if self.values_are_keys else G * dv)      # what biases and convolution cover
        self.gate_col = self.channels
        if self.conv_taps:
            self.keeps_when_reading = (0,)       # the convolution's history is the layer's own whatever keys it reads
        self.w_in = self.wo = self.b_in = self.conv = self.sinks = self.slopes = None

    def _kv_names(self):
        return [] if self.reads_kv else (["k"] if self.values_are_keys else ["k", "v"])

    def params(self):
        H, G, d, dv, w, n = self.n_heads, self.n_kv_heads, self.head_dim, self.v_head_dim, self.hidden_size, self.names
        rows = {"q": H * d, "k": G * d, "v": G * dv}
        out = {n["o"]: ParamSpec((w, H * dv))}
        for key in ["q"] + self._kv_names():
            out[n[key]] = ParamSpec((rows[key], w))
            if self.bias:
                out[n[key + "_bias"]] = ParamSpec((rows[key],), "vector", "small")
            if self.conv_taps:
                out[n[key + "_conv"]] = ParamSpec((rows[key], self.conv_taps), "vector", "wide")
        if self.sink:
            out[n["sink"]] = ParamSpec((H,), "vector", "small")
        if self.gate:
            out[n["g"]] = ParamSpec((H, w))
        return out

    def bind(self, tensors):
        n, keys = self.names, ["q"] + self._kv_names()
        plain = lambda t: t.as_subclass(torch.Tensor)
        rows = [tensors[n[k]] for k in keys] + ([tensors[n["g"]]] if self.gate else [])
        self.w_in = ops.prepare_weight(torch.cat(rows, 0).contiguous())
        self.wo = ops.prepare_weight(tensors[n["o"]])
        if self.bias:
            # a bias for every column of the one input product: those of q, k and v, none for the gate's
            b = torch.cat([plain(tensors[n[k + "_bias"]]).float() for k in keys])
            pad = torch.zeros(self.n_heads if self.gate else 0, dtype=torch.float32, device=b.device)
            self.b_in = ops.glu_params(torch.cat([b, pad]).contiguous())
        if self.conv_taps:
            self.conv = torch.cat([plain(tensors[n[k + "_conv"]]).float() for k in keys], 0).contiguous()
        self.sinks = tensors[n["sink"]] if self.sink else None
        if self.slope_exponent is not None:
            H = self.n_heads
            self.slopes = torch.tensor([2.0 ** (-self.slope_exponent * (h + 1) / H) for h in range(H)], dtype=torch.float64) \
                .to(torch.float32).to(self.wo.device)

    def cache_specs(self):
        kv = KVSpec(self.n_kv_heads, ops.padded_map_dim(self.head_dim), self.keep_window, self.v_head_dim, self.keep_block, "maps")
        if self.conv_taps:
            return [StateSpec((max(self.conv_taps - 1, 1), self.channels), "float32"), kv]
        return [kv]

    def _key_shares(self, ctx) -> int:
        """Workgroups that share a token's keys in a decode step of a 16-bit model (a mask bounds what a token sees)."""
        if self.dtype == torch.float32 or not ctx.is_decode:
            return 1
        # the step counts one wave a (sequence, key/value head, split); here each of those is a workgroup of four waves
        # (measured at 32/8 heads and a mask of 1,024: batch 8 0.82 -> 0.80 ms a step, batch 32 1.06 -> 0.99)
        shares = max(1, ctx.decode_splits(self.n_kv_heads, self.n_heads) // 4)
        for span in (self.block, self.window):
            if span:
                shares = min(shares, max(1, span // 128))
        return shares

    def _splits(self, ctx) -> int:
        """Splits of the keys for the softmax decoder's decode kernel: what the step asks for, but at least two pages a
        split of what the mask leaves (a power of two)."""
        splits = ctx.decode_splits(self.n_kv_heads, self.n_heads)
        for span in (self.block, self.window):
            if span:
                splits = min(splits, max(1, span // 128))
        return 1 << (splits.bit_length() - 1)

    def attend(self, h, ctx, views, owns_cache):
        """The heads' gated outputs side by side, [T, H * dv] in the model's type."""
        if owns_cache == self.reads_kv:
            raise ValueError("gated attention: a layer without key and value tensors reads another run's cache, and only such a layer")
        H, G, d, dv = self.n_heads, self.n_kv_heads, self.head_dim, self.v_head_dim
        kv = views[-1].as_tuple()
        if self.bias:
            proj = ops.linear(h, self.w_in, ops.EPI_BIAS, out_dtype=torch.float32, params=self.b_in)
        else:
            proj = ops.linear(h, self.w_in, out_dtype=torch.float32)
        # the convolution rides in the kernel that turns and stores; the history is brought up to date behind it
        conv = (self.conv, views[0].state) if self.conv_taps else None
        q = ops.rot_store(proj, self.q_col, self.k_col, self.v_col, getattr(self.position, "inv_freq", None) if self.rot else None,
                          self.rot, ctx.pos, ctx.tok_slot, kv, H, 0 if self.reads_kv else G, d, dv, kv[0].dtype, conv)
        if self.conv_taps > 1:
            ops.conv_history(proj, 0, self.channels, self.conv_taps, views[0].state, ctx)
        if self.dtype != torch.float32 and d == dv and d % 16 == 0 and d <= 256:
            # a 16-bit model whose keys and values have one size the kernels take as it is: the softmax decoder's own
            # kernels (prompts: pages through LDS, scores of the next page under the weights of this one; decode steps:
            # a wave per (sequence, key/value head, split of the keys that the mask leaves))
            gate = proj if self.gate else None
            if ctx.is_decode:
                a = ops.attention_decode(q, kv, ctx.seq_slot, ctx.seq_ctx, ctx.n_seqs, H, G, d, self.scale, self.window,
                                         self._splits(ctx), self.block, self.sinks, self.slopes, gate, self.gate_col)
            else:
                a = ops.attention_prefill(q, kv, ops.prefill_meta(ctx), H, G, d, self.scale, self.window, self.block, self.sinks,
                                          self.slopes, gate, self.gate_col)
            return a.view(a.shape[0], H * dv)
        sixteen = self.dtype != torch.float32 and ops.diff_attention_fits(d, dv)
        return ops.diff_attention(q, kv, ctx.pos, ctx.tok_slot, H, G, 1, d, dv, self.scale, self.block, self.window, 0.0, None, 1.0,
                                  self.dtype, ops.diff_tiles(ctx, self.block, self.window) if sixteen else None, sink=self.sinks,
                                  key_shares=self._key_shares(ctx) if sixteen else 1, slopes=self.slopes,
                                  gate=proj if self.gate else None, gate_col=self.gate_col)

    def forward(self, h, ctx, views, residual, owns_cache=True):
        ops.linear(self.attend(h, ctx, views, owns_cache), self.wo, ops.EPI_ADD, out=residual)

    def forward_into(self, h, out, ctx, views, owns_cache=True):
        """The mixer's result written over the float32 rows ``out`` (nothing is added to what they held)."""
        ops.linear(self.attend(h, ctx, views, owns_cache), self.wo, out=out)
        return None
