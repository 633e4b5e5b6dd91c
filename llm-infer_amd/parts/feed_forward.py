from __future__ import annotations

import torch

from ..kernels import ops
from ..registry import register_feed_forward
from ..tensor import Tensor
from ..weights.loader import ParamSpec
from .base import Part


@register_feed_forward("gated_mlp")
class GatedMLP(Part):
    """down(act(gate(x)) * up(x)) added into the residual stream; act is silu, x / (1 + exp(-x)), or
    gelu in the tanh form the reference computes (src/model/block.cpp:200-222,
    include/kernels_cpu.hpp:179-186).

    Gate and up rows are interleaved into one matrix (row 2j = gate_j, row 2j+1 = up_j),
    so that one product yields both and its epilogue applies the activation before
    anything is written; each row's sum is what it would be alone.

    ``activation`` "clamped_swish": with g = min(gate, ``limit``) and u = clamp(up, -limit, limit) the hidden row is
    g sigmoid(``alpha`` g) (u + ``up_shift``), computed in float32 on the product's sums.  ``bias``: gate, up and down
    have biases, added in their products.
    """

    takes_lazy_norm = True      # the normed input goes to ops.linear as it comes
    writes_rows = True          # forward_into overwrites the rows it is handed

    def __init__(self, *, hidden_size, intermediate_size, activation="silu", limit=None, alpha=1.702, up_shift=1.0,
                 bias=False, names=None, prefix, dtype, device):
        """``names``: local tensor names for gate, up and down (and gate_bias, up_bias, down_bias)."""
        self.names = {"gate": "gate_proj.weight", "up": "up_proj.weight", "down": "down_proj.weight",
                      "gate_bias": "gate_proj.bias", "up_bias": "up_proj.bias", "down_bias": "down_proj.bias", **(names or {})}
        if activation not in ("silu", "gelu", "clamped_swish"):
            raise ValueError(f"gated_mlp: activation {activation!r} is not built (silu and gelu are, and clamped_swish with a limit)")
        self.clamped = activation == "clamped_swish"
        if self.clamped and not (limit is not None and float(limit) > 0):
            raise ValueError("gated_mlp: the clamped activation needs a positive limit")
        if bias and not self.clamped:
            raise ValueError("gated_mlp: biases are built for the clamped activation")
        self.mode = ops.EPI_GEGLU if activation == "gelu" else ops.EPI_SWIGLU
        self.limit, self.alpha, self.up_shift = float(limit or 0.0), float(alpha), float(up_shift)
        self.bias = bool(bias)
        self.hidden_size, self.intermediate_size = hidden_size, intermediate_size
        self.prefix, self.dtype, self.device = prefix, dtype, device
        self.w_gate_up = self.w_down = self.b_gate_up = self.b_down = None

    def params(self):
        f, d = self.intermediate_size, self.hidden_size
        n = self.names
        out = {n["gate"]: ParamSpec((f, d)), n["up"]: ParamSpec((f, d)), n["down"]: ParamSpec((d, f))}
        if self.bias:
            out.update({n["gate_bias"]: ParamSpec((f,), "vector", "small"), n["up_bias"]: ParamSpec((f,), "vector", "small"),
                        n["down_bias"]: ParamSpec((d,), "vector", "small")})
        return out

    def bind(self, tensors):
        g, u = tensors[self.names["gate"]], tensors[self.names["up"]]
        if g.dtype != u.dtype:
            g, u = g.float(), u.float()
        gu = torch.stack([g, u], dim=1).reshape(2 * self.intermediate_size, self.hidden_size).contiguous()
        self.w_gate_up = ops.prepare_weight(gu)
        self.w_down = ops.prepare_weight(tensors[self.names["down"]])
        if self.bias:
            plain = lambda name: tensors[self.names[name]].as_subclass(torch.Tensor).float()
            self.b_gate_up = torch.stack([plain("gate_bias"), plain("up_bias")], dim=1).reshape(-1).contiguous()   # interleaved as the rows are
            self.b_down = plain("down_bias").contiguous()
        if self.clamped:
            self.glu = ops.glu_params(self.b_gate_up, self.limit, None, self.alpha, self.up_shift)

    def _hidden(self, h):
        if not self.clamped:
            return ops.linear(h, self.w_gate_up, self.mode, out_dtype=self.dtype)
        # biases, clamps and the activation on the product's float32 sums, in its epilogue
        return ops.linear(h, self.w_gate_up, ops.EPI_CLAMPGLU, out_dtype=self.dtype, params=self.glu)

    def forward(self, h, residual):
        ops.linear(self._hidden(h), self.w_down, ops.EPI_ADD, out=residual)
        if self.b_down is not None:
            ops.add_bias(residual, 0, self.b_down)

    def forward_into(self, h, out, ctx=None, view=None, owns_cache=True):
        """The result written over the float32 rows ``out``; returns the bias that is still to be added to them (or None)."""
        ops.linear(self._hidden(h), self.w_down, out=out)
        return self.b_down


@register_feed_forward("poly_mlp")
class PolyNormMLP(Part):
    """down(PolyNorm(up(x))): no gate.  PolyNorm(z) = a N(z) + b N(z^2) + c N(z^3) + e with the powers taken
    element by element and N the division of a token's vector by its root mean square (``eps`` inside the
    root), computed in float32; (a, b, c, e) are the four numbers of the tensor ``names["act"]``."""

    def __init__(self, *, hidden_size, intermediate_size, eps, names=None, prefix, dtype, device):
        self.hidden_size, self.intermediate_size, self.eps = hidden_size, intermediate_size, float(eps)
        self.names = {"up": "up_proj.weight", "down": "down_proj.weight", "act": "act", **(names or {})}
        self.prefix, self.dtype, self.device = prefix, dtype, device
        self.w_up = self.w_down = self.coef = None

    def params(self):
        f, d, n = self.intermediate_size, self.hidden_size, self.names
        return {n["up"]: ParamSpec((f, d)), n["down"]: ParamSpec((d, f)), n["act"]: ParamSpec((4,), "vector", "ones")}

    def bind(self, tensors):
        n = self.names
        self.w_up, self.w_down = ops.prepare_weight(tensors[n["up"]]), ops.prepare_weight(tensors[n["down"]])
        self.coef = tensors[n["act"]]

    def addends(self, h):
        z = ops.linear(h, self.w_up, out_dtype=torch.float32)
        a = ops.polynorm(z, self.coef, self.eps, self.dtype)
        return [(ops.linear(a, self.w_down, out_dtype=torch.float32), 1.0)]

    def forward(self, h, residual):
        ops.linear(ops.polynorm(ops.linear(h, self.w_up, out_dtype=torch.float32), self.coef, self.eps, self.dtype),
                   self.w_down, ops.EPI_ADD, out=residual)


@register_feed_forward("dense_mlp")
class DenseMLP(Part):
    """down(act(up(x))) added into the residual stream: no gate.  ``activation``: "gelu" (the exact form with
    erf), "gelu_tanh" or "silu", computed in float32 on the product's sums.  ``names``: local tensor names."""

    takes_lazy_norm = True

    def __init__(self, *, hidden_size, intermediate_size, activation="gelu", names=None, prefix, dtype, device):
        if activation not in ops.ACTIVATIONS:
            raise ValueError(f"dense_mlp: activation {activation!r} is not built ({', '.join(ops.ACTIVATIONS)} are)")
        self.hidden_size, self.intermediate_size, self.activation = hidden_size, intermediate_size, activation
        self.names = {"up": "up_proj.weight", "down": "down_proj.weight", **(names or {})}
        self.prefix, self.dtype, self.device = prefix, dtype, device
        self.w_up = self.w_down = None

    def params(self):
        f, d, n = self.intermediate_size, self.hidden_size, self.names
        return {n["up"]: ParamSpec((f, d)), n["down"]: ParamSpec((d, f))}

    def bind(self, tensors):
        n = self.names
        self.w_up, self.w_down = ops.prepare_weight(tensors[n["up"]]), ops.prepare_weight(tensors[n["down"]])

    def forward(self, h, residual):
        z = ops.linear(h, self.w_up, out_dtype=torch.float32)
        ops.linear(ops.activation(z, self.activation, self.dtype), self.w_down, ops.EPI_ADD, out=residual)


@register_feed_forward("routed_experts")
class RoutedExperts(Part):
    """A mixture of ``n_experts`` gated feed-forwards down(silu(gate(h)) * up(h)) of width ``expert_ff`` (tensors
    ``e<i>.gate``, ``e<i>.up``, ``e<i>.down``), of which every token uses ``top``.  ``gated`` False: an expert is
    down(act(up(h))) with ``activation`` one of gelu, gelu_tanh, silu, relu2 (the square of relu), and has no gate
    matrix.  ``scores`` "sigmoid": s is the sigmoid of every router logit instead of their softmax; ``renormalize``
    False: a chosen expert's weight is its own s (times ``route_scale``), not divided by the sum of the chosen;
    ``weight_on`` "input": the weight multiplies what the expert reads, the result is the sum of expert(weight * h)
    (experts without a gate: their up product is linear, so the weight is applied to its sums, act(weight * up(h)),
    in float32).

    The router has n_experts + ``n_identity`` outputs; its logits and everything after them are float32:
    s = softmax(W_router h); the ``top`` outputs with the largest s + correction are chosen (``correction``: a
    tensor with one number an output, used for the choice only); their weights are s / (sum of the chosen s +
    1e-20) * ``route_scale``.  The last ``n_identity`` outputs have no matrices: chosen, they add weight * h.
    ``shared_ff`` > 0: one more expert of that width runs for every token; ``shared_gate``: it is weighted by
    sigmoid(w_sg . h).

    How it runs.  Few tokens (a decode step, a short prompt, and every step of a float32 model): the experts' gate
    and up matrices are stacked (the shared expert's behind them) into one product whose epilogue applies
    silu(gate) * up; every expert's block of the hidden row is multiplied by the token's weight for that expert,
    zero where it was not chosen; one product against the down matrices side by side then sums the experts.
    Every token so runs through every expert's matrices: the same numbers as running only the chosen ones, every
    matrix streamed once, no shapes that depend on the data (a step can be recorded), at n_experts / top times the
    arithmetic.  Many tokens in a 16-bit model (``GROUPED_FROM`` rows an expert on average): the tokens are listed
    by expert on the device, the host reads the eight or so counts, and every expert runs its own two products on
    its own tokens' rows, added into the residual rows expert by expert (a fixed order)."""

    # measured (eight experts of 3,584, two chosen, width 4,096): a prompt of 512 tokens 2.94 ms with every token
    # through every expert and 3.46 sorted by expert (40 launches a layer and a wait for the counts against 3 launches),
    # 1,024 tokens 4.90 and 4.86, 2,048 tokens 8.58 and 7.50
    GROUPED_FROM = 256

    def __init__(self, *, hidden_size, n_experts, expert_ff, top, n_identity=0, route_scale=1.0, correction=True,
                 shared_ff=0, shared_gate=True, gated=True, activation="silu", scores="softmax", renormalize=True,
                 weight_on="output", routing="router", vocab_size=0, limit=None, shared_limit=None, alpha=1.702,
                 up_shift=1.0, names=None, prefix, dtype, device):
        if not 1 <= top <= n_experts + n_identity:
            raise ValueError(f"routed experts: top {top} of {n_experts + n_identity} outputs")
        if scores not in ("softmax", "sigmoid") or weight_on not in ("output", "input"):
            raise ValueError("routed experts: scores 'softmax' or 'sigmoid', weight_on 'output' or 'input'")
        if routing not in ("router", "table"):
            raise ValueError("routed experts: routing 'router' or 'table'")
        if routing == "table" and (n_identity or correction or vocab_size < 1):
            raise ValueError("routed experts: a table names experts with matrices for every token id, without corrections")
        if gated and (activation not in ("silu", "clamped_swish") or weight_on != "output"):
            raise ValueError("routed experts: gated experts are built with silu or clamped_swish and the weight on their output")
        self.clamped = bool(gated) and activation == "clamped_swish"
        if self.clamped and not (limit is not None and float(limit) > 0):
            raise ValueError("routed experts: the clamped activation needs a positive limit")
        self.table_routing, self.vocab_size = routing == "table", int(vocab_size)
        self.takes_ctx = self.table_routing           # the token ids come with the step
        self.limit, self.alpha, self.up_shift = float(limit or 0.0), float(alpha), float(up_shift)
        self.shared_limit = self.limit if shared_limit is None else float(shared_limit)
        if not gated and activation not in ops.ACTIVATIONS:
            raise ValueError(f"routed experts: activation {activation!r} is not built ({', '.join(ops.ACTIVATIONS)} are)")
        self.gated, self.activation, self.sigmoid_scores = bool(gated), activation, scores == "sigmoid"
        self.renormalize, self.on_input = bool(renormalize), weight_on == "input"
        self.hidden_size, self.n_experts, self.expert_ff, self.top = hidden_size, n_experts, expert_ff, top
        self.n_identity, self.route_scale, self.correction = n_identity, float(route_scale), bool(correction)
        self.shared_ff, self.shared_gate = int(shared_ff or 0), bool(shared_gate) and bool(shared_ff)
        self.names = {"router": "router.weight", "correction": "router.correction", "expert": "e{}.", "shared": "shared.",
                      "gate": "gate", "up": "up", "down": "down", "shared_gate": "shared.sg", "table": "table", **(names or {})}
        self.prefix, self.dtype, self.device = prefix, dtype, device
        self.w_router = self.w_gate_up = self.w_down = self.bias = None

    def _experts(self):
        n = self.names
        out = [(n["expert"].format(i), self.expert_ff) for i in range(self.n_experts)]
        return out + ([(n["shared"], self.shared_ff)] if self.shared_ff else [])

    def params(self):
        n, d = self.names, self.hidden_size
        if self.table_routing:
            out = {n["table"]: ParamSpec((self.vocab_size, self.top), "int", f"distinct:{self.n_experts}")}
        else:
            out = {n["router"]: ParamSpec((self.n_experts + self.n_identity, d), "vector", "wide")}
        if self.correction:
            out[n["correction"]] = ParamSpec((self.n_experts + self.n_identity,), "vector", "small")
        for p, f in self._experts():
            out.update({p + n["up"]: ParamSpec((f, d)), p + n["down"]: ParamSpec((d, f))})
            if self.gated:
                out[p + n["gate"]] = ParamSpec((f, d))
        if self.shared_gate:
            out[n["shared_gate"]] = ParamSpec((1, d), "vector", "wide")
        return out

    def bind(self, tensors):
        n, d = self.names, self.hidden_size
        gu, down = [], []
        for p, f in self._experts():
            u = tensors[p + n["up"]]
            if self.gated:
                gu.append(torch.stack([tensors[p + n["gate"]], u], dim=1).reshape(2 * f, d))   # row 2j: gate_j, row 2j + 1: up_j
            else:
                gu.append(u.as_subclass(torch.Tensor))
            down.append(tensors[p + n["down"]])
        self.w_gate_up = ops.prepare_weight(torch.cat(gu, 0).contiguous())
        self.w_down = ops.prepare_weight(torch.cat(down, 1).contiguous())
        # for prompts: every expert's matrices by themselves (gate and up as row ranges of the stacked matrix where
        # its tiles allow, the down matrices as copies of their own)
        self.per_expert = None
        if self.dtype != torch.float32:
            parts, at = [], 0
            for (p, f), g_u, d_ in zip(self._experts(), gu, down):
                rows = 2 * f if self.gated else f
                parts.append((self._rows(self.w_gate_up, at, rows, g_u), ops.prepare_weight(d_.contiguous())))
                at += rows
            self.per_expert = parts
        rows = ([] if self.table_routing else [tensors[n["router"]].float()]) + \
            ([tensors[n["shared_gate"]].float().view(1, d)] if self.shared_gate else [])
        self.w_router = torch.cat(rows, 0).contiguous() if rows else None     # float32: the logits are summed in float32
        self.table = tensors[n["table"]] if self.table_routing else None
        self.bias = tensors[n["correction"]] if self.correction else None

    @staticmethod
    def _rows(stacked, r0, n, own):
        """Rows r0 .. r0 + n of a stacked matrix as a matrix of its own, sharing the storage where the tiled layout
        allows (ranges that begin and end at multiples of 16 rows); else a copy."""
        if ops.is_tiled(stacked) and r0 % 16 == 0 and n % 16 == 0:
            k = ops.matrix_shape(stacked)[1]
            flat = stacked.as_subclass(torch.Tensor)[r0 * k:(r0 + n) * k]
            return Tensor.wrap(flat, "tiled", (n, k), stacked.owner, stacked)
        return ops.prepare_weight(own.contiguous())

    def _hidden(self, rows, w_up, weights, idx, col, blocks, ff, tail):
        """The hidden rows of experts without a gate: the activation of the up product's sums, with the routing weight."""
        z = ops.linear(rows, w_up, out_dtype=torch.float32)
        return ops.expert_act(z, weights, blocks, ff, tail, self.activation, self.on_input, self.dtype, idx, col)

    def _grouped_plain(self, h, residual, weights):
        idx, counts = ops.moe_buckets(weights, self.n_experts)
        for e, n in enumerate(counts):
            if n:
                w_up, w_d = self.per_expert[e]
                t = self._hidden(ops.gather_rows(h, idx[e], n), w_up, weights, idx[e], e, 1, self.expert_ff, 0)
                ops.scatter_add_rows(residual, ops.linear(t, w_d, out_dtype=torch.float32), idx[e], weights, None)
        if self.shared_ff:
            w_up, w_d = self.per_expert[self.n_experts]
            t = self._hidden(h, w_up, weights, None, self.n_experts, 1, self.shared_ff, 0)
            ops.linear(t, w_d, ops.EPI_ADD, out=residual)

    def _gated_hidden(self, rows, w_gu, ff, limit):
        """One gated expert's hidden rows (no routing weight)."""
        if not self.clamped:
            return ops.linear(rows, w_gu, ops.EPI_SWIGLU, out_dtype=self.dtype)
        return ops.linear(rows, w_gu, ops.EPI_CLAMPGLU, out_dtype=self.dtype,
                          params=ops.glu_params(None, limit, None, self.alpha, self.up_shift))

    def _grouped(self, h, residual, weights):
        if not self.gated:
            return self._grouped_plain(h, residual, weights)
        idx, counts = ops.moe_buckets(weights, self.n_experts)
        for e, n in enumerate(counts):
            if n:
                w_gu, w_d = self.per_expert[e]
                t = self._gated_hidden(ops.gather_rows(h, idx[e], n), w_gu, self.expert_ff, self.limit)
                ops.scatter_add_rows(residual, ops.linear(t, w_d, out_dtype=torch.float32), idx[e], weights, e)
        if self.shared_ff:
            w_gu, w_d = self.per_expert[self.n_experts]
            t = self._gated_hidden(h, w_gu, self.shared_ff, self.shared_limit)
            ops.scatter_add_rows(residual, ops.linear(t, w_d, out_dtype=torch.float32), None, weights, self.n_experts)

    def _weights(self, h, residual, ctx):
        """The dense row of routing weights of every token (the shared expert's in the last column)."""
        has_gate = (1 if self.shared_gate else 2) if self.shared_ff else 0
        if self.table_routing:
            if ctx is None:
                raise ValueError("routed experts: a table chooses by token id and needs the step")
            gate = ops.small_logits(h, self.w_router) if self.shared_gate else None
            return ops.table_route(ctx.token_ids, self.table, self.n_experts, gate, has_gate)
        logits = ops.small_logits(h, self.w_router)
        return ops.moe_route(logits, self.bias, h, residual, self.n_experts + self.n_identity, self.n_experts, self.top,
                             has_gate, self.route_scale, self.sigmoid_scores, self.renormalize)

    def forward(self, h, residual, ctx=None):
        weights = self._weights(h, residual, ctx)
        if (self.per_expert is not None and self.n_experts and h.shape[0] * self.top >= self.GROUPED_FROM * self.n_experts
                and not torch.cuda.is_current_stream_capturing()):
            return self._grouped(h, residual, weights)
        if not self.gated:
            t = self._hidden(h, self.w_gate_up, weights, None, None, self.n_experts, self.expert_ff, self.shared_ff)
            return ops.linear(t, self.w_down, ops.EPI_ADD, out=residual)
        if self.clamped:
            # the shared expert's outputs, behind the others', take its own limit
            t = ops.linear(h, self.w_gate_up, ops.EPI_CLAMPGLU, out_dtype=self.dtype,
                           params=ops.glu_params(None, self.limit, self.shared_limit, self.alpha, self.up_shift,
                                                 self.n_experts * self.expert_ff))
        else:
            t = ops.linear(h, self.w_gate_up, ops.EPI_SWIGLU, out_dtype=self.dtype)
        ops.scale_blocks(t, weights, self.n_experts, self.expert_ff, self.shared_ff)
        ops.linear(t, self.w_down, ops.EPI_ADD, out=residual)
