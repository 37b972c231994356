"""Feed-forward parts."""
from typing import Dict, List

from .base import FeedForward, register_feed_forward
from .spec import ParamDecl


@register_feed_forward("dense")
class DenseFeedForward(FeedForward):
    """`act(h W1^T + b1) W2^T + b2`, the activation applied to the float32
    accumulator (reference: hlo.py:550-559; activations.py:20-48)."""

    recordable = True

    def __init__(self, width: int, inner: int, activation: str, up_name: str, down_name: str, bias: bool = True,
                 weight_suffix: str = ".weight", act_name: str = None, eps: float = 1e-5):
        """`up_name`, `down_name`: the checkpoint's names of the two matrices, relative to the part's prefix;
        `weight_suffix`: what a matrix's name adds to them.

        `activation="poly_norm"` is no function of one element: with N(v) = v / sqrt(mean(v^2) + eps) over a
        token's inner values, act(z) = a N(z) + b N(z^2) + c N(z^3) + e, powers element by element, the four
        numbers being the tensor `act_name`. Sums and roots are float32. `activation="relu2"` is the square of
        relu."""
        self.width, self.inner, self.activation, self.has_bias = width, inner, activation, bias
        self.up_name, self.down_name, self.weight_suffix = up_name, down_name, weight_suffix
        self.act_name, self.eps = act_name, float(eps)
        if activation == "poly_norm" and not act_name:
            raise ValueError("activation 'poly_norm' needs `act_name`, the tensor of its four numbers")

    def param_decls(self, prefix: str) -> List[ParamDecl]:
        d = [ParamDecl(f"{prefix}{self.up_name}{self.weight_suffix}", (self.inner, self.width)),
             ParamDecl(f"{prefix}{self.down_name}{self.weight_suffix}", (self.width, self.inner))]
        if self.has_bias:
            d += [ParamDecl(f"{prefix}{self.up_name}.bias", (self.inner,), "vector"),
                  ParamDecl(f"{prefix}{self.down_name}.bias", (self.width,), "vector")]
        if self.activation == "poly_norm":
            d.append(ParamDecl(f"{prefix}{self.act_name}", (4,), "vector", "around_one"))
        return d

    def load(self, tensors: Dict, prefix: str, ops, dtype) -> None:
        super().load(tensors, prefix, ops, dtype)
        self.w1 = ops.prepare_weight(tensors[f"{prefix}{self.up_name}{self.weight_suffix}"])
        self.w2 = ops.prepare_weight(tensors[f"{prefix}{self.down_name}{self.weight_suffix}"])
        self.b1 = tensors.get(f"{prefix}{self.up_name}.bias") if self.has_bias else None
        self.b2 = tensors.get(f"{prefix}{self.down_name}.bias") if self.has_bias else None
        self.coeffs = tensors[f"{prefix}{self.act_name}"] if self.activation == "poly_norm" else None

    def first_weight(self):
        return self.w1

    def forward(self, h, ctx, residual):
        """`residual` None: f(h) alone, in float32 (for an arrangement that norms it before the sum)."""
        if self.activation == "poly_norm":
            inner = self.ops.poly_norm(self.ops.linear(h, self.w1, self.b1, out_f32=True, f32_by_library=True),
                                       self.coeffs, self.eps)
        else:
            inner = self.ops.linear(h, self.w1, self.b1, act=self.activation)
        return self.ops.linear(inner, self.w2, self.b2, residual=residual, out_f32=True, f32_by_library=residual is None)


@register_feed_forward("gated")
class GatedFeedForward(FeedForward):
    """`W_down (act(W_gate h) * (W_up h))`, no biases: gate and up rows are one product, the activation and the
    product of the two halves are made on its float32 sums and rounded once."""

    recordable = True

    def __init__(self, width: int, inner: int, activation: str, names, weight_suffix: str = ""):
        """`names`: the checkpoint's names of the gate, up and down matrices; `activation`: "gelu_new" (the tanh
        form) or "silu"."""
        if activation not in ("gelu_new", "silu"):
            raise ValueError(f"a gated feed-forward's activation is gelu_new or silu, got {activation!r}")
        self.width, self.inner, self.activation = width, inner, activation
        self.names, self.weight_suffix = tuple(names), weight_suffix

    def param_decls(self, prefix: str) -> List[ParamDecl]:
        g, u, d = (f"{prefix}{n}{self.weight_suffix}" for n in self.names)
        return [ParamDecl(g, (self.inner, self.width)), ParamDecl(u, (self.inner, self.width)),
                ParamDecl(d, (self.width, self.inner))]

    def load(self, tensors: Dict, prefix: str, ops, dtype) -> None:
        import torch
        super().load(tensors, prefix, ops, dtype)
        g, u, d = (f"{prefix}{n}{self.weight_suffix}" for n in self.names)
        self.w_in = ops.prepare_weight(torch.cat([tensors[g], tensors[u]], dim=0).contiguous())
        self.w_down = ops.prepare_weight(tensors[d])

    def forward(self, h, ctx, residual):
        inner = self.ops.gated_activation(self.ops.linear(h, self.w_in, None, out_f32=True, f32_by_library=True),
                                          self.activation)
        return self.ops.linear(inner, self.w_down, None, residual=residual, out_f32=True,
                               f32_by_library=residual is None)


@register_feed_forward("none")
class NoFeedForward(FeedForward):
    """A layer without a feed-forward: the stream passes."""

    recordable = True
    absent = True

    def __init__(self, **_):
        pass

    def forward(self, h, ctx, residual):
        return residual


@register_feed_forward("mixture")
class ExpertMixture(FeedForward):
    """A mixture of gated experts, of which a token takes `top`, and optionally one more that every token takes.

    Router: z = W_r h in float32, scores s = sigmoid(z) (`score="sigmoid"`) or softmax(z) (`"softmax"`); a token's
    experts are the `top` with the largest scores (the lower number where two are equal), their weights the
    scores, divided by their sum with `renormalize`. An expert is W_down (act(W_gate x) * (W_up x)), no biases.
    `weight_on="input"`: the result is the sum of expert(w h), the weight applied to what the expert reads;
    `"output"`: the sum of w expert(h). The shared expert (`shared_inner` > 0) is of the same form, reads h and
    is added. The weights enter the float32 sums of the first products, so nothing is rounded twice.

    `correction_name`: a tensor of one number an expert that is added to the scores where the experts are chosen
    and nowhere else (the weights are the scores without it). `route_scale`: the weights times this number.
    `activation="clamped_swiglu"` with `limit` (`shared_limit` for the shared expert): g = min(W_gate x, limit),
    u = clamp(W_up x, -limit, limit), and the expert is W_down (g sigmoid(1.702 g) (u + 1))."""

    recordable = True

    def __init__(self, width: int, experts: int, top: int, inner: int, router_name: str, expert_name: str, names,
                 shared_inner: int = 0, shared_name: str = "shared.", score: str = "sigmoid", renormalize: bool = False,
                 weight_on: str = "output", activation: str = "silu", weight_suffix: str = "",
                 correction_name: str = None, route_scale: float = 1.0, limit: float = None, shared_limit: float = None):
        """`expert_name`: a format string that takes the expert's number ("e{}."); `names`: the names of an
        expert's gate, up and down matrices."""
        if not 1 <= top <= experts:
            raise ValueError(f"a token takes {top} of {experts} experts")
        if score not in ("sigmoid", "softmax") or weight_on not in ("input", "output") \
                or activation not in ("silu", "gelu_new", "clamped_swiglu"):
            raise ValueError(f"mixture: score {score!r}, weight_on {weight_on!r}, activation {activation!r}")
        if activation == "clamped_swiglu":
            if limit is None or not float(limit) > 0 or (shared_inner and not float(shared_limit or 0) > 0):
                raise ValueError("mixture: activation 'clamped_swiglu' needs a positive `limit` (and `shared_limit`)")
            if weight_on != "output":
                raise ValueError("mixture: a clamped expert takes its weight on the output")
        if correction_name and (score != "sigmoid" or renormalize):
            raise ValueError("mixture: a correction of the choice goes with sigmoid scores that are not renormalized")
        self.correction_name, self.route_scale = correction_name, float(route_scale)
        self.limit = float(limit) if limit is not None else None
        self.shared_limit = float(shared_limit) if shared_limit is not None else None
        self.width, self.experts, self.top, self.inner, self.shared_inner = width, experts, top, inner, shared_inner
        self.router_name, self.expert_name, self.shared_name = router_name, expert_name, shared_name
        self.names, self.weight_suffix = tuple(names), weight_suffix
        self.score, self.renormalize, self.weight_on, self.activation = score, bool(renormalize), weight_on, activation

    def _expert_decls(self, prefix: str, inner: int) -> List[ParamDecl]:
        g, u, d = self.names
        s = self.weight_suffix
        return [ParamDecl(f"{prefix}{g}{s}", (inner, self.width)), ParamDecl(f"{prefix}{u}{s}", (inner, self.width)),
                ParamDecl(f"{prefix}{d}{s}", (self.width, inner))]

    def param_decls(self, prefix: str) -> List[ParamDecl]:
        d = []
        for e in range(self.experts):
            d += self._expert_decls(prefix + self.expert_name.format(e), self.inner)
        d.append(ParamDecl(f"{prefix}{self.router_name}{self.weight_suffix}", (self.experts, self.width)))
        if self.correction_name:
            d.append(ParamDecl(f"{prefix}{self.correction_name}", (self.experts,), "vector"))
        if self.shared_inner:
            d += self._expert_decls(prefix + self.shared_name, self.shared_inner)
        return d

    def load(self, tensors: Dict, prefix: str, ops, dtype) -> None:
        import torch
        super().load(tensors, prefix, ops, dtype)
        g, u, d = self.names
        s = self.weight_suffix
        each = [prefix + self.expert_name.format(e) for e in range(self.experts)]
        # an expert's gate rows, then its up rows: `[experts, 2 inner, width]`; the down matrices `[experts, width, inner]`
        self.w_gate_up = torch.stack([torch.cat([tensors[f"{p}{g}{s}"], tensors[f"{p}{u}{s}"]], dim=0) for p in each]).contiguous()
        self.w_down = torch.stack([tensors[f"{p}{d}{s}"] for p in each]).contiguous()
        self.w_router = ops.prepare_weight(tensors[f"{prefix}{self.router_name}{s}"])
        self.correction = tensors[f"{prefix}{self.correction_name}"] if self.correction_name else None
        if self.shared_inner:
            p = prefix + self.shared_name
            self.w_shared_in = ops.prepare_weight(torch.cat([tensors[f"{p}{g}{s}"], tensors[f"{p}{u}{s}"]], dim=0).contiguous())
            self.w_shared_down = ops.prepare_weight(tensors[f"{p}{d}{s}"])

    def flops_per_token(self, keys: float = 0.0) -> float:
        return 2.0 * self.width * (self.experts + 3 * self.top * self.inner + 3 * self.shared_inner)

    def forward(self, h, ctx, residual):
        ops = self.ops
        z = ops.linear(h, self.w_router, None, out_f32=True, f32_by_library=True)
        more = {}
        if self.correction is not None or self.route_scale != 1.0:
            more = dict(correction=self.correction, scale=self.route_scale)
        chosen, weights = ops.route(z, self.top, self.score, self.renormalize, **more)
        limit = dict(limit=self.limit) if self.limit is not None else {}
        # (a step that is being recorded is sized by `length_bound`; any other may let the host read)
        x = ops.expert_mixture(h, chosen, weights, self.w_gate_up, self.w_down, self.activation, self.weight_on, residual,
                               may_wait=ctx is not None and ctx.length_bound is None, **limit)
        if not self.shared_inner:
            return x
        limit = dict(limit=self.shared_limit) if self.shared_limit is not None else {}
        inner = ops.gated_activation(ops.linear(h, self.w_shared_in, None, out_f32=True, f32_by_library=True),
                                     self.activation, **limit)
        return ops.linear(inner, self.w_shared_down, None, residual=x, out_f32=True)
