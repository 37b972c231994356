"""Mixers that carry a state of fixed size from token to token, and the mixer that runs two mixers side by side.

State is laid out by position, as all per-request state of the engine is: the token at position p reads place
(p - 1) & 1 of two and writes place p & 1 (position 0 reads nothing, whatever a slot's former holder left), and the
inputs of a convolution of `taps` taps lie at place p mod taps of `taps`. A step of single tokens that is recorded
and run again reads what it read the first time.
"""
from typing import Dict, List, Optional

import torch

from .base import MIXERS, CacheNeed, Mixer, register_mixer
from .spec import ParamDecl, PartSpec


class _BesideAnother:
    """What a mixer offers so that `side_by_side` can run it beside another: the input of its output product goes
    into a slice of a buffer the two share (`inner_into`, times a factor, before the one rounding), and its
    output matrix is handed over (`out_matrix`) instead of being kept."""

    defer_out = False

    def _keep_out(self, ops, w):
        if self.defer_out:
            self.w_out_raw, self.w_out = w, None
        else:
            self.w_out = ops.prepare_weight(w)

    def out_matrix(self):
        w, self.w_out_raw = self.w_out_raw, None
        return w


@register_mixer("min_gru")
class MinimalGatedRecurrence(_BesideAnother, Mixer):
    """A gated recurrence whose gates read the current token only (minGRU):

        z = sigmoid(W_z h + b_z),  u = W_x h + b_x,  c = u + 1/2 where u >= 0, sigmoid(u) below
        S_t = (1 - z) S_(t-1) + z c      element by element, S = 0 before the first token
        result = W_o (S_t * silu(W_g h))

    The three input matrices are one product; gates, candidate and state are float32."""

    recordable = True

    def __init__(self, width: int, inner: int, names, weight_suffix: str = "", bias_suffix: str = ".b"):
        """`names`: the checkpoint's names of W_z, W_x, W_g and W_o; W_z and W_x have a bias."""
        self.width, self.inner = width, inner
        self.names, self.weight_suffix, self.bias_suffix = tuple(names), weight_suffix, bias_suffix
        if len(self.names) != 4:
            raise ValueError("names: W_z, W_x, W_g and W_o, four names")

    def cache_need(self) -> Optional[CacheNeed]:
        return CacheNeed("state", state_shapes=(("carried", (2, self.inner)),))

    def param_decls(self, prefix: str) -> List[ParamDecl]:
        z, x, g, o = (prefix + n for n in self.names)
        ws, bs = self.weight_suffix, self.bias_suffix
        return [ParamDecl(z + ws, (self.inner, self.width)), ParamDecl(z + bs, (self.inner,), "vector"),
                ParamDecl(x + ws, (self.inner, self.width)), ParamDecl(x + bs, (self.inner,), "vector"),
                ParamDecl(g + ws, (self.inner, self.width)), ParamDecl(o + ws, (self.width, self.inner))]

    def load(self, tensors: Dict, prefix: str, ops, dtype) -> None:
        super().load(tensors, prefix, ops, dtype)
        z, x, g, o = (prefix + n for n in self.names)
        ws, bs = self.weight_suffix, self.bias_suffix
        self.w_in = ops.prepare_weight(torch.cat([tensors[z + ws], tensors[x + ws], tensors[g + ws]], dim=0).contiguous())
        self.b_in = torch.cat([tensors[z + bs], tensors[x + bs], torch.zeros_like(tensors[z + bs])]).contiguous()
        self._keep_out(ops, tensors[o + ws])

    def flops_per_token(self, keys: float = 0.0) -> float:
        return super().flops_per_token(keys) + 6.0 * self.inner

    def inner_width(self) -> int:
        return self.inner

    def inner_into(self, h, ctx, cache, out, scale: float):
        proj = self.ops.linear(h, self.w_in, self.b_in, out_f32=True, f32_by_library=True)
        return self.ops.min_gru(proj, self.inner, ctx, cache.state["carried"], out=out, out_scale=scale)

    def forward(self, h, ctx, cache, residual):
        y = self.inner_into(h, ctx, cache, None, 1.0)
        return self.ops.linear(y, self.w_out, None, residual=residual, out_f32=True, f32_by_library=residual is None)


@register_mixer("rglru")
class GatedLinearRecurrence(_BesideAnother, Mixer):
    """Griffin's recurrent block around a real-gated linear recurrent unit. With `inner` channels in `blocks`
    equal parts:

        y = gelu_tanh(W_y h + b_y),   u = conv(W_x h + b_x) + b_conv     (a causal convolution of `taps` taps a channel)
        r = sigmoid(A_b u_b + a_b),   i = sigmoid(I_b u_b + i_b)         (part b of u through square matrices of its own)
        log a = -8 r softplus(lam),   S_t = a S_(t-1) + sqrt(1 - a^2) (i u),   S = 0 before the first token
        result = W_o (S_t * y)

    The first token has no special case. The two input matrices are one product and the two gates' matrices of a
    part are one. Gates, decay and state are float32; the state also keeps the convolution's last `taps - 1`
    inputs."""

    recordable = True

    def __init__(self, width: int, inner: int, blocks: int, taps: int, names, weight_suffix: str = "",
                 bias_suffix: str = ".b"):
        """`names`: the checkpoint's names of W_y, W_x, the convolution `[inner, taps]`, the two gates' matrices
        `[blocks, inner / blocks, inner / blocks]`, lam and W_o; all but lam and W_o have a bias."""
        if inner % blocks or taps < 1:
            raise ValueError(f"a recurrence of {inner} channels in {blocks} parts with {taps} taps")
        self.width, self.inner, self.blocks, self.taps = width, inner, blocks, taps
        self.names, self.weight_suffix, self.bias_suffix = tuple(names), weight_suffix, bias_suffix
        if len(self.names) != 7:
            raise ValueError("names: W_y, W_x, the convolution, the two gates, lam and W_o, seven names")

    def cache_need(self) -> Optional[CacheNeed]:
        shapes = (("carried", (2, self.inner)),)
        if self.taps > 1:
            shapes += (("inputs", (self.taps, self.inner)),)
        return CacheNeed("state", state_shapes=shapes)

    def param_decls(self, prefix: str) -> List[ParamDecl]:
        y, x, conv, ra, ri, lam, o = (prefix + n for n in self.names)
        ws, bs = self.weight_suffix, self.bias_suffix
        c, b = self.inner, self.blocks
        return [ParamDecl(y + ws, (c, self.width)), ParamDecl(y + bs, (c,), "vector"),
                ParamDecl(x + ws, (c, self.width)), ParamDecl(x + bs, (c,), "vector"),
                ParamDecl(conv, (c, self.taps), "vector"), ParamDecl(conv + bs, (c,), "vector"),
                ParamDecl(ra + ws, (b, c // b, c // b)), ParamDecl(ra + bs, (b, c // b), "vector"),
                ParamDecl(ri + ws, (b, c // b, c // b)), ParamDecl(ri + bs, (b, c // b), "vector"),
                ParamDecl(lam, (c,), "vector"), ParamDecl(o + ws, (self.width, c))]

    def load(self, tensors: Dict, prefix: str, ops, dtype) -> None:
        super().load(tensors, prefix, ops, dtype)
        y, x, conv, ra, ri, lam, o = (prefix + n for n in self.names)
        ws, bs = self.weight_suffix, self.bias_suffix
        self.w_in = ops.prepare_weight(torch.cat([tensors[y + ws], tensors[x + ws]], dim=0).contiguous())
        self.b_in = torch.cat([tensors[y + bs], tensors[x + bs]]).contiguous()
        self.conv_w, self.conv_b = tensors[conv], tensors[conv + bs]
        # a part's two gates through one product: the rows of A_b, then those of I_b
        self.w_gates = torch.cat([tensors[ra + ws], tensors[ri + ws]], dim=1).contiguous()
        self.b_gates = torch.cat([tensors[ra + bs], tensors[ri + bs]], dim=1).contiguous()
        # log a = r * rate, rate = -8 softplus(lam), made once in float32
        self.rate = (-8.0 * torch.nn.functional.softplus(tensors[lam].float())).contiguous()
        self._keep_out(ops, tensors[o + ws])

    def flops_per_token(self, keys: float = 0.0) -> float:
        return super().flops_per_token(keys) + 2.0 * self.inner * self.taps + 10.0 * self.inner

    def inner_width(self) -> int:
        return self.inner

    def inner_into(self, h, ctx, cache, out, scale: float):
        ops, c = self.ops, self.inner
        proj = ops.linear(h, self.w_in, self.b_in, out_f32=True, f32_by_library=True)
        u, u_compute = ops.channel_conv(proj[:, c:], self.conv_w, self.conv_b, ctx, cache.state.get("inputs"))
        gates = ops.batched_linear(u_compute.view(-1, self.blocks, c // self.blocks), self.w_gates, out_f32=True)
        return ops.gated_linear_recurrence(gates, self.b_gates, u, proj[:, :c], self.rate, ctx, cache.state["carried"],
                                           out=out, out_scale=scale)

    def forward(self, h, ctx, cache, residual):
        y = self.inner_into(h, ctx, cache, None, 1.0)
        return self.ops.linear(y, self.w_out, None, residual=residual, out_f32=True, f32_by_library=residual is None)


class _SubCache:
    """The part of a call's cache that one of two mixers side by side sees: the pages as they are, and of the
    state the tensors under its own prefix, named as the mixer names them."""

    def __init__(self, cache, prefix: str):
        self.cache_id, self.group, self.writes, self.pages = cache.cache_id, cache.group, cache.writes, cache.pages
        self.state = {k[len(prefix):]: v for k, v in cache.state.items() if k.startswith(prefix)}

    k_pages = property(lambda self: self.pages.get("k"))
    v_pages = property(lambda self: self.pages.get("v"))


@register_mixer("side_by_side")
class SideBySide(Mixer):
    """Two mixers that read the same input, `left_scale * left(h) + right_scale * right(h)`.

    Both end in an output product; the two are made one: each mixer writes what its output matrix reads, times
    its factor, into its own columns of one buffer (`inner_into`), and the product of that buffer with the two
    output matrices side by side is the weighted sum, added up in float32. At most one of the two keeps pages;
    the state of both lives in the one cache of the call, under the prefixes `left.` and `right.`."""

    def __init__(self, left: PartSpec, right: PartSpec, left_name: str = "left.", right_name: str = "right.",
                 left_scale: float = 1.0, right_scale: float = 1.0):
        self.left, self.right = MIXERS.build(left), MIXERS.build(right)
        for m in (self.left, self.right):
            if not hasattr(m, "inner_into"):
                raise ValueError(f"mixer {m.kind!r} cannot run beside another: it has no `inner_into`")
            m.defer_out = True
        self.left_name, self.right_name = left_name, right_name
        self.left_scale, self.right_scale = float(left_scale), float(right_scale)
        self.recordable = bool(getattr(self.left, "recordable", False) and getattr(self.right, "recordable", False))
        self._subs = {}

    def cache_need(self) -> Optional[CacheNeed]:
        needs = [(m.cache_need(), p) for m, p in ((self.left, "left."), (self.right, "right."))]
        paged = [n for n, _ in needs if n is not None and n.kind == "paged"]
        if len(paged) > 1:
            raise ValueError("of two mixers side by side at most one keeps pages")
        state = tuple((p + name, shape) for n, p in needs if n is not None for name, shape in n.state_shapes)
        if paged:
            n = paged[0]
            return CacheNeed("paged", n.kv_heads, n.head_size, n.window, state, "float32", n.page_tensors)
        return CacheNeed("state", state_shapes=state) if state else None

    def param_decls(self, prefix: str) -> List[ParamDecl]:
        return self.left.param_decls(prefix + self.left_name) + self.right.param_decls(prefix + self.right_name)

    def load(self, tensors: Dict, prefix: str, ops, dtype) -> None:
        super().load(tensors, prefix, ops, dtype)
        self.left.load(tensors, prefix + self.left_name, ops, dtype)
        self.right.load(tensors, prefix + self.right_name, ops, dtype)
        self.split = self.left.inner_width()
        self.w_out = ops.prepare_weight(torch.cat([self.left.out_matrix(), self.right.out_matrix()], dim=1).contiguous())

    def step_planners(self):
        return {**self.left.step_planners(), **self.right.step_planners()}

    def launch_shape(self, step):
        return (self.left.launch_shape(step), self.right.launch_shape(step))

    def flops_per_token(self, keys: float = 0.0) -> float:
        return self.left.flops_per_token(keys) + self.right.flops_per_token(keys)

    def forward(self, h, ctx, cache, residual):
        subs = self._subs.get(id(cache))
        if subs is None or subs[0] is not cache:
            subs = self._subs[id(cache)] = (cache, _SubCache(cache, "left."), _SubCache(cache, "right."))
        both = torch.empty(h.shape[0], self.split + self.right.inner_width(), dtype=self.dtype, device=self.ops.device)
        self.left.inner_into(h, ctx, subs[1], both[:, :self.split], self.left_scale)
        self.right.inner_into(h, ctx, subs[2], both[:, self.split:], self.right_scale)
        return self.ops.linear(both, self.w_out, None, residual=residual, out_f32=True, f32_by_library=residual is None)
