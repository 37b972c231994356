"""Arrangements of a layer's parts around the residual stream."""
from .. import debug
from .base import Block, Stream, register_block


@register_block("pre_norm")
class PreNormBlock(Block):
    """`x = x + mixer(norm(x))`, `x = x + feed_forward(norm(x))`
    (reference: opt/model.py:351-375). The sums are made in float32 by the
    last matrix product of each part."""

    recordable = True

    fold_mixer_norm = fold_feed_forward_norm = False

    def after_load(self) -> None:
        # Each norm's output goes to one part only; where that part does nothing with it but one matrix
        # product, the backend may do the norm inside the product (the few-rows products of decode steps:
        # one launch less for each half of a layer).
        w = self.mixer.first_weight()
        self.fold_mixer_norm = w is not None and self.mixer_norm.fold_into(w)
        w = self.feed_forward.first_weight()
        self.fold_feed_forward_norm = w is not None and self.feed_forward_norm.fold_into(w)

    def forward(self, stream: Stream, ctx, cache) -> Stream:
        h = (self.mixer_norm.deferred(stream.x) if self.fold_mixer_norm
             else self.mixer_norm.forward(stream.x, False, True)[1])
        x = debug.tap("after_mixer", self.mixer.forward(h, ctx, cache, stream.x))
        h = (self.feed_forward_norm.deferred(x) if self.fold_feed_forward_norm
             else self.feed_forward_norm.forward(x, False, True)[1])
        x = self.feed_forward.forward(h, ctx, x)
        return Stream(x, None)


@register_block("post_norm")
class PostNormBlock(Block):
    """`x = norm(x + mixer(x))`, `x = norm(x + feed_forward(x))`: the norm follows
    each sum, and its output is the stream."""

    recordable = True

    reads_compute_copy = True      # the mixer reads the stream itself, in the compute dtype

    def forward(self, stream: Stream, ctx, cache) -> Stream:
        h = stream.compute if stream.compute is not None else self.mixer_norm.ops.cast(stream.x, self.mixer_norm.dtype)
        t = self.mixer.forward(h, ctx, cache, stream.x)
        x, h = self.mixer_norm.forward(t, True, True)
        debug.tap("after_mixer", x)
        t = self.feed_forward.forward(h, ctx, x)
        x, h = self.feed_forward_norm.forward(t, True, True)
        return Stream(x, h)


@register_block("parallel")
class ParallelBlock(Block):
    """`h = norm(x)`, `x = x + mixer(h) + feed_forward(h)`: one norm, and both parts read its output. The sum
    is float32: the mixer's last product adds the stream, the feed-forward's adds that."""

    recordable = True

    def forward(self, stream: Stream, ctx, cache) -> Stream:
        h = self.mixer_norm.forward(stream.x, False, True)[1]
        x = debug.tap("after_mixer", self.mixer.forward(h, ctx, cache, stream.x))
        return Stream(self.feed_forward.forward(h, ctx, x), None)


@register_block("sandwich")
class SandwichBlock(Block):
    """A norm before and after each part, the part's normed result scaled before it joins the stream:

        x = x + mult * post_norm(mixer(conv(norm(x))))        and the same for the feed-forward,

    with, each optional:
    `taps`: what a part reads, h = norm(x), is first replaced by h + conv(h), a causal convolution over the
        request's tokens on every channel, conv(h)_t = sum_j w[:, j] h_(t - taps + 1 + j) (zeros before the
        request's start; weights `[width, taps]`). The last taps - 1 inputs of each part are per-request state
        (kept in `taps` places, by position, so that a step of single tokens can be run again and read the same).
    `side`: a token-keyed input after the feed-forward. With e the `dim` elements from column `offset` on of
        the token's row of a table, g = gelu_tanh(W_gate x) * e, y = W_proj g:
        x = x + mult * y / sqrt(mean(y^2) + eps) * weight.
    `depth_average`: the stream that goes on is a weighted sum of what every call so far has left and of
        the embedded tokens, sum_j w[j] X_j (j = 0 the embedded tokens, j = i + 1 this call's result, the i-th
        of the run order), w a tensor of `depth_average` numbers. `depth_slots` is how many X the model has.
    The sums, the norms and the state are float32.
    """

    recordable = True

    def __init__(self, mixer, feed_forward, mixer_norm, feed_forward_norm, *, mixer_post_norm, feed_forward_post_norm,
                 names, mult: float = 1.0, taps: int = 0, conv_names=None, side=None, depth_average: int = 0,
                 depth_name=None, depth_slots: int = 0):
        """`names`: the checkpoint's names of the two post norms, relative to the layer's prefix; `conv_names`
        those of the two convolutions; `side`: dict(table, dim, offset, gate, proj, norm, eps, columns), `table`
        a full tensor name (layers share it), `columns` its width, the others relative names."""
        super().__init__(mixer, feed_forward, mixer_norm, feed_forward_norm)
        from .base import NORMS
        self.has_ff = not getattr(feed_forward, "absent", False)
        self.mixer_post = NORMS.build(mixer_post_norm)
        self.ff_post = NORMS.build(feed_forward_post_norm) if self.has_ff else None
        self.names, self.conv_names = tuple(names), tuple(conv_names or ())
        self.mult, self.taps = float(mult), int(taps)
        self.side = dict(side) if side else None
        self.depth_average, self.depth_name, self.depth_slots = int(depth_average), depth_name, int(depth_slots)
        self.width = mixer_norm.width

    def _convs(self):
        return (1 if self.taps > 0 else 0) * (2 if self.has_ff else 1)

    def state_need(self):
        if self.taps > 1:
            from .base import CacheNeed
            return CacheNeed("state", state_shapes=(("inputs", (self._convs(), self.taps, self.width)),))
        return None

    def param_decls(self, prefix: str):
        from .spec import ParamDecl
        d = self.mixer_post.param_decls(prefix + self.names[0])
        if self.has_ff:
            d += self.ff_post.param_decls(prefix + self.names[1])
        for name in self.conv_names[:self._convs()]:
            d.append(ParamDecl(prefix + name, (self.width, self.taps), "vector"))
        if self.side:
            s = self.side
            d += [ParamDecl(s["table"], (s["rows"], s["columns"]), "table"),
                  ParamDecl(prefix + s["gate"], (s["dim"], self.width)),
                  ParamDecl(prefix + s["proj"], (self.width, s["dim"])),
                  ParamDecl(prefix + s["norm"], (self.width,), "vector", "around_one")]
        if self.depth_average:
            d.append(ParamDecl(prefix + self.depth_name, (self.depth_average,), "vector", "around_mean"))
        return d

    def load(self, tensors, prefix, ops, dtype) -> None:
        super().load(tensors, prefix, ops, dtype)
        self.mixer_post.load(tensors, prefix + self.names[0], ops, dtype)
        if self.has_ff:
            self.ff_post.load(tensors, prefix + self.names[1], ops, dtype)
        self.conv_w = [tensors[prefix + name] for name in self.conv_names[:self._convs()]]
        if self.side:
            s = self.side
            self.side_table = tensors[s["table"]]
            self.side_gate = ops.prepare_weight(tensors[prefix + s["gate"]])
            self.side_proj = ops.prepare_weight(tensors[prefix + s["proj"]])
            self.side_norm = tensors[prefix + s["norm"]]
        self.depth_w = tensors[prefix + self.depth_name] if self.depth_average else None

    def flops_per_token(self, keys: float = 0.0) -> float:
        return 4.0 * self.side["dim"] * self.width if self.side else 0.0

    def _input(self, norm, x, which, ctx, join=None):
        """What a part reads: the norm of the stream, with the convolution over the request's tokens. `join` =
        (y, post norm): the part before joins the stream first, x + mult * post_norm(y). Returns (the stream,
        what the part reads). One launch where both norms can be applied inside a kernel of the backend's."""
        state = ctx.call_state.state["inputs"] if self.taps > 1 else None
        pre = norm.fused_form() if hasattr(norm, "fused_form") else None
        post = join[1].fused_form() if join is not None and hasattr(join[1], "fused_form") else None
        if self.taps > 0 and pre is not None and (join is None or (post is not None and post[3] == pre[3])) \
                and not debug.tapping():
            joined = (join[0], post[0], post[1], post[2], self.mult) if join is not None else None
            return self.ops.join_norm_conv(x, joined, pre, self.conv_w[which], state, which, ctx, self.dtype)
        if join is not None:
            x = debug.tap("after_mixer", join[1].add_to(join[0], x, self.mult))
        if self.taps <= 0:
            return x, norm.forward(x, False, True)[1]
        h = norm.forward(x, True, False)[0]
        return x, self.ops.input_conv(h, self.conv_w[which], state, which, ctx, self.dtype)

    def forward(self, stream: Stream, ctx, cache) -> Stream:
        ops = self.ops
        x = stream.x
        history, filled = stream.history, stream.filled
        if self.depth_average and history is None:
            history = x.new_empty((self.depth_slots,) + tuple(x.shape))
            history[0].copy_(x)
            filled = 1
        if self.depth_average and not filled < self.depth_slots:
            raise ValueError(f"the average over depth has {self.depth_slots} places and the run order more calls")
        place = history[filled] if self.depth_average else None       # where this call's own result goes

        x, h = self._input(self.mixer_norm, x, 0, ctx)
        y = self.mixer.forward(h, ctx, cache, None)
        compute = None
        if self.has_ff:
            x, h = self._input(self.feed_forward_norm, x, 1, ctx, join=(y, self.mixer_post))
            y = self.feed_forward.forward(h, ctx, None)
            if self.side:
                x, compute = self.ff_post.add_to(y, x, self.mult, None, want_compute=True)
            else:
                x = self.ff_post.add_to(y, x, self.mult, place)
        elif self.side:
            x, compute = self.mixer_post.add_to(y, x, self.mult, None, want_compute=True)
        else:
            x = self.mixer_post.add_to(y, x, self.mult, place)
        if self.side:
            s = self.side
            rows = ctx.memo.get(("table rows", s["table"]))
            if rows is None:        # the tokens' rows, looked up once a step for all layers
                rows = ctx.memo[("table rows", s["table"])] = ops.embed(ctx.token_ids, self.side_table, self.dtype,
                                                                       ctx.kept_tokens)
            g = ops.linear(compute, self.side_gate, None, act="gelu_new")
            g = ops.mul_columns(g, rows, s["offset"])
            y = ops.linear(g, self.side_proj, None, out_f32=True, f32_by_library=True)
            x = ops.norm_add(y, self.side_norm, None, s["eps"], False, x, self.mult, place)
        if not self.depth_average:
            return Stream(x, None)
        if self.depth_average != filled + 1:
            raise ValueError(f"this call averages {self.depth_average} results and {filled + 1} are there")
        debug.tap("own_result", x)
        return Stream(ops.weighted_sum(history, self.depth_w, filled + 1), None, history, filled + 1)


@register_block("hyper")
class HyperConnectionBlock(Block):
    """Pre-norm sublayers around several copies of the residual stream (hyper-connections). The copies x_1 .. x_s
    all start as the embedded tokens. For a sublayer f (the mixer, then the feed-forward, where the layer has one)
    with its own weights `in` [s], `out` [s] and `mix` [s, s] (indexed [from, to]):

        u = sum_a in[a] x_a,   y = f(norm(u)),   x_b <- sum_a mix[a, b] x_a + out[b] y     (all b at once, from the old copies)

    `streams=0` is the plain residual sum x <- x + f(norm(x)): one copy and no weights. With `taps`, what the mixer
    reads is first replaced by h + conv(h), a causal convolution over the request's tokens on every channel
    (weights `[width, taps]`, zeros before the request's start); its last taps - 1 inputs are per-request state.
    The copies, the norms, the sums and the state are float32. When the last call of the run order is through,
    the model sums the copies.

    A sublayer's result does not join the copies at once: it is left `pending` on the stream, and whoever reads
    the copies next (the next sublayer's weighted sum and norm, or the sum at the end) applies it in the same
    launch."""

    recordable = True

    def __init__(self, mixer, feed_forward, mixer_norm, feed_forward_norm, *, streams: int, taps: int = 0,
                 conv_name: str = "conv", names=("hc1.", "hc2."), parts=("in", "out", "mix")):
        """`names`: the prefixes of the mixer's and the feed-forward's stream weights, relative to the layer's;
        `parts`: what the three tensors are called under them."""
        super().__init__(mixer, feed_forward, mixer_norm, feed_forward_norm)
        self.streams, self.taps, self.conv_name = int(streams), int(taps), conv_name
        self.names, self.part_names = tuple(names), tuple(parts)
        self.has_ff = not getattr(feed_forward, "absent", False)
        self.width = mixer_norm.width
        if self.streams < 0 or self.taps < 0:
            raise ValueError(f"hyper-connections with {streams} streams and {taps} taps")
        for norm in (mixer_norm,) + ((feed_forward_norm,) if self.has_ff else ()):
            if not hasattr(norm, "fused_form") or norm.fused_form()[2]:
                raise ValueError("the norm behind the weighted sum of the copies is one that only scales (rms_norm)")

    def state_need(self):
        if self.taps > 1:
            from .base import CacheNeed
            return CacheNeed("state", state_shapes=(("inputs", (1, self.taps, self.width)),))
        return None

    def _sublayers(self):
        return self.names[:2 if self.has_ff else 1]

    def param_decls(self, prefix: str):
        from .spec import ParamDecl
        d = []
        s = self.streams
        if s:
            i, o, m = self.part_names
            for name in self._sublayers():
                d += [ParamDecl(prefix + name + i, (s,), "vector", "around_mean"),
                      ParamDecl(prefix + name + o, (s,), "vector", "around_one"),
                      ParamDecl(prefix + name + m, (s, s), "vector", "around_mean")]
        if self.taps > 0:
            d.append(ParamDecl(prefix + self.conv_name, (self.width, self.taps), "vector"))
        return d

    def load(self, tensors, prefix, ops, dtype) -> None:
        import torch
        super().load(tensors, prefix, ops, dtype)
        self.weights = []
        for name in self._sublayers():
            if self.streams:
                i, o, m = (tensors[prefix + name + p].float().contiguous() for p in self.part_names)
            else:
                one = torch.ones(1, dtype=torch.float32, device=getattr(ops, "device", "cpu"))
                i, o, m = one, one, one.view(1, 1)
            self.weights.append((i, o, m))
        self.conv_w = tensors[prefix + self.conv_name] if self.taps > 0 else None

    def _read(self, stream: Stream, which: int, norm, want_f32: bool):
        """The copies with what is pending joined, and norm(sum_a in[a] x_a) in float32 or in the compute dtype."""
        weight, _, _, eps = norm.fused_form()
        h32, hc = self.ops.hyper_step(stream.copies, stream.pending, self.weights[which][0], weight, eps, self.dtype,
                                      want_f32, not want_f32)
        return h32 if want_f32 else hc

    def forward(self, stream: Stream, ctx, cache) -> Stream:
        ops = self.ops
        copies = stream.copies
        if copies is None:          # the first call of the run order: every copy is the embedded tokens
            copies = stream.x.unsqueeze(0).repeat(max(1, self.streams), 1, 1)
            stream = Stream(None, None, copies=copies)
        elif copies.shape[0] != max(1, self.streams):
            raise ValueError(f"the stream has {copies.shape[0]} copies, this layer {max(1, self.streams)}")
        if self.taps > 0:
            h = self._read(stream, 0, self.mixer_norm, True)
            state = ctx.call_state.state["inputs"] if self.taps > 1 else None
            h = ops.input_conv(h, self.conv_w, state, 0, ctx, self.dtype)
        else:
            h = self._read(stream, 0, self.mixer_norm, False)
        y = self.mixer.forward(h, ctx, cache, None)
        stream = Stream(None, None, copies=copies, pending=(y, self.weights[0][2], self.weights[0][1]))
        if debug.tapping():
            debug.tap("after_mixer", ops.hyper_sum(copies, stream.pending))
            stream.pending = None
        if self.has_ff:
            h = self._read(stream, 1, self.feed_forward_norm, False)
            y = self.feed_forward.forward(h, ctx, None)
            stream = Stream(None, None, copies=copies, pending=(y, self.weights[1][2], self.weights[1][1]))
        if debug.tapping():
            # what a tap of the stream after this call sees: the sum of the copies
            stream.x = ops.hyper_sum(copies, stream.pending)
            stream.pending = None
        return stream
