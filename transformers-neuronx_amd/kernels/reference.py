"""A plain torch rendition of every kernel, with the same call signatures.

It is what each HIP kernel is tested against, and it can stand in for the whole
backend (`EngineConfig(kernels="reference")`) to debug the engine on any
device. It is never chosen by itself: the product path is `kernels.hip`.
All arithmetic is done in float32 and rounded once to the output dtype, which
is what the kernels do with their float32 accumulators.
"""
import math
from typing import Optional

import torch


def philox_uniform(seed: int, counter: int) -> float:
    """Philox-4x32-10 keyed by `seed`, counter `counter`; first word -> [0, 1)."""
    m0, m1, w0, w1, mask = 0xD2511F53, 0xCD9E8D57, 0x9E3779B9, 0xBB67AE85, 0xFFFFFFFF
    c = [counter & mask, (counter >> 32) & mask, 0, 0]
    k = [seed & mask, (seed >> 32) & mask]
    for _ in range(10):
        p0, p1 = m0 * c[0], m1 * c[2]
        c = [((p1 >> 32) ^ c[1] ^ k[0]) & mask, p1 & mask, ((p0 >> 32) ^ c[3] ^ k[1]) & mask, p0 & mask]
        k = [(k[0] + w0) & mask, (k[1] + w1) & mask]
    return (c[0] >> 8) * (1.0 / (1 << 24))


class ReferenceOps:
    name = "reference"

    def __init__(self, dtype: torch.dtype, device="cpu"):
        self.dtype = dtype
        self.device = torch.device(device)

    # ---------------------------------------------------------------- input end

    def embed(self, token_ids, table, dtype=None, kept_tokens=None):
        """Rows of the token table; an id -1 - k is the token kept in `kept_tokens[k]`."""
        ids = token_ids.long()
        if kept_tokens is not None:
            ids = torch.where(ids < 0, kept_tokens.long()[(-1 - ids).clamp(min=0)], ids)
        return table[ids]

    def send_tokens(self, tokens, kept, ctx):
        self.store_tokens(kept, tokens, ctx)
        return tokens

    def receive_tokens(self, sent):
        return sent.tolist()

    def store_tokens(self, kept, tokens, ctx):
        slots = ctx.slots.long()[ctx.token_request.long()[ctx.logits_rows.long()]]
        kept[slots] = tokens.to(kept.dtype)

    def add_positions(self, src, positions, table, offset, dtype, want_compute, scale=1.0):
        x = src.float() * scale + table[(positions + offset).long()].float()
        return x, (x.to(dtype) if want_compute else None)

    def to_stream(self, src, dtype, want_compute, scale=1.0):
        x = src.float() * scale
        return x, (x.to(dtype) if want_compute else None)

    def add_sinusoid(self, src, positions, freqs, dtype, want_compute, scale=1.0):
        """float32 `src * scale` plus, at elements 2i and 2i + 1, the sine and the cosine of position * freqs[i]
        (the angle a float32 product)."""
        angle = positions.float()[:, None] * freqs.float()[None, :]
        x = src.float() * scale + torch.stack([torch.sin(angle), torch.cos(angle)], dim=-1).reshape(src.shape)
        return x, (x.to(dtype) if want_compute else None)

    # ---------------------------------------------------------------- several copies of the stream

    @staticmethod
    def _join(copies, pending):
        """`copies[b] <- sum_a mix[a, b] copies[a] + out[b] y` for pending = (y, mix, out), in place."""
        if pending is not None:
            y, mix, out = pending
            copies.copy_(torch.einsum("ab,atd->btd", mix.float(), copies) + out.float()[:, None, None] * y.float()[None])

    def hyper_step(self, copies, pending, read, norm_weight, eps, dtype, want_f32, want_compute):
        """Joins what is pending to the float32 copies `[s, T, width]` (in place), then
        h = u / sqrt(mean(u^2) + eps) * norm_weight with u = sum_a read[a] copies[a]; returns (h in float32 or None,
        h in `dtype` or None)."""
        self._join(copies, pending)
        u = torch.einsum("a,atd->td", read.float(), copies)
        h = u * torch.rsqrt((u * u).mean(-1, keepdim=True) + eps) * norm_weight.float()
        return (h if want_f32 else None), (h.to(dtype) if want_compute else None)

    def hyper_sum(self, copies, pending):
        """Joins what is pending (in place) and returns the float32 sum of the copies."""
        self._join(copies, pending)
        return copies.sum(0)

    # ---------------------------------------------------------------- norms

    def layernorm(self, x, weight, bias, eps, dtype, want_f32, want_compute, center=True):
        """`center=False`: the norm that only scales, x / sqrt(mean(x^2) + eps) (times weight, plus bias)."""
        x = x.float()
        mean = x.mean(-1, keepdim=True) if center else torch.zeros_like(x[:, :1])
        var = ((x - mean) ** 2).mean(-1, keepdim=True)
        y = (x - mean) * torch.rsqrt(var + eps)
        if weight is not None:
            y = y * weight.float()
        if bias is not None:
            y = y + bias.float()
        return (y if want_f32 else None), (y.to(dtype) if want_compute else None)

    # ---------------------------------------------------------------- matrix products

    def layernorm_deferred(self, x, weight, bias, eps, dtype, center=True):
        """The norm's output for a part that only multiplies it; a backend may hand back something a
        product resolves instead (`HipOps.layernorm_deferred`)."""
        return self.layernorm(x, weight, bias, eps, dtype, False, True, center)[1]

    def fold_norm(self, w, weight, bias, center=True) -> bool:
        return False

    def prepare_weight(self, w):
        """Matrices are used as they are here."""
        return w

    @staticmethod
    def activation(y, act):
        if act is None or act == "none":
            return y
        if act == "relu":
            return torch.relu(y)
        if act == "gelu":
            return 0.5 * y * (1.0 + torch.erf(y / math.sqrt(2.0)))
        if act == "gelu_new":
            return 0.5 * y * (1.0 + torch.tanh(math.sqrt(2.0 / math.pi) * (y + 0.044715 * y * y * y)))
        if act == "relu2":
            return torch.relu(y) ** 2
        raise ValueError(f"unknown activation {act!r}")

    def linear(self, x, w, bias=None, act=None, residual=None, out_f32=False, f32_by_library=False):
        """`act(x w^T + bias) + residual`, `w` being `[out, in]`. An operand in the
        narrower dtype decides what the other is rounded to, except that a
        float32 matrix keeps the product in float32."""
        if w.dtype == torch.float32:
            xa = x.float()
        else:
            xa = x.to(w.dtype).float()
        y = xa @ w.float().t()
        if bias is not None:
            y = y + bias.float()
        y = self.activation(y, act)
        if residual is not None:
            y = y + residual.float()
        return y if out_f32 else y.to(self.dtype)

    # ---------------------------------------------------------------- attention

    def qkv_project(self, h, w, bias, num_heads, num_kv_write, head_size, scale, ctx, view, k_pages, v_pages, turn=None):
        """The projection to queries, keys and values (`w` holds the three stacked by rows), then
        `qkv_write`."""
        return self.qkv_write(self.linear(h, w, None), bias, num_heads, num_kv_write, head_size, scale, ctx, view,
                              k_pages, v_pages, turn)

    def qkv_write(self, qkv, bias, num_heads, num_kv_write, head_size, scale, ctx, view, k_pages, v_pages, turn=None):
        """Bias, then `turn` = (a, b), float32 `[positions, head_size]`: element d of every query and key head
        of a token at position p becomes a[p, d] x[d] + b[p, d] x[d ^ 1]; then the query scale, and the step's
        keys and values into their pages: page `table[run][position // page_size]`, place `position % page_size`."""
        t = qkv.shape[0]
        y = qkv.float()
        if bias is not None:
            y = y + bias.float()
        nq = num_heads * head_size
        if turn is not None:
            a, b = turn
            turned = nq + num_kv_write * head_size
            at = ctx.positions.long().clamp(0, a.shape[0] - 1)
            x = y[:, :turned].reshape(t, -1, head_size)
            beside = x.reshape(t, -1, head_size // 2, 2).flip(-1).reshape(t, -1, head_size)
            y = torch.cat([(a[at][:, None, :] * x + b[at][:, None, :] * beside).reshape(t, turned), y[:, turned:]], dim=1)
        q = (y[:, :nq] * scale).to(self.dtype)
        if num_kv_write:
            nk = num_kv_write * head_size
            k = y[:, nq:nq + nk].reshape(t, num_kv_write, head_size).to(k_pages.dtype)
            v = y[:, nq + nk:nq + 2 * nk].reshape(t, num_kv_write, head_size).to(v_pages.dtype)
            pos = ctx.positions.long()
            page = view.block_table[ctx.token_request.long(), pos // view.page_size].long()
            if int(page.min()) < 0:
                raise RuntimeError("a token of this step has no page")
            off = pos % view.page_size
            k_pages[page, :, off, :] = k
            v_pages[page, :, :, off] = v
        return q.contiguous()

    def attention(self, q, num_heads, num_kv_heads, head_size, ctx, view, k_pages, v_pages, window=None):
        """For every token: softmax over the keys of its own request at positions
        `<=` its own (`> position - window` with a window), times the values."""
        t = q.shape[0]
        out = torch.empty(t, num_heads * head_size, dtype=torch.float32, device=q.device)
        ps = view.page_size
        group = num_heads // num_kv_heads
        starts = ctx.run_start.tolist()
        for r in range(ctx.num_requests):
            s, e = starts[r], starts[r + 1]
            if e == s:
                continue
            total = int(ctx.cached_lens_host[r]) + (e - s)
            nb = -(-total // ps)
            pages = view.block_table[r, :nb].long().clamp(min=0)
            keys = k_pages[pages].float().permute(1, 0, 2, 3).reshape(num_kv_heads, nb * ps, head_size)[:, :total]
            vals = v_pages[pages].float().permute(1, 2, 0, 3).reshape(num_kv_heads, head_size, nb * ps)[:, :, :total]
            # pages that were given back may hold anything: what the mask hides must not reach the sum
            vals = torch.where(torch.isfinite(vals), vals, torch.zeros_like(vals))
            qr = q[s:e].float().reshape(e - s, num_heads, head_size).permute(1, 0, 2)
            keys = keys.repeat_interleave(group, dim=0)
            vals = vals.repeat_interleave(group, dim=0)
            scores = qr @ keys.transpose(1, 2)                       # [heads, run, total]
            pos = ctx.positions[s:e].long().unsqueeze(1)
            j = torch.arange(total, device=q.device).unsqueeze(0)
            allowed = j <= pos
            if window is not None:
                allowed &= j > pos - window
            scores = scores.masked_fill(~allowed.unsqueeze(0), float("-inf"))
            p = torch.softmax(scores, dim=-1)
            o = p @ vals.transpose(1, 2)                             # [heads, run, head_size]
            out[s:e] = o.permute(1, 0, 2).reshape(e - s, num_heads * head_size)
        return out.to(self.dtype)


    # ---------------------------------------------------------------- parts of other designs

    def _resolved(self, token_ids, kept_tokens):
        ids = token_ids.long()
        if kept_tokens is not None:
            ids = torch.where(ids < 0, kept_tokens.long()[(-1 - ids).clamp(min=0)], ids)
        return ids

    def embed_pairs(self, token_ids, table, pairs, buckets, mul_prev, mul_cur, ctx, last_token, kept_tokens=None):
        """float32 `table[token] + pairs[row]`, row = (previous * mul_prev + token * mul_cur) mod buckets, and
        `buckets` at position 0. `last_token` `[slots, 2]` keeps a request's last token at place (its position) & 1:
        the token before a step's first of a request is read there, and the step's last is written."""
        ids = self._resolved(token_ids, kept_tokens)
        starts = ctx.run_start.long()
        first = torch.zeros_like(ids, dtype=torch.bool)
        first[starts[:-1]] = True
        slots = ctx.slots.long()
        before = torch.roll(ids, 1)
        pos = ctx.positions.long()
        before[starts[:-1]] = last_token[slots, (pos[starts[:-1]] - 1) & 1].long()
        rows = (before * mul_prev + ids * mul_cur) % buckets
        rows = torch.where(ctx.positions.long() == 0, torch.full_like(rows, buckets), rows)
        last_token[slots, pos[starts[1:] - 1] & 1] = ids[starts[1:] - 1].to(last_token.dtype)
        return table[ids].float() + pairs[rows].float()

    def norm_add(self, y, weight, bias, eps, center, residual, mult=1.0, out=None, want_compute=False):
        """float32 `residual + mult * norm(y)`; `center` as in `layernorm`. With `want_compute` the pair (result,
        its copy in the compute dtype)."""
        normed = self.layernorm(y, weight, bias, eps, torch.float32, True, False, center)[0]
        result = residual.float() + mult * normed
        if out is not None:
            out.copy_(result)
            result = out
        return (result, result.to(self.dtype)) if want_compute else result

    def join_norm_conv(self, x, join, pre, conv_w, state, which, ctx, dtype):
        """What a part reads: `h = pre_norm(x')`, the result `h + conv(h)` as `input_conv` makes it, with `x' = x`,
        or for `join` = (y, weight, bias, center, mult), `x' = x + mult * post_norm(y)`. `pre` = (weight, bias,
        center, eps), one eps for both norms. Returns (x', the result in `dtype`)."""
        pw, pb, pc, eps = pre
        if join is not None:
            x = self.norm_add(join[0], join[1], join[2], eps, join[3], x, join[4])
        h = self.layernorm(x, pw, pb, eps, torch.float32, True, False, pc)[0]
        return x, self.input_conv(h, conv_w, state, which, ctx, dtype)

    def input_conv(self, h, weight, state, which, ctx, dtype):
        """`h + conv(h)`: conv(h)_t = sum_j weight[:, j] h_(t - taps + 1 + j) over the tokens of t's own request;
        the taps - 1 inputs before a step's first token of a request come from `state[slot, which]`
        (`[taps, width]`: the input at position p at place p mod taps; zeros before a request's start), which
        then takes the run's last ones."""
        taps = weight.shape[1]
        out = torch.empty_like(h)
        start = 0
        for r in range(ctx.num_requests):
            n, slot, have = int(ctx.run_lens_host[r]), int(ctx.slots_host[r]), int(ctx.cached_lens_host[r])
            run = h[start:start + n].float()
            if taps > 1:
                before = [state[slot, which, p % taps].float() if p >= 0 else torch.zeros_like(run[0])
                          for p in range(have - (taps - 1), have)]
                seq = torch.cat([torch.stack(before), run], dim=0)
                for i in range(max(0, n - (taps - 1)), n):
                    state[slot, which, (have + i) % taps] = run[i]
            else:
                seq = run
            acc = run.clone()
            for j in range(taps):
                acc = acc + weight[:, j].float()[None, :] * seq[j:j + n]
            out[start:start + n] = acc
            start += n
        return out.to(dtype)

    def poly_norm(self, z, coeffs, eps):
        """a N(z) + b N(z^2) + c N(z^3) + e, N(v) = v / sqrt(mean(v^2) + eps) over a row; float32 in, compute
        dtype out."""
        z = z.float()
        c = coeffs.float()

        def unit(v):
            return v * torch.rsqrt((v * v).mean(-1, keepdim=True) + eps)
        return (c[0] * unit(z) + c[1] * unit(z * z) + c[2] * unit(z * z * z) + c[3]).to(self.dtype)

    def mul_columns(self, g, rows, offset):
        """`g * rows[:, offset:offset + g.shape[1]]`, rounded once."""
        return (g.float() * rows[:, offset:offset + g.shape[1]].float()).to(self.dtype)

    def weighted_sum(self, history, weights, count):
        """float32 `sum_j weights[j] history[j]` over the first `count` slots of `history` `[slots, T, width]`."""
        out = torch.zeros_like(history[0])
        for j in range(count):
            out = out + weights[j] * history[j]
        return out

    @staticmethod
    def _turn(x, positions, freqs):
        """Pairs (2i, 2i + 1) of the last axis of `x` `[T, ..., r]` turned by positions * freqs[i]; float32."""
        dims = 2 * freqs.numel()
        angle = positions.float().reshape([-1] + [1] * (x.dim() - 1)) * freqs.float()
        cos, sin = torch.cos(angle), torch.sin(angle)
        u, v = x[..., 0:dims:2], x[..., 1:dims:2]
        out = x.clone()
        out[..., 0:dims:2] = u * cos - v * sin
        out[..., 1:dims:2] = v * cos + u * sin
        return out

    def latent_norms(self, down, q_rank, kv_rank, rot, q_weight, kv_weight, eps, freqs, ctx, view, latent_pages,
                     rotated_pages, across_pages=None):
        """`down` float32 `[T, q_rank + kv_rank + rot]`: the first q_rank elements, scaled to unit root mean
        square and weighted, come back in the compute dtype; the next kv_rank likewise go to the tokens' places
        in `latent_pages` (and, the page's tokens side by side, in `across_pages` `[pages, kv_rank, page_size]`), the
        last `rot`, turned by the position, to `rotated_pages` (kv_rank 0: none). The rows of `down` may hold more
        behind these; q_rank 0: no query latent, and nothing comes back."""
        x = down.float()

        def rms(v, w):
            return v * torch.rsqrt((v * v).mean(-1, keepdim=True) + eps) * w.float()
        c_q = rms(x[:, :q_rank], q_weight).to(self.dtype) if q_rank else None
        if kv_rank:
            pos = ctx.positions.long()
            page = view.block_table[ctx.token_request.long(), pos // view.page_size].long()
            if int(page.min()) < 0:
                raise RuntimeError("a token of this step has no page")
            off = pos % view.page_size
            latent_pages[page, off] = rms(x[:, q_rank:q_rank + kv_rank], kv_weight).to(latent_pages.dtype)
            if across_pages is not None:
                across_pages[page, :, off] = latent_pages[page, off]
            turned = self._turn(x[:, q_rank + kv_rank:q_rank + kv_rank + rot], pos, freqs)
            rotated_pages[page, off] = turned.to(rotated_pages.dtype)
        return c_q

    def batched_linear(self, x, w, alpha=1.0, out_f32=False):
        """`out[t, h, :] = alpha * w[h] x[t, h, :]`: x `[T, H, K]` (a view whose last axis is dense), w `[H, N, K]`."""
        y = torch.einsum("thk,hnk->thn", x.to(w.dtype).float(), w.float()) * alpha
        return (y if out_f32 else y.to(self.dtype)).contiguous()

    @staticmethod
    def _with_sink(scores, allowed, sink):
        """Softmax over the allowed keys of `scores` `[H, I, J]`; `sink` `[H]`: the denominator also holds
        exp(sink) of the head, once."""
        scores = scores.masked_fill(~allowed.unsqueeze(0), float("-inf"))
        if sink is None:
            p = torch.softmax(scores, dim=-1)
        else:
            heads, rows, _ = scores.shape
            beside = sink.float().reshape(heads, 1, 1).expand(heads, rows, 1)
            p = torch.softmax(torch.cat([scores, beside], dim=-1), dim=-1)[..., :-1]
        return torch.where(allowed.unsqueeze(0), p, torch.zeros_like(p))

    def latent_attention(self, q, q_lat, num_heads, head_size, rot, kv_rank, freqs, scale, ctx, view, latent_pages,
                         rotated_pages, across_pages=None, window=None, sink=None, gate=None):
        """For every token and head: scores scale * (q_lat . c[j] + turn(q_r) . k_r[j]) over the cached tokens j
        of its request with j <= position (and position - j < window), softmax, and the weighted sum of the
        c[j]: `[T, H, kv_rank]`. `q` `[T, H * (head_size + rot)]` holds q_r, unturned, behind each head's
        `head_size` elements; `q_lat` is `[T, H, kv_rank]`. `across_pages` hold the c[j] once more, a page's
        tokens side by side, for kernels that sum from there. `sink` (float32 `[H]`): the softmax's denominator
        also holds exp(sink) of the head; `gate` (float32 `[T, H]`, rows may lie apart): a head's result is
        multiplied by sigmoid(gate)."""
        t = q.shape[0]
        ps = view.page_size
        out = torch.empty(t, num_heads, kv_rank, dtype=torch.float32, device=q.device)
        q_r = q.view(t, num_heads, head_size + rot)[:, :, head_size:].float()
        q_r = self._turn(q_r, ctx.positions.long(), freqs)
        starts = ctx.run_start.tolist()
        for r in range(ctx.num_requests):
            s, e = starts[r], starts[r + 1]
            if e == s:
                continue
            total = int(ctx.cached_lens_host[r]) + (e - s)
            nb = -(-total // ps)
            pages = view.block_table[r, :nb].long().clamp(min=0)
            c = latent_pages[pages].float().reshape(nb * ps, kv_rank)[:total]
            k_r = rotated_pages[pages].float().reshape(nb * ps, rot)[:total]
            scores = (torch.einsum("ihd,jd->hij", q_lat[s:e].float(), c) + torch.einsum("ihd,jd->hij", q_r[s:e], k_r)) * scale
            pos = ctx.positions[s:e].long().unsqueeze(1)
            j = torch.arange(total, device=q.device).unsqueeze(0)
            allowed = j <= pos
            if window is not None:
                allowed &= pos - j < window
            p = self._with_sink(scores, allowed, sink)
            # pages that were given back may hold anything: what the mask hides must not reach the sum
            c = torch.where(torch.isfinite(c), c, torch.zeros_like(c))
            out[s:e] = torch.einsum("hij,jd->ihd", p, c)
        if gate is not None:
            out = out * torch.sigmoid(gate.float())[:, :, None]
        return out.to(self.dtype)

    expand_prompts = False     # tests set it: steps of prompts' runs alone take `latent_attention_expanded`

    def latent_expands(self, ctx, head_size, rot, value_size, kv_rank) -> bool:
        return bool(self.expand_prompts and int(ctx.run_lens_host.min()) > 1)

    def latent_attention_expanded(self, q, w_uk, w_uv, num_heads, head_size, rot, value_size, kv_rank, freqs, scale, ctx,
                                  view, latent_pages, rotated_pages, window=None, sink=None, gate=None):
        """Attention with the keys W_uk c and values W_uv c of the cached tokens made explicitly:
        `[T, H * value_size]`, what `latent_attention` and the product with W_uv give by the other order."""
        t, ps = q.shape[0], view.page_size
        out = torch.empty(t, num_heads * value_size, dtype=torch.float32, device=q.device)
        qh = q.view(t, num_heads, head_size + rot).float()
        q_r = self._turn(qh[:, :, head_size:], ctx.positions.long(), freqs)
        starts = ctx.run_start.tolist()
        for r in range(ctx.num_requests):
            s, e = starts[r], starts[r + 1]
            total = int(ctx.cached_lens_host[r]) + (e - s)
            nb = -(-total // ps)
            pages = view.block_table[r, :nb].long().clamp(min=0)
            c = latent_pages[pages].reshape(nb * ps, kv_rank)[:total]
            c = torch.where(torch.isfinite(c.float()), c.float(), torch.zeros_like(c.float())).to(latent_pages.dtype)
            k_r = rotated_pages[pages].float().reshape(nb * ps, rot)[:total]
            k_n = self.linear(c, w_uk).float().view(total, num_heads, head_size)
            val = self.linear(c, w_uv).float().view(total, num_heads, value_size)
            scores = (torch.einsum("ihd,jhd->hij", qh[s:e, :, :head_size], k_n) + torch.einsum("ihd,jd->hij", q_r[s:e], k_r)) * scale
            pos = ctx.positions[s:e].long().unsqueeze(1)
            j = torch.arange(total, device=q.device).unsqueeze(0)
            allowed = j <= pos
            if window is not None:
                allowed &= pos - j < window
            p = self._with_sink(scores, allowed, sink)
            out[s:e] = torch.einsum("hij,jhd->ihd", p, val).reshape(e - s, num_heads * value_size)
        if gate is not None:
            out = (out.view(t, num_heads, value_size) * torch.sigmoid(gate.float())[:, :, None]).reshape(t, -1)
        return out.to(self.dtype)


    # ---------------------------------------------------------------- normed, turned and blended projections

    def qkv_prepare(self, proj, num_heads, num_kv, head_size, value_size, cache_head, q_weight, k_weight, eps, freqs,
                    interleaved, scale, mix_weight, first_values, ctx, view, k_pages, v_pages, per_head=False,
                    values_at=None, head_scale=None):
        """From the float32 projections `proj` `[T, H n + G n + G v]` (bias added) to the queries and the cache:
        the queries and the keys are each scaled to unit root mean square over their whole width and weighted
        (`q_weight`, `k_weight`; None: not), the first `2 len(freqs)` elements of every head are turned by
        position * freqs (pairs (i, i + half), or neighbours with `interleaved`; `freqs` None: not), the queries
        are multiplied by `scale`, the values become (1 - l) v + l first_values with l = `mix_weight[0]`
        (`first_values` float32 `[T, G v]`, a view whose rows may lie apart; None: not). Keys and values go to their
        tokens' places in the pages, heads filled up with zeros to `cache_head` elements; the queries come back
        `[T, H cache_head]`, filled up alike, in the compute dtype. `values_at`: the column of a row where the
        values begin, if not behind the keys (the keys' own first column: the values are the keys as projected).
        `head_scale` (float32 `[H]`): a query head's elements are multiplied by its number as well."""
        t = proj.shape[0]
        nq, nk, nv = num_heads * head_size, num_kv * head_size, num_kv * value_size
        x = proj.float()
        at = nq + nk if values_at is None else int(values_at)
        q, k, v = x[:, :nq], x[:, nq:nq + nk], x[:, at:at + nv]
        if per_head:
            # every head to unit root mean square by itself; the weights, if any, are still one a projection element
            q, k = q.reshape(t, num_heads, head_size), k.reshape(t, num_kv, head_size)
            q = (q * torch.rsqrt((q * q).mean(-1, keepdim=True) + eps)).reshape(t, nq)
            k = (k * torch.rsqrt((k * k).mean(-1, keepdim=True) + eps)).reshape(t, nk)
            if q_weight is not None:
                q, k = q * q_weight.float(), k * k_weight.float()
        elif q_weight is not None:
            q = q * torch.rsqrt((q * q).mean(-1, keepdim=True) + eps) * q_weight.float()
            k = k * torch.rsqrt((k * k).mean(-1, keepdim=True) + eps) * k_weight.float()
        q, k = q.reshape(t, num_heads, head_size), k.reshape(t, num_kv, head_size)
        if freqs is not None:
            pos = ctx.positions.long()
            if interleaved:
                q, k = self._turn(q, pos, freqs), self._turn(k, pos, freqs)
            else:
                half = freqs.numel()
                angle = pos.float()[:, None, None] * freqs.float()[None, None, :]
                cos, sin = torch.cos(angle), torch.sin(angle)

                def turned(y):
                    a, b = y[..., :half], y[..., half:2 * half]
                    return torch.cat([a * cos - b * sin, b * cos + a * sin, y[..., 2 * half:]], dim=-1)
                q, k = turned(q), turned(k)
        if first_values is not None:
            lam = mix_weight.float()[0]
            v = (1.0 - lam) * v + lam * first_values.float()
        v = v.reshape(t, num_kv, value_size)
        pos = ctx.positions.long()
        page = view.block_table[ctx.token_request.long(), pos // view.page_size].long()
        if int(page.min()) < 0:
            raise RuntimeError("a token of this step has no page")
        off = pos % view.page_size
        k_pages[page, :, off, :] = 0
        k_pages[page, :, off, :head_size] = k.to(k_pages.dtype)
        v_pages[page, :, :, off] = 0
        v_pages[page, :, :value_size, off] = v.to(v_pages.dtype)
        out = torch.zeros(t, num_heads, cache_head, dtype=self.dtype, device=proj.device)
        if head_scale is not None:
            q = q * head_scale.float()[None, :, None]
        out[:, :, :head_size] = (q * scale).to(self.dtype)
        return out.reshape(t, num_heads * cache_head)

    def attention_scored(self, q, num_heads, num_kv_heads, head_size, ctx, view, k_pages, v_pages, window=None,
                         chunk=None, softcap=None, distance_bias=None, gate=None, value_size=None, out=None,
                         out_scale=1.0, gate_per_head=False):
        """Attention whose scores or mask are not the plain ones. For a query at position i and a key at j <= i of
        its request: s = q . k (the query comes scaled); with `softcap` c, s <- c tanh(s / c); with
        `distance_bias` (float32 `[heads, D + 1]`), s <- s + distance_bias[head, min(i - j, D)]. Visible are the
        keys with i - j < window (if given) and floor(j / chunk) = floor(i / chunk) (if given). Softmax over the
        visible keys, times the values. `gate` (float32 `[T, heads * value_size]`, rows may lie apart): the first
        `value_size` elements of every head are multiplied by sigmoid(gate) (`gate_per_head`: `[T, heads]`, one
        number for all elements of a head). The result times `out_scale` goes to
        `out` (`[T, heads * head_size]` in the compute dtype, rows may lie apart) or to a new tensor."""
        t = q.shape[0]
        value_size = head_size if value_size is None else value_size
        res = torch.empty(t, num_heads, head_size, dtype=torch.float32, device=q.device)
        ps = view.page_size
        group = num_heads // num_kv_heads
        starts = ctx.run_start.tolist()
        for r in range(ctx.num_requests):
            s, e = starts[r], starts[r + 1]
            if e == s:
                continue
            total = int(ctx.cached_lens_host[r]) + (e - s)
            nb = -(-total // ps)
            pages = view.block_table[r, :nb].long().clamp(min=0)
            keys = k_pages[pages].float().permute(1, 0, 2, 3).reshape(num_kv_heads, nb * ps, head_size)[:, :total]
            vals = v_pages[pages].float().permute(1, 2, 0, 3).reshape(num_kv_heads, head_size, nb * ps)[:, :, :total]
            vals = torch.where(torch.isfinite(vals), vals, torch.zeros_like(vals))
            keys = torch.where(torch.isfinite(keys), keys, torch.zeros_like(keys))
            qr = q[s:e].float().reshape(e - s, num_heads, head_size).permute(1, 0, 2)
            keys = keys.repeat_interleave(group, dim=0)
            vals = vals.repeat_interleave(group, dim=0)
            scores = qr @ keys.transpose(1, 2)                       # [heads, run, total]
            if softcap:
                scores = softcap * torch.tanh(scores / softcap)
            pos = ctx.positions[s:e].long().unsqueeze(1)
            j = torch.arange(total, device=q.device).unsqueeze(0)
            allowed = j <= pos
            if distance_bias is not None:
                far = distance_bias.shape[1] - 1
                scores = scores + distance_bias.float()[:, (pos - j).clamp(0, far)]
            if window is not None:
                allowed &= j > pos - window
            if chunk is not None:
                allowed &= (j // chunk) == (pos // chunk)
            scores = scores.masked_fill(~allowed.unsqueeze(0), float("-inf"))
            p = torch.softmax(scores, dim=-1)
            res[s:e] = (p @ vals.transpose(1, 2)).permute(1, 0, 2)
        if gate is not None:
            res[:, :, :value_size] *= torch.sigmoid(gate.float()).reshape(t, num_heads, 1 if gate_per_head else value_size)
        res = (res * out_scale).reshape(t, num_heads * head_size)
        if out is None:
            return res.to(self.dtype)
        out.copy_(res)
        return out

    # ---------------------------------------------------------------- recurrences

    def min_gru(self, proj, inner, ctx, carried, out=None, out_scale=1.0):
        """The minimal gated recurrence over a step's runs. `proj` float32 `[T, 3 inner]` = [z' | u | g] (biases
        added): z = sigmoid(z'), c = u + 1/2 where u >= 0 and sigmoid(u) below, S <- (1 - z) S + z c; the result
        is S silu(g) times `out_scale`, `[T, inner]` in the compute dtype (into `out`, whose rows may lie apart).
        `carried` float32 `[slots, 2, inner]`: the token at position p reads place (p - 1) & 1 (zeros at p = 0) and
        writes place p & 1."""
        x = proj.float()
        z, u, g = torch.sigmoid(x[:, :inner]), x[:, inner:2 * inner], x[:, 2 * inner:3 * inner]
        cand = torch.where(u >= 0, u + 0.5, torch.sigmoid(u))
        res = torch.empty(x.shape[0], inner, dtype=torch.float32, device=x.device)
        start = 0
        for r in range(ctx.num_requests):
            n, slot, have = int(ctx.run_lens_host[r]), int(ctx.slots_host[r]), int(ctx.cached_lens_host[r])
            s = carried[slot, (have - 1) & 1].clone() if have > 0 else torch.zeros_like(carried[slot, 0])
            for i in range(start, start + n):
                s = (1.0 - z[i]) * s + z[i] * cand[i]
                res[i] = s
            if n:
                carried[slot, (have + n - 1) & 1] = s
            start += n
        res = res * (g * torch.sigmoid(g)) * out_scale
        if out is None:
            return res.to(self.dtype)
        out.copy_(res)
        return out

    def channel_conv(self, x, weight, bias, ctx, state):
        """A causal convolution over the request's tokens on every channel, with a bias:
        u_t = bias + sum_j weight[:, j] x_(t - taps + 1 + j), zeros before the request's start. `x` float32
        `[T, channels]` (rows may lie apart), `weight` `[channels, taps]`. `state` float32 `[slots, taps, channels]`
        holds the input at position p at place p mod taps and takes the run's last ones. Returns (u in float32, u
        in the compute dtype)."""
        taps = weight.shape[1]
        x = x.float()
        out = torch.empty_like(x)
        start = 0
        for r in range(ctx.num_requests):
            n, slot, have = int(ctx.run_lens_host[r]), int(ctx.slots_host[r]), int(ctx.cached_lens_host[r])
            run = x[start:start + n]
            if taps > 1:
                before = [state[slot, p % taps].float() if p >= 0 else torch.zeros_like(run[0])
                          for p in range(have - (taps - 1), have)]
                seq = torch.cat([torch.stack(before), run], dim=0)
                for i in range(max(0, n - (taps - 1)), n):
                    state[slot, (have + i) % taps] = run[i]
            else:
                seq = run
            acc = bias.float()[None, :].expand(n, -1).clone()
            for j in range(taps):
                acc = acc + weight[:, j].float()[None, :] * seq[j:j + n]
            out[start:start + n] = acc
            start += n
        return out, out.to(self.dtype)

    def gated_linear_recurrence(self, gates, gate_bias, u, y, rate, ctx, carried, out=None, out_scale=1.0):
        """The real-gated linear recurrence over a step's runs. `gates` float32 `[T, blocks, 2 w]`: a part's
        pre-activations of the recurrence gate (the first w) and of the input gate, `gate_bias` `[blocks, 2 w]`
        their biases; `u` float32 `[T, blocks w]`; `y` float32 `[T, blocks w]` (rows may lie apart), through
        gelu_tanh here; `rate` `[blocks w]` = -8 softplus(lam).
        a = exp(rate sigmoid(r')), S <- a S + sqrt(1 - a^2) sigmoid(i') u; the result S gelu_tanh(y) times
        `out_scale` in the compute dtype. `carried` as in `min_gru`."""
        t, blocks, two_w = gates.shape
        w = two_w // 2
        pre = gates.float() + gate_bias.float()[None]
        r = torch.sigmoid(pre[:, :, :w]).reshape(t, blocks * w)
        i = torch.sigmoid(pre[:, :, w:]).reshape(t, blocks * w)
        log_a = rate.float()[None, :] * r
        a = torch.exp(log_a)
        inp = torch.sqrt(-torch.expm1(2.0 * log_a)) * i * u.float()      # sqrt(1 - a^2) without the cancellation near a = 1
        res = torch.empty(t, blocks * w, dtype=torch.float32, device=u.device)
        start = 0
        for q in range(ctx.num_requests):
            n, slot, have = int(ctx.run_lens_host[q]), int(ctx.slots_host[q]), int(ctx.cached_lens_host[q])
            s = carried[slot, (have - 1) & 1].clone() if have > 0 else torch.zeros_like(carried[slot, 0])
            for k in range(start, start + n):
                s = a[k] * s + inp[k]
                res[k] = s
            if n:
                carried[slot, (have + n - 1) & 1] = s
            start += n
        res = res * self.activation(y.float(), "gelu_new") * out_scale
        if out is None:
            return res.to(self.dtype)
        out.copy_(res)
        return out

    # ---------------------------------------------------------------- the matrix memory

    def matrix_memory(self, proj, num_heads, head_size, value_size, gate_cap, eps, norm_weight, ctx, memory, normalizer,
                      peak):
        """The recurrence of the matrix-memory mixer over a step's runs and what follows it up to the output
        projection. `proj` float32 `[T, 2 H n + 2 H v + 2 H]`: queries, keys, values, output gates, and a head's
        input and forget pre-activations (bias added). State float32, in two places by the parity of the
        position: `memory` `[slots, 2, H, v, n]` (a column's rows side by side), `normalizer` `[slots, 2, H, n]`, `peak`
        `[slots, 2, H]`; the token
        at position p reads place (p - 1) & 1 (nothing at p = 0: all zeros) and writes place p & 1. Returns
        `[T, H v]` in the compute dtype: each head's result at unit root mean square, weighted, times
        sigmoid(gate)."""
        t = proj.shape[0]
        h, n, v = num_heads, head_size, value_size
        x = proj.float()
        q = x[:, :h * n].reshape(t, h, n) * (n ** -0.5)
        k = x[:, h * n:2 * h * n].reshape(t, h, n)
        val = x[:, 2 * h * n:2 * h * n + h * v].reshape(t, h, v)
        gate = x[:, 2 * h * n + h * v:2 * h * n + 2 * h * v]
        gi = gate_cap * torch.tanh(x[:, -2 * h:-h] / gate_cap)
        gf = torch.nn.functional.logsigmoid(gate_cap * torch.tanh(x[:, -h:] / gate_cap))
        out = torch.empty(t, h, v, dtype=torch.float32, device=proj.device)
        start = 0
        for r in range(ctx.num_requests):
            count, slot, have = int(ctx.run_lens_host[r]), int(ctx.slots_host[r]), int(ctx.cached_lens_host[r])
            if have > 0:
                at = (have - 1) & 1
                mem, nrm, pk = memory[slot, at].transpose(1, 2).clone(), normalizer[slot, at].clone(), peak[slot, at].clone()
            else:
                mem = torch.zeros_like(memory[slot, 0]).transpose(1, 2).clone()
                nrm, pk = torch.zeros_like(normalizer[slot, 0]), torch.zeros_like(peak[slot, 0])
            for i in range(start, start + count):
                new = torch.maximum(gf[i] + pk, gi[i])
                keep, take = torch.exp(gf[i] + pk - new), torch.exp(gi[i] - new)
                mem = keep[:, None, None] * mem + take[:, None, None] * (k[i][:, :, None] * val[i][:, None, :])
                nrm = keep[:, None] * nrm + take[:, None] * k[i]
                pk = new
                below = torch.maximum((nrm * q[i]).sum(-1).abs(), torch.exp(-pk)) + 1e-6
                out[i] = torch.einsum("hnv,hn->hv", mem, q[i]) / below[:, None]
            at = (have + count - 1) & 1
            memory[slot, at], normalizer[slot, at], peak[slot, at] = mem.transpose(1, 2), nrm, pk
            start += count
        out = out * torch.rsqrt((out * out).mean(-1, keepdim=True) + eps)
        y = out.reshape(t, h * v) * norm_weight.float() * torch.sigmoid(gate)
        return y.to(self.dtype)

    # ---------------------------------------------------------------- experts

    def route(self, z, top, score="sigmoid", renormalize=False, correction=None, scale=1.0):
        """float32 router logits `[T, E]` -> (int32 `[T, top]` the experts with the largest scores, the lower
        number first where two are equal; float32 `[T, top]` their scores, sigmoid(z) or softmax(z), divided by
        their sum with `renormalize`). The ranking is by the logits, which both scores grow with: two large
        logits that float32 still tells apart can have scores that it does not. With `correction` (float32 `[E]`)
        the ranking is by score + correction, and the weights are the scores without it; `scale` multiplies the
        weights."""
        s = torch.sigmoid(z.float()) if score == "sigmoid" else torch.softmax(z.float(), dim=-1)
        ranked = z.float() if correction is None else s + correction.float()
        order = torch.sort(ranked, dim=-1, descending=True, stable=True).indices[:, :top]
        w = torch.gather(s, 1, order)
        if renormalize:
            w = w / w.sum(-1, keepdim=True)
        if scale != 1.0:
            w = w * scale
        return order.to(torch.int32).contiguous(), w.contiguous()

    @staticmethod
    def _gated(g, u, activation, limit=None):
        """What a gated expert makes of its two halves: act(g) * u; "clamped_swiglu": with g' = min(g, limit) and
        u' = clamp(u, -limit, limit), g' sigmoid(1.702 g') (u' + 1)."""
        if activation == "clamped_swiglu":
            g, u = g.clamp(max=limit), u.clamp(min=-limit, max=limit)
            return g * torch.sigmoid(1.702 * g) * (u + 1.0)
        if activation == "silu":
            return g * torch.sigmoid(g) * u
        return ReferenceOps.activation(g, activation) * u

    def gated_activation(self, gate_up, activation, row_weights=None, limit=None):
        """`act(g) * u` from float32 `[T, 2 F]` = [g | u], in the compute dtype; `row_weights` `[T]`: a factor a
        row on both g and u."""
        f = gate_up.shape[1] // 2
        g, u = gate_up[:, :f].float(), gate_up[:, f:].float()
        if row_weights is not None:
            g, u = g * row_weights.float()[:, None], u * row_weights.float()[:, None]
        return self._gated(g, u, activation, limit).to(self.dtype)

    def expert_mixture(self, h, chosen, weights, w_gate_up, w_down, activation, weight_on, residual=None, may_wait=False,
                       limit=None):
        """float32 `residual + sum_c expert_(chosen[t, c])(h[t])` with the weights `weights[t, c]` on the expert's
        input (`weight_on="input"`: act(w g) * (w u), the float32 sums of the first product times w) or on its
        output. `w_gate_up` `[E, 2 F, D]` (gate rows, then up rows), `w_down` `[E, D, F]`."""
        t, top = chosen.shape
        f = w_down.shape[2]
        out = residual.float().clone() if residual is not None else torch.zeros(t, w_down.shape[1], dtype=torch.float32,
                                                                                device=h.device)
        x = h.to(w_gate_up.dtype).float()
        for c in range(top):
            e = chosen[:, c].long()
            gu = torch.einsum("tk,tnk->tn", x, w_gate_up[e].float())
            w = weights[:, c].float()[:, None]
            if weight_on == "input":
                gu = gu * w
            inner = self._gated(gu[:, :f], gu[:, f:], activation, limit).to(self.dtype)
            y = torch.einsum("tf,tdf->td", inner.to(w_down.dtype).float(), w_down[e].float())
            out = out + (y if weight_on == "input" else y * w)
        return out

    # ---------------------------------------------------------------- output end

    def gather_rows(self, x, rows):
        return x[rows.long()]

    def cast(self, x, dtype):
        return x.to(dtype)

    def ban_tokens(self, logits, tokens):
        rows = torch.nonzero(tokens >= 0).flatten()
        logits[rows, tokens[rows].long()] = float("-inf")
        return logits

    def ban_pairs(self, logits, rows, tokens):
        logits[rows.long(), tokens.long()] = float("-inf")
        return logits

    def argmax(self, logits):
        return logits.argmax(dim=-1).to(torch.int32)

    def sample(self, logits, temperature, top_k, top_p, seeds, counters, min_keep=None):
        """One token per row. Row i: logits / temperature[i]; the top_k[i] largest
        are kept (0 keeps all; ties go to the lower token id); of these, in
        descending order, the shortest prefix whose softmax mass reaches
        top_p[i] (>= 1 keeps all); neither keeps fewer than min_keep[i] tokens
        (1 if not given); the draw is by inverse CDF over the kept
        tokens in ascending order of token id with the uniform number
        `philox_uniform(seeds[i], counters[i])`, or 0.5 for a counter below zero.
        temperature 0 is argmax."""
        m, v = logits.shape
        out = torch.empty(m, dtype=torch.int32)
        for i in range(m):
            row = logits[i].float().cpu()
            temp = float(temperature[i])
            if temp == 0.0:
                out[i] = int(row.argmax())
                continue
            row = row / temp
            values, indices = torch.sort(row, descending=True, stable=True)
            least = max(1, int(min_keep[i])) if min_keep is not None else 1
            k = int(top_k[i])
            if k > 0:
                k = max(k, least)
            if 0 < k < v:
                values, indices = values[:k], indices[:k]
            p = float(top_p[i])
            if p < 1.0:
                cum = torch.cumsum(torch.softmax(values, -1, dtype=torch.float32), -1)
                keep = torch.cat([torch.ones(1, dtype=torch.bool), (cum < p)[:-1]])
                keep[:least] = True
                values, indices = values[keep], indices[keep]
            order = torch.argsort(indices)
            values, indices = values[order], indices[order]
            w = torch.exp(values - values.max()).double()
            cum = torch.cumsum(w, -1)
            u = 0.5 if int(counters[i]) < 0 else philox_uniform(int(seeds[i]), int(counters[i]))
            pick = int((cum <= u * float(cum[-1])).sum())
            out[i] = int(indices[min(pick, len(indices) - 1)])
        return out.to(logits.device)

    def synchronize(self):
        if self.device.type == "cuda":
            torch.cuda.synchronize(self.device)
