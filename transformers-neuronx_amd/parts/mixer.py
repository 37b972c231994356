"""Token mixers."""
import math
from typing import Dict, List, Optional

import torch

from .base import POSITIONS, CacheNeed, Mixer, register_mixer
from .spec import ParamDecl


def distance_bucket(n: int, rows: int, max_distance: int) -> int:
    """The row of a distance-bias table for the distance n >= 0 between a query and a key: the distance itself
    below rows / 2, then logarithmic steps that reach the last row at `max_distance`."""
    half = rows // 2
    if n < half:
        return n
    return min(rows - 1, half + int(math.floor(math.log(n / half) / math.log(max_distance / half) * (rows - half))))


def bias_by_distance(table: torch.Tensor, max_distance: int) -> torch.Tensor:
    """float32 `[heads, max_distance + 1]` from a table `[rows, heads]`: what a head adds to the score of a key n
    tokens back, at column min(n, max_distance) (every distance from `max_distance` on falls into the last row).
    The buckets are worked out once, on the host, in double precision."""
    rows = table.shape[0]
    if rows < 2 or max_distance <= rows // 2:
        raise ValueError(f"a distance bias of {rows} rows up to distance {max_distance}: the rows beyond the first "
                         f"half need a distance beyond {rows // 2} to spread over")
    rows_of = torch.tensor([distance_bucket(n, rows, max_distance) for n in range(max_distance)] + [rows - 1],
                           dtype=torch.long, device=table.device)
    return table.float()[rows_of].t().contiguous()


@register_mixer("attention")
class Attention(Mixer):
    """Softmax attention over a paged key/value cache.

    `Q = (h Wq^T + bq) * scale`, keys and values of the step's tokens are stored
    into the request's pages, each query attends to the keys of its own request
    at positions `<=` its own (and `> position - window` when a window is set),
    softmax in float32, then the output projection (reference:
    opt/model.py:444-523; scale layers/attention.py:428-437; masks
    hlo.py:1030-1042 and the bottom-right block-diagonal form hlo.py:3211-3309;
    cache scatter by slot hlo.py:3665-3704).

    `num_kv_heads < num_heads` groups query heads over shared key/value heads.
    `own_kv=False` builds a mixer without key/value projections that reads the
    cache another call of the run order writes. `rotation` names a position
    encoding (a `PartSpec` of the position registry) that turns the queries and
    keys before they are scaled and stored: through its `pair_tables`, inside the
    projection's launch, or else through its `on_query_key`; OPT has none.
    """

    recordable = True

    def __init__(self, width: int, num_heads: int, head_size: int, names, num_kv_heads: Optional[int] = None,
                 bias: bool = True, window: Optional[int] = None, scale: Optional[float] = None,
                 own_kv: bool = True, rotation=None, value_size: Optional[int] = None, out_bias: Optional[bool] = None,
                 qk_norm=None, value_mix=None, weight_suffix: str = ".weight", bias_suffix: str = ".bias",
                 softcap: Optional[float] = None, distance_bias=None, chunk: Optional[int] = None,
                 out_gate: Optional[str] = None, out_gate_per_head: bool = False, values_from_keys: bool = False,
                 head_scale: Optional[str] = None):
        """`names`: the checkpoint's names of the query, key, value and output projections, relative to
        the mixer's prefix (the architecture's spec gives them); a matrix's name adds `weight_suffix`, a bias's
        `bias_suffix`. `out_bias`: whether the output projection has a bias (as the others, if not said).

        `value_size`: elements of a value head where they differ from a query/key head's `head_size`.
        `qk_norm` = {eps, suffix}: queries and keys are scaled to unit root mean square over the whole
        projection, all heads at once, and weighted (the tensors `<query name><suffix>`, `<key name><suffix>`),
        after the bias and before the rotation. `value_mix` = {key, first, name}: the layers that give the same
        `key` blend their values with those the `first` of them made for the same token,
        v = (1 - l) v + l v_first with l the scalar tensor `name`; the blended values are what is cached. The
        first blends nothing and has no such tensor. A rotation whose pairs are not neighbours
        (`interleaved=False`) hands its frequencies to the kernel that norms, turns and stores.
        With `per_head` in `qk_norm` every head is scaled to unit root mean square by itself, and with
        `weighted=False` there are no weight tensors.
        These take the float32 route: the projection's float32 result goes through one kernel (`ops.qkv_prepare`)
        that norms, turns, scales, blends and stores, and heads of unequal sizes are cached filled up with
        zeros to one size, a multiple of 16.

        What changes the scores or the mask (the route above, and `ops.attention_scored` in the place of
        `ops.attention`): `softcap` c: a score s becomes c tanh(s / c) (after the scale). `distance_bias` =
        {name, max_distance, rows}: the tensor `name` `[rows, heads]` holds a bias a head for every bucket of the
        distance n = i - j between query and key, added after the cap: bucket(n) = n below rows / 2, and from
        there on logarithmic steps up to `max_distance`, min(rows - 1, rows/2 + floor(ln(n / (rows/2)) /
        ln(max_distance / (rows/2)) * (rows - rows/2))); `rows` None: the checkpoint's tensor says. `chunk` m: a
        query at position i sees the keys j <= i with floor(j / m) = floor(i / m), positions counted from the
        request's start. `out_gate`: the name of a matrix W_g `[heads * value_size, width]`; the heads' results
        side by side are multiplied by sigmoid(W_g h) before the output projection (the gate's rows ride in the
        one input projection); with `out_gate_per_head` W_g is `[heads, width]` and a head's whole result is
        multiplied by its one number.

        `values_from_keys`: there is no value projection (its name in `names` is not read): a token's values are
        its keys as projected, before their norm and turn. `head_scale`: the name of a tensor of one number a query
        head that multiplies the head's scores (beside `scale`). With `shared` in `qk_norm` (which implies
        `per_head`) the two weight tensors hold one head's `head_size` elements, the same for every head."""
        self.width, self.num_heads, self.head_size = width, num_heads, head_size
        self.num_kv_heads = num_kv_heads if num_kv_heads is not None else num_heads
        if self.num_heads % self.num_kv_heads:
            raise ValueError(f"num_heads ({num_heads}) must be a multiple of num_kv_heads ({self.num_kv_heads})")
        self.value_size = value_size if value_size is not None else head_size
        self.qk_norm = dict(qk_norm) if qk_norm else None
        self.value_mix = dict(value_mix) if value_mix else None
        self.rotation = POSITIONS.build(rotation) if rotation is not None else None
        halves = self.rotation is not None and not getattr(self.rotation, "interleaved", True)
        self.softcap = float(softcap) if softcap else None
        self.distance_bias = dict(distance_bias) if distance_bias else None
        self.chunk = int(chunk) if chunk else None
        self.out_gate, self.out_gate_per_head = out_gate, bool(out_gate_per_head) and bool(out_gate)
        self.values_from_keys, self.head_scale = bool(values_from_keys), head_scale
        if self.qk_norm and self.qk_norm.get("shared"):
            self.qk_norm["per_head"] = True
        if self.values_from_keys and self.value_size != head_size:
            raise ValueError(f"values that are the keys have the keys' size ({head_size}), not {self.value_size}")
        if self.values_from_keys and self.value_mix:
            raise ValueError("values that are the keys are not blended")
        if self.chunk is not None and window is not None:
            raise ValueError("an attention mixer masks by a window or by chunks, not both")
        self.scored = bool(self.softcap or self.distance_bias or self.chunk or out_gate)
        self.prepared = bool(self.qk_norm or self.value_mix or halves or self.value_size != head_size or self.scored
                             or self.values_from_keys or head_scale)
        self.defer_out = False      # set by a mixer that runs this one beside another and owns the output product
        if self.prepared:
            if not own_kv:
                raise ValueError("a mixer that norms, blends or fills up its heads makes its own keys and values")
            if self.rotation is not None and not hasattr(self.rotation, "frequencies"):
                raise ValueError("the float32 route turns by a rotation that gives `frequencies()`")
            self.cache_head = -(-max(head_size, self.value_size) // 16) * 16
        else:
            self.cache_head = head_size
        if self.cache_head % 16 or not 16 <= self.cache_head <= 256:
            raise ValueError(f"head_size must be a multiple of 16 between 16 and 256, got {head_size}")
        self.has_bias, self.window, self.own_kv = bias, window, own_kv
        self.has_out_bias = bias if out_bias is None else bool(out_bias)
        self.weight_suffix, self.bias_suffix = weight_suffix, bias_suffix
        self.scale = float(scale) if scale is not None else 1.0 / math.sqrt(head_size)
        self.names = tuple(names)
        if self.rotation is not None and not getattr(self.rotation, "recordable", False):
            self.recordable = False
        if len(self.names) != 4:
            raise ValueError("names: the query, key, value and output projections, four names")

    def cache_need(self) -> Optional[CacheNeed]:
        return CacheNeed("paged", kv_heads=self.num_kv_heads, head_size=self.cache_head, window=self.window)

    def param_decls(self, prefix: str) -> List[ParamDecl]:
        qn, kn, vn, on = self.names
        ws, bs = self.weight_suffix, self.bias_suffix
        q_out = self.num_heads * self.head_size
        kv_out = self.num_kv_heads * self.head_size
        v_out = self.num_kv_heads * self.value_size
        outs = [(qn, q_out)] + ([(kn, kv_out)] + ([] if self.values_from_keys else [(vn, v_out)]) if self.own_kv else [])
        d = []
        for n, out in outs:
            d.append(ParamDecl(f"{prefix}{n}{ws}", (out, self.width)))
            if self.has_bias:
                d.append(ParamDecl(f"{prefix}{n}{bs}", (out,), "vector"))
        d.append(ParamDecl(f"{prefix}{on}{ws}", (self.width, self.num_heads * self.value_size)))
        if self.has_out_bias:
            d.append(ParamDecl(f"{prefix}{on}{bs}", (self.width,), "vector"))
        if self.qk_norm and self.qk_norm.get("weighted", True):
            shared = self.qk_norm.get("shared")
            d += [ParamDecl(f"{prefix}{qn}{self.qk_norm['suffix']}", (self.head_size if shared else q_out,), "vector", "around_one"),
                  ParamDecl(f"{prefix}{kn}{self.qk_norm['suffix']}", (self.head_size if shared else kv_out,), "vector", "around_one")]
        if self.head_scale:
            d.append(ParamDecl(f"{prefix}{self.head_scale}", (self.num_heads,), "vector", "around_one"))
        if self.distance_bias:
            d.append(ParamDecl(f"{prefix}{self.distance_bias['name']}", (self.distance_bias.get("rows"), self.num_heads),
                               "vector"))
        if self.out_gate:
            d.append(ParamDecl(f"{prefix}{self.out_gate}{ws}",
                               (self.num_heads * (1 if self.out_gate_per_head else self.value_size), self.width)))
        if self.value_mix and not self.value_mix["first"]:
            d.append(ParamDecl(f"{prefix}{self.value_mix['name']}", (), "vector", "around_half"))
        if self.rotation is not None:
            d += self.rotation.param_decls(prefix + "rotation")
        return d

    def load(self, tensors: Dict, prefix: str, ops, dtype) -> None:
        super().load(tensors, prefix, ops, dtype)
        qn, kn, vn, on = self.names
        ws, bs = self.weight_suffix, self.bias_suffix
        ins = ([qn] + ([kn] + ([] if self.values_from_keys else [vn]) if self.own_kv else [])
               + ([self.out_gate] if self.out_gate else []))
        # One fused projection: a plain concatenation of the rows (the reference's
        # fused form interleaves per tensor-parallel shard, utils.py:189-242).
        self.w_qkv = ops.prepare_weight(torch.cat([tensors[f"{prefix}{n}{ws}"] for n in ins], dim=0).contiguous())
        self.b_qkv = (torch.cat([tensors[f"{prefix}{n}{bs}"] for n in ins], dim=0).contiguous()
                      if self.has_bias else None)
        w_out = tensors[f"{prefix}{on}{ws}"]
        if self.cache_head != self.value_size:
            # the attention's result has heads of the cache's size: the columns that meet the filling are zeros
            wide = w_out.new_zeros(self.width, self.num_heads, self.cache_head)
            wide[:, :, :self.value_size] = w_out.view(self.width, self.num_heads, self.value_size)
            w_out = wide.view(self.width, self.num_heads * self.cache_head).contiguous()
        if self.defer_out:
            self.w_out_raw, self.w_out = w_out, None
        else:
            self.w_out = ops.prepare_weight(w_out)
        self.b_out = tensors[f"{prefix}{on}{bs}"] if self.has_out_bias else None
        self.bias_by_distance = None
        if self.distance_bias:
            self.bias_by_distance = bias_by_distance(tensors[f"{prefix}{self.distance_bias['name']}"],
                                                     int(self.distance_bias["max_distance"]))
        self.turn = None
        self.q_norm = self.k_norm = self.mix_weight = self.freqs = None
        if self.rotation is not None:
            self.rotation.load(tensors, prefix + "rotation", ops, dtype)
            if self.prepared:
                self.freqs = self.rotation.frequencies()
            else:
                self.turn = self.rotation.pair_tables(self.head_size)     # the pairwise form: applied by the projection
        if self.qk_norm and self.qk_norm.get("weighted", True):
            self.q_norm = tensors[f"{prefix}{qn}{self.qk_norm['suffix']}"]
            self.k_norm = tensors[f"{prefix}{kn}{self.qk_norm['suffix']}"]
            if self.qk_norm.get("shared"):      # one head's weights, the same for every head: spread once
                self.q_norm = self.q_norm.repeat(self.num_heads).contiguous()
                self.k_norm = self.k_norm.repeat(self.num_kv_heads).contiguous()
        self.head_scales = tensors[f"{prefix}{self.head_scale}"] if self.head_scale else None
        if self.value_mix and not self.value_mix["first"]:
            self.mix_weight = tensors[f"{prefix}{self.value_mix['name']}"].reshape(1)

    def first_weight(self):
        return None if self.prepared else self.w_qkv

    def step_planners(self):
        from ..kernels.attention_plan import attention_plan
        return {"attention": attention_plan}

    def launch_shape(self, step):
        shape = getattr(self.ops, "attention_launch_shape", None)
        return shape(step, self.num_heads, self.window, self.cache_head, self.num_kv_heads) if shape is not None else None

    def flops_per_token(self, keys: float = 0.0) -> float:
        seen = min(keys, self.window) if self.window else keys
        if self.chunk:
            seen = min(keys, (self.chunk + 1) / 2.0)      # a query sees half a chunk on average
        # q k^T and p v
        return super().flops_per_token(keys) + 2.0 * self.num_heads * (self.head_size + self.value_size) * seen

    # ---- beside another mixer (`side_by_side`): the heads' results go into a slice of a buffer that the two
    # share, and the mixer that runs them owns the one output product

    def inner_width(self) -> int:
        return self.num_heads * self.cache_head

    def out_matrix(self):
        w, self.w_out_raw = self.w_out_raw, None
        return w

    def inner_into(self, h, ctx, cache, out, scale: float) -> None:
        if not self.prepared or self.has_out_bias:
            raise ValueError("an attention mixer beside another takes the float32 route and has no output bias")
        self._inner_prepared(h, ctx, cache, ctx.groups[cache.group], out, scale)

    def _forward_prepared(self, h, ctx, cache, residual, view):
        """The float32 route: projection with its bias, one kernel that norms, turns, scales, blends and stores,
        attention over heads of the cache's size, the output projection."""
        ops = self.ops
        c = self._inner_prepared(h, ctx, cache, view, None, 1.0)
        return ops.linear(c, self.w_out, self.b_out, residual=residual, out_f32=True)

    def _inner_prepared(self, h, ctx, cache, view, out, out_scale):
        ops = self.ops
        proj = ops.linear(h, self.w_qkv, self.b_qkv, out_f32=True, f32_by_library=True)
        first = None
        if self.value_mix:
            key = ("value mix", self.value_mix["key"])
            if self.value_mix["first"]:
                # what the later layers blend with: this step's values as this layer made them
                at = (self.num_heads + self.num_kv_heads) * self.head_size
                ctx.memo[key] = proj[:, at:at + self.num_kv_heads * self.value_size]
            else:
                first = ctx.memo.get(key)
                if first is None:
                    raise ValueError("a layer blends its values with those of a layer that has not run in this pass")
        rot = self.rotation
        more = {"per_head": True} if (self.qk_norm or {}).get("per_head") else {}
        if self.values_from_keys:
            more["values_at"] = self.num_heads * self.head_size        # the keys' columns are read a second time
        if self.head_scales is not None:
            more["head_scale"] = self.head_scales
        q = ops.qkv_prepare(proj, self.num_heads, self.num_kv_heads, self.head_size, self.value_size, self.cache_head,
                            self.q_norm, self.k_norm, self.qk_norm["eps"] if self.qk_norm else 0.0, self.freqs,
                            bool(rot.interleaved) if rot is not None else False, self.scale, self.mix_weight, first,
                            ctx, view, cache.k_pages, cache.v_pages, **more)
        if not self.scored and out is None:
            return ops.attention(q, self.num_heads, self.num_kv_heads, self.cache_head, ctx, view, cache.k_pages,
                                 cache.v_pages, self.window)
        gate, more = None, {}
        if self.out_gate:
            at = self.num_heads * self.head_size + self.num_kv_heads * (
                self.head_size + (0 if self.values_from_keys else self.value_size))
            gate = proj[:, at:at + self.num_heads * (1 if self.out_gate_per_head else self.value_size)]
            if self.out_gate_per_head:
                more["gate_per_head"] = True
        return ops.attention_scored(q, self.num_heads, self.num_kv_heads, self.cache_head, ctx, view, cache.k_pages,
                                    cache.v_pages, window=self.window, chunk=self.chunk, softcap=self.softcap,
                                    distance_bias=self.bias_by_distance, gate=gate, value_size=self.value_size,
                                    out=out, out_scale=out_scale, **more)

    def forward(self, h, ctx, cache, residual):
        if cache.writes != self.own_kv:
            raise ValueError("an attention mixer with own_kv writes its cache; one without reads another's")
        view = ctx.groups[cache.group]
        if self.prepared:
            return self._forward_prepared(h, ctx, cache, residual, view)
        kv_write = self.num_kv_heads if self.own_kv else 0
        if self.rotation is not None and self.turn is None:
            # the projections with their bias, turned by the encoding, then scaled and stored
            qkv = self.ops.linear(h, self.w_qkv, self.b_qkv)
            qkv = self.rotation.on_query_key(qkv, ctx, self.num_heads, kv_write, self.head_size)
            q = self.ops.qkv_write(qkv, None, self.num_heads, kv_write, self.head_size, self.scale, ctx, view,
                                   cache.k_pages, cache.v_pages)
            c = self.ops.attention(q, self.num_heads, self.num_kv_heads, self.head_size, ctx, view,
                                   cache.k_pages, cache.v_pages, self.window)
            return self.ops.linear(c, self.w_out, self.b_out, residual=residual, out_f32=True)
        q = self.ops.qkv_project(h, self.w_qkv, self.b_qkv, self.num_heads,
                                 self.num_kv_heads if self.own_kv else 0, self.head_size, self.scale, ctx, view,
                                 cache.k_pages, cache.v_pages, **({"turn": self.turn} if self.turn is not None else {}))
        c = self.ops.attention(q, self.num_heads, self.num_kv_heads, self.head_size, ctx, view,
                               cache.k_pages, cache.v_pages, self.window)
        return self.ops.linear(c, self.w_out, self.b_out, residual=residual, out_f32=True)


@register_mixer("latent_attention")
class LatentAttention(Mixer):
    """Softmax attention whose keys and values are made from one small vector a token, and only that vector
    is cached.

    With H heads, per head n unrotated and r rotated query/key elements and v value elements, a key/value
    latent of R and a query latent of Q elements:
        c_q = rms_norm(W_dq h),  q = W_uq c_q  laid out head by head as [n | r]
        [c' | k_r'] = W_dkv h,   c = rms_norm(c'),  k_r = turn(k_r')      (R and r elements; k_r is shared by the heads)
        score(i, j, head) = scale * (q_n[i] . (W_uk c[j]) + turn(q_r[i]) . k_r[j]),   value = W_uv c[j]
    over the keys of the query's own request at positions j <= i (and i - j < window with a window), softmax
    in float32, then W_o on the heads side by side. `turn` is the `rotation` (a `rotary` position part).

    The cache holds c and k_r, in pages of their own shapes. The products with W_uk and W_uv are moved to the
    query's side, so that a cached token is read as it lies: q_lat = W_uk^T q_n (R elements a head),
    score = scale * (q_lat . c + q_r . k_r), and the weighted sum of the c[j] goes through W_uv afterwards.
    c is kept twice, the second time with a page's tokens side by side (`across`), as the other designs'
    values are: the weighted sum contracts over tokens, and the matrix unit wants them next to each other.
    That order is the one for decoding, where what is read counts. A step of prompts' runs alone may take the
    other (`ops.latent_expands`): the keys W_uk c and values W_uv c of what the runs can see are made once for
    the step, and a (query, key) pair costs 2 (n + r + v) multiply-adds a head instead of 2 (2R + r).

    `q_rank=None`: no query latent: q = W_q h, one matrix (the second of `names`; the first is not read).
    `sink`: the name of a tensor of one number a head; the softmax's denominator also holds exp(sink), once, a term
    that stands for no token. `out_gate`: the name of a matrix W_g `[heads, width]`; a head's result is multiplied
    by sigmoid(W_g h) of that head before W_o (its rows ride in the product with W_dkv). A rotation that pairs
    element i with i + dims / 2 is brought to neighbouring pairs by putting the rows of the matrices that make
    q_r and k_r in the order (0, dims/2, 1, dims/2 + 1, ...) once, at load: q_r and k_r meet in a dot product
    only, which does not see the order.

    `own_kv=False`: no W_dkv; the mixer reads the cache of another call of the run order, whose R, r and
    rotation are its own. `keep`: the tokens the cache keeps: a number, "all", or None for the mixer's own window;
    a cache that is read by mixers of different windows keeps the most any of them sees.
    """

    recordable = True

    def __init__(self, width: int, num_heads: int, head_size: int, rot_size: int, value_size: int, kv_rank: int,
                 q_rank: Optional[int], scale: float, eps: float, rotation, names, window: Optional[int] = None,
                 keep=None, own_kv: bool = True, norm_suffix: str = ".norm", weight_suffix: str = "",
                 sink: Optional[str] = None, out_gate: Optional[str] = None):
        """`names`: the checkpoint's names, relative to the mixer's prefix, of W_dq, W_uq, W_dkv, W_uk, W_uv and
        W_o; a latent's norm weight is its down-projection's name with `norm_suffix`."""
        self.width, self.num_heads, self.head_size, self.rot_size = width, num_heads, head_size, rot_size
        self.value_size, self.kv_rank, self.q_rank = value_size, kv_rank, q_rank
        self.scale, self.eps, self.window, self.own_kv = float(scale), float(eps), window, own_kv
        self.keep = keep if own_kv else None
        if keep is not None and keep != "all" and (not isinstance(keep, int) or keep < 1):
            raise ValueError(f"keep is a number of tokens, \"all\" or None, got {keep!r}")
        if own_kv and isinstance(keep, int) and (window is None or keep < window):
            raise ValueError(f"a cache that keeps {keep} tokens cannot serve a window of {window}")
        self.names = tuple(names)
        if len(self.names) != 6:
            raise ValueError("names: W_dq, W_uq, W_dkv, W_uk, W_uv, W_o, six names")
        self.norm_suffix, self.weight_suffix = norm_suffix, weight_suffix
        self.sink, self.out_gate = sink, out_gate
        if out_gate and not own_kv:
            raise ValueError("a latent-attention mixer with a gate on its heads makes its own latents")
        self.rotation = POSITIONS.build(rotation)
        if rot_size % 2 or self.rotation.dims > rot_size:
            raise ValueError(f"the rotated part has {rot_size} elements; the rotation turns {self.rotation.dims}")

    def cache_need(self) -> Optional[CacheNeed]:
        keep = None if self.keep == "all" else (self.keep if self.keep is not None else self.window)
        return CacheNeed("paged", window=keep,
                         page_tensors=(("latent", ("page", self.kv_rank)), ("rotated", ("page", self.rot_size)),
                                       ("across", (self.kv_rank, "page"))))

    def step_planners(self):
        from ..kernels.attention_plan import attention_plan
        return {"attention": attention_plan}

    def param_decls(self, prefix: str) -> List[ParamDecl]:
        dq, uq, dkv, uk, uv, o = (prefix + (n or "") for n in self.names)
        s, h = self.weight_suffix, self.num_heads
        if self.q_rank is None:
            d = [ParamDecl(uq + s, (h * (self.head_size + self.rot_size), self.width))]
        else:
            d = [ParamDecl(dq + s, (self.q_rank, self.width)),
                 ParamDecl(dq + self.norm_suffix, (self.q_rank,), "vector", "around_one"),
                 ParamDecl(uq + s, (h * (self.head_size + self.rot_size), self.q_rank))]
        if self.sink:
            d.append(ParamDecl(prefix + self.sink, (h,), "vector"))
        if self.out_gate:
            d.append(ParamDecl(prefix + self.out_gate + s, (h, self.width)))
        if self.own_kv:
            d += [ParamDecl(dkv + s, (self.kv_rank + self.rot_size, self.width)),
                  ParamDecl(dkv + self.norm_suffix, (self.kv_rank,), "vector", "around_one")]
        d += [ParamDecl(uk + s, (h * self.head_size, self.kv_rank)),
              ParamDecl(uv + s, (h * self.value_size, self.kv_rank)),
              ParamDecl(o + s, (self.width, h * self.value_size))]
        return d

    def load(self, tensors: Dict, prefix: str, ops, dtype) -> None:
        super().load(tensors, prefix, ops, dtype)
        dq, uq, dkv, uk, uv, o = (prefix + (n or "") for n in self.names)
        s, h = self.weight_suffix, self.num_heads
        self.rotation.load(tensors, prefix + "rotation", ops, dtype)
        self.freqs = self.rotation.frequencies()
        n, r, dims = self.head_size, self.rot_size, self.rotation.dims
        w_uq, w_dkv = tensors[uq + s], (tensors[dkv + s] if self.own_kv else None)
        if not self.rotation.interleaved:
            if not self.own_kv:
                raise ValueError("a rotation by halves is brought to neighbouring pairs in the matrices that make "
                                 "both q_r and k_r: the mixer must own the latter")
            # element i and element i + dims / 2 of the rotated part become neighbours
            order = torch.arange(r, device=w_uq.device)
            order[:dims] = torch.stack([torch.arange(dims // 2), torch.arange(dims // 2) + dims // 2], dim=1).reshape(-1) \
                .to(w_uq.device)
            rows = (torch.arange(h, device=w_uq.device)[:, None] * (n + r) + n + order[None, :]).reshape(-1)
            w_uq = w_uq.clone()
            w_uq.view(h, n + r, -1)[:, n:] = tensors[uq + s][rows].view(h, r, -1)
            w_dkv = torch.cat([w_dkv[:self.kv_rank], w_dkv[self.kv_rank + order]], dim=0)
        # one product for what is wanted in float32: the rows of W_dq, then those of W_dkv, then the gate's
        down = (([tensors[dq + s]] if self.q_rank is not None else []) + ([w_dkv] if self.own_kv else [])
                + ([tensors[prefix + self.out_gate + s]] if self.out_gate else []))
        self.w_down = ops.prepare_weight(torch.cat(down, dim=0).contiguous())
        self.q_norm = tensors[dq + self.norm_suffix] if self.q_rank is not None else None
        self.kv_norm = tensors[dkv + self.norm_suffix] if self.own_kv else None
        self.sinks = tensors[prefix + self.sink] if self.sink else None
        self.w_uq = ops.prepare_weight(w_uq.contiguous())
        # W_uk a head, transposed: [H, R, n], the matrix that takes a head's q_n to its q_lat
        self.w_uk_t = tensors[uk + s].view(h, self.head_size, self.kv_rank).transpose(1, 2).contiguous()
        self.w_uv = tensors[uv + s].view(h, self.value_size, self.kv_rank).contiguous()
        # the whole matrices, for steps whose keys and values are made explicitly
        self.w_uk_whole = ops.prepare_weight(tensors[uk + s])
        self.w_uv_whole = tensors[uv + s]
        self.w_o = ops.prepare_weight(tensors[o + s])

    def first_weight(self):
        return None          # the product's float32 result goes to two norms: the norm before it stays a kernel

    def flops_per_token(self, keys: float = 0.0) -> float:
        seen = min(keys, self.window) if self.window else keys
        return super().flops_per_token(keys) + 2.0 * self.num_heads * (2 * self.kv_rank + self.rot_size) * seen

    def forward(self, h, ctx, cache, residual):
        if cache.writes != self.own_kv:
            raise ValueError("a latent-attention mixer with own_kv writes its cache; one without reads another's")
        ops, view = self.ops, ctx.groups[cache.group]
        heads, n, r = self.num_heads, self.head_size, self.rot_size
        latent, rotated, across = cache.pages["latent"], cache.pages["rotated"], cache.pages["across"]
        if latent.shape[-1] != self.kv_rank or rotated.shape[-1] != r:
            raise ValueError(f"the cache holds latents of {latent.shape[-1]} + {rotated.shape[-1]} elements, "
                             f"this mixer reads {self.kv_rank} + {r}")
        down = ops.linear(h, self.w_down, None, out_f32=True, f32_by_library=True)
        q_rank = self.q_rank or 0
        c_q = ops.latent_norms(down, q_rank, self.kv_rank if self.own_kv else 0, r if self.own_kv else 0,
                               self.q_norm, self.kv_norm, self.eps, self.freqs, ctx, view, latent, rotated, across)
        q = ops.linear(c_q if self.q_rank is not None else h, self.w_uq, None)
        more = {}
        if self.sinks is not None:
            more["sink"] = self.sinks
        if self.out_gate:
            at = q_rank + self.kv_rank + r
            more["gate"] = down[:, at:at + heads]
        if ops.latent_expands(ctx, n, r, self.value_size, self.kv_rank):
            # a step of prompts' runs alone: keys and values made from the latents, attention on them
            values = ops.latent_attention_expanded(q, self.w_uk_whole, self.w_uv_whole, heads, n, r, self.value_size,
                                                   self.kv_rank, self.freqs, self.scale, ctx, view, latent, rotated,
                                                   self.window, **more)
            return ops.linear(values, self.w_o, None, residual=residual, out_f32=True, f32_by_library=residual is None)
        q_lat = ops.batched_linear(q.view(-1, heads, n + r)[:, :, :n], self.w_uk_t)
        o_lat = ops.latent_attention(q, q_lat, heads, n, r, self.kv_rank, self.freqs, self.scale, ctx, view,
                                     latent, rotated, across, self.window, **more)
        values = ops.batched_linear(o_lat, self.w_uv)
        return ops.linear(values.view(-1, heads * self.value_size), self.w_o, None, residual=residual, out_f32=True,
                          f32_by_library=residual is None)


@register_mixer("mlstm")
class MatrixMemory(Mixer):
    """A matrix memory a head that is carried from token to token (the mLSTM cell of xLSTM): no cache that grows,
    a state of fixed size a request.

    With H heads, n query/key and v value elements a head, for the token at step t:
        q = W_q h / sqrt(n),  k = W_k h,  val = W_v h
        i = cap tanh((W_i h + b_i) / cap),  f = logsigmoid(cap tanh((W_f h + b_f) / cap))        (a number a head each)
        m_t = max(f + m_(t-1), i)
        S_t = exp(f + m_(t-1) - m_t) S_(t-1) + exp(i - m_t) k val^T,   n_t likewise with k alone
        o = S_t^T q / (max(|n_t . q|, exp(-m_t)) + 1e-6)
    S, n and m start at zero. Each head's o is scaled to unit root mean square, the heads side by side are
    weighted by `norm`, multiplied by sigmoid(W_g h), and W_o follows. Gates, state and norms are float32.

    The state is kept in two places by the parity of the position: the token at position p reads place
    (p - 1) & 1 and writes place p & 1, so that a step of single tokens that is run again reads what it read the
    first time. Position 0 reads nothing.
    """

    recordable = True

    def __init__(self, width: int, num_heads: int, head_size: int, value_size: int, gate_cap: float, eps: float, names,
                 weight_suffix: str = "", bias_suffix: str = ".b"):
        """`names`: the checkpoint's names, relative to the mixer's prefix, of W_q, W_k, W_v, W_g, W_o, W_i, W_f
        (the two gates have a bias, their name with `bias_suffix`) and of the weight of the norm after the cell."""
        self.width, self.num_heads, self.head_size, self.value_size = width, num_heads, head_size, value_size
        self.gate_cap, self.eps = float(gate_cap), float(eps)
        self.names = tuple(names)
        if len(self.names) != 8:
            raise ValueError("names: W_q, W_k, W_v, W_g, W_o, W_i, W_f and the norm, eight names")
        self.weight_suffix, self.bias_suffix = weight_suffix, bias_suffix

    def cache_need(self) -> Optional[CacheNeed]:
        h, n, v = self.num_heads, self.head_size, self.value_size
        # (a column's rows side by side: what a lane of the kernel holds are neighbours in memory)
        return CacheNeed("state", state_shapes=(("memory", (2, h, v, n)), ("normalizer", (2, h, n)), ("peak", (2, h))))

    def _rows(self):
        h, n, v = self.num_heads, self.head_size, self.value_size
        q, k, val, g, o, i, f, norm = self.names
        return [(q, h * n), (k, h * n), (val, h * v), (g, h * v), (i, h), (f, h)]

    def param_decls(self, prefix: str) -> List[ParamDecl]:
        ws, bs = self.weight_suffix, self.bias_suffix
        q, k, val, g, o, i, f, norm = self.names
        d = [ParamDecl(f"{prefix}{name}{ws}", (rows, self.width)) for name, rows in self._rows()]
        d += [ParamDecl(f"{prefix}{i}{bs}", (self.num_heads,), "vector"),
              ParamDecl(f"{prefix}{f}{bs}", (self.num_heads,), "vector"),
              ParamDecl(f"{prefix}{o}{ws}", (self.width, self.num_heads * self.value_size)),
              ParamDecl(f"{prefix}{norm}", (self.num_heads * self.value_size,), "vector", "around_one")]
        return d

    def load(self, tensors: Dict, prefix: str, ops, dtype) -> None:
        super().load(tensors, prefix, ops, dtype)
        ws, bs = self.weight_suffix, self.bias_suffix
        q, k, val, g, o, i, f, norm = self.names
        # one product for everything the cell reads: the rows of W_q, W_k, W_v, W_g, W_i, W_f
        self.w_in = ops.prepare_weight(torch.cat([tensors[f"{prefix}{name}{ws}"] for name, _ in self._rows()], dim=0)
                                       .contiguous())
        gates = torch.cat([tensors[f"{prefix}{i}{bs}"], tensors[f"{prefix}{f}{bs}"]])
        bias = gates.new_zeros(self.w_in.shape[0])
        bias[-2 * self.num_heads:] = gates
        self.b_in = bias.contiguous()
        self.w_out = ops.prepare_weight(tensors[f"{prefix}{o}{ws}"])
        self.norm_weight = tensors[f"{prefix}{norm}"]

    def flops_per_token(self, keys: float = 0.0) -> float:
        # the memory's update and its product with the query, a head
        return super().flops_per_token(keys) + 4.0 * self.num_heads * self.head_size * self.value_size

    def forward(self, h, ctx, cache, residual):
        ops = self.ops
        proj = ops.linear(h, self.w_in, self.b_in, out_f32=True, f32_by_library=True)
        st = cache.state
        y = ops.matrix_memory(proj, self.num_heads, self.head_size, self.value_size, self.gate_cap, self.eps,
                              self.norm_weight, ctx, st["memory"], st["normalizer"], st["peak"])
        return ops.linear(y, self.w_out, None, residual=residual, out_f32=True)
