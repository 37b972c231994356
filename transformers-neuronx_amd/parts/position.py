"""Position encodings."""
from typing import Dict, List

from .base import PositionEncoding, register_position
from .spec import ParamDecl


@register_position("learned")
class LearnedPositions(PositionEncoding):
    """A table with one row per position, added to the embedded tokens; row
    `position + offset` is read (reference: opt/model.py:232-244, where the
    offset is 2, and decoder.py:562-572)."""

    recordable = True

    def __init__(self, width: int, max_positions: int, offset: int = 0):
        self.width, self.max_positions, self.offset = width, max_positions, offset
        self.table = None

    def param_decls(self, prefix: str) -> List[ParamDecl]:
        return [ParamDecl(prefix + ".weight", (self.max_positions + self.offset, self.width), "table")]

    def load(self, tensors: Dict, prefix: str, ops, dtype) -> None:
        super().load(tensors, prefix, ops, dtype)
        self.table = tensors[prefix + ".weight"]

    def at_input(self, x, positions, want_compute: bool, scale: float = 1.0):
        """x `[T, width]` (any float dtype) -> (float32 sum, compute-dtype copy or None); `scale` multiplies the
        token's row before the position's joins it."""
        return self.ops.add_positions(x, positions, self.table, self.offset, self.dtype, want_compute, scale=scale)


@register_position("none")
class NoPositions(PositionEncoding):
    """No encoding at the input: the embedded tokens pass as they are."""

    recordable = True

    def __init__(self, **_):
        pass

    def at_input(self, x, positions, want_compute: bool, scale: float = 1.0):
        return self.ops.to_stream(x, self.dtype, want_compute, scale=scale)


@register_position("sinusoidal")
class SinusoidalPositions(PositionEncoding):
    """Fixed sines and cosines added to the embedded tokens: element 2i of the token at position p gets
    sin(p * base^(-2i / width)), element 2i + 1 the cosine of the same angle. No table: the kernel that starts the
    stream makes the angles, in float32, so there is no longest request."""

    recordable = True

    def __init__(self, width: int, base: float = 10000.0):
        if width % 2:
            raise ValueError(f"sines and cosines come in pairs: the width must be even, got {width}")
        self.width, self.base = width, float(base)

    def load(self, tensors: Dict, prefix: str, ops, dtype) -> None:
        super().load(tensors, prefix, ops, dtype)
        import torch
        # base^(-2i / width), made in float64 and rounded once
        i = torch.arange(self.width // 2, dtype=torch.float64)
        self.freqs = (self.base ** (-2.0 * i / self.width)).to(torch.float32).to(getattr(ops, "device", "cpu"))

    def at_input(self, x, positions, want_compute: bool, scale: float = 1.0):
        return self.ops.add_sinusoid(x, positions, self.freqs, self.dtype, want_compute, scale=scale)


@register_position("rotary")
class RotaryPositions(PositionEncoding):
    """Turns pairs of query and key elements by an angle that grows with the position: of the first `dims`
    elements of a head, element 2i is paired with 2i + 1 (`interleaved`) or element i with i + dims / 2, and the
    pair (u, v) at position p becomes (u cos a - v sin a, v cos a + u sin a), a = p * base^(-2i / dims). The
    elements beyond `dims` pass. Positions, frequencies and angles are float32.

    `scaling` = {factor, low, high, original} stretches the slow turns for requests longer than `original`
    tokens: a frequency f with wavelength l = 2 pi / f is kept where l < original / high, becomes f / factor
    where l > original / low, and between the two (1 - s) f / factor + s f with
    s = (original / l - low) / (high - low). `scaling` = {factor} alone divides every frequency by the factor
    (positions stretched linearly).

    Two ways to use it: `pair_tables` (the attention mixer's pairwise form, for `max_positions` positions,
    interleaved pairs only), or `frequencies()`, for a mixer whose kernels make the angles themselves."""

    recordable = True

    def __init__(self, base: float, dims: int, max_positions: int = 0, interleaved: bool = True, scaling=None):
        if dims % 2 or dims < 0:
            raise ValueError(f"rotary positions turn pairs: dims must be even, got {dims}")
        self.base, self.dims, self.max_positions, self.interleaved = float(base), dims, max_positions, interleaved
        self.scaling = dict(scaling) if scaling else None
        self.linear_scaling = bool(self.scaling) and set(self.scaling) == {"factor"}
        if self.linear_scaling:
            if not float(self.scaling["factor"]) > 0:
                raise ValueError(f"scaling of rotary frequencies: a positive factor, got {self.scaling!r}")
        elif self.scaling:
            missing = [k for k in ("factor", "low", "high", "original") if k not in self.scaling]
            if missing or self.scaling["high"] == self.scaling["low"]:
                raise ValueError(f"scaling of rotary frequencies: factor, low, high (other than low) and original; "
                                 f"got {self.scaling!r}")
        self.device = "cpu"

    def load(self, tensors: Dict, prefix: str, ops, dtype) -> None:
        super().load(tensors, prefix, ops, dtype)
        self.device = getattr(ops, "device", "cpu")
        self._freqs = None

    def frequencies(self):
        """float32 `[dims / 2]` on the device: base^(-2i / dims), made in float64 and rounded once."""
        if getattr(self, "_freqs", None) is None:
            import torch
            i = torch.arange(self.dims // 2, dtype=torch.float64)
            f = self.base ** (-2.0 * i / max(self.dims, 1))
            if self.linear_scaling:
                f = f / float(self.scaling["factor"])
            elif self.scaling:
                import math
                c = self.scaling
                turns = float(c["original"]) * f / (2.0 * math.pi)        # original / wavelength
                s = (turns - c["low"]) / (c["high"] - c["low"])
                blend = (1.0 - s) * f / c["factor"] + s * f
                f = torch.where(turns > c["high"], f, torch.where(turns < c["low"], f / c["factor"], blend))
            self._freqs = f.to(torch.float32).to(self.device)
        return self._freqs

    def pair_tables(self, head_size: int):
        import torch
        if not self.interleaved or self.max_positions <= 0 or self.dims > head_size:
            return None
        angle = torch.arange(self.max_positions, dtype=torch.float32)[:, None] * self.frequencies().cpu()[None, :]
        cos, sin = torch.cos(angle), torch.sin(angle)
        a = torch.ones(self.max_positions, head_size, dtype=torch.float32)
        b = torch.zeros(self.max_positions, head_size, dtype=torch.float32)
        a[:, :self.dims] = torch.stack([cos, cos], dim=-1).reshape(self.max_positions, self.dims)
        b[:, :self.dims] = torch.stack([-sin, sin], dim=-1).reshape(self.max_positions, self.dims)
        return a.contiguous().to(self.device), b.contiguous().to(self.device)
