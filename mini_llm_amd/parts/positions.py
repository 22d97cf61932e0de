"""Position encodings. GPT-2 has learned absolute positions: a table row per position, added to
the token row at the embedding (engine/src/embedding.c:9-16)."""

from __future__ import annotations

from ..weights.spec import TABLE, Normal, TensorSpec
from .base import PositionEncoding, register_part


class LearnedPositions(PositionEncoding):
    """``tensor_name``: the table's name behind the part's prefix ("" where the part's own name is the tensor's)."""

    stage = "embedding"

    def __init__(self, n_positions: int, width: int, tensor_name: str = "weight", std: float = 0.02):
        self.n_positions, self.width = n_positions, width
        self._tensor_name, self._std = tensor_name, std
        self.weight = None

    def tensor_specs(self):
        return {self._tensor_name: TensorSpec((self.n_positions, self.width), TABLE, Normal(self._std))}

    def bind(self, tensors):
        self.weight = tensors[self._tensor_name]

    def max_positions(self) -> int:
        return self.n_positions


class RotaryEncoding(PositionEncoding):
    """Rotation of the first ``dims`` elements of a head by an angle that grows with the position: pair i turns by p * f_i with
    f_i = base^(-2i / dims). ``pairing`` says which elements make pair i: "half" pairs element i with element i + dims / 2,
    "neighbours" pairs element 2i with element 2i + 1, (u, v) -> (u cos a - v sin a, v cos a + u sin a). It has no tensors; the
    mixer that holds it applies it to its queries and keys (``stage`` "mixer") with ``frequencies`` and ``magnitude``.

    ``scaling`` stretches the slow pairs for sequences longer than ``original`` positions, in one of two ways (``kind``):

    "yarn" (the default), {factor, original, fast, slow} (YaRN: Peng, Quesnelle, Fan, Shippole, "YaRN: Efficient Context Window
    Extension of Large Language Models"): with pair(t) = dims * ln(original / (2 pi t)) / (2 ln base), the pair that turns t
    times within the original length, lo = max(floor(pair(fast)), 0), hi = min(ceil(pair(slow)), dims - 1) and ramp_i =
    clamp((i - lo) / max(hi - lo, 0.001), 0, 1), the frequency becomes f_i / factor * ramp_i + f_i * (1 - ramp_i), and cos and
    sin are multiplied by 0.1 ln(factor) + 1.

    "wavelength", {factor, low, high, original}: by a pair's wavelength l = 2 pi / f. A pair with l < original / high keeps f; one
    with l > original / low gets f / factor; between the two, with s = (original / l - low) / (high - low), the frequency is
    (1 - s) f / factor + s f. cos and sin keep their size."""

    stage = "mixer"

    def __init__(self, dims: int, base: float, scaling: dict | None = None, pairing: str = "half"):
        import math

        if dims < 0 or dims % 2:
            raise ValueError(f"a rotation pairs elements: {dims} is not an even number of them")
        if not base > 0:
            raise ValueError(f"the base must be positive, not {base}")
        if pairing not in ("half", "neighbours"):
            raise ValueError(f"unknown pairing {pairing!r}: half or neighbours")
        self.dims, self.base, self.scaling, self.pairing = dims, float(base), dict(scaling) if scaling else None, pairing
        values = [self.base ** (-2.0 * i / dims) for i in range(dims // 2)]
        self.magnitude = 1.0
        kind = (self.scaling or {}).get("kind", "yarn")
        if self.scaling and kind == "yarn":
            factor, original = float(self.scaling["factor"]), float(self.scaling["original"])
            pair = lambda turns: dims * math.log(original / (2.0 * math.pi * turns)) / (2.0 * math.log(self.base))
            lo = max(math.floor(pair(float(self.scaling["fast"]))), 0)
            hi = min(math.ceil(pair(float(self.scaling["slow"]))), dims - 1)
            for i, f in enumerate(values):
                ramp = min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0)
                values[i] = f / factor * ramp + f * (1.0 - ramp)
            self.magnitude = 0.1 * math.log(factor) + 1.0
        elif self.scaling and kind == "wavelength":
            factor, original = float(self.scaling["factor"]), float(self.scaling["original"])
            low, high = float(self.scaling["low"]), float(self.scaling["high"])
            for i, f in enumerate(values):
                wavelength = 2.0 * math.pi / f
                if wavelength < original / high:
                    continue
                if low > 0 and wavelength > original / low:   # (with low = 0 no wavelength is past original / low)
                    values[i] = f / factor
                else:
                    s = (original / wavelength - low) / (high - low)
                    values[i] = (1.0 - s) * f / factor + s * f
        elif self.scaling:
            raise ValueError(f"unknown kind of scaling {kind!r}: yarn or wavelength")
        self.values = values   # float64 on the host; ``frequencies`` rounds them to 32-bit on the device, ``frequencies64`` does not
        self._on_device = {}

    def frequencies(self, device):
        import torch

        key = str(device)
        if key not in self._on_device:
            self._on_device[key] = torch.tensor(self.values or [0.0], dtype=torch.float64).to(torch.float32).to(device)
        return self._on_device[key]

    def frequencies64(self, device):
        """The same numbers unrounded, for a kernel that takes its angles in 64-bit."""
        import torch

        key = (str(device), 64)
        if key not in self._on_device:
            self._on_device[key] = torch.tensor(self.values or [0.0], dtype=torch.float64).to(device)
        return self._on_device[key]


register_part("position_encoding", "learned", LearnedPositions)
register_part("position_encoding", "rotary", RotaryEncoding)
