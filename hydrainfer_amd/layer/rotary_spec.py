"""What config.json says about a rotation: how many channels of a head turn, the base of the frequencies and, optionally,
YaRN scaling.  No table: kernels take the angle of every pair per position and form cos and sin from the position."""
import math
from dataclasses import dataclass
from typing import List, Optional, Tuple


@dataclass
class RotarySpec:
    dims: int
    base: float
    factor: Optional[float] = None      # YaRN: None = plain frequencies
    original: float = 0.0
    fast: float = 32.0
    slow: float = 1.0

    def frequencies(self) -> Tuple[List[float], float]:
        """(angle per position of every pair [dims / 2], factor on cos and sin).  With YaRN the pairs that turn fast keep
        their frequency, the slow ones are divided by `factor`, with a linear ramp between."""
        f = [self.base ** (-2.0 * i / self.dims) for i in range(self.dims // 2)]
        if not self.factor:
            return f, 1.0
        turn = lambda t: self.dims * math.log(self.original / (2.0 * math.pi * t)) / (2.0 * math.log(self.base))
        lo = max(math.floor(turn(self.fast)), 0)
        hi = min(math.ceil(turn(self.slow)), self.dims - 1)
        ramp = [min(max((i - lo) / max(hi - lo, 0.001), 0.0), 1.0) for i in range(self.dims // 2)]
        return [fi / self.factor * r + fi * (1.0 - r) for fi, r in zip(f, ramp)], 0.1 * math.log(self.factor) + 1.0

    @classmethod
    def from_config(cls, rot: Optional[dict]) -> Optional["RotarySpec"]:
        """rot: {"dims", "base", "scaling": {"factor", "original", "fast", "slow"} or absent}; None stays None."""
        if not rot:
            return None
        sc = rot.get("scaling") or {}
        return cls(int(rot["dims"]), float(rot["base"]), float(sc["factor"]) if sc.get("factor") else None,
                   float(sc.get("original", 0.0)), float(sc.get("fast", 32.0)), float(sc.get("slow", 1.0)))

    def to_config(self) -> dict:
        out = {"base": self.base, "dims": self.dims}
        if self.factor:
            out["scaling"] = {"factor": self.factor, "original": self.original, "fast": self.fast, "slow": self.slow}
        return out
