"""RotaryEmbedding (reference: src/positional.rs:8-31)."""
from __future__ import annotations

import enum


class RotaryEmbedding(enum.IntEnum):
    ROPE = 0
    ALIBI = 1  # the reference's default (src/positional.rs:12-13)
    POPE = 2

    def as_str(self) -> str:
        return self.name.lower()

    @classmethod
    def default(cls) -> "RotaryEmbedding":
        return cls.ALIBI

    @classmethod
    def parse(cls, value) -> "RotaryEmbedding":
        if isinstance(value, cls):
            return value
        if isinstance(value, str):
            return cls[value.upper()]
        return cls(int(value))
