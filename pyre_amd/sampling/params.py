"""How a request's next tokens are chosen and when it stops."""

from __future__ import annotations

from dataclasses import dataclass


@dataclass(frozen=True)
class SamplingParams:
    """``temperature`` 0 is the reference's argmax (`pyre/scheduler.py:80,94`); above 0
    the token is drawn from softmax(logits / temperature). A request ends after
    ``max_new_tokens`` tokens or with ``eos_id`` (which is kept in the output,
    `pyre/scheduler.py:82-83,96-97`) unless ``ignore_eos``."""

    max_new_tokens: int = 16
    temperature: float = 0.0
    eos_id: int | None = None
    ignore_eos: bool = False
    seed: int = 0

    def __post_init__(self) -> None:
        if self.max_new_tokens < 1:
            raise ValueError("max_new_tokens must be at least 1")
        if self.temperature < 0:
            raise ValueError("temperature must not be negative")
