"""Result record of one request (reference: src/tokamak/engine/outputs.py:12-38)."""

from __future__ import annotations

from dataclasses import dataclass

from tokamak_amd.engine.request import FinishReason


@dataclass(frozen=True)
class RequestOutput:
    request_id: int
    prompt: str | None
    prompt_token_ids: list[int]
    output_text: str | None
    output_token_ids: list[int]
    finish_reason: FinishReason
    ttft_s: float | None = None
    latency_s: float | None = None
