"""What a caller hands in and gets back.  Names follow the reference's
src/minigpt_infer/engine/request.py:20-75; text fields are left out because the engine's
contract is token ids in, token ids out."""

from __future__ import annotations

from dataclasses import dataclass, field
from typing import List, Optional

from ..config.engine_config import SamplingParams


@dataclass
class Request:
    request_id: str
    prompt_token_ids: List[int]
    sampling_params: SamplingParams = field(default_factory=SamplingParams)
    eot_token_id: Optional[int] = None


@dataclass
class RequestOutput:
    request_id: str
    new_token_ids: List[int]
    finished: bool
    finish_reason: Optional[str] = None   # "eot", "length", "cancelled"
