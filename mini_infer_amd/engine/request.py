"""Request types, with the reference's names (scheduler/request_state.py:30-116)."""

from __future__ import annotations

import dataclasses
import enum
import threading
from typing import Literal, Sequence

from mini_infer_amd.sampling.params import SamplingParams

FinishReason = Literal["stop", "length", "cancelled"]


@dataclasses.dataclass(frozen=True)
class Request:
    """`prompt` is text (needs the model folder's tokenizer) or a list of token ids."""

    prompt: str | Sequence[int]
    sampling_params: SamplingParams = SamplingParams()
    max_tokens: int = 16


@dataclasses.dataclass(frozen=True)
class GenerationResult:
    text: str
    tokens: list[int]
    finish_reason: FinishReason
    prompt_tokens: int


@dataclasses.dataclass(frozen=True)
class GenerationStep:
    """One streamed step; `finish_reason` is set on the last one only."""

    text: str
    finish_reason: FinishReason | None = None
    num_tokens: int = 0
    tokens: tuple[int, ...] = ()


class RequestState(str, enum.Enum):
    WAITING = "waiting"
    PREFILLING = "prefilling"
    CHUNKED_PREFILLING = "chunked_prefilling"
    DECODING = "decoding"
    DONE = "done"


@dataclasses.dataclass
class RunningRequest:
    """Scheduler-side state of one request."""

    request_id: int
    request: Request
    prompt_token_ids: list[int]
    seed: int
    state: RequestState = RequestState.WAITING
    # tokens fed so far count against `feed`: the prompt, then generated tokens
    # (after a preemption the generated tokens are fed again as part of the prompt)
    tokens_fed: int = 0
    tokens_generated: list[int] = dataclasses.field(default_factory=list)
    finish_reason: FinishReason | None = None
    cancel_requested: bool = False
    admitted_order: int = -1
    preemptions: int = 0
    # index of the request's next draw, as read from its state slot when it was preempted
    # (while it runs, the slot itself holds the counter)
    draws: int = 0
    steps: list[GenerationStep] = dataclasses.field(default_factory=list)
    done_event: threading.Event = dataclasses.field(default_factory=threading.Event)
    # asynchronous sampling: the request's newest token has been sampled but not read by the
    # host yet; it is this row of the scheduler's pending sample
    pending_row: int | None = None

    @property
    def feed(self) -> list[int]:
        """Everything that must be in the cache before the next token can be sampled."""
        return self.prompt_token_ids + self.tokens_generated

    @property
    def prefill_remaining(self) -> int:
        return len(self.prompt_token_ids) + len(self.tokens_generated) - self.tokens_fed
