"""What one step is asked to run."""

from __future__ import annotations

import dataclasses
from typing import Hashable, Sequence


@dataclasses.dataclass
class StepEntry:
    """A request's next tokens, and the places among them whose logits are wanted.

    A portion of a prompt (any length, cut anywhere) or a single decoded token.
    `want` indexes into `tokens`; it is empty for a portion in the middle of a prompt.
    `device_row`, if given, says that the entry's ONE token is not known to the host yet: it
    is row `device_row` of the `device_tokens` tensor handed to `step` (ids a previous step
    sampled and left on the device); `tokens` then holds one placeholder.
    """

    request_id: Hashable
    tokens: Sequence[int]
    want: Sequence[int] = ()
    device_row: int | None = None
