"""One generation request as the scheduler sees it: the prompt, the tokens generated so far, the
row it occupies in the KV caches and a completion signal for the thread that submitted it.
Same attributes and methods as the reference's request object
(src/chunk_attn/models/sequence.py:6-36), plus a timeout on get_result."""
from __future__ import annotations

import threading
import uuid
from dataclasses import dataclass, field
from typing import List, Optional


@dataclass(eq=False)
class Sequence:
    prompt_tokens: List[int]
    max_tokens: int = 2048
    # filled in by the scheduler
    index: Optional[int] = None            # row in the KV caches once the prompt is prefilled
    error: Optional[BaseException] = None  # what ended the request early, if anything did
    id: str = field(default_factory=lambda: str(uuid.uuid4()))
    tokens: List[int] = field(init=False)  # prompt followed by everything generated
    result_ready: threading.Event = field(default_factory=threading.Event, repr=False)

    def __post_init__(self) -> None:
        self.tokens = list(self.prompt_tokens)

    # ---- scheduler side --------------------------------------------------------------------
    def append(self, token: int) -> None:
        self.tokens.append(token)

    def set_result_ready(self) -> None:
        self.result_ready.set()

    def set_error(self, error: BaseException) -> None:
        self.error = error
        self.result_ready.set()

    # ---- submitter side --------------------------------------------------------------------
    def get_result(self, timeout: Optional[float] = None) -> List[int]:
        """Blocks until the request is finished (or `timeout` seconds have passed) and returns all
        its tokens; re-raises what the scheduler recorded with set_error."""
        finished = self.result_ready.wait(timeout)
        if not finished:
            raise TimeoutError(f"sequence {self.id} is not finished")
        if self.error is not None:
            raise self.error
        return self.tokens

    def __len__(self) -> int:
        return len(self.tokens)

    def __getitem__(self, position):
        return self.tokens[position]
