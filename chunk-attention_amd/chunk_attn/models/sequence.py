"""One generation request (reference: src/chunk_attn/models/sequence.py:6-36)."""
from __future__ import annotations

import uuid
from threading import Event
from typing import Any, List, Optional


class Sequence:
    def __init__(self, prompt_tokens: List[int], max_tokens: int = 2048) -> None:
        self.id = str(uuid.uuid4())
        self.prompt_tokens = prompt_tokens
        self.max_tokens = max_tokens
        self.tokens = list(prompt_tokens)
        self.index: Optional[int] = None    # position in the KV caches, set by prefill
        self.error: Optional[Exception] = None
        self.result_ready = Event()

    def get_result(self, timeout: Optional[float] = None) -> Any:
        if not self.result_ready.wait(timeout):
            raise TimeoutError(f"sequence {self.id} is not finished")
        if self.error is not None:
            raise self.error
        return self.tokens

    def set_result_ready(self) -> None:
        self.result_ready.set()

    def set_error(self, error: Exception) -> None:
        self.error = error
        self.result_ready.set()

    def append(self, token: int) -> None:
        self.tokens.append(token)

    def __len__(self) -> int:
        return len(self.tokens)

    def __getitem__(self, index):
        return self.tokens[index]
