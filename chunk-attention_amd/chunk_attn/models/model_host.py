"""Iteration-level scheduler over the prefix-tree KV caches (reference:
src/chunk_attn/models/model_host.py:13-134).

Every iteration: drop finished sequences from the caches, admit queued requests (prefill),
run one decode step for everything running.  `running_seqs` is kept in cache order: prefill
reports the index the prefix tree inserted a sequence at (next to the sequences it shares a
prefix with), finished sequences are removed by index.  Admission is prefix-aware: requests
admitted together are prefilled in prompt order, so arrivals with a common prefix enter the
tree back to back and every shared chunk keeps covering one contiguous range of sequences.
A model error fails the sequences it hit instead of killing the worker thread.
"""
from __future__ import annotations

import queue
import threading
from types import TracebackType
from typing import List, Optional, Type

import torch

from .sequence import Sequence


class ModelHost:
    def __init__(self, model_obj, kv_caches, max_batch_size: int = 32, prefix_aware: bool = True):
        self.model_obj = model_obj          # callable(seqs, kv_caches, prefill) -> next token per sequence
        self.kv_caches = kv_caches
        self.running_seqs: List[Sequence] = []
        self.max_batch_size = max_batch_size
        self.prefix_aware = prefix_aware
        self.peak_batch_size = 0
        self.iterations = 0
        self.stopped = True
        self.cycle_time = 1.0               # seconds an idle worker waits for a request per round
        # room for a whole batch beyond the one being admitted: producers rarely wait on put()
        self.batch_queue: "queue.Queue[Sequence]" = queue.Queue(maxsize=2 * max_batch_size)
        self.thread: Optional[threading.Thread] = None

    def predict_async(self, prompt_tokens: List[int], max_tokens: int) -> Sequence:
        """Queues a request; the returned Sequence delivers tokens (or the error) when done."""
        request = Sequence(prompt_tokens=prompt_tokens, max_tokens=max_tokens)
        if self.stopped:
            raise RuntimeError("model host is stopped: start() it before asking for predictions")
        self.batch_queue.put(request)
        return request

    def predict(self, prompt_tokens: List[int], max_tokens: int) -> List[int]:
        return self.predict_async(prompt_tokens, max_tokens).get_result()

    def start(self) -> None:
        if self.thread is not None or not self.stopped:
            raise RuntimeError("model host is already started")
        worker = threading.Thread(target=self.run_iterations, name="chunk-attn-model-host", daemon=True)
        self.stopped = False
        self.thread = worker
        worker.start()

    def stop(self) -> None:
        self.stopped = True
        if self.thread is not None:
            self.thread.join()
            self.thread = None

    def get_new_requests(self) -> List[Sequence]:
        """Requests to admit this iteration: as many as fit beside the running sequences.  An idle
        host waits up to cycle_time for the first one instead of spinning."""
        room = self.max_batch_size - len(self.running_seqs)
        admitted: List[Sequence] = []
        wait = self.cycle_time if not self.running_seqs else None
        while len(admitted) < room:
            try:
                if wait is not None and not admitted:
                    admitted.append(self.batch_queue.get(timeout=wait))
                else:
                    admitted.append(self.batch_queue.get_nowait())
            except queue.Empty:
                break
        if self.prefix_aware:
            admitted.sort(key=lambda s: s.prompt_tokens)   # stable: equal prompts keep arrival order
        return admitted

    def _remove_finished(self) -> None:
        finished = [i for i, seq in enumerate(self.running_seqs)
                    if len(seq) >= seq.max_tokens + len(seq.prompt_tokens)]
        for n_removed, i in enumerate(finished):
            i -= n_removed
            seq = self.running_seqs.pop(i)
            for kv_cache in self.kv_caches:
                kv_cache.remove_seq(i)
            seq.set_result_ready()

    def _fail(self, seqs: List[Sequence], error: Exception) -> None:
        for seq in seqs:
            seq.set_error(error)

    @torch.inference_mode()
    def run_iterations(self) -> None:
        while not self.stopped:
            self._remove_finished()
            sequences = self.get_new_requests()
            # prefill one request at a time: prompts differ in length, and each insertion index
            # refers to the caches as they are after the previous insertion
            for seq in sequences:
                try:
                    seq.append(self.model_obj([seq], self.kv_caches, prefill=True)[0])
                except Exception as e:  # noqa: BLE001  (reported through the sequence)
                    self._fail([seq], e)
                    continue
                self.running_seqs.insert(seq.index, seq)
            self.peak_batch_size = max(self.peak_batch_size, len(self.running_seqs))
            if self.running_seqs:
                try:
                    new_tokens = self.model_obj(self.running_seqs, self.kv_caches, prefill=False)
                except Exception as e:  # noqa: BLE001
                    self._fail(self.running_seqs, e)
                    self.running_seqs = []
                    for kv_cache in self.kv_caches:
                        kv_cache.clear()
                    continue
                for seq, tok in zip(self.running_seqs, new_tokens):
                    seq.append(tok)
                self.iterations += 1
        # leaving: nothing is left waiting forever
        self._fail([s for s in self.running_seqs if not s.result_ready.is_set()],
                   RuntimeError("model host stopped before the sequence finished"))

    def __enter__(self) -> "ModelHost":
        self.start()
        return self

    def __exit__(self, exc_type: Optional[Type[BaseException]], exc_val: Optional[BaseException],
                 exc_tb: Optional[TracebackType]) -> bool:
        self.stop()
        return False   # an exception raised inside the with-block goes on to the caller
