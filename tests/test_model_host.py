"""Host logic of the iteration-level scheduler (chunk_attn/models/model_host.py, mirror of the
reference's src/chunk_attn/models/model_host.py) with a fake model: the oracle prefix tree
stands in for the KV caches, so the test sees whether `running_seqs` stays in cache order
through admissions and removals."""
import threading
import time

import pytest

from chunk_attn.models import ModelHost, Sequence
from oracle.prefix_tree import PrefixTree


class FakeCache:
    """What the scheduler calls on a cache, recorded on the oracle tree."""

    def __init__(self, chunk_size=4):
        self.tree = PrefixTree(chunk_size, 100000)
        self.removed = 0

    def remove_seq(self, idx):
        self.tree.remove_seq(idx)
        self.removed += 1

    def clear(self):
        self.tree = PrefixTree(self.tree.chunk_size, 100000)

    def all_tokens(self):
        return [self.tree.seq_tokens(i) for i in range(self.tree.n_seqs)]


class FakeModel:
    """Next token = a function of the whole history; checks the batch against the cache."""

    def __init__(self, fail_on=None):
        self.decode_batches = []
        self.fail_on = fail_on

    @staticmethod
    def next_token(tokens):
        return (sum(tokens) * 31 + len(tokens)) % 997

    def __call__(self, seqs, kv_caches, prefill):
        cache = kv_caches[0]
        if prefill:
            assert len(seqs) == 1
            if self.fail_on is not None and self.fail_on in seqs[0].tokens:
                raise ValueError("bad prompt")
            idx, _ = cache.tree.add_seq(list(seqs[0].tokens))
            seqs[0].index = idx
            return [self.next_token(seqs[0].tokens)]
        # decode: batch row i must be cache sequence i, holding everything but the newest token
        assert [s.tokens[:-1] for s in seqs] == cache.all_tokens()
        cache.tree.append_token([s[-1] for s in seqs])
        self.decode_batches.append(len(seqs))
        return [self.next_token(s.tokens) for s in seqs]


def expected(prompt, n):
    toks = list(prompt)
    for _ in range(n):
        toks.append(FakeModel.next_token(toks))
    return toks


def test_results_order_and_batch_limit():
    model, cache = FakeModel(), FakeCache()
    shared = list(range(10))
    prompts = [shared + [100 + i] * (1 + i % 3) for i in range(9)] + [[500 + i, 7] for i in range(3)]
    budgets = [3 + (5 * i) % 11 for i in range(len(prompts))]
    with ModelHost(model, [cache], max_batch_size=4) as host:
        seqs = [host.predict_async(p, n) for p, n in zip(prompts, budgets)]
        results = [s.get_result(timeout=30) for s in seqs]
    for p, n, r in zip(prompts, budgets, results):
        assert r == expected(p, n)
    assert host.peak_batch_size <= 4 and max(model.decode_batches) <= 4
    assert cache.removed == len(prompts) and cache.all_tokens() == []


def test_prefix_aware_admission_sorts_arrivals():
    host = ModelHost(FakeModel(), [FakeCache()], max_batch_size=8)
    host.stopped = False
    for p in ([5, 1], [1, 2, 3], [5, 0], [1, 2]):
        host.batch_queue.put(Sequence(p, 1))
    assert [s.prompt_tokens for s in host.get_new_requests()] == [[1, 2], [1, 2, 3], [5, 0], [5, 1]]


def test_errors_reach_the_caller_and_the_host_survives():
    model, cache = FakeModel(fail_on=666), FakeCache()
    with ModelHost(model, [cache], max_batch_size=4) as host:
        bad = host.predict_async([1, 666, 2], 4)
        good = host.predict_async([1, 2, 3], 4)
        with pytest.raises(ValueError, match="bad prompt"):
            bad.get_result(timeout=30)
        assert good.get_result(timeout=30) == expected([1, 2, 3], 4)
    with pytest.raises(RuntimeError, match="stopped"):
        host.predict_async([1], 1)
    with pytest.raises(RuntimeError, match="already started"):
        host.start()
        try:
            host.start()
        finally:
            host.stop()


def test_stop_fails_unfinished_sequences():
    model, cache = FakeModel(), FakeCache()
    host = ModelHost(model, [cache], max_batch_size=2)
    host.start()
    seq = host.predict_async([1, 2, 3], 10_000_000)
    time.sleep(0.2)
    host.stop()
    with pytest.raises(RuntimeError, match="stopped before"):
        seq.get_result(timeout=5)
