#!/usr/bin/env python3
"""Decode-attention benchmark on one MI355X.

One "step" = one forward of the prefix-tree decode attention (chunk-first launches +
sequence-first launch + merge) over a synthetic batch whose K/V already sit in the HBM pool
and whose device tables are valid -- the protocol of the reference's own microbenchmark
(tests/benchmark_chunk_attn.py:60-97 there: warm-up, then timed forwards between device syncs).

Prints one JSON line: metric = decode-attention us/step (lower is better) with the achieved
HBM rate of the dominant kernel against the 8 TB/s roofline and the CPU baseline next to it.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.join(ROOT, "chunk-attention_amd"))
sys.path.insert(0, ROOT)

HBM_PEAK_GBPS = 8000.0


def build_cache(w, torch, capi, seed=0, tpp_threshold=1):
    import numpy as np
    dev = torch.device("cuda:0")
    need = sum(w.seq_len(s) // w.chunk_size + 2 for s in range(w.n_seqs)) + 2048 // w.chunk_size + 10   # + room for side_costs
    per_chunk = w.chunk_size * w.n_heads * w.d_head * 2 * 2
    memory_mb = -(-need * per_chunk // (1 << 20))
    attn = capi.Attention(n_heads=w.n_heads, d_head=w.d_head, chunk_size=w.chunk_size, memory_mb=memory_mb,
                          share_prefix=True, tpp_threshold=tpp_threshold, dtype=torch.float16, device=dev)
    for s in range(w.n_seqs):
        k, v = w.kv(s, seed)
        idx = attn.add_seq(w.tokens(s), torch.from_numpy(np.ascontiguousarray(k)).to(dev),
                           torch.from_numpy(np.ascontiguousarray(v)).to(dev))
        assert idx == s
    return attn


def time_forward(attn, q, out, steps, warmup, torch, partition=0):
    stream = torch.cuda.current_stream().cuda_stream
    n = q.shape[0]
    attn.refresh_kernel_context()
    for _ in range(warmup):
        attn.ctx.attention(q.data_ptr(), out.data_ptr(), n, partition, stream)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        attn.ctx.attention(q.data_ptr(), out.data_ptr(), n, partition, stream)
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e3 / steps


def phase_times(attn, q, out, steps, torch, mode, partition=0):
    """HIP-event times per forward, recorded inside the library on the launch stream.
    mode 1: the fused launch; mode 2: three separate launches (chunk-first, sequence-first, merge)."""
    stream = torch.cuda.current_stream().cuda_stream
    attn.ctx.set_timing(mode)
    attn.ctx.read_timing(reset=True)
    for _ in range(steps):
        attn.ctx.attention(q.data_ptr(), out.data_ptr(), q.shape[0], partition, stream)
    t = attn.ctx.read_timing(reset=True)
    attn.ctx.set_timing(0)
    n = max(t["calls"], 1)
    return {k: t[k] / n for k in ("shared_ms", "stream_ms", "merge_ms")}


def measured_traffic(workload, info):
    """HBM bytes per decode launch from the committed rocprofv3 --pmc summary, when it was taken
    for this workload with this work list; None otherwise (counters cannot be read from here)."""
    path = os.path.join(ROOT, "profiles", "hbm_traffic.json")
    try:
        with open(path) as f:
            table = json.load(f)
    except (OSError, ValueError):
        return None, "no counter summary"
    e = table.get(workload)
    if not e or e.get("shared_items") != info.n_shared_items or e.get("stream_items") != info.n_stream_items:
        return None, "no counter summary for this workload / work list"
    return int(e["decode_kernel_bytes"]), e.get("how", "")


def cold_forward_us(attn, q, out, torch, reps=20, hints=(("default_policy", 0), ("non_temporal_forced", 1))):
    """The forward when nothing it attends is still cached: a read of 1 GiB of other memory (four
    times the last-level cache; a read, so that no dirty lines are left to write back) runs in
    front of every timed forward, HIP events on the launch stream around the forward alone.  What
    a model with many layers sees; the benchmark protocol repeats one forward.  Also returned: the
    decode launch alone under the same protocol (events recorded inside the library around that
    launch, default policy)."""
    stream = torch.cuda.current_stream().cuda_stream
    flush = torch.zeros(1 << 27, dtype=torch.int64, device="cuda:0")
    res = {}
    for name, hint in hints:
        attn.ctx.set_stream_hint(hint)
        attn.refresh_kernel_context()
        total = 0.0
        for i in range(reps + 2):
            flush.sum()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            attn.ctx.attention(q.data_ptr(), out.data_ptr(), q.shape[0], 0, stream)
            e1.record()
            e1.synchronize()
            if i >= 2:
                total += e0.elapsed_time(e1)
        res[name + "_us"] = round(total * 1e3 / reps, 2)
    attn.ctx.set_stream_hint(0)
    attn.refresh_kernel_context()
    attn.ctx.set_timing(1)
    for i in range(reps + 2):
        if i == 2:
            attn.ctx.read_timing(reset=True)
        flush.sum()
        attn.ctx.attention(q.data_ptr(), out.data_ptr(), q.shape[0], 0, stream)
    t = attn.ctx.read_timing(reset=True)
    attn.ctx.set_timing(0)
    res["decode_launch_us"] = round(t["shared_ms"] * 1e3 / max(t["calls"], 1), 2)
    del flush
    return res


def plain_read_gbps(ctx, n_bytes, torch, reps=20, wgs_per_cu=2):
    """What a read with no structure reaches on this GPU: the library's read probe (wgs_per_cu
    workgroups per compute unit, non-temporal 16-byte loads, nothing kept) over a buffer of
    n_bytes under the decode launch's two protocols (warm: a back-to-back train between two HIP
    events; cold: after a read of 1 GiB of other memory, events around the single launch), and
    over 2 GiB, where no cache helps and the launch's start and end no longer weigh.  A yardstick
    beside the published peak, not a replacement for it."""
    stream = torch.cuda.current_stream().cuda_stream
    flush = torch.zeros(1 << 27, dtype=torch.int64, device="cuda:0")
    res = {}
    for name, size, cold in (("warm", n_bytes, False), ("cold", n_bytes, True), ("2GiB", 2 << 30, False)):
        buf = torch.ones(max(size // 8, 2), dtype=torch.int64, device="cuda:0")
        nb = buf.numel() * 8
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        if cold:
            total = 0.0
            for i in range(reps + 2):
                flush.sum()
                e0.record()
                ctx.bench_read_probe(buf.data_ptr(), nb, wgs_per_cu, stream)
                e1.record()
                e1.synchronize()
                if i >= 2:
                    total += e0.elapsed_time(e1)
            ms = total / reps
        else:
            n = reps if size <= (1 << 30) else 5
            for _ in range(2):
                ctx.bench_read_probe(buf.data_ptr(), nb, wgs_per_cu, stream)
            e0.record()
            for _ in range(n):
                ctx.bench_read_probe(buf.data_ptr(), nb, wgs_per_cu, stream)
            e1.record()
            e1.synchronize()
            ms = e0.elapsed_time(e1) / n
        res[name] = round(nb / (ms * 1e-3) / 1e9, 1)
        del buf
    del flush
    res["wgs_per_cu"] = wgs_per_cu
    return res


def pybind_forward_us(w, q, steps, warmup, torch, seed):
    """The drop-in class as a caller of the reference would use it: chunk_attn.Attention.forward
    (output allocation, validity check and both launches), same protocol as time_forward.  Returns
    (us per forward, us per forward of the C-ABI call on the same cache with a preallocated output)."""
    import numpy as np
    import chunk_attn
    attn = pybind_cache(w, torch, seed, extra_chunks_per_seq=10)
    for _ in range(warmup):
        out = attn.forward(q)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(steps):
        out = attn.forward(q)
    torch.cuda.synchronize()
    us = (time.perf_counter() - t0) * 1e6 / steps
    # table refresh through the class, host time per call (the upload is asynchronous):
    # "tree changed" = forced rebuild (tree walk, plan, upload); "tails rolled" = what a decode
    # step pays when last chunks fill up: reserve() + the in-place patch of the tables
    # (three in a row at a time: the uploads come from a ring of four staging buffers, and a
    # longer train would time the wait for the device to release one)
    rebuild_us = 0.0
    for _ in range(5):
        torch.cuda.synchronize()
        attn.forward(q)
        t0 = time.perf_counter()
        for _ in range(3):
            attn.refresh_kernel_context(True)
        rebuild_us += (time.perf_counter() - t0) * 1e6 / 15
    torch.cuda.synchronize()
    kz = torch.zeros((w.n_seqs, w.n_heads, w.d_head), dtype=torch.float16, device="cuda:0")
    reserve_t, roll_t, n_rolled, rolls = [], [], 0, 0
    c = w.chunk_size
    for t in range(8 * c):
        attn.append_token([1_900_000_000 - t * 4096 - s for s in range(w.n_seqs)], kz, kz)
        if any(x.n_tokens == c for x in attn.tails):     # full last chunks: the next reserve rolls them
            # (no device sync in front: the first launch after one costs the host 10 us more)
            t0 = time.perf_counter()
            fresh = attn.reserve()                       # tree work + one Python object per new chunk
            t1 = time.perf_counter()
            attn.refresh_kernel_context()                # the tables: patched in place, upload queued
            t2 = time.perf_counter()
            if rolls or t >= c:                          # the first patch is not timed
                reserve_t.append((t1 - t0) * 1e6)
                roll_t.append((t2 - t1) * 1e6)
                n_rolled += len(fresh)
            rolls += 1
    torch.cuda.synchronize()
    # one beam-search step with four candidates through the class (three copies of the last chunk
    # and four K/V rows in one launch): from an idle device to completion, and eight in a row
    k4 = torch.zeros((4, w.n_heads, w.d_head), dtype=torch.float16, device="cuda:0")
    for rep in range(2):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        attn.append_completion(0, [-5 - 4 * rep, -6 - 4 * rep, -7 - 4 * rep, -8 - 4 * rep], k4, k4)
        torch.cuda.synchronize()
        beam_synced = (time.perf_counter() - t0) * 1e6
        for i in (3, 2, 1):
            attn.remove_seq(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for rep in range(8):
        attn.append_completion(0, [-100 - 4 * rep, -101 - 4 * rep, -102 - 4 * rep, -103 - 4 * rep], k4, k4)
    beam_host = (time.perf_counter() - t0) * 1e6 / 8
    torch.cuda.synchronize()
    beam_free = (time.perf_counter() - t0) * 1e6 / 8
    for i in range(24, 0, -1):
        attn.remove_seq(i)
    beam = {"synced_us": round(beam_synced, 1), "free_running_us": round(beam_free, 1), "host_us": round(beam_host, 1),
            "note": "append_completion with four candidates through chunk_attn.Attention (pybind11): one step from an "
                    "idle device to its completion; eight steps in a row and one sync; host time per step of those"}
    timed = max(rolls - 1, 1)
    tables = {"tree_changed_us": round(rebuild_us, 1), "tails_rolled_us": round(float(np.median(roll_t)), 1),
              "tails_rolled_max_us": round(max(roll_t), 1),
              "reserve_call_us": round(float(np.median(reserve_t)), 1),
              "tails_rolled_per_patch": n_rolled // timed, "patches_timed": rolls - 1,
              "note": "host time per call through chunk_attn.Attention; tree_changed = refresh_kernel_context(True): tree "
                      "walk + tables + upload; tails_rolled = refresh_kernel_context() after reserve() gave full last "
                      "chunks a successor: tables patched in place + upload (reserve_call_us is that reserve(), which "
                      "also builds one Python object per new chunk); medians over the patches timed, max = the "
                      "patch that outgrew a device buffer, if one did (buffers double)"}
    return us, out, tables, beam


def pybind_cache(w, torch, seed, extra_chunks_per_seq=1):
    """The workload in a cache of the pybind11 class."""
    import numpy as np
    import chunk_attn
    need = sum(w.seq_len(s) // w.chunk_size + 1 + extra_chunks_per_seq for s in range(w.n_seqs)) + 8
    per_chunk = w.chunk_size * w.n_heads * w.d_head * 2 * 2
    attn = chunk_attn.Attention(n_heads=w.n_heads, d_head=w.d_head, chunk_size=w.chunk_size,
                                memory_mb=-(-need * per_chunk // (1 << 20)), dtype=torch.float16,
                                device=torch.device("cuda:0"))
    for s in range(w.n_seqs):
        k, v = w.kv(s, seed)
        attn.add_seq(w.tokens(s), torch.from_numpy(np.ascontiguousarray(k)).to("cuda:0"),
                     torch.from_numpy(np.ascontiguousarray(v)).to("cuda:0"))
    return attn


def decode_launch_us(attn, q, out, steps, torch, what=0):
    """Average duration of the decode launch (what 0), or of its sequence-first workgroups alone
    (what 1): a back-to-back train of that launch between two HIP events on the launch stream
    (events around every single launch add 2-3 us each).  `out` is left incomplete."""
    stream = torch.cuda.current_stream().cuda_stream
    for _ in range(5):
        attn.ctx.bench_decode_launch(q.data_ptr(), out.data_ptr(), q.shape[0], what, stream)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(steps):
        attn.ctx.bench_decode_launch(q.data_ptr(), out.data_ptr(), q.shape[0], what, stream)
    e1.record()
    e1.synchronize()
    return e0.elapsed_time(e1) * 1e3 / steps


def side_costs(attn, w, torch, capi, operators=False):
    """Per-decode-step costs outside the timed forward: a forced table rebuild (tree walk, plan,
    upload) and the append kernel, as wall-clock microseconds between device syncs."""
    import numpy as np
    stream = torch.cuda.current_stream().cuda_stream
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    reps = 20
    for _ in range(reps):
        attn.refresh_kernel_context(force=True)
    torch.cuda.synchronize()
    refresh_us = (time.perf_counter() - t0) * 1e6 / reps
    k = torch.zeros((w.n_seqs, w.n_heads, w.d_head), dtype=torch.float16, device="cuda:0")
    attn.refresh_kernel_context()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(reps):   # rewrites the same free row of every tail: the cache is not advanced
        attn.ctx.append_kv(k.data_ptr(), k.data_ptr(), w.n_seqs, stream)
    torch.cuda.synchronize()
    append_us = (time.perf_counter() - t0) * 1e6 / reps
    # the decode step's rotary embedding: as its own launch before the append (the reference's
    # sequence), and folded into the append launch
    qr = torch.zeros_like(k)
    cache = torch.zeros((8192, w.d_head), dtype=torch.float16, device="cuda:0")
    pos = torch.zeros(w.n_seqs, dtype=torch.int64, device="cuda:0")
    q2, k2 = qr.view(w.n_seqs, -1), k.view(w.n_seqs, -1)
    capi.rotary_embedding(pos, q2, k2, w.d_head, cache, True)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(reps):
        capi.rotary_embedding(pos, q2, k2, w.d_head, cache, True)
        attn.ctx.append_kv(k.data_ptr(), k.data_ptr(), w.n_seqs, stream)
    torch.cuda.synchronize()
    two_us = (time.perf_counter() - t0) * 1e6 / reps
    t0 = time.perf_counter()
    for _ in range(reps):
        attn.ctx.rope_append_kv(0, qr.data_ptr(), k.data_ptr(), k.data_ptr(), cache.data_ptr(), 8192, w.d_head,
                                True, w.n_seqs, stream)
    torch.cuda.synchronize()
    fused_us = (time.perf_counter() - t0) * 1e6 / reps
    # prefill copy-in: a 2048-token sequence that shares nothing (every K/V row is scattered into
    # fresh chunks), inserted and removed again; wall clock with a device sync per insertion
    T = 2048
    pk = torch.zeros((T, w.n_heads, w.d_head), dtype=torch.float16, device="cuda:0")
    toks = [-(10 ** 9) - i for i in range(T)]
    idx = attn.add_seq(toks, pk, pk)
    attn.remove_seq(idx)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(5):
        idx = attn.add_seq(toks, pk, pk)
        torch.cuda.synchronize()
        attn.remove_seq(idx)
    add_us = (time.perf_counter() - t0) * 1e6 / 5
    # the copy-in launch by itself: the same rows scattered again into the chunks of one such
    # sequence (a launch train between events; nothing else owns those chunks)
    idx = attn.add_seq(toks, pk, pk)
    own = [int(r[0]) for r in attn.get_chunks() if r[2] == idx and r[3] == idx + 1 and r[1] > 0]
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    attn.ctx.scatter_kv(pk.data_ptr(), pk.data_ptr(), T, 0, own, stream)
    e0.record()
    for _ in range(reps):
        attn.ctx.scatter_kv(pk.data_ptr(), pk.data_ptr(), T, 0, own, stream)
    e1.record()
    torch.cuda.synchronize()
    scatter_us = e0.elapsed_time(e1) * 1e3 / reps
    # one beam-search step on that sequence: four candidates = three tail-chunk copies and four
    # K/V rows (wall clock with a device sync; the three new sequences are removed again)
    k4 = torch.zeros((4, w.n_heads, w.d_head), dtype=torch.float16, device="cuda:0")
    for rep in range(2):            # the first step is a warm-up: timed is the second
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        attn.append_completion(idx, [-5 - 4 * rep, -6 - 4 * rep, -7 - 4 * rep, -8 - 4 * rep], k4, k4)
        torch.cuda.synchronize()
        beam_us = (time.perf_counter() - t0) * 1e6
        for i in (3, 2, 1):
            attn.remove_seq(idx + i)
    # the same step eight times in a row without waiting for the device in between (candidate 0
    # keeps extending the sequence; the 24 sequences it spawns are removed afterwards)
    n_free = 8
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for rep in range(n_free):
        attn.append_completion(idx, [-100 - 4 * rep, -101 - 4 * rep, -102 - 4 * rep, -103 - 4 * rep], k4, k4)
    host_us = (time.perf_counter() - t0) * 1e6 / n_free
    torch.cuda.synchronize()
    beam_free_us = (time.perf_counter() - t0) * 1e6 / n_free
    for i in range(3 * n_free, 0, -1):
        attn.remove_seq(idx + i)
    attn.remove_seq(idx)
    attn.refresh_kernel_context()
    torch.cuda.synchronize()
    copy_bytes = 2 * 2 * T * w.n_heads * w.d_head * 2   # K and V, read and written
    base = {"table_rebuild_us": round(refresh_us, 1), "append_kv_us": round(append_us, 1),
            "add_seq_2048_tokens_us": round(add_us, 1), "add_seq_copy_GBps": round(copy_bytes / add_us / 1e3, 1),
            "beam_step_4_candidates_us": round(beam_us, 1), "beam_step_free_running_us": round(beam_free_us, 1), "beam_step_host_us": round(host_us, 1),
            "scatter_kernel_2048_tokens_us": round(scatter_us, 1), "scatter_kernel_GBps": round(copy_bytes / scatter_us / 1e3, 1),
            "rotary_then_append_us": round(two_us, 1), "rotary_append_fused_us": round(fused_us, 1),
            "chunk_rows": int(attn.ctx.plan_info().n_chunks),
            "beam_note": "beam_step_4_candidates_us: one step from an idle device to its completion, wall clock "
                         "with a device sync (launch + sync of an idle device alone is about 15 us); "
                         "beam_step_free_running_us: eight steps in a row and one sync; beam_step_host_us: host time per step of those"}
    if not operators:
        return base
    # the layer's norm operators on a prefill batch of 16384 rows of H*d (128 MiB per tensor, so
    # that a launch outlasts the host's ~10 us per call; launch trains timed with events on the
    # current stream): rms_norm reads and writes the rows once, the fused form reads and writes
    # both the activation and the residual
    hidden = w.n_heads * w.d_head
    TN = 16384
    x = torch.randn((TN, hidden), device="cuda:0").half()
    res, y = torch.randn_like(x), torch.empty_like(x)
    wt = torch.ones(hidden, dtype=torch.float16, device="cuda:0")
    norm = {}
    for name, fn, passes in (("rms_norm", lambda: capi.rms_norm(y, x, wt, 1e-6), 2),
                             ("fused_add_rms_norm", lambda: capi.fused_add_rms_norm(x, res, wt, 1e-6), 4)):
        fn()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(reps):
            fn()
        e1.record()
        torch.cuda.synchronize()
        us = e0.elapsed_time(e1) * 1e3 / reps
        norm[name + "_%dx%d_us" % (TN, hidden)] = round(us, 1)
        norm[name + "_GBps"] = round(passes * TN * hidden * 2 / us / 1e3, 1)
    # the rotary operator on the same batch: q and k rows of H*d, read and written once
    kq = torch.randn((TN, hidden), device="cuda:0").half()
    posn = torch.arange(TN, device="cuda:0", dtype=torch.int64) % 8192
    capi.rotary_embedding(posn, x, kq, w.d_head, cache, True)
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(reps):
        capi.rotary_embedding(posn, x, kq, w.d_head, cache, True)
    e1.record()
    torch.cuda.synchronize()
    us = e0.elapsed_time(e1) * 1e3 / reps
    norm["rotary_embedding_%dx%d_us" % (TN, hidden)] = round(us, 1)
    norm["rotary_embedding_GBps"] = round(4 * TN * hidden * 2 / us / 1e3, 1)
    return {**norm, **base}


def decode_loop(w, torch, capi, synth, seed, unique_tokens, fused=False):
    """The configuration's decode loop on a fresh cache of the pybind11 class: per step one
    append_token (K/V rows of every sequence into the last chunks; when those are full: reserve,
    new chunks, tables patched in place) and one forward, host work included -- or, fused, one
    decode_step, whose attention launch writes the new rows itself.  us_per_step: the loop
    free-running; per-step figures: a second pass with a device sync after every step."""
    lw = synth.two_level_workload(w.name + "-loop", 8, 8, w.chunk_size, 1024, 512, unique_tokens,
                                  n_heads=w.n_heads, append_steps=w.append_steps)
    res = {}
    for timed_per_step in (False, True):
        attn = pybind_cache(lw, torch, seed, extra_chunks_per_seq=2)
        q = torch.from_numpy(lw.q(seed)).to("cuda:0")
        kv = [tuple(torch.from_numpy(a).to("cuda:0") for a in lw.append_kv(t, seed)) for t in range(lw.append_steps)]
        toks = [lw.append_tokens(t) for t in range(lw.append_steps)]
        attn.forward(q)
        torch.cuda.synchronize()
        new_chunks, per_step, t0 = [], [], time.perf_counter()
        for t in range(lw.append_steps):
            t1 = time.perf_counter()
            if fused:
                before = attn.peak_memory_allocated()
                attn.decode_step(toks[t], q, kv[t][0], kv[t][1])
                new_chunks.append(int(attn.peak_memory_allocated() > before))
            else:
                new_chunks.append(len(attn.append_token(toks[t], kv[t][0], kv[t][1])))
                attn.forward(q)
            if timed_per_step:
                torch.cuda.synchronize()
                per_step.append((time.perf_counter() - t1) * 1e6)
        torch.cuda.synchronize()
        if not timed_per_step:
            res["us_per_step"] = round((time.perf_counter() - t0) * 1e6 / lw.append_steps, 1)
        else:
            rolled = [i for i, n in enumerate(new_chunks) if n]
            plain = sorted(x for i, x in enumerate(per_step) if i not in rolled and i > 0)
            res["synced_step_median_us"] = round(plain[len(plain) // 2], 1)
            res["synced_steps_that_added_chunks_us"] = {str(i): round(per_step[i], 1) for i in rolled}
        del attn
    return {"steps": lw.append_steps, "unique_tokens_at_start": unique_tokens, "form": "decode_step" if fused else "append_token + forward",
            **res, "steps_that_added_chunks": int(sum(1 for x in new_chunks if x)),
            "note": "per step through chunk_attn.Attention (pybind11), host work included"}


def decode_step_us(w, q, torch, capi, seed, steps=48):
    """One decode step through the C-ABI on a fresh cache, free-running (no sync inside the loop):
    the two-call form (ca_append_kv, delta_tokens + 1, ca_attention) against the fused one
    (ca_decode_step), the two-call form with the rotary embedding of the step's rows folded into its
    append (ca_rope_append_kv + ca_attention), and the forward alone under the
    same protocol beside them (last chunks stay empty there: it attends fewer tokens than the
    others, whose last chunks fill up step by step).  Few enough steps that no last chunk fills
    (no table work in the loop)."""
    res = {}
    k = torch.zeros((w.n_seqs, w.n_heads, w.d_head), dtype=torch.float16, device="cuda:0")
    out = torch.empty_like(q)
    cache = torch.zeros((16384, w.d_head), dtype=torch.float16, device="cuda:0")
    stream = torch.cuda.current_stream().cuda_stream
    for form in ("forward_only", "two_call", "fused", "rotary_two_call"):
        attn = build_cache(w, torch, capi, seed)
        attn.refresh_kernel_context()
        ctx, n = attn.ctx, w.n_seqs
        # free rows in the fullest last chunk (the last row of get_chunks covering a sequence is its tail)
        fill = {}
        for slot, n_tok, b, e in attn.get_chunks().tolist():
            for s in range(b, e):
                fill[s] = n_tok
        room = w.chunk_size - max(fill.values())
        n_steps = max(2, min(steps, room - 1))
        qr = q.clone()   # the two-call rotary form rotates it in place

        def one():
            if form == "forward_only":
                ctx.attention(q.data_ptr(), out.data_ptr(), n, 0, stream)
            elif form == "fused":
                ctx.decode_step(q.data_ptr(), k.data_ptr(), k.data_ptr(), out.data_ptr(), n, stream)
            elif form == "two_call":
                ctx.append_kv(k.data_ptr(), k.data_ptr(), n, stream)
                ctx.delta_tokens = ctx.delta_tokens + 1
                ctx.attention(q.data_ptr(), out.data_ptr(), n, 0, stream)
            else:
                ctx.rope_append_kv(0, qr.data_ptr(), k.data_ptr(), k.data_ptr(), cache.data_ptr(), 16384, w.d_head,
                                   True, n, stream)
                ctx.delta_tokens = ctx.delta_tokens + 1
                ctx.attention(qr.data_ptr(), out.data_ptr(), n, 0, stream)
        one()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(n_steps - 1):
            one()
        torch.cuda.synchronize()
        res[form + "_us"] = round((time.perf_counter() - t0) * 1e6 / (n_steps - 1), 2)
        res["steps"] = n_steps - 1
        del attn
    res["note"] = ("append + forward per decode step through the C-ABI, free-running: ca_append_kv + ca_attention (three "
                   "launches) against ca_decode_step (two: the decode launch attends the new rows from the caller's "
                   "tensors, the merge launch writes them into the pool); rotary_two_call: ca_rope_append_kv + "
                   "ca_attention; forward_only attends the cache as built (empty last chunks)")
    return res


def decode_long(w, torch, capi, seed, steps=2048):
    """A long decode on the configuration: `steps` tokens appended to every sequence through
    Attention.decode_step (ctypes class), tables patched at every roll-over, with the re-planning
    policy off (patch only: work-item sizes stay those of the first step) and on (full rebuild
    whenever the attended tokens moved by more than 25 % since the last one).  Wall clock per step
    over the whole run and over its last quarter, host work included."""
    import numpy as np
    res = {}
    per_chunk = w.chunk_size * w.n_heads * w.d_head * 2 * 2
    need = sum((w.seq_len(s) + steps) // w.chunk_size + 3 for s in range(w.n_seqs)) + 64
    kz = torch.zeros((w.n_seqs, w.n_heads, w.d_head), dtype=torch.float16, device="cuda:0")
    q = torch.from_numpy(w.q(seed)).to("cuda:0")
    outs = {}
    for name, percent in (("patch_only", 0), ("replan_25", 25)):
        attn = capi.Attention(n_heads=w.n_heads, d_head=w.d_head, chunk_size=w.chunk_size,
                              memory_mb=-(-need * per_chunk // (1 << 20)), dtype=torch.float16, device=torch.device("cuda:0"))
        for s in range(w.n_seqs):
            k, v = w.kv(s, seed)
            attn.add_seq(w.tokens(s), torch.from_numpy(np.ascontiguousarray(k)).to("cuda:0"),
                         torch.from_numpy(np.ascontiguousarray(v)).to("cuda:0"))
        attn.ctx.set_replan(percent)
        attn.forward(q)
        torch.cuda.synchronize()
        marks = []
        t0 = time.perf_counter()
        for t in range(steps):
            out = attn.decode_step([1_500_000_000 - t * 4096 - s for s in range(w.n_seqs)], q, kz, kz)
            if (t + 1) % (steps // 4) == 0:
                torch.cuda.synchronize()
                marks.append(time.perf_counter())
        full, patches = attn.ctx.table_stats()
        info = attn.ctx.plan_info()
        res[name] = {"us_per_step": round((marks[-1] - t0) * 1e6 / steps, 2),
                     "last_quarter_us_per_step": round((marks[-1] - marks[-2]) * 1e6 / (steps // 4), 2),
                     "full_builds": full, "patches": patches,
                     "final_work_items": [info.n_shared_items, info.n_stream_items], "final_partial_rows": info.n_part_rows}
        outs[name] = out.float()
        del attn
    res["max_abs_diff_between_the_two"] = float((outs["patch_only"] - outs["replan_25"]).abs().max())
    res["steps"] = steps
    res["note"] = ("decode_step per step through the ctypes Attention class, zero K/V rows appended; the two runs attend "
                   "the same cache with differently cut work lists")
    return res


def cpu_baseline(attn, q_np, budget_s, torch):
    """The CPU restatement of the reference's MKL path on the same cache contents (fp16 values
    widened to fp32), timed on this machine's host cores."""
    import numpy as np
    from oracle.attention_ref import CpuAttention
    rows = attn.get_chunks()
    top = int(rows[:, 0].max()) + 1
    kp, vp = attn.pool_views()
    kpool = kp[:top].float().cpu().numpy()
    vpool = vp[:top].float().cpu().numpy()
    cpu = CpuAttention("auto")
    threads = min(cpu.max_threads, torch.get_num_threads())
    qf = q_np.astype(np.float32)
    res = {}
    for name, part in (("chunk_first", 0), ("seq_first", 2)):
        cpu.attention(qf, rows, kpool, vpool, part, threads)  # warm-up
        n, t0 = 0, time.perf_counter()
        while True:
            ref = cpu.attention(qf, rows, kpool, vpool, part, threads)
            n += 1
            el = time.perf_counter() - t0
            if el > budget_s / 2 or n >= 100:
                break
        res[name] = (el / n * 1e6, n)
    return res, threads, cpu.blas_source, ref


def main() -> int:
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--config", type=int, default=1, help="0-based index into the benchmark configurations (default: batch 32, 2048 shared + 512 unique, chunk 64)")
    ap.add_argument("--fraction", type=float, default=0.5, help="shared fraction for configuration 2")
    ap.add_argument("--heads", type=int, default=32, help="number of heads (the configurations have 32; others for measurements of what depends on it)")
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="CPU-baseline time budget, 0 to skip")
    ap.add_argument("--no-paged", action="store_true", help="skip the private-copies baseline")
    ap.add_argument("--operators", action="store_true",
                    help="also time the layer operators around the attention call (rms_norm, fused_add_rms_norm and "
                         "rotary_embedding on a prefill-sized batch): outside the metric, off by default")
    ap.add_argument("--no-pybind", action="store_true", help="skip timing the forward through the pybind11 class")
    ap.add_argument("--no-side-costs", action="store_true",
                    help="skip the per-step side costs and the decode-step legs (profiling runs that only want the forward)")
    ap.add_argument("--no-decode-long", action="store_true", help="skip the 2048-step decode with and without re-planning (default configuration only)")
    ap.add_argument("--markers", action="store_true",
                    help="named roctx ranges around refreshes, patches, attention calls and appends (for rocprofv3 --marker-trace)")
    ap.add_argument("--seg-chunks", type=int, default=0)
    ap.add_argument("--stream-chunks", type=int, default=0)
    ap.add_argument("--stream-hint", type=int, default=0, help="non-temporal loads of private chunks: 0 by working-set size (default), 1 always, 2 never")
    ap.add_argument("--schedule", type=int, default=0, help="0 producer launch + merge launch (default), 1 single launch with in-kernel merge")
    ap.add_argument("--seed", type=int, default=0)
    ap.add_argument("--calibrate-copy", type=int, default=0, metavar="MiB",
                    help="only run 20 plain device copies of this many MiB (a known-size reference for HBM traffic counters) and exit")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: the decode path has no multi-GPU component (run with --gpus 1)", file=sys.stderr)
        return 2

    import numpy as np
    import torch
    import synth
    from chunk_attn import capi
    if not torch.cuda.is_available():
        print("bench.py needs an MI355X: no HIP device visible and there is no CPU fallback", file=sys.stderr)
        return 3
    torch.cuda.set_device(0)

    if args.calibrate_copy > 0:
        n = args.calibrate_copy << 20
        src = torch.empty(n, dtype=torch.uint8, device="cuda:0").random_(0, 255)
        dst = torch.empty_like(src)
        torch.cuda.synchronize()
        for _ in range(20):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"calibrate_copy_MiB": args.calibrate_copy, "copies": 20, "bytes_read_per_copy": n, "bytes_written_per_copy": n}))
        return 0

    if args.markers:
        capi.set_markers(True)
    w = synth.baseline_config(args.config, args.fraction, args.heads)
    attn = build_cache(w, torch, capi, args.seed)
    if args.seg_chunks or args.stream_chunks:
        attn.ctx.set_plan(args.seg_chunks, args.stream_chunks)
    attn.ctx.set_schedule(args.schedule)
    attn.ctx.set_stream_hint(args.stream_hint)
    q_np = w.q(args.seed)
    q = torch.from_numpy(q_np).to("cuda:0")
    out = torch.empty_like(q)

    ms = time_forward(attn, q, out, args.steps, args.warmup, torch)
    scratch_out = torch.empty_like(q)   # the launch-only measurements leave their output incomplete
    decode_ms = decode_launch_us(attn, q, scratch_out, min(args.steps, 200), torch) * 1e-3
    merge_ms = max(ms - decode_ms, 0.0)  # the step is the two launches back to back
    ph = phase_times(attn, q, out, min(args.steps, 50), torch, 2)
    info = attn.ctx.plan_info()
    H, d = w.n_heads, w.d_head
    tok_bytes = 4 * H * d  # K and V rows of one token, all heads, fp16
    stream_bytes = tok_bytes * info.stream_tokens
    shared_bytes = tok_bytes * info.shared_tokens
    qo_bytes = 4 * w.n_seqs * H * d
    step_bytes = stream_bytes + shared_bytes + qo_bytes
    # dominant kernel = the decode launch: it reads every attended K/V row once, plus Q
    decode_bytes = stream_bytes + shared_bytes + qo_bytes // 2
    achieved = decode_bytes / (decode_ms * 1e-3) / 1e9 if decode_ms > 0 else 0.0
    traffic, traffic_note = measured_traffic(w.name, info)
    stream_us = decode_launch_us(attn, q, scratch_out, min(args.steps, 200), torch, what=1) if info.n_stream_items else 0.0
    train_gbps = stream_bytes / (stream_us * 1e-6) / 1e9 if stream_us > 0 else 0.0
    stream_gbps = stream_bytes / (ph["stream_ms"] * 1e-3) / 1e9 if ph["stream_ms"] > 0 else 0.0

    result = {
        "metric": "decode attention us/step",
        "value": round(ms * 1e3, 3),
        "unit": "us/step",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms, 6),
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f16",
        "data": "synthetic",
        "config": {"workload": w.name, "n_seqs": w.n_seqs, "n_heads": H, "d_head": d, "chunk_size": w.chunk_size,
                   "shared_tokens": int(info.shared_tokens), "stream_tokens": int(info.stream_tokens),
                   "shared_items": info.n_shared_items, "stream_items": info.n_stream_items,
                   "partial_rows": info.n_part_rows},
        "step_bytes": step_bytes,
        "step_GBps": round(step_bytes / (ms * 1e-3) / 1e9, 1),
        "step_frac_of_hbm_peak": round(step_bytes / (ms * 1e-3) / 1e9 / HBM_PEAK_GBPS, 4),
        "split_phases_us": {k.replace("_ms", ""): round(v * 1e3, 2) for k, v in ph.items()},
        "unique_kv_streaming": {"GBps": round(stream_gbps, 1), "frac_of_hbm_peak": round(stream_gbps / HBM_PEAK_GBPS, 4),
                                "bytes": stream_bytes, "launch_train_us": round(stream_us, 2),
                                "launch_train_GBps": round(train_gbps, 1),
                                "note": "sequence-first phase launched alone.  GBps: HIP events around every single launch "
                                        "(split_phases_us.stream; the events add 2-3 us).  launch_train: a back-to-back train "
                                        "of the launch between two events (consecutive launches overlap tail and ramp a "
                                        "little).  The launch's duration in the committed rocprofv3 kernel trace lies between."},
        "launches_us": {"decode_kernel": round(decode_ms * 1e3, 2), "merge_kernel": round(merge_ms * 1e3, 2)},
        "roofline": {"bound": "hbm", "kernel": "decode_kernel", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBPS,
                     "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBPS, 4), "traffic": traffic,
                     "traffic_note": traffic_note,
                     "bytes_per_launch": decode_bytes, "avg_launch_us": round(decode_ms * 1e3, 2)},
    }

    cold = None
    if args.stream_hint == 0:
        cold = cold_forward_us(attn, q, out, torch)
        result["cold_cache_forward"] = cold
        # FETCH_SIZE counts L2 misses, which the 256 MiB last-level cache may serve: when the
        # attended bytes fit it, repeated forwards are not an HBM measurement and the cold
        # figure is the HBM fraction to quote
        cold_gbps = decode_bytes / (cold["decode_launch_us"] * 1e-6) / 1e9
        result["roofline"]["achieved_cold"] = round(cold_gbps, 1)
        result["roofline"]["frac_cold"] = round(cold_gbps / HBM_PEAK_GBPS, 4)
        result["roofline"]["cold_launch_us"] = cold["decode_launch_us"]
        result["roofline"]["fits_last_level_cache"] = bool(stream_bytes + shared_bytes <= (256 << 20))
        result["roofline"]["cold_note"] = ("decode launch after 1 GiB of other memory was read, HIP events recorded inside "
                                           "the library around that launch (they add about 2 us: the fraction is a lower bound)")
        result["roofline"]["plain_read_GBps"] = plain_read_gbps(attn.ctx, decode_bytes, torch)
        result["roofline"]["plain_read_1_wg_per_cu_GBps"] = plain_read_gbps(attn.ctx, decode_bytes, torch, wgs_per_cu=1)
        result["roofline"]["plain_read_note"] = ("a kernel that only reads (non-temporal 16-byte loads, eight per lane in flight, "
                                                 "two workgroups of 256 threads per compute unit as the decode launch has, and "
                                                 "one) over bytes_per_launch bytes under the same two protocols (repeated; after "
                                                 "the 1 GiB read) and over 2 GiB, HIP events around the launch")
    if not args.no_pybind:
        pyb_us, pyb_out, pyb_tables, pyb_beam = pybind_forward_us(w, q, args.steps, args.warmup, torch, args.seed)
        torch.cuda.synchronize()
        result["table_refresh_pybind"] = pyb_tables
        result["beam_step_pybind"] = pyb_beam
        result["forward_pybind_us"] = round(pyb_us, 2)
        result["forward_pybind_minus_c_abi_us"] = round(pyb_us - ms * 1e3, 2)
        result["forward_pybind_max_abs_diff"] = float((pyb_out.float() - out.float()).abs().max())
        del pyb_out
    if not args.no_side_costs:
        result["per_step_side_costs"] = side_costs(attn, w, torch, capi, args.operators)
        result["decode_step"] = decode_step_us(w, q, torch, capi, args.seed)
    if args.config == 1 and not args.no_decode_long:
        result["decode_long"] = decode_long(w, torch, capi, args.seed)
    if args.config == 3:
        # the two-level configuration's 32 decode steps: as given (tails never fill) and with
        # 100 private tokens, where every tail fills at step 28 (reserve + table rebuild)
        result["decode_loop"] = [decode_loop(w, torch, capi, synth, args.seed, u, fused) for u in (128, 100)
                                 for fused in (False, True)]

    if not args.no_paged:
        pw = synth.paged_variant(w)
        pattn = build_cache(pw, torch, capi, args.seed)
        pout = torch.empty_like(q)
        pms = time_forward(pattn, q, pout, max(args.steps // 4, 10), max(args.warmup // 4, 2), torch)
        logical = tok_bytes * w.logical_tokens()
        physical = stream_bytes + shared_bytes
        torch.cuda.synchronize()
        diff = float((pout.float() - out.float()).abs().max())
        ratio = logical / physical
        result["paged_baseline"] = {"us_per_step": round(pms * 1e3, 2), "speedup": round(pms / ms, 3),
                                    "kv_sharing_ratio": round(ratio, 3),
                                    "speedup_over_ratio": round(pms / ms / ratio, 3),
                                    "GBps": round((logical + qo_bytes) / (pms * 1e-3) / 1e9, 1),
                                    "max_abs_diff_vs_shared": diff}
        if cold is not None:
            pcold = cold_forward_us(pattn, q, pout, torch, reps=8, hints=(("default_policy", 0),))
            result["paged_baseline"]["cold_us_per_step"] = pcold["default_policy_us"]
            result["paged_baseline"]["cold_speedup"] = round(pcold["default_policy_us"] / cold["default_policy_us"], 3)
            result["paged_baseline"]["cold_speedup_over_ratio"] = round(
                pcold["default_policy_us"] / cold["default_policy_us"] / ratio, 3)
        del pattn

    if args.cpu_seconds > 0:
        res, threads, blas, ref = cpu_baseline(attn, q_np, args.cpu_seconds, torch)
        err = float(np.abs(out.float().cpu().numpy() - ref).max())
        result["cpu_baseline"] = {"value": round(res["chunk_first"][0], 1), "unit": "us/step", "cores": threads,
                                  "kind": "port",
                                  "sample": "%s, full workload, fp32; chunk-first x%d forwards (value), sequence-first x%d forwards = %.1f us/step; host has %d logical cpus; %s" % (
                                      w.name, res["chunk_first"][1], res["seq_first"][1], res["seq_first"][0],
                                      os.cpu_count(), blas)}
        result["max_abs_err_vs_cpu"] = err
    print(json.dumps(result))
    return 0


if __name__ == "__main__":
    sys.exit(main())
