"""GPU parity with chunks that sit beyond the first 4 GiB of each pool: every kernel's chunk
offset (slot * H * chunk_size * d halves) must be formed in 64 bits.  A cache sized for this
part's HBM is far larger than 4 GiB; the allocator hands out low slots first, so the ordinary
tests never reach such offsets.  Here the kernel seam of the C-ABI is driven directly with
chunk rows that name high slots of a 5 GiB + 5 GiB pool (the memory is only touched where the
rows point)."""
import numpy as np
import pytest
import torch

from chunk_attn import capi
from gpu_helpers import assert_close, dev, to_dev
from oracle.attention_ref import CpuAttention, textbook_attention

pytestmark = pytest.mark.gpu

H, C, D = 32, 64, 128
N_SLOTS = 10240 + 256          # 512 KiB per chunk and pool: slot 8192 starts at 4 GiB
FIRST_HIGH = 8192 + 5


def build_case(n_seqs, rng):
    """Rows in the manager's order (parents first, children last to first): two full chunks shared
    by everyone, then per sequence one full private chunk and a partly filled tail.  Slots are
    drawn without order from the region above 4 GiB."""
    slots = list(rng.permutation(np.arange(FIRST_HIGH, N_SLOTS))[: 2 + 2 * n_seqs])
    rows = [[slots[0], C, 0, n_seqs], [slots[1], C, 0, n_seqs]]
    for s in range(n_seqs - 1, -1, -1):
        rows.append([slots[2 + 2 * s], C, s, s + 1])
        rows.append([slots[3 + 2 * s], 3 + (7 * s) % (C - 4), s, s + 1])
    return np.array(rows, np.int32)


def compact(rows, kp, vp):
    """The used chunks as small numpy pools and the rows renumbered into them, for the oracle."""
    used = sorted(set(int(r[0]) for r in rows))
    new = {slot: i for i, slot in enumerate(used)}
    idx = torch.tensor(used, device=dev())
    torch.cuda.synchronize()
    k = kp[idx].float().cpu().numpy()
    v = vp[idx].float().cpu().numpy()
    r2 = rows.copy()
    r2[:, 0] = [new[int(s)] for s in rows[:, 0]]
    return r2, k, v


@pytest.mark.parametrize("n_seqs", [5, 100])      # narrow and wide chunk-first form
def test_chunks_beyond_4_gib(n_seqs):
    rng = np.random.default_rng(100 + n_seqs)
    kp = torch.empty((N_SLOTS, H, C, D), dtype=torch.float16, device=dev())
    vp = torch.empty_like(kp)
    assert kp[FIRST_HIGH].data_ptr() - kp.data_ptr() > (1 << 32)
    rows = build_case(n_seqs, rng)
    for slot, n_tok, _, _ in rows:
        kp[int(slot)] = to_dev(rng.standard_normal((H, C, D)).astype(np.float16))
        vp[int(slot)] = to_dev(rng.standard_normal((H, C, D)).astype(np.float16))
    ctx = capi.KernelContext(H, D, C, kp.data_ptr(), vp.data_ptr(), N_SLOTS)
    stream = torch.cuda.current_stream().cuda_stream
    q = rng.standard_normal((n_seqs, H, D)).astype(np.float16)
    tq, out = to_dev(q), torch.empty((n_seqs, H, D), dtype=torch.float16, device=dev())
    ctx.refresh(rows, n_seqs, stream)
    r2, k_np, v_np = compact(rows, kp, vp)
    want = textbook_attention(q.astype(np.float32), r2.tolist(), k_np, v_np)
    for partition in (0, 1, 2):
        out.zero_()
        ctx.attention(tq.data_ptr(), out.data_ptr(), n_seqs, partition, stream)
        assert_close(out, want)
    cpu = CpuAttention().attention(q.astype(np.float32), r2.tolist(), k_np, v_np, 0)
    assert_close(out, cpu.astype(np.float64))

    # one decode step: a new K/V row into every tail (high slots again), then the forward
    k_new = rng.standard_normal((n_seqs, H, D)).astype(np.float16)
    v_new = rng.standard_normal((n_seqs, H, D)).astype(np.float16)
    tk, tv = to_dev(k_new), to_dev(v_new)
    ctx.append_kv(tk.data_ptr(), tv.data_ptr(), n_seqs, stream)
    ctx.delta_tokens = 1
    ctx.attention(tq.data_ptr(), out.data_ptr(), n_seqs, 0, stream)
    grown = rows.copy()
    for s in range(n_seqs):
        tail = [i for i, r in enumerate(rows) if r[2] == s and r[3] == s + 1][-1]
        slot, fill = int(rows[tail][0]), int(rows[tail][1])
        torch.cuda.synchronize()
        assert np.array_equal(kp[slot, :, fill].cpu().numpy(), k_new[s])     # bit-exact row writes
        assert np.array_equal(vp[slot, :, fill].cpu().numpy(), v_new[s])
        grown[tail][1] = fill + 1
    r3, k_np, v_np = compact(grown, kp, vp)
    assert_close(out, textbook_attention(q.astype(np.float32), r3.tolist(), k_np, v_np))


def test_copy_in_and_chunk_copy_beyond_4_gib():
    rng = np.random.default_rng(7)
    kp = torch.empty((N_SLOTS, H, C, D), dtype=torch.float16, device=dev())
    vp = torch.empty_like(kp)
    ctx = capi.KernelContext(H, D, C, kp.data_ptr(), vp.data_ptr(), N_SLOTS)
    stream = torch.cuda.current_stream().cuda_stream
    T = 2 * C + 9                                     # two full chunks and a partial one
    k = rng.standard_normal((T, H, D)).astype(np.float16)
    v = rng.standard_normal((T, H, D)).astype(np.float16)
    slots = [N_SLOTS - 1, FIRST_HIGH + 3, N_SLOTS - 77]
    tk, tv = to_dev(k), to_dev(v)
    ctx.scatter_kv(tk.data_ptr(), tv.data_ptr(), T, 0, slots, stream)
    torch.cuda.synchronize()
    for i, slot in enumerate(slots):
        n = min(C, T - i * C)
        assert np.array_equal(kp[slot, :, :n].cpu().numpy(), k[i * C:i * C + n].transpose(1, 0, 2))
        assert np.array_equal(vp[slot, :, :n].cpu().numpy(), v[i * C:i * C + n].transpose(1, 0, 2))
    ctx.copy_chunk(N_SLOTS - 1, FIRST_HIGH + 40, stream)
    torch.cuda.synchronize()
    assert torch.equal(kp[FIRST_HIGH + 40], kp[N_SLOTS - 1]) and torch.equal(vp[FIRST_HIGH + 40], vp[N_SLOTS - 1])


def test_row_writes_beyond_4_gib_and_bad_targets():
    rng = np.random.default_rng(8)
    kp = torch.empty((N_SLOTS, H, C, D), dtype=torch.float16, device=dev())
    vp = torch.empty_like(kp)
    ctx = capi.KernelContext(H, D, C, kp.data_ptr(), vp.data_ptr(), N_SLOTS)
    stream = torch.cuda.current_stream().cuda_stream
    n = 70                                             # more than one launch's worth of targets
    k = rng.standard_normal((n, H, D)).astype(np.float16)
    v = rng.standard_normal((n, H, D)).astype(np.float16)
    targets = [(int(FIRST_HIGH + 3 * i), int((5 * i) % C)) for i in range(n)]
    tk, tv = to_dev(k), to_dev(v)
    ctx.put_kv_rows(tk.data_ptr(), tv.data_ptr(), targets, stream)
    torch.cuda.synchronize()
    for i, (slot, row) in enumerate(targets):
        assert np.array_equal(kp[slot, :, row].cpu().numpy(), k[i])
        assert np.array_equal(vp[slot, :, row].cpu().numpy(), v[i])
    for bad in [(N_SLOTS, 0), (-1, 0), (5, C), (5, -1)]:
        with pytest.raises(capi.ChunkAttnError, match="outside the pool or the chunk"):
            ctx.put_kv_rows(tk.data_ptr(), tv.data_ptr(), [bad], stream)
