"""The pybind11/libtorch `Attention` class as a drop-in: the reference's own test scenarios
(tests/test_chunk_attn_cpu.py and tests/test_chunk_attn_cuda.py there) run against it on the
GPU, with node identity (`attn.tails == [n3]`) as those tests rely on it."""
import math

import numpy as np
import pytest
import torch

from kats import ADD_SEQ_STEPS, APPEND_CASE, REMOVE_CASE

pytestmark = pytest.mark.gpu


@pytest.fixture()
def mod():
    import chunk_attn
    return chunk_attn


def small(mod, **kw):
    args = dict(n_heads=2, d_head=4, chunk_size=2, memory_mb=1, dtype=torch.float16, device=torch.device("cuda"))
    args.update(kw)
    return mod.Attention(**args)


def ones(n, H=2, d=4):
    return torch.ones((n, H, d), dtype=torch.float16, device="cuda")


def tree_of(node):
    return (node.n_seqs, tuple(node.tokens), [tree_of(c) for c in node.children])


def node_at(root, path):
    for i in path:
        root = root.children[i]
    return root


def test_add_seq(mod):
    attn = small(mod)
    trie = attn.get_trie()
    for (tokens, want_tree, want_tails), want_idx in zip(ADD_SEQ_STEPS, [0, 1, 2, 3, 3, 3]):
        assert attn.add_seq(tokens=tokens, k=ones(len(tokens)), v=ones(len(tokens))) == want_idx
        assert (trie.n_seqs, trie.n_tokens, trie.tokens) == (want_tree[0], 0, [])
        assert tree_of(trie) == want_tree
        assert attn.tails == [node_at(trie, p) for p in want_tails]      # same node objects
    n1 = trie.children[0]
    assert (n1.n_seqs, n1.n_tokens, n1.tokens, n1.capacity) == (5, 2, [1, 2], 2)


def test_append_token_and_remove(mod):
    attn = small(mod)
    for tokens in APPEND_CASE["adds"]:
        attn.add_seq(tokens=tokens, k=ones(len(tokens)), v=ones(len(tokens)))
    new = attn.append_token(tokens=APPEND_CASE["append"], k=ones(2), v=ones(2))
    assert new == []
    trie = attn.get_trie()
    assert tree_of(trie) == APPEND_CASE["tree"]
    assert attn.tails == [node_at(trie, p) for p in APPEND_CASE["tails"]]
    # K rows landed where the tree says (chunk [5, 8] holds the appended row at index 1)
    n3 = node_at(trie, (0, 0, 0))
    assert attn.key(n3).shape == (2, 2, 4)
    assert torch.equal(attn.key(n3)[:, 1, :], torch.ones((2, 4), dtype=torch.float16, device="cuda"))

    attn2 = small(mod)
    for tokens in REMOVE_CASE["adds"]:
        attn2.add_seq(tokens=tokens, k=ones(len(tokens)), v=ones(len(tokens)))
    peak = attn2.peak_memory_allocated()
    assert peak == 4 * (2 * 2 * 4 * 2 * 2)          # four chunks of K+V
    attn2.remove_seq(REMOVE_CASE["remove"])
    assert tree_of(attn2.get_trie()) == REMOVE_CASE["tree"]
    assert attn2.peak_memory_allocated() == peak
    attn2.clear()
    assert tree_of(attn2.get_trie()) == (0, (), [])


def test_unsupported_shape_fails_at_forward_like_the_reference(mod):
    attn = small(mod)
    attn.add_seq(tokens=[1, 2, 3], k=ones(3), v=ones(3))
    with pytest.raises(RuntimeError, match="unsupported head dim 4"):
        attn.forward(q=ones(1))


def torch_reference(qs, keys, values, d_head):
    # the reference's check (tests/test_chunk_attn_cuda.py:37-44): fp32 softmax, fp16 P, matmul
    outs = []
    for q, k, v in zip(qs, keys, values):
        score = torch.matmul(q.transpose(0, 1).float(), k.transpose(0, 1).transpose(1, 2).float())
        score = torch.softmax(score / math.sqrt(d_head), dim=-1)
        outs.append(torch.matmul(score, v.transpose(0, 1).float()).transpose(0, 1))
    return torch.cat(outs, dim=0)


@pytest.mark.parametrize("chunk_size", [32, 64, 128])
def test_check_result_with_pytorch(mod, chunk_size):
    torch.manual_seed(0)
    seq_len, n_shared, n_heads, d_head, n_requests = 2000, 1000, 2, 128, 32
    f16 = dict(dtype=torch.float16, device="cuda")
    shared_k, shared_v = torch.randn((n_shared, n_heads, d_head), **f16), torch.randn((n_shared, n_heads, d_head), **f16)
    keys = [torch.randn((seq_len, n_heads, d_head), **f16) for _ in range(n_requests)]
    values = [torch.randn((seq_len, n_heads, d_head), **f16) for _ in range(n_requests)]
    for k, v in zip(keys, values):
        k[:n_shared], v[:n_shared] = shared_k, shared_v
    qs = [torch.randn((1, n_heads, d_head), **f16) for _ in range(n_requests)]
    want = torch_reference(qs, keys, values, d_head)
    attn = mod.Attention(n_heads=n_heads, d_head=d_head, chunk_size=chunk_size, memory_mb=512, dtype=torch.float16,
                         device=torch.device("cuda"))
    rng = np.random.default_rng(0)
    for i in range(n_requests):
        toks = list(range(n_shared)) + (n_shared + 1 + i * seq_len + np.arange(seq_len - n_shared)).tolist()
        assert attn.add_seq(tokens=toks, k=keys[i], v=values[i]) == i
    q = torch.cat(qs, dim=0)
    out = attn.forward(q=q)
    assert out.dtype == torch.float16 and out.shape == (n_requests, n_heads, d_head)
    assert torch.allclose(out.float(), want, atol=2e-3, rtol=1e-2)
    assert torch.allclose(attn.forward(q=q, partition=2).float(), want, atol=2e-3, rtol=1e-2)
    # the shared prefix is stored once
    shared_chunks = [c for (c, b, e) in attn.get_chunks() if e - b > 1]
    assert len(shared_chunks) == n_shared // chunk_size and all(e - b == n_requests for (c, b, e) in attn.get_chunks() if e - b > 1)


def test_decode_loop_like_the_model(mod):
    # the caller order of the reference's model layer: append_token -> forward -> reserve -> refresh
    torch.manual_seed(1)
    H, c = 4, 32
    f16 = dict(dtype=torch.float16, device="cuda")
    attn = mod.Attention(n_heads=H, d_head=128, chunk_size=c, memory_mb=64, dtype=torch.float16, device=torch.device("cuda"))
    lens = [30, 31, 45]
    ks = [torch.randn((n, H, 128), **f16) for n in lens]
    vs = [torch.randn((n, H, 128), **f16) for n in lens]
    for i, n in enumerate(lens):
        attn.add_seq(tokens=[1000 * i + t for t in range(n)], k=ks[i], v=vs[i])
    for step in range(40):
        k, v = torch.randn((3, H, 128), **f16), torch.randn((3, H, 128), **f16)
        attn.append_token(tokens=[7, 8, 9], k=k, v=v)
        for i in range(3):
            ks[i] = torch.cat([ks[i], k[i:i + 1]])
            vs[i] = torch.cat([vs[i], v[i:i + 1]])
        q = torch.randn((3, H, 128), **f16)
        out = attn.forward(q)
        attn.reserve()
        attn.refresh_kernel_context(False)
        want = torch_reference([q[i:i + 1] for i in range(3)], ks, vs, 128)
        assert torch.allclose(out.float(), want, atol=2e-3, rtol=1e-2), step


def test_copy_constructor_duplicate_and_completion(mod):
    torch.manual_seed(2)
    H, c = 2, 32
    f16 = dict(dtype=torch.float16, device="cuda")
    base = mod.Attention(n_heads=H, d_head=128, chunk_size=c, memory_mb=32, dtype=torch.float16, device=torch.device("cuda"))
    layer2 = mod.Attention(base)          # same configuration, empty cache
    k, v = torch.randn((40, H, 128), **f16), torch.randn((40, H, 128), **f16)
    layer2.add_seq(tokens=list(range(40)), k=k, v=v)
    assert base.get_trie().n_seqs == 0 and layer2.get_trie().n_seqs == 1
    layer2.duplicate(0, 2)
    assert layer2.get_trie().n_seqs == 3 and len(layer2.tails) == 3
    q = torch.randn((3, H, 128), **f16)
    out = layer2.forward(q)
    want = torch_reference([q[i:i + 1] for i in range(3)], [k] * 3, [v] * 3, 128)
    assert torch.allclose(out.float(), want, atol=2e-3, rtol=1e-2)
    # beam step on sequence 1: two candidates -> sequences 1 and 2 continue differently
    nk, nv = torch.randn((2, H, 128), **f16), torch.randn((2, H, 128), **f16)
    toks = [500, 501]
    assert layer2.append_completion(1, toks, nk, nv) == 1
    assert layer2.get_trie().n_seqs == 4
    q = torch.randn((4, H, 128), **f16)
    out = layer2.forward(q)
    ks = [k, torch.cat([k, nk[0:1]]), torch.cat([k, nk[1:2]]), k]
    vs = [v, torch.cat([v, nv[0:1]]), torch.cat([v, nv[1:2]]), v]
    want = torch_reference([q[i:i + 1] for i in range(4)], ks, vs, 128)
    assert torch.allclose(out.float(), want, atol=2e-3, rtol=1e-2)


def test_errors_and_defaults(mod):
    with pytest.raises(RuntimeError, match="device is not CUDA"):
        mod.Attention(n_heads=2, d_head=128, chunk_size=64, memory_mb=1, dtype=torch.float16, device=torch.device("cpu"))
    attn = mod.Attention(n_heads=2, d_head=128, chunk_size=64, memory_mb=1, dtype=torch.float16, device=torch.device("cuda"))
    k = torch.ones((3, 2, 128), dtype=torch.float16, device="cuda")
    attn.add_seq(tokens=[1, 2, 3], k=k, v=k)
    with pytest.raises(RuntimeError, match="q is not contiguous"):
        attn.forward(torch.ones((1, 2, 256), dtype=torch.float16, device="cuda")[:, :, :128])
    with pytest.raises(RuntimeError, match="num of seqs is not equal to num of tokens"):
        attn.append_token(tokens=[1, 2], k=k[:2], v=k[:2])
    with pytest.raises(RuntimeError, match="has bugs"):
        attn.add_seq_async(tokens=[1], k=k[:1], v=k[:1])
    with pytest.raises(RuntimeError, match="capacity reached"):
        for i in range(10):
            attn.add_seq(tokens=[100 + i] * 64, k=torch.ones((64, 2, 128), dtype=torch.float16, device="cuda"),
                         v=torch.ones((64, 2, 128), dtype=torch.float16, device="cuda"))
    attn.print()


def test_rotary_ops_and_fused_append_match_the_c_abi_binding(mod):
    """chunk_attn.ops.rotary_embedding (reference python_exports_ops.cpp:13) and
    Attention.append_token_rotary go through the same C-ABI entry points as the ctypes binding:
    identical results, and the fused step equals rotary followed by append_token."""
    from chunk_attn import capi
    from oracle.rotary import cos_sin_cache, rotary_embedding
    rng = np.random.default_rng(21)
    H, d, c, n = 2, 128, 32, 3
    cache_np = cos_sin_cache(d, 256)
    cache = torch.from_numpy(cache_np).cuda()
    pos_np = np.array([5, 0, 77], dtype=np.int64)
    q_np = rng.standard_normal((n, H * d)).astype(np.float16)
    k_np = rng.standard_normal((n, H * d)).astype(np.float16)
    q, k, pos = torch.from_numpy(q_np).cuda(), torch.from_numpy(k_np).cuda(), torch.from_numpy(pos_np).cuda()
    mod.ops.rotary_embedding(pos, q, k, d, cache, True)
    q2, k2 = torch.from_numpy(q_np).cuda(), torch.from_numpy(k_np).cuda()
    capi.rotary_embedding(pos, q2, k2, d, cache, True)
    assert torch.equal(q, q2) and torch.equal(k, k2)
    wq, wk = rotary_embedding(pos_np, q_np, k_np, d, cache_np, True)
    np.testing.assert_allclose(q.float().cpu().numpy(), wq.astype(np.float32), atol=2e-3, rtol=1e-2)
    np.testing.assert_allclose(k.float().cpu().numpy(), wk.astype(np.float32), atol=2e-3, rtol=1e-2)

    def cache_with_two_seqs():
        a = mod.Attention(n_heads=H, d_head=d, chunk_size=c, memory_mb=4, dtype=torch.float16,
                          device=torch.device("cuda"))
        g = torch.Generator().manual_seed(3)
        for s, T in enumerate((40, 45)):
            toks = list(range(32)) + [1000 * (s + 1) + i for i in range(T - 32)]
            kk = torch.randn((T, H, d), generator=g).half()
            vv = torch.randn((T, H, d), generator=g).half()
            if s:
                kk[:32], vv[:32] = first[0][:32], first[1][:32]
            else:
                first = (kk, vv)
            assert a.add_seq(tokens=toks, k=kk.cuda(), v=vv.cuda()) == s
        return a

    fused, plain = cache_with_two_seqs(), cache_with_two_seqs()
    for step in range(30):      # sequence 0 crosses into a new chunk at step 24
        qn = torch.randn((2, H, d)).half().cuda()
        kn = torch.randn((2, H, d)).half().cuda()
        vn = torch.randn((2, H, d)).half().cuda()
        lens = torch.tensor([40 + step, 45 + step], dtype=torch.int64, device="cuda")
        qf, qp, kp = qn.clone(), qn.clone(), kn.clone()
        fresh = fused.append_token_rotary(tokens=[step, step], q=qf, k=kn, v=vn, cos_sin_cache=cache)
        mod.ops.rotary_embedding(lens, qp.view(2, H * d), kp.view(2, H * d), d, cache, True)
        fresh_p = plain.append_token(tokens=[step, step], k=kp, v=vn)
        assert len(fresh) == len(fresh_p)
        # same fp32 arithmetic in both kernels; the final rounding to fp16 may differ by one place
        assert ((qf.float() - qp.float()).abs() <= 2.0 ** -10 * qf.float().abs() + 2.0 ** -24).all()
        np.testing.assert_allclose(fused.forward(qf).float().cpu().numpy(), plain.forward(qp).float().cpu().numpy(),
                                   atol=2e-3, rtol=1e-2)
    with pytest.raises(RuntimeError, match="positions"):
        fused.append_token_rotary(tokens=[1, 2], q=qf, k=kn, v=vn, cos_sin_cache=cache,
                                  positions=torch.zeros(3, dtype=torch.int64, device="cuda"))
