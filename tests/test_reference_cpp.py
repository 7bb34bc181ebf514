"""The plain C++ references of the kernels against the plain Python implementation, part by part, on the
CPU; and their self-test under the host's sanitizers. (On the GPU the kernels are held against both.)"""
import math
import subprocess

import pytest
import torch

import cache_order
import plain_llama as P
from reference_cpp import CppReference


@pytest.fixture(scope="module")
def ref():
    return CppReference()


def rand(*shape, seed=0, scale=1.0):
    return torch.randn(*shape, generator=torch.Generator().manual_seed(seed)) * scale


def close(a, b, tol=2e-5):
    assert a.shape == b.shape
    assert float((a.double() - b.double()).abs().max()) <= tol * (1.0 + float(b.double().abs().max()))


def test_selftest_runs_clean_under_the_sanitizers():
    from xeno_rt_amd.ops import build
    program = build.build_reference_selftest(sanitize=True)
    done = subprocess.run([program], capture_output=True, text=True, timeout=120)
    assert done.returncode == 0, done.stdout + done.stderr
    assert "reference selftest ok" in done.stdout


def test_block_size_is_the_caches(ref):
    from xeno_rt_amd.cache import BLOCK_TOKENS
    assert ref.lib.xrt_ref_block_tokens() == BLOCK_TOKENS


def test_norm_products_and_gate(ref):
    x, w = rand(5, 96, seed=1, scale=3.0), rand(96, seed=2) + 1.0
    close(ref.rmsnorm(x, w, 1e-3), P.rmsnorm(x, w, 1e-3))
    rows = torch.tensor([4, 0, 4], dtype=torch.int32)
    assert torch.equal(ref.rmsnorm(x, w, 1e-3, rows=rows), ref.rmsnorm(x, w, 1e-3)[rows.long()])
    a, m = rand(7, 40, seed=3), rand(24, 40, seed=4, scale=0.3)
    close(ref.linear(a, m), P.linear(a, m))
    base = rand(7, 24, seed=5)
    close(ref.linear(a, m, base=base), base + P.linear(a, m))
    both = P.linear(a, m)
    close(ref.linear_glu(a, m), P.swiglu(both[:, :12], both[:, 12:]))
    table = rand(50, 8, seed=6)
    assert torch.equal(ref.embed(table, torch.tensor([3, 49, 3])), table[[3, 49, 3]])


@pytest.mark.parametrize("nh,nkv,hd,rope_dim,norms", [(4, 2, 16, 16, False), (6, 3, 32, 32, True), (2, 1, 48, 32, True)])
def test_preparation_and_attention_over_the_cache(ref, nh, nkv, hd, rope_dim, norms):
    """One sequence of 150 tokens through the preparation (head norms, rotation, cache write) and the attention
    over the cache's blocks, against the plain functions on whole tensors."""
    tokens, base, eps = 150, 10000.0, 1e-4
    width = (nh + 2 * nkv) * hd
    qkv = rand(tokens, width, seed=hd)
    positions = torch.arange(tokens, dtype=torch.int32)
    slots = torch.zeros(tokens, dtype=torch.int32)
    qn, kn = (rand(hd, seed=1) + 1.0, rand(hd, seed=2) + 1.0) if norms else (None, None)
    theta = P.rope_inverse_frequencies(rope_dim, base)
    table = torch.tensor([[2, 0, 1]], dtype=torch.int32)           # three blocks, not in order
    k = torch.zeros(3, nkv, 64, hd)
    v = torch.zeros(3, nkv, hd, 64)
    got = ref.qkv_prepare(qkv, nh, nkv, hd, positions, slots, qn, kn, eps, theta, rope_dim, 1.0, kv=(k, v, table))
    q, kk, vv = qkv[:, :nh * hd], qkv[:, nh * hd:(nh + nkv) * hd], qkv[:, (nh + nkv) * hd:]
    if norms:
        q, kk = P.head_rmsnorm(q, nh, hd, qn, eps), P.head_rmsnorm(kk, nkv, hd, kn, eps)
    q, kk = P.rope(q, nh, hd, positions, rope_dim, base), P.rope(kk, nkv, hd, positions, rope_dim, base)
    close(got[:, :nh * hd], q, 1e-4)
    close(got[:, nh * hd:(nh + nkv) * hd], kk, 1e-4)
    assert torch.equal(got[:, (nh + nkv) * hd:], vv)
    # the cache: token 70 lies in logical block 1 = physical block 0, place 6
    close(cache_order.plain_keys(k)[0, :, 6, :].reshape(-1), kk[70], 1e-4)
    assert torch.equal(cache_order.plain_values(v)[0, :, :, 6].reshape(-1), vv[70])
    out = ref.attention(got, nh, nkv, hd, k, v, table, positions, slots, 1.0 / math.sqrt(hd))
    close(out, P.causal_attention(q, kk, vv, nh, nkv, hd), 1e-4)
    # a window of 20: the plain attention over the 20 last keys of every query
    windowed = ref.attention(got, nh, nkv, hd, k, v, table, positions, slots, 1.0 / math.sqrt(hd), window=20)
    for t in (0, 19, 20, 149):
        first = max(0, t - 19)
        want = P.causal_attention(q[t:t + 1], kk[first:t + 1], vv[first:t + 1], nh, nkv, hd, start_position=t - first)
        close(windowed[t:t + 1], want, 1e-4)


def test_sampling_against_the_plain_distribution(ref):
    vocab, draws = 300, 600
    row = rand(vocab, seed=9, scale=2.0)
    history = [3, 7, 7, vocab - 1]
    u = ((torch.arange(draws) + 0.5) / draws).tolist()
    for temperature, top_k, top_p, penalty in [(1.0, 0, 1.0, 1.0), (0.7, 40, 0.95, 1.1), (1.5, 5, 1.0, 2.0), (1.0, 0, 0.5, 1.0)]:
        adjusted = P.apply_repetition_penalty(row, history, penalty)
        dist = P.sampling_distribution(adjusted, temperature, top_k, top_p)
        picks = ref.sample(row[None, :].expand(draws, vocab), [temperature] * draws, [top_k] * draws, [top_p] * draws,
                           [penalty] * draws, history, [0, len(history)] * draws, u)
        counts = torch.bincount(torch.tensor(picks), minlength=vocab).double() / draws
        assert float((counts - dist).abs().max()) <= 1.5 / draws + 1e-6
        greedy = ref.sample(row[None, :], [0.0], [top_k], [top_p], [penalty], history, [0, len(history)], [0.5])
        assert greedy == [P.greedy(adjusted)]
    assert ref.sample(torch.tensor([[1.0, 3.0, 3.0, float("nan")]]), [0.0], [0], [1.0], [1.0], [0], [0, 0], [0.5]) == [1]


def test_random_weights_and_packing(ref):
    from xeno_rt_amd.weights import random_init
    key = random_init.tensor_key(4, "some.weight")
    scale = random_init.normal_scale(0.02)
    assert torch.equal(ref.random_normal(5000, key, scale), random_init.normal_values(key, 0, 5000, scale))
    assert torch.equal(ref.random_normal(100, key, scale, 1.0), random_init.normal_values(key, 0, 100, scale) + 1.0)
    w = rand(40, 64, seed=3)
    flat = ref.pack(w)
    place = lambda row, k: ((row // 16) * 2 + k // 32) * 512 + ((k % 32 // 8) * 16 + row % 16) * 8 + k % 8
    for row, k in ((0, 0), (39, 63), (17, 9), (15, 32)):
        assert flat[place(row, k)] == w[row, k]
    assert float(flat[place(45, 3)]) == 0.0
    pairs = ref.pack(rand(32, 64, seed=4), kind=2, gated_n=16)
    assert pairs[place(8, 5)] == rand(32, 64, seed=4)[16, 5]           # the first up row follows the first eight gate rows
