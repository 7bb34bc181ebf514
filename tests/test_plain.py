"""Pins the plain implementation by what fixes it beside the reference's text: vectors
that the reference's own tests hold, special cases that reduce to a library routine,
and invariants. Each is chosen so that a plausible mistake fails it."""
import math

import numpy as np
import pytest
import torch

import plain_llama as P


def close(a, b, tol=1e-6):
    a, b = torch.as_tensor(a, dtype=torch.float64), torch.as_tensor(b, dtype=torch.float64)
    assert a.shape == b.shape
    assert float((a - b).abs().max()) <= tol, (a, b)


# ---- RMSNorm ---------------------------------------------------------------------

def test_rmsnorm_reference_vector():
    # tests/kernels_test.rs:75-91 of the reference
    x = torch.tensor([1.0, 2.0, 3.0, 4.0])
    w = torch.tensor([1.0, 1.5, 2.0, 2.5])
    inv = 1.0 / math.sqrt((1 + 4 + 9 + 16) / 4 + 1e-5)
    close(P.rmsnorm(x, w, 1e-5), [1 * inv * 1.0, 2 * inv * 1.5, 3 * inv * 2.0, 4 * inv * 2.5])


def test_rmsnorm_reduces_to_numpy_and_is_scale_invariant():
    x = torch.randn(5, 24, dtype=torch.float64)
    ones = torch.ones(24, dtype=torch.float64)
    want = x.numpy() / np.linalg.norm(x.numpy(), axis=-1, keepdims=True) * math.sqrt(24)
    close(P.rmsnorm(x, ones, 0.0), want, 1e-12)
    close(P.rmsnorm(3.7 * x, ones, 0.0), P.rmsnorm(x, ones, 0.0), 1e-12)
    # the weight multiplies (it is not 1 + w): zero weight gives zero
    close(P.rmsnorm(x, torch.zeros(24, dtype=torch.float64), 1e-5), torch.zeros(5, 24))


def test_rmsnorm_eps_is_inside_the_root():
    x = torch.tensor([[3.0, 4.0]])
    close(P.rmsnorm(x, torch.ones(2), 0.5), x / math.sqrt(12.5 + 0.5))


def test_head_rmsnorm_reduces_to_rmsnorm():
    x = torch.randn(3, 32, dtype=torch.float64)
    w = torch.randn(32, dtype=torch.float64)
    close(P.head_rmsnorm(x, 1, 32, w, 1e-6), P.rmsnorm(x, w, 1e-6), 1e-12)      # one head of full width
    w8 = torch.randn(8, dtype=torch.float64)
    rows = P.rmsnorm(x.reshape(3 * 4, 8), w8, 1e-6).reshape(3, 32)                # heads are rows
    close(P.head_rmsnorm(x, 4, 8, w8, 1e-6), rows, 1e-12)


# ---- rotation --------------------------------------------------------------------

def test_rope_reference_vector():
    # tests/kernels_test.rs:94-108: one head of 4, position 2, base 1e4: angles 2 and 0.02,
    # pairs (0, 2) and (1, 3)
    x = torch.tensor([[1.0, 2.0, 3.0, 4.0]])
    a0, a1 = 2.0, 2.0 / 100.0
    want = [[1 * math.cos(a0) - 3 * math.sin(a0), 2 * math.cos(a1) - 4 * math.sin(a1),
             1 * math.sin(a0) + 3 * math.cos(a0), 2 * math.sin(a1) + 4 * math.cos(a1)]]
    close(P.rope(x, 1, 4, torch.tensor([2]), 4, 10000.0), want)


def test_rope_position_zero_is_identity_and_pairs_keep_their_norm():
    x = torch.randn(4, 2 * 16)
    close(P.rope(x, 2, 16, torch.zeros(4, dtype=torch.long), 16, 1e4), x, 0)
    y = P.rope(x, 2, 16, torch.tensor([1, 7, 30, 100]), 16, 1e4).reshape(4, 2, 16)
    xr = x.reshape(4, 2, 16)
    close(y[..., :8] ** 2 + y[..., 8:] ** 2, xr[..., :8] ** 2 + xr[..., 8:] ** 2, 1e-5)


def test_rope_is_a_complex_multiplication_of_half_split_pairs():
    x = torch.randn(1, 8, dtype=torch.float64)
    pos, base = 5, 100.0
    theta = np.array([base ** (2 * i / 8) for i in range(4)])
    z = (x[0, :4].numpy() + 1j * x[0, 4:].numpy()) * np.exp(1j * pos / theta)
    got = P.rope(x, 1, 8, torch.tensor([pos]), 8, base)
    close(got[0, :4], z.real, 1e-6)
    close(got[0, 4:], z.imag, 1e-6)
    # interleaved pairing (2i, 2i+1) would give something else on this data
    zi = (x[0, 0::2].numpy() + 1j * x[0, 1::2].numpy()) * np.exp(1j * pos / theta)
    assert np.abs(got[0, :4].numpy() - zi.real).max() > 1e-3


def test_rope_scores_depend_on_distance_only():
    q, k = torch.randn(1, 32, dtype=torch.float64), torch.randn(1, 32, dtype=torch.float64)
    def score(m, n):
        return float(P.rope(q, 1, 32, torch.tensor([m]), 32, 1e4) @ P.rope(k, 1, 32, torch.tensor([n]), 32, 1e4).t())
    assert abs(score(9, 4) - score(109, 104)) < 1e-4      # float32 angles limit this
    assert abs(score(9, 4) - score(4, 9)) > 1e-3          # the sign of the distance matters


def test_rope_leaves_the_tail_beyond_rope_dim():
    x = torch.randn(2, 16)
    y = P.rope(x, 1, 16, torch.tensor([3, 4]), 8, 1e4)
    close(y[:, 8:], x[:, 8:], 0)
    assert float((y[:, :8] - x[:, :8]).abs().max()) > 1e-3


def test_rope_scale_multiplies_the_position():
    """rope.rs:25, 63, 109: angle = position * scale / theta. Position 8 at scale 0.25 is position 2 at scale 1; a scale
    that divided the position, or multiplied theta, would make it position 32."""
    x = torch.randn(3, 2 * 16)
    at = lambda p: torch.tensor([p, p, p])
    close(P.rope(x, 2, 16, at(8), 16, 1e4, 0.25), P.rope(x, 2, 16, at(2), 16, 1e4, 1.0), 1e-6)
    assert float((P.rope(x, 2, 16, at(8), 16, 1e4, 0.25) - P.rope(x, 2, 16, at(32), 16, 1e4, 1.0)).abs().max()) > 1e-2
    # with fewer dims rotated the pairs are (i, i + rope_dim / 2) of the first rope_dim dims, and theta's exponent is over rope_dim
    y = P.rope(x, 2, 16, at(5), 8, 1e4, 0.5)
    z = (x.view(3, 2, 16)[:, :, :4].double().numpy() + 1j * x.view(3, 2, 16)[:, :, 4:8].double().numpy()) \
        * np.exp(1j * 5 * 0.5 / (1e4 ** (np.arange(4) * 2.0 / 8)))
    close(y.view(3, 2, 16)[:, :, :4], z.real, 1e-5)
    close(y.view(3, 2, 16)[:, :, 4:8], z.imag, 1e-5)


def test_the_plain_model_reads_the_rotation_s_options(tmp_path):
    """The second tiny configuration rotates half of a head and divides positions by 4; the plain model must see both
    (a model that ignored them would agree with the engine only if the engine ignored them too)."""
    from conftest import TINY, make_folder
    model = P.PlainModel(make_folder(TINY["qwen3"], tmp_path / "m", seed=5))
    assert model.config.rope_dim == 16 and model.config.head_dim == 32 and model.config.rope_scale == 0.25
    ids = list(range(3, 23))
    with_options = model.logits(ids)
    model.config.rope_scale, model.config.rope_dim = 1.0, 32
    assert float((model.logits(ids) - with_options).abs().max()) > 1e-3 * float(with_options.abs().max())


# ---- softmax, silu, linear ---------------------------------------------------------

def test_softmax_reference_vector():
    # tests/kernels_test.rs:110-124
    d = math.exp(-2) + math.exp(-1) + 1
    got = P.softmax(torch.tensor([1.0, 2.0, 3.0]))
    close(got, [math.exp(-2) / d, math.exp(-1) / d, 1 / d])
    assert abs(float(got.sum()) - 1) < 1e-6
    x = torch.randn(7, dtype=torch.float64)
    close(P.softmax(x), torch.softmax(x, 0), 1e-12)
    close(P.softmax(x + 1000.0), P.softmax(x), 1e-9)


def test_silu_reference_vector():
    # tests/kernels_test.rs:126-136
    x = torch.tensor([-2.0, -0.5, 0.0, 1.5])
    close(P.silu(x), [v * (1 / (1 + math.exp(-v))) for v in x.tolist()])
    g, u = torch.randn(9, dtype=torch.float64), torch.randn(9, dtype=torch.float64)
    close(P.swiglu(g, u), torch.nn.functional.silu(g) * u, 1e-12)
    assert float(P.silu(torch.tensor(0.0))) == 0.0


def test_linear_layout_is_out_by_in():
    # tests/kernels_test.rs:138-153 holds A[2x3].B[3x2]; here the weight is B transposed
    a = torch.tensor([[1.0, 2.0, 3.0], [4.0, 5.0, 6.0]])
    b = torch.tensor([[7.0, 8.0], [9.0, 10.0], [11.0, 12.0]])
    close(P.linear(a, b.t().contiguous()), [[58.0, 64.0], [139.0, 154.0]])
    w = torch.randn(5, 3)
    close(P.linear(torch.tensor([[0.0, 1.0, 0.0]]), w), w[:, 1][None, :], 0)   # one-hot input returns a column


# ---- attention ---------------------------------------------------------------------

def test_attention_without_groups_is_library_causal_attention():
    t, nh, hd = 9, 3, 8
    q, k, v = (torch.randn(t, nh * hd, dtype=torch.float64) for _ in range(3))
    got = P.causal_attention(q, k, v, nh, nh, hd)
    lib = torch.nn.functional.scaled_dot_product_attention(
        q.reshape(t, nh, hd).transpose(0, 1), k.reshape(t, nh, hd).transpose(0, 1),
        v.reshape(t, nh, hd).transpose(0, 1), is_causal=True).transpose(0, 1).reshape(t, nh * hd)
    close(got, lib, 1e-10)


def test_attention_one_token_returns_the_value_row():
    q, k, v = torch.randn(1, 4 * 8), torch.randn(1, 2 * 8), torch.randn(1, 2 * 8)
    got = P.causal_attention(q, k, v, 4, 2, 8).reshape(4, 8)
    vh = v.reshape(2, 8)
    close(got, torch.stack([vh[0], vh[0], vh[1], vh[1]]), 1e-6)   # consecutive query heads share a kv head


def test_attention_groups_equal_expanded_heads():
    t, nh, nkv, hd = 7, 6, 2, 4
    q = torch.randn(t, nh * hd, dtype=torch.float64)
    k, v = torch.randn(t, nkv * hd, dtype=torch.float64), torch.randn(t, nkv * hd, dtype=torch.float64)
    expand = lambda x: x.reshape(t, nkv, 1, hd).expand(t, nkv, nh // nkv, hd).reshape(t, nh * hd)
    close(P.causal_attention(q, k, v, nh, nkv, hd), P.causal_attention(q, expand(k), expand(v), nh, nh, hd), 1e-12)


def test_attention_is_causal_and_start_position_counts():
    t, nh, nkv, hd = 6, 2, 1, 8
    q, k, v = torch.randn(t, nh * hd), torch.randn(t, nkv * hd), torch.randn(t, nkv * hd)
    base = P.causal_attention(q, k, v, nh, nkv, hd)
    k2, v2 = k.clone(), v.clone()
    k2[4:], v2[4:] = 9.0, -9.0
    close(P.causal_attention(q, k2, v2, nh, nkv, hd)[:4], base[:4], 0)       # later tokens change nothing earlier
    close(P.causal_attention(q[3:], k, v, nh, nkv, hd, start_position=3), base[3:], 1e-6)


def test_attention_scale_is_inverse_root_of_head_dim():
    hd = 16
    q = torch.zeros(2, hd); q[1, 0] = 4.0
    k = torch.zeros(2, hd); k[0, 0] = 1.0
    v = torch.tensor([[1.0] + [0.0] * (hd - 1), [0.0] * hd])
    w0 = math.exp(4.0 / math.sqrt(hd)) / (math.exp(4.0 / math.sqrt(hd)) + 1.0)
    assert abs(float(P.causal_attention(q, k, v, 1, 1, hd)[1, 0]) - w0) < 1e-6


# ---- block / model -------------------------------------------------------------------

def _model(tmp_path, name, **changes):
    from conftest import TINY, make_folder
    raw = dict(TINY[name], **changes)
    return P.PlainModel(make_folder(raw, tmp_path / name, seed=3, std=0.2))


def test_model_with_silenced_blocks_is_norm_and_head(tmp_path):
    model = _model(tmp_path, "llama")
    for name in list(model.weights):
        if name.endswith("o_proj.weight") or name.endswith("down_proj.weight"):
            model.weights[name].zero_()
    ids = [5, 9, 200]
    want = P.linear(P.rmsnorm(model.w("model.embed_tokens.weight")[ids], model.w("model.norm.weight"),
                              model.config.eps), model.w("lm_head.weight"))
    close(model.logits(ids), want, 1e-5)


def test_tied_model_uses_the_embedding_as_head(tmp_path):
    model = _model(tmp_path, "qwen3")
    assert model.config.tied and "lm_head.weight" not in model.weights
    for name in list(model.weights):
        if name.endswith("o_proj.weight") or name.endswith("down_proj.weight"):
            model.weights[name].zero_()
    e = model.w("model.embed_tokens.weight")
    close(model.logits([7]), P.rmsnorm(e[[7]], model.w("model.norm.weight"), model.config.eps) @ e.t(), 1e-5)


def test_model_is_causal_and_float64_agrees(tmp_path):
    model = _model(tmp_path, "qwen3")
    ids = list(range(3, 15))
    full = model.logits(ids)
    close(model.logits(ids[:7]), full[:7], 1e-5)
    other = list(ids); other[9] = 300
    close(model.logits(other)[:9], full[:9], 1e-5)
    double = P.PlainModel(str(tmp_path / "qwen3"), dtype=torch.float64).logits(ids)
    assert float((double - full).abs().max()) < 1e-4


def test_norm_weights_and_qk_norm_matter(tmp_path):
    # guards the tests themselves: the fixtures' norm weights are not all ones, and the
    # per-head norm of q and k changes the logits
    model = _model(tmp_path, "qwen3")
    ids = list(range(10, 30))
    base = model.logits(ids)
    assert float((model.w("model.layers.0.input_layernorm.weight") - 1).abs().max()) > 0.05
    model.config.qk_norm = False
    assert float((model.logits(ids) - base).abs().max()) > 1e-2


def test_a_block_sees_positions_only_as_distances(tmp_path):
    """Keys and queries are normed per head and then rotated, values are not rotated at all: then every
    score depends on the distance between query and key alone, and a block gives the same output when all
    positions are shifted. The head norm after the rotation (its weights differ along the head, so they
    would break the pairs' rotation) or a rotated value fails this."""
    model = _model(tmp_path, "qwen3")
    c = model.config
    p = "model.layers.1.self_attn."
    assert float((model.w(p + "q_norm.weight") - 1).abs().max()) > 0.05         # the fixture's head norms are not ones
    x = torch.randn(9, c.hidden, generator=torch.Generator().manual_seed(4))
    positions = torch.arange(9)
    base = model.block(1, x, positions)
    close(model.block(1, x, positions + 37), base, 1e-5 * float(base.abs().max()))     # float32 angles round differently
    # the guard: the same parts with the norm after the rotation do depend on absolute positions
    def scores_with_norm_last(at):
        normed = P.rmsnorm(x, model.w("model.layers.1.input_layernorm.weight"), c.eps)
        q = P.rope(P.linear(normed, model.w(p + "q_proj.weight")), c.n_heads, c.head_dim, at, c.rope_dim, c.rope_theta)
        k = P.rope(P.linear(normed, model.w(p + "k_proj.weight")), c.n_kv_heads, c.head_dim, at, c.rope_dim, c.rope_theta)
        q = P.head_rmsnorm(q, c.n_heads, c.head_dim, model.w(p + "q_norm.weight"), c.eps)
        k = P.head_rmsnorm(k, c.n_kv_heads, c.head_dim, model.w(p + "k_norm.weight"), c.eps)
        return q[:, :c.head_dim] @ k[:, :c.head_dim].t()
    assert float((scores_with_norm_last(positions) - scores_with_norm_last(positions + 37)).abs().max()) > 1e-3


def test_the_feed_forward_reads_the_stream_after_the_attention_was_added(tmp_path):
    """norm, attention, add, norm, feed-forward, add: with the feed-forward silenced a block returns
    x1 = x + attention; with both live it returns x1 + feed_forward(norm2(x1)). A block whose two halves
    both read the incoming stream (a parallel block), or a norm after the sum, fails this."""
    model = _model(tmp_path, "llama")
    c = model.config
    p = "model.layers.0."
    x = torch.randn(6, c.hidden, generator=torch.Generator().manual_seed(8))
    positions = torch.arange(6)
    both = model.block(0, x, positions)
    kept = model.w(p + "mlp.down_proj.weight").clone()
    model.weights[p + "mlp.down_proj.weight"].zero_()
    x1 = model.block(0, x, positions)
    model.weights[p + "mlp.down_proj.weight"].copy_(kept)
    normed = P.rmsnorm(x1, model.w(p + "post_attention_layernorm.weight"), c.eps)
    want = x1 + P.linear(P.swiglu(P.linear(normed, model.w(p + "mlp.gate_proj.weight")),
                                  P.linear(normed, model.w(p + "mlp.up_proj.weight"))), kept)
    close(both, want, 1e-5)
    parallel = P.rmsnorm(x, model.w(p + "post_attention_layernorm.weight"), c.eps)
    wrong = x1 + P.linear(P.swiglu(P.linear(parallel, model.w(p + "mlp.gate_proj.weight")),
                                   P.linear(parallel, model.w(p + "mlp.up_proj.weight"))), kept)
    assert float((both - wrong).abs().max()) > 1e-2


def test_logits_of_the_last_positions_alone_are_those_of_the_whole(tmp_path):
    for name in ("llama", "qwen3"):
        model = _model(tmp_path, name)
        ids = list(range(20, 61))
        whole = model.logits(ids)
        for tail in (1, 5, len(ids), len(ids) + 3):
            close(model.logits(ids, tail=tail), whole[-tail:], 1e-5)


def test_model_from_tensors_is_the_model_from_the_folder(tmp_path):
    import json, os
    model = _model(tmp_path, "qwen3")
    raw = json.load(open(os.path.join(str(tmp_path / "qwen3"), "config.json")))
    again = P.PlainModel.from_weights(raw, {name: tensor.clone() for name, tensor in model.weights.items()})
    ids = [3, 1, 4, 1, 5, 9, 2, 6]
    assert torch.equal(again.logits(ids), model.logits(ids))


# ---- sampling and the loop -------------------------------------------------------------

def test_greedy_and_penalty_reference_cases():
    # tests/sampler_test.rs:101-127
    assert P.greedy(torch.tensor([-1.0, 0.5, 3.25, 2.0])) == 2
    assert P.greedy(P.apply_repetition_penalty(torch.tensor([1.2, 1.5]), [1], 2.0)) == 0
    assert P.greedy(torch.tensor([1.0, 3.0, 3.0])) == 1                       # ties go to the lowest id
    close(P.apply_repetition_penalty(torch.tensor([-1.0, 2.0]), [0, 1], 2.0), [-2.0, 1.0])
    close(P.apply_repetition_penalty(torch.tensor([-1.0, 2.0]), [0, 1], 1.0), [-1.0, 2.0])


def test_sampling_distribution_reference_cases():
    # tests/sampler_test.rs:24-98
    e = math.exp
    cold = P.sampling_distribution(torch.tensor([2.0, 1.0, 0.0]), 0.5)
    close(cold[0], e(4) / (e(4) + e(2) + 1), 1e-9)
    hot = P.sampling_distribution(torch.tensor([2.0, 1.0, 0.0]), 2.0)
    close(hot[:2], [e(1) / (e(1) + e(0.5) + 1), e(0.5) / (e(1) + e(0.5) + 1)], 1e-9)
    logits = torch.tensor([4.0, 3.0, 2.0, 1.0])
    top2 = P.sampling_distribution(logits, 1.0, top_k=2)
    close(top2, [e(4) / (e(4) + e(3)), e(3) / (e(4) + e(3)), 0, 0], 1e-9)
    nucleus = P.sampling_distribution(logits, 1.0, top_p=0.85)       # p0 + p1 = 0.88 >= 0.85
    close(nucleus, top2, 1e-9)
    close(P.sampling_distribution(logits, 1.0).sum(), 1.0, 1e-12)


def test_generation_loop_stops(tmp_path):
    model = _model(tmp_path, "llama")
    prompt = [4, 8, 15]
    free = P.generate_greedy(model, prompt, 6, stop_ids=[])
    assert len(free) == 6
    stopped = P.generate_greedy(model, prompt, 6, stop_ids=[free[2]])
    assert stopped == free[:free.index(free[2])]            # the stop token is not returned
    with pytest.raises(ValueError):
        P.generate_greedy(model, list(range(200)), 1)        # longer than the context
    model.config.bos_id = None
    with pytest.raises(ValueError):
        P.generate_greedy(model, [], 1)
