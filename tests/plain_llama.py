"""Plain, slow implementation of the Llama / Qwen3 dense decoder.

Whole sequences, no cache, one function for each part, written from the
formulas of the reference (cited as file:line of the reference's own tree). It
shares no code with the engine: it reads the model folder with the
`safetensors` package and `json`, and computes with elementary torch tensor
operations on the CPU (float32 by default, float64 on request).
"""
from __future__ import annotations

import json
import math
import os

import torch


# ----------------------------------------------------------------------------
# parts
# ----------------------------------------------------------------------------

def rmsnorm(x: torch.Tensor, weight: torch.Tensor, eps: float) -> torch.Tensor:
    """y_i = (x_i * r) * w_i with r = 1/sqrt(mean(x^2) + eps), over the last axis.

    crates/xrt-kernels/src/cpu/rmsnorm.rs:26-32 (mean square, inverse root)
    and :43 (product order); the weight is used as it is, not as 1+w.
    """
    mean_square = (x * x).sum(dim=-1, keepdim=True) / x.shape[-1]
    inv_rms = 1.0 / torch.sqrt(mean_square + eps)
    return (x * inv_rms) * weight


def head_rmsnorm(x: torch.Tensor, n_heads: int, head_dim: int, weight: torch.Tensor,
                 eps: float) -> torch.Tensor:
    """RMSNorm of every head slice of width head_dim, one weight [head_dim] for all heads.

    crates/xrt-models/src/llama.rs:1025-1040.
    """
    tokens = x.shape[0]
    heads = x.reshape(tokens, n_heads, head_dim)
    sum_sq = (heads * heads).sum(dim=-1, keepdim=True)
    inv_rms = 1.0 / torch.sqrt(sum_sq / head_dim + eps)
    return (heads * inv_rms * weight).reshape(tokens, n_heads * head_dim)


def rope_inverse_frequencies(rope_dim: int, base: float, dtype=torch.float32) -> torch.Tensor:
    """theta_i = base^(2i/rope_dim) for i in [0, rope_dim/2).

    crates/xrt-kernels/src/cpu/rope.rs:10-16 (the table holds theta, the angle
    divides by it). Computed in float32 like the reference's powf.
    """
    half = rope_dim // 2
    pair = torch.arange(half, dtype=torch.float32)
    theta = torch.tensor(base, dtype=torch.float32) ** ((2.0 * pair) / float(rope_dim))
    return theta.to(dtype)


def rope(x: torch.Tensor, n_heads: int, head_dim: int, positions: torch.Tensor,
         rope_dim: int, base: float, scale: float = 1.0) -> torch.Tensor:
    """Rotate pairs (i, i+half) of every head by angle = pos*scale/theta_i.

    crates/xrt-kernels/src/cpu/rope.rs:59-68 (angle) and :71-89 (rotation:
    d[i] = a*cos - b*sin, d[i+half] = a*sin + b*cos). Elements beyond
    rope_dim are left as they are.
    """
    tokens = x.shape[0]
    rotary = min(rope_dim, head_dim)
    half = rotary // 2
    theta = rope_inverse_frequencies(rotary, base, dtype=torch.float32)
    angle = (positions.to(torch.float32)[:, None] * scale) / theta[None, :]
    sin = torch.sin(angle).to(x.dtype)[:, None, :]
    cos = torch.cos(angle).to(x.dtype)[:, None, :]
    heads = x.reshape(tokens, n_heads, head_dim).clone()
    a = heads[:, :, :half].clone()
    b = heads[:, :, half:2 * half].clone()
    heads[:, :, :half] = a * cos - b * sin
    heads[:, :, half:2 * half] = a * sin + b * cos
    return heads.reshape(tokens, n_heads * head_dim)


def softmax(scores: torch.Tensor) -> torch.Tensor:
    """exp(x - max) / sum over the last axis.

    crates/xrt-kernels/src/cpu/softmax.rs:14-109.
    """
    shifted = scores - scores.max(dim=-1, keepdim=True).values
    e = torch.exp(shifted)
    return e / e.sum(dim=-1, keepdim=True)


def silu(x: torch.Tensor) -> torch.Tensor:
    """x / (1 + exp(-x)).  crates/xrt-kernels/src/cpu/silu.rs:1-3."""
    return x / (1.0 + torch.exp(-x))


def swiglu(gate: torch.Tensor, up: torch.Tensor) -> torch.Tensor:
    """silu(gate) * up.  crates/xrt-kernels/src/cpu/silu.rs:22-24."""
    return silu(gate) * up


def linear(x: torch.Tensor, weight: torch.Tensor) -> torch.Tensor:
    """out[t, r] = sum_c W[r, c] * x[t, c]; W is [out][in], no bias.

    crates/xrt-kernels/src/cpu/matmul.rs:153-167 (row-major matvec).
    """
    return x @ weight.t()


def causal_attention(q: torch.Tensor, k: torch.Tensor, v: torch.Tensor, n_heads: int,
                     n_kv_heads: int, head_dim: int, start_position: int = 0) -> torch.Tensor:
    """Causal attention of one sequence with grouped KV heads.

    q is [T, n_heads*head_dim] for the tokens at positions start_position..,
    k and v are [start_position+T, n_kv_heads*head_dim] for all positions.
    Query head h reads KV head h // (n_heads // n_kv_heads); the token at
    absolute position P sees keys 0..P inclusive; scale 1/sqrt(head_dim).
    crates/xrt-models/src/llama.rs:727-770 (prefill) and :504-574 (decode).
    """
    tokens = q.shape[0]
    group = n_heads // n_kv_heads
    scale = 1.0 / math.sqrt(head_dim)
    qh = q.reshape(tokens, n_heads, head_dim)
    kh = k.reshape(k.shape[0], n_kv_heads, head_dim)
    vh = v.reshape(v.shape[0], n_kv_heads, head_dim)
    out = torch.zeros_like(qh)
    # attend_len = start_position + t + 1 (llama.rs:736): key j is hidden from query t if j > start_position + t
    hidden = torch.arange(k.shape[0])[None, :] > (start_position + torch.arange(tokens))[:, None]
    for head in range(n_heads):
        kv_head = head // group                                  # llama.rs:741
        scores = (qh[:, head, :] @ kh[:, kv_head, :].t()) * scale            # :744-751, all queries of the head at once
        probs = softmax(scores.masked_fill(hidden, -math.inf))   # :753 over the keys each query sees
        out[:, head, :] = probs @ vh[:, kv_head, :]              # :756-768
    return out.reshape(tokens, n_heads * head_dim)


# ----------------------------------------------------------------------------
# model folder
# ----------------------------------------------------------------------------

class PlainConfig:
    """The numbers of config.json that the formulas need (llama.rs:24-137)."""

    def __init__(self, raw: dict):
        self.architecture = raw["architectures"][0]
        self.vocab_size = int(raw["vocab_size"])
        self.hidden = int(raw["hidden_size"])
        self.intermediate = int(raw["intermediate_size"])
        self.layers = int(raw["num_hidden_layers"])
        self.n_heads = int(raw["num_attention_heads"])
        self.n_kv_heads = int(raw.get("num_key_value_heads", self.n_heads))    # llama.rs:68-70
        self.head_dim = int(raw.get("head_dim") or self.hidden // self.n_heads)  # llama.rs:125-128
        self.eps = float(raw.get("rms_norm_eps", 1e-5))                        # llama.rs:95-98
        self.rope_theta = float(raw.get("rope_theta", 10000.0))                # llama.rs:99-102
        # llama.rs:92-94 (dims of a head that are rotated) and :103-106 (what multiplies a position, rope.rs:25); in a
        # config.json a share of the head and a linear rule whose factor divides the positions
        rule = raw.get("rope_scaling") or {}
        self.rope_dim = int(self.head_dim * float(raw.get("partial_rotary_factor") or 1.0))
        self.rope_scale = 1.0 / float(rule["factor"]) if rule.get("rope_type", rule.get("type")) == "linear" else 1.0
        self.tied = bool(raw.get("tie_word_embeddings", False))
        self.qk_norm = self.architecture == "Qwen3ForCausalLM"
        self.max_position = int(raw["max_position_embeddings"])
        eos = raw.get("eos_token_id")
        self.eos_ids = [] if eos is None else ([int(e) for e in eos] if isinstance(eos, list) else [int(eos)])
        self.bos_id = raw.get("bos_token_id")


class PlainModel:
    """Weights of a model folder as float tensors on the CPU, by checkpoint name."""

    def __init__(self, folder: str, dtype=torch.float32):
        from safetensors import safe_open

        with open(os.path.join(folder, "config.json")) as handle:
            self.config = PlainConfig(json.load(handle))
        self.dtype = dtype
        self.weights = {}
        with safe_open(os.path.join(folder, "model.safetensors"), framework="pt") as handle:
            for name in handle.keys():
                self.weights[name] = handle.get_tensor(name).to(dtype)

    @classmethod
    def from_weights(cls, raw_config: dict, weights: dict, dtype=torch.float32) -> "PlainModel":
        """From config.json's contents and tensors by checkpoint name (any float type)."""
        model = cls.__new__(cls)
        model.config = PlainConfig(raw_config)
        model.dtype = dtype
        model.weights = {name: tensor.to(dtype) for name, tensor in weights.items()}
        return model

    def w(self, name: str) -> torch.Tensor:
        return self.weights[name]

    # -- one block: norm -> attention -> add -> norm -> feed-forward -> add ----
    def block(self, layer: int, x: torch.Tensor, positions: torch.Tensor, tail: int = 0) -> torch.Tensor:
        """crates/xrt-models/src/llama.rs:433-602 (decode) / 676-810 (prefill).

        With tail = n only the last n positions are returned: keys and values are made for every
        position, queries and everything after the attention only for those n (what the reference's
        decode step computes for one position, llama.rs:447-602, against the keys before it)."""
        c = self.config
        p = f"model.layers.{layer}."
        first = x.shape[0] - tail if tail else 0
        normed = rmsnorm(x, self.w(p + "input_layernorm.weight"), c.eps)           # :441-442
        q = linear(normed[first:], self.w(p + "self_attn.q_proj.weight"))         # :447-486
        k = linear(normed, self.w(p + "self_attn.k_proj.weight"))
        v = linear(normed, self.w(p + "self_attn.v_proj.weight"))
        if c.qk_norm:                                                              # :489-496
            q = head_rmsnorm(q, c.n_heads, c.head_dim, self.w(p + "self_attn.q_norm.weight"), c.eps)
            k = head_rmsnorm(k, c.n_kv_heads, c.head_dim, self.w(p + "self_attn.k_norm.weight"), c.eps)
        q = rope(q, c.n_heads, c.head_dim, positions[first:], c.rope_dim, c.rope_theta, c.rope_scale)    # :498-500
        k = rope(k, c.n_kv_heads, c.head_dim, positions, c.rope_dim, c.rope_theta, c.rope_scale)
        attn = causal_attention(q, k, v, c.n_heads, c.n_kv_heads, c.head_dim, start_position=first)   # :504-574
        x = x[first:] + linear(attn, self.w(p + "self_attn.o_proj.weight"))       # :576-577
        normed = rmsnorm(x, self.w(p + "post_attention_layernorm.weight"), c.eps)  # :579-580
        gate = linear(normed, self.w(p + "mlp.gate_proj.weight"))                 # :584-598
        up = linear(normed, self.w(p + "mlp.up_proj.weight"))
        x = x + linear(swiglu(gate, up), self.w(p + "mlp.down_proj.weight"))      # :599-601
        return x

    def logits(self, token_ids, tail: int = 0) -> torch.Tensor:
        """Logits [T, V] at every position of one whole sequence, positions 0..T-1; with tail = n only
        at the last n positions (the layers before the last still run every position: their outputs
        make the next layer's keys and values).

        crates/xrt-models/src/llama.rs:830-1009 (forward_batch_all_logits).
        """
        c = self.config
        ids = torch.as_tensor(list(token_ids), dtype=torch.long)
        if ids.numel() == 0:
            raise ValueError("empty sequence")                                    # :624-626
        if int(ids.max()) >= c.vocab_size or int(ids.min()) < 0:
            raise ValueError("token id exceeds embedding rows")                   # :1044-1049
        positions = torch.arange(ids.numel())
        x = self.w("model.embed_tokens.weight")[ids]                              # :666-669
        tail = min(int(tail), ids.numel())
        for layer in range(c.layers):
            x = self.block(layer, x, positions, tail=tail if layer == c.layers - 1 else 0)
        normed = rmsnorm(x, self.w("model.norm.weight"), c.eps)                   # :604-609
        head = self.w("model.embed_tokens.weight") if c.tied else self.w("lm_head.weight")  # :301-305
        return linear(normed, head)                                               # :613


# ----------------------------------------------------------------------------
# sampling and the generation loop
# ----------------------------------------------------------------------------

def apply_repetition_penalty(logits: torch.Tensor, history, penalty: float) -> torch.Tensor:
    """logit > 0 ? logit / pen : logit * pen for ids in history; only if pen > 1.

    crates/xrt-runtime/src/sampler.rs:77-91 and :110-125.
    """
    out = logits.clone()
    if penalty > 1.0 and len(history) > 0:
        for token in set(int(t) for t in history):
            value = out[token]
            out[token] = value / penalty if value > 0 else value * penalty
    return out


def greedy(logits: torch.Tensor) -> int:
    """First index of the maximum (strict >, ties to the lowest id).

    crates/xrt-runtime/src/sampler.rs:83-98.
    """
    best, best_value = 0, -math.inf
    for index, value in enumerate(logits.tolist()):
        if value > best_value:
            best, best_value = index, value
    return best


def sampling_distribution(logits: torch.Tensor, temperature: float, top_k: int = 0,
                          top_p: float = 1.0) -> torch.Tensor:
    """Probability of every token id under temperature / top-k / top-p.

    crates/xrt-runtime/src/sampler.rs:107-183: keep the k largest (0 = all),
    softmax of (logit - max)/T over them, keep the shortest descending prefix
    whose cumulative probability reaches top_p, renormalise.
    """
    vocab = logits.numel()
    k = top_k if top_k > 0 else vocab
    order = sorted(range(vocab), key=lambda i: (-float(logits[i]), i))[:k]
    kept = torch.tensor([float(logits[i]) for i in order], dtype=torch.float64)
    probs = torch.exp((kept - kept[0]) / temperature)
    probs = probs / probs.sum()
    keep = len(order)
    if top_p < 1.0:
        cumulative = 0.0
        for i, p in enumerate(probs.tolist()):
            cumulative += p
            if cumulative >= top_p:
                keep = i + 1
                break
        probs = probs[:keep] / probs[:keep].sum()
    dist = torch.zeros(vocab, dtype=torch.float64)
    for i in range(keep):
        dist[order[i]] = probs[i]
    return dist


def generate_greedy(model: PlainModel, prompt, max_tokens: int, stop_ids=None,
                    repetition_penalty: float = 1.0):
    """The reference's loop for one request with greedy sampling and no cache.

    crates/xrt-runtime/src/session.rs:69-141: sample from the last logits;
    a stop token ends the request and is neither stored nor returned; a full
    context ends it; otherwise the token is stored and run.
    """
    c = model.config
    stops = set(c.eos_ids if stop_ids is None else stop_ids)
    tokens = list(prompt)
    if not tokens:                                                                # :78-86
        if c.bos_id is None:
            raise ValueError("empty prompt and no BOS token")
        tokens = [int(c.bos_id)]
    if len(tokens) > c.max_position:                                              # :87-93
        raise ValueError("prompt longer than the context")
    produced = []
    while len(produced) < max_tokens:                                             # :115
        last = model.logits(tokens)[-1]
        nxt = greedy(apply_repetition_penalty(last, tokens, repetition_penalty))  # :116
        if nxt in stops:                                                          # :117-119
            break
        if len(tokens) >= c.max_position:                                         # :120-122
            break
        tokens.append(nxt)                                                        # :124
        produced.append(nxt)
    return produced
