"""A stand-in for the HIP kernels, for tests only: each operation of the kernel
library written with elementary torch operations in float32 on whatever device
the tensors are on.

It has two uses. On a machine without a GPU it lets the tests drive the engine's
own step function, cache and generation loop (everything except the kernels). On
the GPU it is the plain reference that each kernel is compared with, alone and at
sizes other than the engine's. The engine itself never falls back to it.

Layout facts it shares with the kernels (they are the contract, not code):
qkv rows are [q heads | k heads | v heads]; a cache block holds BLOCK tokens of
every key/value head, in the order that cache_order.py spells out.
"""
from __future__ import annotations

import math

import torch

import cache_order
from xeno_rt_amd.cache import BLOCK_TOKENS as BLOCK      # the cache's own constant: blocks are its unit


class EmulatedOps:
    name = "emulation"

    # -- elementwise / gather ---------------------------------------------------
    def embed(self, table, ids, out):
        out.copy_(table[ids.long()].to(torch.float32))

    def add(self, residual, delta):
        residual.add_(delta.to(torch.float32))

    def rmsnorm(self, x, weight, eps, out, rows=None):
        src = x if rows is None else x[rows.long()]
        src = src.to(torch.float32)
        inv = 1.0 / torch.sqrt((src * src).sum(-1, keepdim=True) / src.shape[-1] + eps)
        out.copy_(((src * inv) * weight.to(torch.float32)).to(out.dtype))

    # -- products ---------------------------------------------------------------
    # An RMSNorm between two products may be done by the two of them (the kernels do so for steps
    # of few rows): the first returns the updated rows times the gain with their sums of squares,
    # the second divides by the rms.
    norms_between_products = True

    class Prescaled:
        def __init__(self, values, squares, eps):
            self.values, self.squares, self.eps = values, squares, eps
            self.shape = values.shape

    def _rows(self, a):
        if isinstance(a, self.Prescaled):
            inv = 1.0 / torch.sqrt(a.squares / a.values.shape[-1] + a.eps)
            return a.values.to(torch.float32), inv[:, None]
        return a.to(torch.float32), 1.0

    def linear(self, a, w, out, accumulate=False, then_norm=None):
        rows, inv = self._rows(a)
        result = (rows @ w.to(torch.float32).t()) * inv
        if accumulate:
            out.add_(result.to(out.dtype))
        else:
            out.copy_(result.to(out.dtype))
        if then_norm is not None and accumulate and self.norms_between_products:
            gain, eps = then_norm
            fresh = out.to(torch.float32)
            return self.Prescaled((fresh * gain.to(torch.float32)).to(w.dtype), (fresh * fresh).sum(-1), eps)
        return None

    def linear_glu(self, a, w_gate_up, out, activation="silu"):
        assert activation == "silu"
        inter = w_gate_up.shape[0] // 2
        rows, inv = self._rows(a)
        both = (rows @ w_gate_up.to(torch.float32).t()) * inv
        gate, up = both[:, :inter], both[:, inter:]
        out.copy_(((gate / (1.0 + torch.exp(-gate))) * up).to(out.dtype))

    # -- attention --------------------------------------------------------------
    def linear_qkv(self, a, w, qkv, *args, **kwargs):
        self.linear(a, w, qkv)
        self.qkv_prepare(qkv, *args, **kwargs)

    def qkv_prepare(self, qkv, n_heads, n_kv_heads, head_dim, positions, slots,
                    q_norm=None, k_norm=None, norm_eps=0.0, rope_theta=None, rope_dim=0,
                    rope_scale=1.0, kv=None, longest_run=0):
        tokens = qkv.shape[0]
        qw, kw = n_heads * head_dim, n_kv_heads * head_dim
        work = qkv.to(torch.float32)
        q = work[:, :qw].reshape(tokens, n_heads, head_dim).clone()
        k = work[:, qw:qw + kw].reshape(tokens, n_kv_heads, head_dim).clone()
        v = work[:, qw + kw:].reshape(tokens, n_kv_heads, head_dim)
        if q_norm is not None:
            q = q * (1.0 / torch.sqrt((q * q).sum(-1, keepdim=True) / head_dim + norm_eps)) * q_norm.float()
        if k_norm is not None:
            k = k * (1.0 / torch.sqrt((k * k).sum(-1, keepdim=True) / head_dim + norm_eps)) * k_norm.float()
        if rope_theta is not None:
            half = rope_dim // 2
            angle = (positions.to(torch.float32)[:, None] * rope_scale) / rope_theta[None, :].float()
            sin, cos = torch.sin(angle)[:, None, :], torch.cos(angle)[:, None, :]
            for t in (q, k):
                a, b = t[..., :half].clone(), t[..., half:2 * half].clone()
                t[..., :half] = a * cos - b * sin
                t[..., half:2 * half] = a * sin + b * cos
        qkv[:, :qw] = q.reshape(tokens, qw).to(qkv.dtype)
        qkv[:, qw:qw + kw] = k.reshape(tokens, kw).to(qkv.dtype)
        if kv is not None:
            table = kv.block_table
            for t in range(tokens):
                slot = int(slots[t])
                if slot < 0:
                    continue
                pos = int(positions[t])
                block = int(table[slot, pos // BLOCK])
                assert block >= 0, "write into a block that the sequence does not hold"
                cache_order.write_key(kv.k, block, pos % BLOCK, qkv[t, qw:qw + kw].reshape(n_kv_heads, head_dim))
                cache_order.write_value(kv.v, block, pos % BLOCK, v[t])

    def attention(self, qkv, n_heads, n_kv_heads, head_dim, kv, batch, out, scale, window=None, distance_slopes=None):
        tokens = qkv.shape[0]
        group = n_heads // n_kv_heads
        q = qkv[:, :n_heads * head_dim].to(torch.float32).reshape(tokens, n_heads, head_dim)
        table = kv.block_table
        for t in range(tokens):
            slot = int(batch.slots[t])
            if slot < 0:
                out[t] = 0
                continue
            pos = int(batch.positions[t])
            first = 0 if window is None else max(0, pos - window + 1)
            index = torch.arange(first, pos + 1)
            blocks = table[slot, (index // BLOCK).to(table.device)].long()
            assert int(blocks.min()) >= 0, "read from a block that the sequence does not hold"
            within = (index % BLOCK).to(blocks.device)
            keys = cache_order.read_keys(kv.k, blocks, within).to(torch.float32)        # [n, kv_heads, dim]
            values = cache_order.read_values(kv.v, blocks, within).to(torch.float32)    # [n, kv_heads, dim]
            for head in range(n_heads):
                kvh = head // group
                scores = (keys[:, kvh, :] @ q[t, head]) * scale
                if distance_slopes is not None:
                    scores = scores + float(distance_slopes[head]) * (index - pos).to(torch.float32)
                probs = torch.softmax(scores, dim=0)
                out[t, head * head_dim:(head + 1) * head_dim] = (probs @ values[:, kvh, :]).to(out.dtype)

    # -- sampling ---------------------------------------------------------------
    def sample(self, logits, out, temperature, top_k, top_p, penalty, history, history_spans, uniforms,
               small_top_k=False, append_at=None):
        rows, vocab = logits.shape
        for r in range(rows):
            self._sample_row(r, logits, out, temperature, top_k, top_p, penalty, history, history_spans, uniforms)
            if append_at is not None and int(append_at[r]) >= 0:
                history[int(append_at[r])] = out[r]

    def _sample_row(self, r, logits, out, temperature, top_k, top_p, penalty, history, history_spans, uniforms):
        vocab = logits.shape[1]
        for _ in range(1):
            row = logits[r].to(torch.float32).clone()
            seen = history[int(history_spans[2 * r]):int(history_spans[2 * r + 1])].long()
            pen = float(penalty[r])
            if pen > 1.0 and seen.numel() > 0:
                seen = torch.unique(seen)
                vals = row[seen]
                row[seen] = torch.where(vals > 0, vals / pen, vals * pen)
            temp = float(temperature[r])
            if temp <= 1e-5:
                out[r] = int(torch.argmax(row))        # first index of the maximum
                continue
            k = int(top_k[r]) if int(top_k[r]) > 0 else vocab
            keep = torch.ones(vocab, dtype=torch.bool, device=row.device)
            if k < vocab:
                kth = torch.topk(row, k).values[-1]
                keep = row >= kth
            weights = torch.where(keep, torch.exp((row - row.max()) / temp), torch.zeros_like(row))
            p = float(top_p[r])
            if p < 1.0:
                total = weights.sum()
                order = torch.argsort(weights, descending=True, stable=True)
                cumulative = torch.cumsum(weights[order], 0)
                cut = int((cumulative >= p * total).nonzero()[0]) + 1
                threshold = weights[order[cut - 1]]
                weights = torch.where(weights >= threshold, weights, torch.zeros_like(weights))
            cumulative = torch.cumsum(weights, 0)
            target = float(uniforms[r]) * float(cumulative[-1])
            pick = int((cumulative > target).nonzero()[0]) if bool((cumulative > target).any()) else int(torch.argmax(weights))
            out[r] = pick
