"""Each part alone on the GPU against the plain function of the same name, and the proof
that the framework takes parts it has never seen: a toy mixer with state of its own, a toy
position encoding and a schedule that runs a layer twice and shares a cache, all defined
here, registered, built and stepped without touching the framework's files."""
import math

import pytest
import torch

import plain_llama as P
from helpers import assert_logits, run_tail_decoded, run_whole, token_ids

pytestmark = pytest.mark.gpu
DEV = "cuda:0"
DT = {"float32": torch.float32, "bfloat16": torch.bfloat16}
TOL = {"float32": 2e-5, "bfloat16": 2e-2}


def runtime(dtype):
    from xeno_rt_amd.ops import load_ops
    from xeno_rt_amd.parts import Runtime
    return Runtime(load_ops(), DT[dtype], DEV)


def weights_for(part, seed, dtype=torch.bfloat16, std=0.3):
    out = {}
    g = torch.Generator().manual_seed(seed)
    for name, spec in part.weight_specs().items():
        base = 1.0 if spec.init == "ones" else 0.0
        out[name] = (base + std * torch.randn(spec.shape, generator=g)).to(dtype)
    return out


def rel(got, want):
    return float((got.double().cpu() - want.double()).abs().max()) / float(want.double().abs().max())


def batch_for(cache, slots, counts):
    from xeno_rt_amd.engine.batch import build_batch
    starts = [cache.length(s) for s in slots]
    for s, n, c in zip(slots, starts, counts):
        cache.reserve(s, n + c)
    cache.sync()
    batch = build_batch(slots, [[0] * c for c in counts], starts, [[] for _ in slots], DEV)
    return batch, starts


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_rmsnorm_part(dtype):
    from xeno_rt_amd.parts import RMSNorm
    part = RMSNorm("n.", 200, 1e-4)
    w = weights_for(part, 1)
    part.bind(w, runtime(dtype))
    x = torch.randn(6, 200, device=DEV) * 4
    want = P.rmsnorm(x.cpu().double(), w["n.weight"].double(), 1e-4)
    assert rel(part.forward(x), want) < TOL[dtype]
    rows = torch.tensor([5, 2], dtype=torch.int32, device=DEV)
    assert rel(part.forward(x, rows=rows), want[[5, 2]]) < TOL[dtype]
    # a weight stored in 32-bit stays 32-bit, on the bfloat16 path too
    part.bind({"n.weight": w["n.weight"].float() + 1e-4}, runtime(dtype))
    assert part.weight.dtype == torch.float32


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_gated_mlp_part(dtype):
    from xeno_rt_amd.parts import GatedMLP
    part = GatedMLP("m.", 96, 176)
    w = weights_for(part, 2)
    rt = runtime(dtype)
    part.bind(w, rt)
    h = (torch.randn(5, 96) * 2).to(DT[dtype])
    residual = torch.randn(5, 96, device=DEV)
    start = residual.clone()
    part.forward(h.to(DEV), None, residual)
    hd = h.double()
    want = P.linear(P.swiglu(P.linear(hd, w["m.gate_proj.weight"].double()), P.linear(hd, w["m.up_proj.weight"].double())),
                    w["m.down_proj.weight"].double())
    assert rel(residual - start, want) < TOL[dtype]
    with pytest.raises(ValueError, match="activation"):
        GatedMLP("m.", 8, 8, activation="gelu")


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("nh,nkv,hd,qk_norm,table", [(4, 2, 16, False, 0), (6, 3, 32, True, 0), (8, 8, 64, True, 0), (8, 1, 128, False, 0),
                                                     (8, 8, 64, True, 140), (6, 2, 128, True, 1000), (6, 3, 32, True, 1000)])
def test_attention_part_prompt_then_decode(dtype, nh, nkv, hd, qk_norm, table):
    """The mixer with its cache: a prompt in one step, then single tokens, two sequences of
    unequal lengths; compared with plain attention over the whole sequences. table: positions whose cosines and sines
    the rotation keeps: with them the attention of a bfloat16 decode step with head norms finishes q, k and v itself,
    as long as the table covers the step (140: the longer sequence's last steps lie beyond it and take the two kernels)."""
    from xeno_rt_amd.cache import SequenceCache
    from xeno_rt_amd.parts import Attention, Rotary
    hidden = 72
    part = Attention("a.", hidden, nh, nkv, hd, position=Rotary(hd, 7000.0, table_positions=table), qk_norm=qk_norm, qk_norm_eps=1e-5)
    # scores come out with a spread of about two: sharp attention, not a saturated one
    w = weights_for(part, 3, std=0.15)
    rt = runtime(dtype)
    part.bind(w, rt)
    cache = SequenceCache([part.cache_needs()], [0], 512, 2, 256, DT[dtype], DEV)
    lengths = [150, 70]
    hs = [torch.randn(n, hidden, generator=torch.Generator().manual_seed(n)).to(DT[dtype]) for n in lengths]

    def plain(h):
        x = h.double()
        pos = torch.arange(x.shape[0])
        q, k, v = (P.linear(x, w[f"a.{n}_proj.weight"].double()) for n in "qkv")
        if qk_norm:
            q = P.head_rmsnorm(q, nh, hd, w["a.q_norm.weight"].double(), 1e-5)
            k = P.head_rmsnorm(k, nkv, hd, w["a.k_norm.weight"].double(), 1e-5)
        q, k = P.rope(q, nh, hd, pos, hd, 7000.0), P.rope(k, nkv, hd, pos, hd, 7000.0)
        return P.linear(P.causal_attention(q, k, v, nh, nkv, hd), w["a.o_proj.weight"].double())

    want = [plain(h) for h in hs]
    slots = [cache.alloc_slot(), cache.alloc_slot()]
    got = [[], []]
    prompts = [130, 1]
    batch, starts = batch_for(cache, slots, prompts)
    residual = torch.zeros(sum(prompts), hidden, device=DEV)
    part.forward(torch.cat([hs[0][:130], hs[1][:1]]).to(DEV), batch, cache.layer_cache(0), residual)
    got[0].append(residual[:130]); got[1].append(residual[130:])
    for s, c in zip(slots, prompts):
        cache.commit(s, c)
    at = list(prompts)
    finished_here = []
    while any(a < n for a, n in zip(at, lengths)):
        live = [i for i in range(2) if at[i] < lengths[i]]
        batch, _ = batch_for(cache, [slots[i] for i in live], [1] * len(live))
        residual = torch.zeros(len(live), hidden, device=DEV)
        finished_here.append((batch.max_context, bool(qk_norm and rt.ops.attention_finishes_qkv(DT[dtype], nh, nkv, hd, batch, None, hd, part.position.table))))
        part.forward(torch.stack([hs[i][at[i]] for i in live]).to(DEV), batch, cache.layer_cache(0), residual)
        for row, i in enumerate(live):
            got[i].append(residual[row:row + 1].clone())
            at[i] += 1
            cache.commit(slots[i], at[i])
    for i in range(2):
        assert rel(torch.cat(got[i]), want[i]) < TOL[dtype], i
    assert part.scale == 1.0 / math.sqrt(hd)
    # which steps the one kernel took: those that the table covers
    takes = dtype == "bfloat16" and qk_norm and table > 0 and hd in (64, 128)
    assert [took for _, took in finished_here] == [takes and longest <= table for longest, _ in finished_here]
    assert [longest for longest, _ in finished_here][:20] == list(range(131, 151))


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
@pytest.mark.parametrize("hidden,nh,nkv,hd,rope_dim", [(4096, 32, 8, 128, 128), (96, 4, 2, 32, 16)])
def test_a_rotation_defined_here_takes_the_fused_path_without_being_the_library_s_rotary(dtype, hidden, nh, nkv, hd, rope_dim):
    """An encoding of this file that rotates half-split pairs by angles from a table of its own (no power law) says so
    with `rotation()`; the attention part then packs the projection for it and lets the projection's kernel rotate,
    knowing nothing of the class. A prompt of 20 tokens, then 8 single tokens (at the first sizes: the packed product
    with the rotation and the cache write in its epilogue), against plain arithmetic."""
    from xeno_rt_amd.cache import SequenceCache
    from xeno_rt_amd.parts import Attention
    from xeno_rt_amd.parts.base import HalfSplitRotation, PositionEncoding

    class TableRotation(PositionEncoding):
        capturable = True

        def __init__(self, rope_dim, scale):
            self.rope_dim, self.scale = rope_dim, scale
            self.table = 1.0 + 3.0 * torch.arange(rope_dim // 2, dtype=torch.float32) ** 1.5

        def bind(self, tensors, runtime):
            super().bind(tensors, runtime)
            self.theta = self.table.to(runtime.device)

        def rotation(self):
            return HalfSplitRotation(self.rope_dim, self.scale, self.theta)

        def apply(self, qkv, n_heads, n_kv_heads, head_dim, batch):
            raise AssertionError("a rotation that describes itself is done by the projection's kernel")

    position = TableRotation(rope_dim, 0.5)
    part = Attention("a.", hidden, nh, nkv, hd, position=position)
    w = weights_for(part, 3, std=1.5 / math.sqrt(hidden))
    rt = runtime(dtype)
    part.bind(w, rt)
    if dtype == "bfloat16" and hidden == 4096:
        assert hasattr(part.w_qkv, "unpacked") and part.w_qkv.packing.rotated_heads == nh + nkv      # the pairs side by side
    length, prompt = 28, 20
    h = torch.randn(length, hidden, generator=torch.Generator().manual_seed(8)).to(DT[dtype])

    def rotate(x, heads):
        x = x.reshape(length, heads, hd).clone()
        angle = (torch.arange(length, dtype=torch.float32)[:, None] * 0.5 / position.table[None, :]).double()
        a, b = x[:, :, :rope_dim // 2].clone(), x[:, :, rope_dim // 2:rope_dim].clone()
        x[:, :, :rope_dim // 2] = a * angle.cos()[:, None] - b * angle.sin()[:, None]
        x[:, :, rope_dim // 2:rope_dim] = a * angle.sin()[:, None] + b * angle.cos()[:, None]
        return x.reshape(length, heads * hd)

    q, k, v = (P.linear(h.double(), w[f"a.{n}_proj.weight"].double()) for n in "qkv")
    want = P.linear(P.causal_attention(rotate(q, nh), rotate(k, nkv), v, nh, nkv, hd), w["a.o_proj.weight"].double())
    cache = SequenceCache([part.cache_needs()], [0], 128, 1, 128, DT[dtype], DEV)
    slot = cache.alloc_slot()
    got = []
    for first, count in [(0, prompt)] + [(t, 1) for t in range(prompt, length)]:
        batch, _ = batch_for(cache, [slot], [count])
        residual = torch.zeros(count, hidden, device=DEV)
        part.forward(h[first:first + count].to(DEV), batch, cache.layer_cache(0), residual)
        got.append(residual)
        cache.commit(slot, first + count)
    assert rel(torch.cat(got), want) < TOL[dtype]


def attention_with_scores_biased_by_distance(rt, dtype, device):
    """A position encoding defined here, which leaves q and k alone and lowers the scores of far keys instead
    (one slope per head): the attention part hands its slopes to the kernel. A prompt, then single tokens.
    Returns (what the part added to the residual, the same by plain arithmetic, the same without the slopes)."""
    from xeno_rt_amd.cache import SequenceCache
    from xeno_rt_amd.parts import Attention
    from xeno_rt_amd.parts.base import PositionEncoding

    class DistanceBias(PositionEncoding):
        capturable = True

        def __init__(self, n_heads):
            self.values = [2.0 ** -(h + 2) for h in range(n_heads)]

        def bind(self, tensors, runtime):
            super().bind(tensors, runtime)
            self.slopes = torch.tensor(self.values, dtype=torch.float32, device=runtime.device)

        def apply(self, qkv, n_heads, n_kv_heads, head_dim, batch):
            return None

        def score_slopes(self):
            return self.slopes

    hidden, nh, nkv, hd, length, prompt = 80, 4, 2, 128, 100, 70
    part = Attention("a.", hidden, nh, nkv, hd, position=DistanceBias(nh))
    w = weights_for(part, 5, std=0.15)
    part.bind(w, rt)
    cache = SequenceCache([part.cache_needs()], [0], 256, 1, 128, DT[dtype], device)
    h = torch.randn(length, hidden, generator=torch.Generator().manual_seed(4)).to(DT[dtype])
    x = h.double()
    q, k, v = (P.linear(x, w[f"a.{n}_proj.weight"].double()) for n in "qkv")
    distance = torch.arange(length, dtype=torch.float64)[None, :] - torch.arange(length, dtype=torch.float64)[:, None]
    mixed = torch.empty(length, nh * hd, dtype=torch.float64)
    for head in range(nh):
        kv_head = head // (nh // nkv)
        scores = q[:, head * hd:(head + 1) * hd] @ k[:, kv_head * hd:(kv_head + 1) * hd].T / math.sqrt(hd)
        scores = scores + part.position.values[head] * distance
        scores = scores.masked_fill(distance > 0, -float("inf"))
        mixed[:, head * hd:(head + 1) * hd] = torch.softmax(scores, dim=1) @ v[:, kv_head * hd:(kv_head + 1) * hd]
    want = P.linear(mixed, w["a.o_proj.weight"].double())
    unbiased = P.linear(P.causal_attention(q, k, v, nh, nkv, hd), w["a.o_proj.weight"].double())
    slot = cache.alloc_slot()
    got = []
    at = 0
    for count in [prompt] + [1] * (length - prompt):
        from xeno_rt_amd.engine.batch import build_batch
        cache.reserve(slot, at + count)
        cache.sync()
        batch = build_batch([slot], [[0] * count], [at], [[]], device)
        residual = torch.zeros(count, hidden, device=device)
        part.forward(h[at:at + count].to(device), batch, cache.layer_cache(0), residual)
        got.append(residual.clone())
        at += count
        cache.commit(slot, at)
    return torch.cat(got), want, unbiased


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_attention_part_with_a_position_encoding_on_the_scores(dtype):
    got, want, unbiased = attention_with_scores_biased_by_distance(runtime(dtype), dtype, DEV)
    assert rel(got, want) < TOL[dtype]
    assert rel(unbiased, want) > 10 * TOL[dtype]                # the slopes do change the result


def test_parts_are_found_by_kind_and_name():
    from xeno_rt_amd.parts import create_part, registered_parts, RMSNorm, Rotary
    assert "attention" in registered_parts("mixer") and "gated_mlp" in registered_parts("feed_forward")
    assert isinstance(create_part("norm", "rmsnorm", prefix="x.", dim=8, eps=1e-5), RMSNorm)
    assert isinstance(create_part("position", "rotary", rope_dim=8, base=10.0), Rotary)
    with pytest.raises(KeyError, match="no mixer named"):
        create_part("mixer", "nonesuch")
    assert create_part("mixer", "attention", prefix="a.", hidden=8, n_heads=2, n_kv_heads=1, head_dim=20).head_dim == 20
    with pytest.raises(ValueError, match="even"):
        create_part("mixer", "attention", prefix="a.", hidden=8, n_heads=2, n_kv_heads=1, head_dim=21)
    with pytest.raises(ValueError, match="multiple"):
        create_part("mixer", "attention", prefix="a.", hidden=8, n_heads=3, n_kv_heads=2, head_dim=16)


# ----------------------------------------------------------------------------------------------
# a toy architecture made of parts that exist only in this file
# ----------------------------------------------------------------------------------------------

def define_toy():
    from dataclasses import dataclass
    from xeno_rt_amd.config import register_architecture
    from xeno_rt_amd.models import LayerCall, ModelSpec
    from xeno_rt_amd.parts import (Attention, CacheNeeds, Embedding, FeedForward, GatedMLP, Mixer, OutputHead,
                                   PositionEncoding, PreNormBlock, RMSNorm, StateSpec, WeightSpec,
                                   register_part)

    class DecayMixer(Mixer):
        """out_t = W (s_t), s_t = decay * s_{t-1} + h_t: a running state of fixed size per
        sequence, kept in the cache's state area, updated token by token in sequence order."""

        def __init__(self, prefix, hidden, decay):
            self.prefix, self.hidden, self.decay = prefix, hidden, decay

        def weight_specs(self):
            return {self.prefix + "mix.weight": WeightSpec((self.hidden, self.hidden))}

        def cache_needs(self):
            return CacheNeeds(state=StateSpec((self.hidden,), torch.float32))

        def bind(self, tensors, runtime):
            super().bind(tensors, runtime)
            self.weight = runtime.matrix(tensors[self.prefix + "mix.weight"])

        def forward(self, h, batch, cache, residual):
            rt = self.runtime
            states = torch.empty(h.shape[0], self.hidden, dtype=torch.float32, device=h.device)
            at = 0
            for slot, count in zip(batch.host_slots, batch.host_counts):
                s = cache.state[slot]
                for t in range(at, at + count):
                    s.mul_(self.decay).add_(h[t].float())
                    states[t] = s
                at += count
            out = rt.empty((h.shape[0], self.hidden), torch.float32)
            rt.ops.linear(states.to(rt.dtype), self.weight, out)
            rt.ops.add(residual, out)

    class ShiftPosition(PositionEncoding):
        """Adds pos * step to the first element of every q and k head: not a rotation, so the
        attention part must take its general path (norms, this, then the cache write)."""

        def __init__(self, step):
            self.step = step

        def apply(self, qkv, n_heads, n_kv_heads, head_dim, batch):
            bump = (batch.positions.float() * self.step).to(qkv.dtype)
            for head in range(n_heads + n_kv_heads):
                qkv[:, head * head_dim] += bump

    class MixtureMLP(FeedForward):
        """Several gated MLPs, each weighted by the softmax of a router's logits (float32): a
        feed-forward made of the framework's own part, several times, behind a router. Every expert
        gets every token, so that a rounding error cannot flip a choice and the comparison with
        the plain model stays one of tolerances."""

        def __init__(self, prefix, hidden, inner, experts, sharpness):
            self.prefix, self.hidden, self.sharpness = prefix, hidden, sharpness
            self.experts = [GatedMLP(f"{prefix}experts.{e}.", hidden, inner) for e in range(experts)]

        def weight_specs(self):
            specs = {self.prefix + "router.weight": WeightSpec((len(self.experts), self.hidden))}
            for expert in self.experts:
                specs.update(expert.weight_specs())
            return specs

        def bind(self, tensors, runtime):
            super().bind(tensors, runtime)
            self.router = runtime.matrix(tensors[self.prefix + "router.weight"])
            for expert in self.experts:
                expert.bind(tensors, runtime)

        def forward(self, h, batch, residual):
            rt = self.runtime
            logits = rt.empty((h.shape[0], len(self.experts)), torch.float32)
            rt.ops.linear(h, self.router, logits)
            weights = torch.softmax(logits * self.sharpness, dim=-1)
            for e, expert in enumerate(self.experts):
                share = torch.zeros_like(residual)
                expert.forward(h, batch, share)
                residual.addcmul_(share, weights[:, e:e + 1])

    register_part("mixer", "toy_decay", DecayMixer)
    register_part("position", "toy_shift", ShiftPosition)
    register_part("feed_forward", "toy_mixture", MixtureMLP)

    @dataclass(frozen=True)
    class ToyConfig:
        architecture: str
        vocab_size: int
        hidden_size: int
        decay: float
        max_position_embeddings: int
        eos_token_ids: tuple = ()
        bos_token_id: int = 0

        @classmethod
        def from_dict(cls, raw):
            return cls(raw["architectures"][0], raw["vocab_size"], raw["hidden_size"], raw["decay"],
                       raw["max_position_embeddings"])

        def to_dict(self):
            return {"architectures": [self.architecture], "vocab_size": self.vocab_size,
                    "hidden_size": self.hidden_size, "decay": self.decay,
                    "max_position_embeddings": self.max_position_embeddings}

    def build(c):
        from xeno_rt_amd.parts import create_part
        h = c.hidden_size
        norm = lambda p: RMSNorm(p, h, 1e-5)
        layers = [
            # layer 0: the stateful toy mixer
            PreNormBlock(norm("l0.n1."), create_part("mixer", "toy_decay", prefix="l0.", hidden=h, decay=c.decay),
                         norm("l0.n2."), GatedMLP("l0.mlp.", h, 2 * h + 8)),
            # layer 1: attention with the toy position encoding; it is run twice
            PreNormBlock(norm("l1.n1."), Attention("l1.attn.", h, 4, 2, 16, qk_norm=True, qk_norm_eps=1e-5,
                                                   position=create_part("position", "toy_shift", step=0.01)),
                         norm("l1.n2."), GatedMLP("l1.mlp.", h, 2 * h + 8)),
            # layer 2: attention without position encoding, reading the cache of the first call of layer 1
            # ... and with a feed-forward of three experts behind a router
            PreNormBlock(norm("l2.n1."), Attention("l2.attn.", h, 4, 2, 16, qk_norm=True, qk_norm_eps=1e-5),
                         norm("l2.n2."), create_part("feed_forward", "toy_mixture", prefix="l2.moe.", hidden=h,
                                                     inner=h + 24, experts=3, sharpness=4.0)),
        ]
        emb = Embedding("emb.", c.vocab_size, h)
        schedule = [LayerCall(0), LayerCall(1), LayerCall(1), LayerCall(2, reads_cache_of=1)]
        return ModelSpec(c, emb, layers, RMSNorm("final.", h, 1e-5), OutputHead("head.", c.vocab_size, h),
                         schedule=schedule)

    register_architecture("ToyForCausalLM", ToyConfig, build)
    return ToyConfig("ToyForCausalLM", 150, 48, 0.8, 200)


def plain_toy(w, config, ids):
    """The toy model on whole sequences, with the plain functions."""
    h = config.hidden_size
    x = w["emb.weight"][ids]
    pos = torch.arange(len(ids)).double()

    def mlp(p, y):
        return P.linear(P.swiglu(P.linear(y, w[p + "gate_proj.weight"]), P.linear(y, w[p + "up_proj.weight"])),
                        w[p + "down_proj.weight"])

    def attend(p, y, shift, shared=None):
        q, k, v = (P.linear(y, w[f"{p}{n}_proj.weight"]) for n in "qkv")
        q = P.head_rmsnorm(q, 4, 16, w[p + "q_norm.weight"], 1e-5)
        k = P.head_rmsnorm(k, 2, 16, w[p + "k_norm.weight"], 1e-5)
        if shift:
            q = q.clone(); k = k.clone()
            q[:, 0::16] += (pos * shift)[:, None]
            k[:, 0::16] += (pos * shift)[:, None]
        if shared is not None:
            k, v = shared
        return P.linear(P.causal_attention(q, k, v, 4, 2, 16), w[p + "o_proj.weight"]), (k, v)

    # layer 0
    y = P.rmsnorm(x, w["l0.n1.weight"], 1e-5)
    s, states = torch.zeros(h, dtype=x.dtype), []
    for t in range(len(ids)):
        s = config.decay * s + y[t]
        states.append(s)
    x = x + P.linear(torch.stack(states), w["l0.mix.weight"])
    x = x + mlp("l0.mlp.", P.rmsnorm(x, w["l0.n2.weight"], 1e-5))
    # layer 1 twice
    first_kv = None
    for call in range(2):
        out, kv = attend("l1.attn.", P.rmsnorm(x, w["l1.n1.weight"], 1e-5), 0.01)
        first_kv = first_kv or kv
        x = x + out
        x = x + mlp("l1.mlp.", P.rmsnorm(x, w["l1.n2.weight"], 1e-5))
    # layer 2 reads the keys and values that the first call of layer 1 cached
    out, _ = attend("l2.attn.", P.rmsnorm(x, w["l2.n1.weight"], 1e-5), 0.0, shared=first_kv)
    x = x + out
    y = P.rmsnorm(x, w["l2.n2.weight"], 1e-5)
    share = torch.softmax(P.linear(y, w["l2.moe.router.weight"]) * 4.0, dim=-1)
    x = x + sum(share[:, e:e + 1] * mlp(f"l2.moe.experts.{e}.", y) for e in range(3))
    return P.linear(P.rmsnorm(x, w["final.weight"], 1e-5), w["head.weight"])


@pytest.mark.parametrize("dtype", ["float32", "bfloat16"])
def test_toy_architecture_with_parts_of_its_own(dtype, tmp_path):
    from xeno_rt_amd.config import load_config, save_config
    from xeno_rt_amd.engine import Engine, GenerateRequest, generate
    from xeno_rt_amd.weights import SafetensorsFile, write_random_model
    from helpers import run_batched

    config = define_toy()
    folder = str(tmp_path / "toy")
    write_random_model(config, folder, seed=3, std=0.25)          # the framework's own random-weights mode
    assert load_config(folder) == config
    engine = Engine.load(folder, dtype=dtype, max_tokens=512, max_slots=3)
    assert len(engine.cache.groups) == 1 and engine.cache.groups[0].calls == [1, 2]   # the shared call owns none
    assert list(engine.cache.states) == [0]

    with SafetensorsFile(folder + "/model.safetensors") as file:
        w = {n: file.read(n).double() for n in file.names()}
    requests = [token_ids(150, n, seed=n) for n in (90, 33, 140)]
    want = [plain_toy(w, config, ids) for ids in requests]
    for ids, logits in zip(requests, want):
        assert_logits(run_whole(engine, ids), logits, dtype, "toy whole")
        assert_logits(run_tail_decoded(engine, ids), logits, dtype, "toy decoded tail")
    for got, logits in zip(run_batched(engine, requests, [50, 33, 100]), want):
        assert_logits(got, logits, dtype, "toy batch")
    # slots are used again: the state of the next sequence starts from zero
    for got, logits in zip(run_batched(engine, requests[::-1], [1, 20, 60]), want[::-1]):
        assert_logits(got, logits, dtype, "toy batch in used slots")
    out = generate(engine, [GenerateRequest(requests[1][:5], max_tokens=4, temperature=0.0, repetition_penalty=1.0),
                            GenerateRequest(requests[2][:3], max_tokens=6, temperature=0.0, repetition_penalty=1.3)])
    assert [len(o.tokens) for o in out] == [4, 6]
    from helpers import assert_greedy_tokens
    logits_of = lambda ids: plain_toy(w, config, ids)
    assert_greedy_tokens(logits_of, requests[1][:5], out[0].tokens, dtype, 1.0, "toy generation")
    assert_greedy_tokens(logits_of, requests[2][:3], out[1].tokens, dtype, 1.3, "toy generation with a penalty")
    engine.cache.check()
