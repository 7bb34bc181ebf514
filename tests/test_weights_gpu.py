"""Weights on the GPU: the random-weights kernel against the host's generator, what a loaded model
keeps on the device, and a float16 checkpoint on the 32-bit path."""
import os

import pytest
import torch

from conftest import TINY, make_folder
from helpers import assert_logits, plain_matrix, run_whole, token_ids
import plain_llama as P

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("dtype", [torch.float32, torch.bfloat16])
@pytest.mark.parametrize("count", [1, 63, 4097, (1 << 22) + 5])
def test_random_kernel_equals_the_host_generator_bit_for_bit(dtype, count):
    from xeno_rt_amd.ops import load_ops
    from xeno_rt_amd.weights import random_init

    ops = load_ops()
    key = random_init.tensor_key(9, "model.layers.3.mlp.up_proj.weight")
    for std, offset in ((0.02, 0.0), (0.3, 1.0)):
        scale = random_init.normal_scale(std)
        out = torch.empty(count, dtype=dtype, device="cuda")
        ops.random_normal(out, key, scale, offset)
        want = torch.cat([random_init.normal_values(key, first, min(1 << 20, count - first), scale)
                          for first in range(0, count, 1 << 20)])
        if offset:
            want = want + offset
        assert torch.equal(out.cpu(), want.to(dtype)), (dtype, count, std)


def test_a_model_in_memory_is_the_model_of_the_written_folder(tmp_path):
    from xeno_rt_amd.config import parse_config
    from xeno_rt_amd.engine import Engine
    from xeno_rt_amd.weights import write_random_model

    config = parse_config(TINY["qwen3"])
    folder = write_random_model(config, str(tmp_path / "m"), seed=12, std=0.2, gain_std=0.2)
    ids = token_ids(config.vocab_size, 50, seed=1)
    for dtype in ("float32", "bfloat16"):
        loaded = Engine.load(folder, dtype=dtype, max_tokens=256)
        made = Engine.random(config, seed=12, std=0.2, gain_std=0.2, dtype=dtype, max_tokens=256)
        if dtype == "bfloat16":     # the folder holds bfloat16: the same numbers as the model made in bfloat16
            assert torch.equal(run_whole(loaded, ids), run_whole(made, ids))
        assert_logits(run_whole(made, ids), P.PlainModel.from_weights(
            TINY["qwen3"], {n: made.get_tensor(n).float() for n in made.tensors.keys()}).logits(ids), dtype, "made in memory")


def test_a_loaded_model_holds_every_weight_once(tmp_path):
    """After Engine.load the device holds the weights in the form the parts bound them (q, k, v and gate, up
    stacked) and nothing else of the checkpoint: no second copy under the checkpoint's names."""
    from xeno_rt_amd.config import parse_config
    from xeno_rt_amd.engine import Engine
    from xeno_rt_amd.weights import write_random_model

    raw = dict(TINY["llama"], hidden_size=512, intermediate_size=1408, num_hidden_layers=6, num_attention_heads=8,
               num_key_value_heads=4, vocab_size=2048, max_position_embeddings=256)
    config = parse_config(raw)
    folder = write_random_model(config, str(tmp_path / "m"), seed=1)
    file_bytes = os.path.getsize(os.path.join(folder, "model.safetensors"))
    torch.cuda.synchronize()
    torch.cuda.empty_cache()
    for dtype, factor in (("bfloat16", 1.0), ("float32", 2.0)):
        torch.cuda.reset_peak_memory_stats()
        before = torch.cuda.memory_allocated()
        engine = Engine.load(folder, dtype=dtype, max_tokens=64, max_slots=1, graphs=False)
        torch.cuda.synchronize()
        held = torch.cuda.memory_allocated() - before
        peak = torch.cuda.max_memory_allocated() - before
        cache_bytes = sum(g.k.numel() * g.k.element_size() * 2 for g in engine.cache.groups)
        assert held - cache_bytes <= 1.02 * factor * file_bytes + (1 << 20), (dtype, held, cache_bytes, file_bytes)
        assert peak - cache_bytes <= 1.05 * factor * file_bytes + (4 << 20), (dtype, peak, file_bytes)
        name = "model.layers.4.self_attn.k_proj.weight"
        assert torch.equal(engine.get_tensor(name).to(engine.dtype), plain_matrix(engine.model.spec.layers[4].mixer.w_qkv)[
            config.q_width:config.q_width + config.kv_width].cpu())
        del engine


def test_float16_checkpoint_on_the_32_bit_path_equals_the_plain_model(tmp_path):
    """A float16 file widens exactly on the 32-bit path; held as bfloat16 it would be off by 1e-3."""
    from safetensors.torch import load_file, save_file
    from xeno_rt_amd.engine import Engine

    folder = make_folder(TINY["qwen3"], tmp_path / "f16", seed=5, std=0.2)
    path = os.path.join(folder, "model.safetensors")
    tensors = {name: (tensor.float() * 1.37).to(torch.float16) for name, tensor in load_file(path).items()}
    save_file(tensors, path, metadata={"format": "pt"})
    plain = P.PlainModel(folder)
    assert plain.w("model.norm.weight").dtype == torch.float32
    ids = token_ids(plain.config.vocab_size, 70, seed=2)
    engine = Engine.load(folder, dtype="float32", max_tokens=256)
    assert engine.model.spec.layers[0].mixer.w_o.dtype == torch.float32
    assert_logits(run_whole(engine, ids), plain.logits(ids), "float32", "float16 checkpoint, 32-bit path")
    assert_logits(run_whole(Engine.load(folder, dtype="bfloat16", max_tokens=256), ids), plain.logits(ids), "bfloat16",
                  "float16 checkpoint, bfloat16 path")
