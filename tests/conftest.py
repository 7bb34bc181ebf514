"""Shared fixtures: the two tiny configurations, model folders with random weights,
and the GPU marker."""
import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for path in (ROOT, os.path.dirname(os.path.abspath(__file__))):
    if path not in sys.path:
        sys.path.insert(0, path)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu)")


def pytest_terminal_summary(terminalreporter):
    """The largest errors against the plain model that the run has seen, next to their limits."""
    import helpers
    for dtype, (worst, rms, what) in sorted(helpers.SEEN.items()):
        limit = helpers.TOLERANCE[dtype]
        terminalreporter.write_line(f"logit errors seen [{dtype}]: max {worst:.2e} (limit {limit['max']:.1e}), "
                                    f"rms {rms:.2e} (limit {limit['rms']:.1e}); the largest in: {what or 'unnamed'}")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU here")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


# Two tiny configurations that differ in every size and option.
TINY_LLAMA = {
    "architectures": ["LlamaForCausalLM"],
    "vocab_size": 256, "hidden_size": 64, "intermediate_size": 176, "num_hidden_layers": 2,
    "num_attention_heads": 4, "num_key_value_heads": 2, "rms_norm_eps": 1e-5, "rope_theta": 10000.0,
    "max_position_embeddings": 128, "tie_word_embeddings": False, "hidden_act": "silu",
    "eos_token_id": 1, "bos_token_id": 0, "torch_dtype": "bfloat16",
}
TINY_QWEN3 = {
    "architectures": ["Qwen3ForCausalLM"],
    "vocab_size": 384, "hidden_size": 96, "intermediate_size": 256, "num_hidden_layers": 3,
    "num_attention_heads": 6, "num_key_value_heads": 3, "head_dim": 32, "rms_norm_eps": 1e-6,
    "rope_theta": 1000000.0, "max_position_embeddings": 256, "tie_word_embeddings": True,
    "hidden_act": "silu", "eos_token_id": [2, 5], "bos_token_id": 3, "torch_dtype": "bfloat16",
    # the rotation's two options (llama.rs:92-94, 103-106): half of a head rotated, positions divided by 4
    "partial_rotary_factor": 0.5, "rope_scaling": {"rope_type": "linear", "factor": 4.0},
}
TINY = {"llama": TINY_LLAMA, "qwen3": TINY_QWEN3}
# On top of a tiny configuration: the whole head is rotated again (the positions' scale stays). For tests that are after
# what only such a model takes: the rotation in a projection's epilogue, the attention that finishes q, k and v itself.
WHOLE_ROTATION = {"partial_rotary_factor": 1.0}


def make_folder(raw_config, folder, seed, std=0.02, randomize_norms=True):
    """Write a model folder with the engine's random-weights mode. Norm weights are then
    replaced by random values near 1, so that a norm in the wrong place, or a weight
    that is not applied, changes the logits."""
    from xeno_rt_amd.config import parse_config
    from xeno_rt_amd.weights import SafetensorsFile, write_random_model, write_safetensors

    config = parse_config(raw_config)
    write_random_model(config, str(folder), seed=seed, std=std)
    if randomize_norms:
        path = os.path.join(str(folder), "model.safetensors")
        with SafetensorsFile(path) as file:
            tensors = {name: file.read(name) for name in file.names()}
        generator = torch.Generator().manual_seed(seed + 77)
        for name, tensor in tensors.items():
            if tensor.dim() == 1:
                tensors[name] = (1.0 + 0.3 * torch.randn(tensor.shape, generator=generator)).to(tensor.dtype)
        write_safetensors(path, tensors)
    return str(folder)


@pytest.fixture(scope="session", params=["llama", "qwen3"])
def tiny_folder(request, tmp_path_factory):
    """(name, folder) of a tiny model with random weights of std 0.2: large enough that
    attention is far from uniform and every part matters to the logits."""
    folder = tmp_path_factory.mktemp(f"tiny_{request.param}")
    return request.param, make_folder(TINY[request.param], folder, seed=11 if request.param == "llama" else 23,
                                      std=0.2)
