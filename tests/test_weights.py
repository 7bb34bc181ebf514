"""The safetensors reader and writer, binding by name, and random weights."""
import json
import os
import struct

import pytest
import torch

from conftest import TINY
from xeno_rt_amd.config import architecture, parse_config
from xeno_rt_amd.weights import (SafetensorsError, SafetensorsFile, WeightError, load_tensors,
                                 write_random_model, write_safetensors)


def raw_file(path, header, data=b""):
    blob = json.dumps(header).encode() if not isinstance(header, bytes) else header
    with open(path, "wb") as handle:
        handle.write(struct.pack("<Q", len(blob)) + blob + data)
    return str(path)


def test_written_files_are_read_by_the_safetensors_package(tmp_path):
    from safetensors import safe_open
    tensors = {"a": torch.randn(3, 5), "b": torch.randn(7).to(torch.bfloat16),
               "c": torch.arange(6, dtype=torch.int32).reshape(2, 3), "d": torch.randn(2, 2).to(torch.float16)}
    path = str(tmp_path / "x.safetensors")
    write_safetensors(path, tensors, metadata={"format": "pt"})
    with safe_open(path, framework="pt") as handle:
        assert set(handle.keys()) == set(tensors)
        for name, tensor in tensors.items():
            assert torch.equal(handle.get_tensor(name), tensor)


def test_files_of_the_safetensors_package_are_read(tmp_path):
    from safetensors.torch import save_file
    tensors = {"w": torch.randn(4, 6).to(torch.bfloat16), "v": torch.randn(9), "i": torch.arange(5)}
    path = str(tmp_path / "y.safetensors")
    save_file(tensors, path)
    with SafetensorsFile(path) as file:
        assert sorted(file.names()) == ["i", "v", "w"]
        assert file.entry("w").dtype == "BF16" and file.entry("w").shape == (4, 6)
        for name, tensor in tensors.items():
            assert torch.equal(file.read(name), tensor)
        with pytest.raises(SafetensorsError, match="missing tensor nope"):
            file.entry("nope")


def test_malformed_files_are_refused(tmp_path):
    ok = {"dtype": "F32", "shape": [2], "data_offsets": [0, 8]}
    cases = [
        (lambda p: open(p, "wb").write(b"\x01\x02") and str(p), "truncated"),
        (lambda p: open(p, "wb").write(struct.pack("<Q", 1000) + b"{}") and str(p), "exceeds the file size"),
        (lambda p: raw_file(p, b"{not json"), "invalid header JSON"),
        (lambda p: raw_file(p, {"t": dict(ok, dtype="F8_E4M3")}, b"\0" * 8), "unsupported dtype"),
        (lambda p: raw_file(p, {"t": dict(ok, data_offsets=[0, 16])}, b"\0" * 8), "outside the data section"),
        (lambda p: raw_file(p, {"t": dict(ok, shape=[3])}, b"\0" * 8), "needs 12 bytes"),
        (lambda p: raw_file(p, {"t": ok, "u": dict(ok, data_offsets=[4, 12])}, b"\0" * 12), "overlap"),
        (lambda p: raw_file(p, b'{"t": %s, "t": %s}' % (json.dumps(ok).encode(), json.dumps(ok).encode()), b"\0" * 8),
         "duplicate tensor name"),
        (lambda p: raw_file(p, {"t": {"dtype": "F32", "shape": [2]}}, b"\0" * 8), "lacks"),
        (lambda p: raw_file(p, {"t": dict(ok, shape=[-2])}, b"\0" * 8), "invalid shape"),
    ]
    for index, (make, text) in enumerate(cases):
        with pytest.raises(SafetensorsError, match=text):
            SafetensorsFile(make(tmp_path / f"bad{index}.safetensors"))
    with pytest.raises(SafetensorsError, match="no such file"):
        SafetensorsFile(str(tmp_path / "absent.safetensors"))


def folder_with(tmp_path, name, edit):
    """A tiny model folder whose tensors were changed by edit(dict)."""
    config = parse_config(TINY[name])
    folder = str(tmp_path / name)
    write_random_model(config, folder, seed=1)
    path = os.path.join(folder, "model.safetensors")
    with SafetensorsFile(path) as file:
        tensors = {n: file.read(n) for n in file.names()}
    edit(tensors)
    write_safetensors(path, tensors)
    spec = architecture(config.architecture).build(config)
    return folder, spec


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    def edit(t):
        del t["model.layers.1.mlp.up_proj.weight"]
        del t["model.norm.weight"]
        t["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)
        t["model.layers.0.self_attn.k_proj.weight"] = torch.zeros(64, 64, dtype=torch.bfloat16)
        t["model.layers.0.input_layernorm.weight"] = torch.zeros(64, dtype=torch.int32)
    folder, spec = folder_with(tmp_path, "llama", edit)
    with pytest.raises(WeightError) as caught:
        load_tensors(folder, spec.weight_specs(), spec.ignored_names())
    error = caught.value
    assert error.missing == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert error.unexpected == ["model.layers.0.self_attn.rotary_emb.inv_freq"]
    assert error.wrong_shape == [("model.layers.0.self_attn.k_proj.weight", (32, 64), (64, 64))]
    assert [w[0] for w in error.wrong_dtype] == ["model.layers.0.input_layernorm.weight"]
    text = str(error)
    for fragment in ("missing tensors (2)", "unexpected tensors (1)", "expected [32, 64] found [64, 64]",
                     "model.norm.weight", "rotary_emb.inv_freq"):
        assert fragment in text


def test_tied_head_in_the_file_is_ignored_untied_head_is_required(tmp_path):
    folder, spec = folder_with(tmp_path, "qwen3", lambda t: t.update({"lm_head.weight": torch.zeros(384, 96)}))
    with pytest.warns(UserWarning, match="lm_head.weight ignored"):        # left alone, and said so
        assert "lm_head.weight" not in load_tensors(folder, spec.weight_specs(), spec.ignored_names())
    folder, spec = folder_with(tmp_path, "llama", lambda t: t.pop("lm_head.weight"))
    with pytest.raises(WeightError, match="lm_head.weight"):
        load_tensors(folder, spec.weight_specs(), spec.ignored_names())


def test_stored_precision_is_kept(tmp_path):
    def edit(t):
        t["model.norm.weight"] = t["model.norm.weight"].to(torch.float32) * 1.001
        t["model.layers.0.mlp.up_proj.weight"] = t["model.layers.0.mlp.up_proj.weight"].to(torch.float16)
    folder, spec = folder_with(tmp_path, "llama", edit)
    tensors = load_tensors(folder, spec.weight_specs())
    assert tensors["model.norm.weight"].dtype == torch.float32                 # 32-bit stays 32-bit
    assert float(tensors["model.norm.weight"][0]) == pytest.approx(1.001, abs=1e-7)
    assert tensors["model.layers.0.mlp.up_proj.weight"].dtype == torch.float16    # as stored: the binder converts
    assert tensors["model.embed_tokens.weight"].dtype == torch.bfloat16


def test_float16_checkpoint_widens_exactly_on_the_32_bit_path_and_is_rounded_only_on_the_other(tmp_path):
    """What the parts bind: a float32 model holds float16(w) exactly, a bfloat16 model its rounding."""
    from ops_emulation import EmulatedOps
    from xeno_rt_amd.engine import Engine

    stored = {}

    def edit(t):
        for name in list(t):
            t[name] = (t[name].float() * 1.37).to(torch.float16)     # values that bfloat16 cannot hold
        stored.update({name: value.clone() for name, value in t.items()})
    folder, spec = folder_with(tmp_path, "llama", edit)
    engine = Engine.load(folder, dtype="float32", max_tokens=128, device="cpu", ops=EmulatedOps())
    mixer, mlp = engine.model.spec.layers[1].mixer, engine.model.spec.layers[1].feed_forward
    p = "model.layers.1."
    want_qkv = torch.cat([stored[p + f"self_attn.{n}_proj.weight"].float() for n in "qkv"])
    assert mixer.w_qkv.dtype == torch.float32 and torch.equal(mixer.w_qkv, want_qkv)
    assert torch.equal(mlp.w_down, stored[p + "mlp.down_proj.weight"].float())
    norm = engine.model.spec.final_norm.weight
    assert norm.dtype == torch.float32 and torch.equal(norm, stored["model.norm.weight"].float())
    assert torch.equal(engine.get_tensor(p + "mlp.up_proj.weight"), stored[p + "mlp.up_proj.weight"])
    rounded = Engine.load(folder, dtype="bfloat16", max_tokens=128, device="cpu", ops=EmulatedOps())
    assert torch.equal(rounded.model.spec.layers[1].mixer.w_qkv, want_qkv.to(torch.bfloat16))
    assert not torch.equal(want_qkv.to(torch.bfloat16).float(), want_qkv)
    # a float16 vector is never squeezed into bfloat16: it widens
    assert rounded.model.spec.final_norm.weight.dtype == torch.float32


def test_random_weights_are_the_same_in_the_file_in_memory_and_in_any_pieces(tmp_path):
    """Every element depends on (seed, tensor name, element index) alone."""
    from ops_emulation import EmulatedOps
    from xeno_rt_amd.engine import Engine
    from xeno_rt_amd.weights import make_tensor
    from xeno_rt_amd.weights import random_init
    from xeno_rt_amd.parts.base import WeightSpec

    config = parse_config(TINY["qwen3"])
    folder = write_random_model(config, str(tmp_path / "m"), seed=5, std=0.05, gain_std=0.1)
    engine = Engine.random(config, seed=5, std=0.05, gain_std=0.1, dtype="bfloat16", max_tokens=128, device="cpu",
                           ops=EmulatedOps())
    with SafetensorsFile(os.path.join(folder, "model.safetensors")) as file:
        for name in file.names():
            assert torch.equal(file.read(name), engine.get_tensor(name)), name
        gains = file.read("model.layers.0.input_layernorm.weight").float()
        assert 0.05 < float((gains - 1).abs().mean()) < 0.15
    p = "model.layers.2.self_attn."
    bound = engine.model.spec.layers[2].mixer.w_qkv
    assert torch.equal(bound, torch.cat([engine.get_tensor(p + f"{n}_proj.weight") for n in "qkv"]))
    # float32 and bfloat16 models of one seed hold the same numbers before rounding
    wide = Engine.random(config, seed=5, std=0.05, dtype="float32", max_tokens=128, device="cpu", ops=EmulatedOps())
    name = "model.layers.1.mlp.gate_proj.weight"
    assert torch.equal(wide.get_tensor(name).to(torch.bfloat16), engine.get_tensor(name))
    # pieces: elements 1000 .. 1010 made alone equal those of the whole; another name or seed gives other values
    key = random_init.tensor_key(5, name)
    whole = random_init.normal_values(key, 0, 5000, 1.0)
    assert torch.equal(random_init.normal_values(key, 1000, 10, 1.0), whole[1000:1010])
    # the tensor arithmetic against the generator written out on Python integers
    for i in (0, 1, 999, 4999):
        words = [random_init._mix((key + (2 * i + j) * random_init._GOLDEN) & random_init._MASK) for j in (0, 1)]
        total = sum((word >> (10 * field)) & 1023 for word in words for field in range(6))
        assert float(whole[i]) == float(2 * total - 12 * 1023)
    assert not (random_init.normal_values(random_init.tensor_key(5, name + "x"), 0, 5000, 1.0) == whole).all()
    assert not (random_init.normal_values(random_init.tensor_key(6, name), 0, 5000, 1.0) == whole).all()
    # a tensor's values do not depend on the other tensors of the model, nor on its shape's cut
    spec = WeightSpec((50, 100))
    assert torch.equal(make_tensor(spec, 5, name, 0.05, torch.float32).reshape(-1),
                       make_tensor(WeightSpec((5000,)), 5, name, 0.05, torch.float32))
    # and they are normal enough: moments of a large sample
    sample = random_init.normal_values(key, 0, 1 << 20, random_init.normal_scale(1.0)).double()
    assert abs(float(sample.mean())) < 4e-3 and abs(float(sample.std()) - 1.0) < 4e-3
    assert abs(float((sample ** 4).mean()) - 3.0) < 0.15          # twelve uniforms: kurtosis 2.9
    assert 0.0015 < float((sample.abs() > 3.0).double().mean()) < 0.0035      # normal: 0.0027


def test_random_weights_follow_seed_and_rule(tmp_path):
    config = parse_config(TINY["qwen3"])
    a = write_random_model(config, str(tmp_path / "a"), seed=7)
    b = write_random_model(config, str(tmp_path / "b"), seed=7)
    c = write_random_model(config, str(tmp_path / "c"), seed=8)
    read = lambda folder: SafetensorsFile(os.path.join(folder, "model.safetensors"))
    with read(a) as fa, read(b) as fb, read(c) as fc:
        assert fa.names() == fb.names() and len(fa.names()) == 1 + 3 * 11 + 1
        for name in fa.names():
            assert torch.equal(fa.read(name), fb.read(name))
        w = fa.read("model.layers.1.mlp.gate_proj.weight").float()
        assert not torch.equal(fa.read("model.layers.1.mlp.gate_proj.weight"), fc.read("model.layers.1.mlp.gate_proj.weight"))
        assert abs(float(w.std()) - 0.02) < 0.002 and abs(float(w.mean())) < 0.001
        assert torch.equal(fa.read("model.layers.2.self_attn.q_norm.weight"), torch.ones(32, dtype=torch.bfloat16))
        assert torch.equal(fa.read("model.norm.weight"), torch.ones(96, dtype=torch.bfloat16))
    assert json.load(open(os.path.join(a, "config.json")))["architectures"] == ["Qwen3ForCausalLM"]


def test_sharded_checkpoints_are_read_through_the_index(tmp_path):
    folder, spec = folder_with(tmp_path, "llama", lambda t: None)
    path = os.path.join(folder, "model.safetensors")
    with SafetensorsFile(path) as file:
        tensors = {n: file.read(n) for n in file.names()}
    os.remove(path)
    names = sorted(tensors)
    shards = {"model-00001-of-00002.safetensors": names[:7], "model-00002-of-00002.safetensors": names[7:]}
    weight_map = {}
    for shard, members in shards.items():
        write_safetensors(os.path.join(folder, shard), {n: tensors[n] for n in members})
        weight_map.update({n: shard for n in members})
    with open(os.path.join(folder, "model.safetensors.index.json"), "w") as handle:
        json.dump({"weight_map": weight_map}, handle)
    loaded = load_tensors(folder, spec.weight_specs())
    assert all(torch.equal(loaded[n], tensors[n]) for n in names)


def test_an_engine_closes_the_files_of_its_checkpoint_once_the_weights_are_bound(tmp_path):
    """A tied model whose file also carries the head's matrix: a warning, the same logits; the shards are closed when
    the parts have bound their tensors, and get_tensor opens them again for its one read."""
    import warnings
    from ops_emulation import EmulatedOps
    from xeno_rt_amd.engine import Engine
    from xeno_rt_amd.weights import CheckpointSource
    folder, spec = folder_with(tmp_path, "qwen3", lambda t: None)
    with warnings.catch_warnings():
        warnings.simplefilter("error")                                      # nothing to warn of here
        plain = Engine.load(folder, dtype="float32", max_tokens=128, device="cpu", ops=EmulatedOps())
    assert isinstance(plain.tensors, CheckpointSource) and not plain.tensors.is_open
    again = plain.get_tensor("model.norm.weight")
    assert not plain.tensors.is_open and again.shape == (96,)
    with SafetensorsFile(os.path.join(folder, "model.safetensors")) as file:
        tensors = {name: file.read(name) for name in file.names()}
    assert torch.equal(again, tensors["model.norm.weight"])
    tensors["lm_head.weight"] = torch.full((384, 96), 3.0)
    write_safetensors(os.path.join(folder, "model.safetensors"), tensors)
    with pytest.warns(UserWarning, match="lm_head.weight ignored"):
        carrying = Engine.load(folder, dtype="float32", max_tokens=128, device="cpu", ops=EmulatedOps())
    ids = [5, 9, 200, 31]
    rows = []
    for engine in (plain, carrying):
        slot = engine.alloc_slot()
        rows.append(engine.step([(slot, ids, [3])]))
        engine.free_slot(slot)
    assert torch.equal(*rows)
