"""Configuration reading, the registry, safetensors by name, weight errors and
the random-weights mode (no GPU)."""
import json
import os

import pytest
import torch

from helpers import ARCH, TINY, config_json
from tiny_llm_infer_amd import lookup_architecture, register_architecture
from tiny_llm_infer_amd.config import ConfigError, Qwen3Config
from tiny_llm_infer_amd.engine.model import Model
from tiny_llm_infer_amd.registry import architecture_of, load_config
from tiny_llm_infer_amd.weights import (Checkpoint, TensorDecl, WeightError, WeightFileError,
                                        load_tensors, write_safetensors)


def test_config_reads_every_key_and_derives_sizes():
    cfg = Qwen3Config.from_dict(config_json("B"))
    assert (cfg.hidden_size, cfg.intermediate_size, cfg.num_hidden_layers) == (96, 160, 3)
    assert (cfg.num_attention_heads, cfg.num_key_value_heads, cfg.head_dim) == (6, 3, 32)
    assert cfg.query_dim == 192 and cfg.kv_dim == 96          # head_dim != hidden / heads
    assert cfg.rms_norm_eps == 1e-5 and cfg.rope_theta == 1e6 and not cfg.tie_word_embeddings
    assert cfg.layer_windows() == (None, 40, 40)
    assert Qwen3Config.from_dict(config_json("C")).layer_windows() == (19, None, 19, None)
    assert Qwen3Config.from_dict(config_json("A")).layer_windows() == (None, None)


def test_config_defaults_follow_the_reference():
    base = dict(architectures=[ARCH], hidden_size=64, intermediate_size=128, num_hidden_layers=2,
                num_attention_heads=4, num_key_value_heads=2, vocab_size=100, max_position_embeddings=64)
    cfg = Qwen3Config.from_dict(base)
    assert cfg.head_dim == 16 and cfg.rms_norm_eps == 1e-6 and cfg.rope_theta == 1e6
    assert cfg.tie_word_embeddings is False and cfg.eos_token_ids == ()
    assert Qwen3Config.from_dict({**base, "eos_token_id": 7}).eos_token_ids == (7,)
    assert Qwen3Config.from_dict({**base, "eos_token_id": [7, 9]}).eos_token_ids == (7, 9)
    # what is written is read back unchanged
    assert Qwen3Config.from_dict(cfg.to_dict()) == cfg


@pytest.mark.parametrize("change, word", [
    ({"hidden_size": None}, "hidden_size"), ({"vocab_size": "many"}, "vocab_size"),
    ({"num_key_value_heads": 3}, "multiple"), ({"head_dim": 15}, "even"),
    ({"attention_bias": True}, "attention_bias"), ({"hidden_act": "gelu"}, "hidden_act"),
    ({"rope_scaling": {"type": "yarn"}}, "rope_scaling"), ({"model_type": "llama"}, "model_type"),
    ({"use_sliding_window": True, "sliding_window": None}, "sliding_window"),
    ({"layer_types": ["full_attention"]}, "layer_types"), ({"rms_norm_eps": 0}, "rms_norm_eps"),
    ({"num_hidden_layers": 0}, "num_hidden_layers"),
])
def test_config_errors_name_the_key(change, word):
    data = config_json("A")
    data.update(change)
    with pytest.raises(ConfigError) as err:
        Qwen3Config.from_dict(data)
    assert word in str(err.value)


def test_registry_maps_the_architecture_name():
    arch = lookup_architecture(ARCH)
    spec = arch.make_spec(arch.read_config(config_json("A"), "x"))
    assert spec.architecture == ARCH and len(spec.blocks) == 2 and len(spec.schedule) == 2
    with pytest.raises(ConfigError) as err:
        architecture_of({"architectures": ["LlamaForCausalLM"]})
    assert "LlamaForCausalLM" in str(err.value) and ARCH in str(err.value)
    with pytest.raises(ConfigError):
        architecture_of({})
    with pytest.raises(ValueError):
        register_architecture(ARCH, None, None)


def test_no_size_of_the_configuration_stands_in_the_spec():
    """Every size in the spec follows the config: change one key, see it move."""
    for key, new in [("hidden_size", 128), ("intermediate_size", 72), ("vocab_size", 999),
                     ("head_dim", 24), ("rms_norm_eps", 2e-3), ("rope_theta", 123.0)]:
        data = config_json("A")
        a = repr(lookup_architecture(ARCH).make_spec(Qwen3Config.from_dict(data)))
        data[key] = new
        b = repr(lookup_architecture(ARCH).make_spec(Qwen3Config.from_dict(data)))
        assert a != b, key


def _decls(name):
    arch = lookup_architecture(ARCH)
    return Model(arch.make_spec(arch.read_config(config_json(name), "x"))).tensors()


def test_model_declares_the_reference_tensor_names():
    names = {d.name: d.shape for d in _decls("B")}
    assert names["model.embed_tokens.weight"] == (384, 96)
    assert names["lm_head.weight"] == (384, 96)
    assert names["model.layers.2.self_attn.q_proj.weight"] == (192, 96)
    assert names["model.layers.2.self_attn.k_proj.weight"] == (96, 96)
    assert names["model.layers.0.self_attn.o_proj.weight"] == (96, 192)
    assert names["model.layers.1.self_attn.q_norm.weight"] == (32,)
    assert names["model.layers.1.mlp.down_proj.weight"] == (96, 160)
    assert names["model.norm.weight"] == (96,)
    assert len(names) == 2 + 1 + 3 * 11
    assert "lm_head.weight" not in {d.name for d in _decls("A")}      # tied


def test_random_weights_folder_round_trip(model_folders):
    folder = model_folders["B"]
    arch, cfg = load_config(folder)
    assert cfg == Qwen3Config.from_dict(config_json("B"))
    ck = Checkpoint(folder)
    decls = _decls("B")
    assert sorted(ck.names()) == sorted(d.name for d in decls)
    assert ck.dtype("model.norm.weight") == torch.bfloat16
    w = ck.read("model.layers.0.mlp.up_proj.weight").float()
    assert abs(float(w.std()) - 0.02) < 0.002 and abs(float(w.mean())) < 0.002
    n = ck.read("model.layers.0.input_layernorm.weight").float()
    assert abs(float(n.mean()) - 1.0) < 0.02
    # same seed, same bytes; another seed, other weights
    from helpers import make_model_folder
    again = Checkpoint(make_model_folder(os.path.join(folder, "again"), "B"))
    assert torch.equal(again.read("lm_head.weight"), ck.read("lm_head.weight"))


def test_random_weights_are_a_function_of_seed_tensor_and_element(model_folders):
    """The file of a random model against the rule written out again in numpy (tests/plain_random.py,
    its quantiles from the standard library): every tensor bit for bit.  An element does not
    depend on the tensor's shape or on what else is drawn."""
    import numpy as np
    import plain_random
    from tiny_llm_infer_amd.weights.random_init import draw_normal
    for name in ("A", "C"):
        decls = _decls(name)
        want = plain_random.model_weights([(d.name, d.shape, d.init) for d in decls], TINY[name]["seed"])
        ck = Checkpoint(model_folders[name])
        for d in decls:
            got = ck.read(d.name)
            assert got.dtype == torch.bfloat16
            assert np.array_equal(got.double().numpy(), want[d.name]), d.name
        ck.close()
    a = draw_normal((7, 1000), 5, 3, 0.02)
    b = draw_normal((7000,), 5, 3, 0.02)
    assert torch.equal(a.reshape(-1), b) and torch.equal(draw_normal((10,), 5, 3, 0.02), b[:10])
    assert not torch.equal(draw_normal((7000,), 5, 4, 0.02), b) and not torch.equal(draw_normal((7000,), 6, 3, 0.02), b)
    big = draw_normal((2000000,), 1, 0, 1.0).double()
    assert abs(float(big.mean())) < 3e-3 and abs(float(big.std()) - 1) < 3e-3
    assert abs(float((big ** 4).mean()) - 3) < 0.03 and 4.2 < float(big.abs().max()) < 4.5       # normal, cut at 4.5 sigma


def test_storage_rule(tmp_path):
    """16-bit floats -> bfloat16 (or widened for a float32 run); 32-bit stays;
    integer tables -> int32."""
    path = str(tmp_path / "model.safetensors")
    write_safetensors(path, [("a", torch.ones(2, 3, dtype=torch.bfloat16)),
                             ("b", torch.full((4,), 0.1, dtype=torch.float16)),
                             ("c", torch.full((4,), 0.1, dtype=torch.float32)),
                             ("d", torch.arange(5, dtype=torch.int64))])
    decls = [TensorDecl("a", (2, 3)), TensorDecl("b", (4,)), TensorDecl("c", (4,)), TensorDecl("d", (5,), "int")]
    bf = dict(load_tensors(str(tmp_path), decls, torch.bfloat16, "cpu"))
    assert [bf[k].dtype for k in "abcd"] == [torch.bfloat16, torch.bfloat16, torch.float32, torch.int32]
    f32 = dict(load_tensors(str(tmp_path), decls, torch.float32, "cpu"))
    assert [f32[k].dtype for k in "abcd"] == [torch.float32, torch.float32, torch.float32, torch.int32]
    assert float(f32["b"][0]) == float(torch.tensor(0.1, dtype=torch.float16))   # widened exactly


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    write_safetensors(str(tmp_path / "model.safetensors"),
                      [("keep", torch.zeros(2, 2, dtype=torch.bfloat16)),
                       ("bad", torch.zeros(3, 2, dtype=torch.bfloat16)),
                       ("extra1", torch.zeros(1, dtype=torch.bfloat16)),
                       ("extra2", torch.zeros(1, dtype=torch.bfloat16)),
                       ("ints", torch.zeros(2, dtype=torch.int32))])
    decls = [TensorDecl("keep", (2, 2)), TensorDecl("bad", (2, 3)), TensorDecl("gone1", (1,)),
             TensorDecl("gone2", (1,)), TensorDecl("ints", (2,))]
    with pytest.raises(WeightError) as err:
        list(load_tensors(str(tmp_path), decls, torch.bfloat16, "cpu"))
    e = err.value
    assert e.missing == ["gone1", "gone2"] and e.unexpected == ["extra1", "extra2"]
    assert e.wrong_shape == [("bad", (3, 2), (2, 3))] and e.bad_dtype[0][0] == "ints"
    for word in ("gone1", "gone2", "extra1", "extra2", "bad is [3, 2], expected [2, 3]"):
        assert word in str(e)


def test_sharded_checkpoint_and_broken_files(tmp_path):
    a, b = torch.randn(2, 2).bfloat16(), torch.randn(3).bfloat16()
    write_safetensors(str(tmp_path / "s1.safetensors"), [("a", a)])
    write_safetensors(str(tmp_path / "s2.safetensors"), [("b", b)])
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps(
        {"weight_map": {"a": "s1.safetensors", "b": "s2.safetensors"}}))
    ck = Checkpoint(str(tmp_path))
    assert torch.equal(ck.read("a"), a) and torch.equal(ck.read("b"), b)
    # a truncated file and offsets outside the file are refused
    blob = (tmp_path / "s1.safetensors").read_bytes()
    (tmp_path / "cut.safetensors").write_bytes(blob[:-3])
    with pytest.raises(WeightFileError):
        Checkpoint(str(tmp_path / "cut.safetensors"))
    (tmp_path / "short.safetensors").write_bytes(b"\x01\x02")
    with pytest.raises(WeightFileError):
        Checkpoint(str(tmp_path / "short.safetensors"))
    empty = tmp_path / "empty"
    empty.mkdir()
    with pytest.raises(WeightFileError):
        Checkpoint(str(empty))


def test_files_of_the_safetensors_package_are_read_and_ours_are_read_by_it(tmp_path):
    """A file that the ``safetensors`` package wrote (its own header padding, a ``__metadata__``
    entry, its order of tensors, tensors in bfloat16, float16 and float32, sharded with an
    index) is read tensor for tensor, and a file that this repository wrote opens in the
    package with the same contents."""
    st = pytest.importorskip("safetensors.torch")
    from safetensors import safe_open
    g = torch.Generator().manual_seed(3)
    tensors = {"z.last": torch.randn(5, 7, generator=g).bfloat16(),
               "a.first": torch.randn(3, generator=g).half(),
               "m.mid": torch.randn(2, 3, 4, generator=g),
               "i.table": torch.arange(6, dtype=torch.int64).reshape(2, 3),
               "s.scalarish": torch.randn(1, generator=g).bfloat16()}
    st.save_file(tensors, str(tmp_path / "model.safetensors"), metadata={"format": "pt", "note": "written by the package"})
    ck = Checkpoint(str(tmp_path))
    assert sorted(ck.names()) == sorted(tensors)
    for name, t in tensors.items():
        assert ck.dtype(name) == t.dtype and tuple(ck.shape(name)) == tuple(t.shape)
        assert torch.equal(ck.read(name), t)
    ck.close()
    decls = [TensorDecl("z.last", (5, 7)), TensorDecl("a.first", (3,)), TensorDecl("m.mid", (2, 3, 4)),
             TensorDecl("i.table", (2, 3), "int"), TensorDecl("s.scalarish", (1,))]
    got = dict(load_tensors(str(tmp_path), decls, torch.bfloat16, "cpu"))
    assert [got[d.name].dtype for d in decls] == [torch.bfloat16, torch.bfloat16, torch.float32, torch.int32, torch.bfloat16]
    assert torch.equal(got["a.first"], tensors["a.first"].to(torch.bfloat16)) and torch.equal(got["m.mid"], tensors["m.mid"])
    # sharded by the package's writer, with an index that also carries metadata
    shards = tmp_path / "sharded"
    shards.mkdir()
    names = list(tensors)
    st.save_file({n: tensors[n] for n in names[:2]}, str(shards / "model-00001-of-00002.safetensors"), metadata={"format": "pt"})
    st.save_file({n: tensors[n] for n in names[2:]}, str(shards / "model-00002-of-00002.safetensors"))
    (shards / "model.safetensors.index.json").write_text(json.dumps({
        "metadata": {"total_size": 1},
        "weight_map": {n: f"model-0000{1 if i < 2 else 2}-of-00002.safetensors" for i, n in enumerate(names)}}))
    ck = Checkpoint(str(shards))
    assert all(torch.equal(ck.read(n), t) for n, t in tensors.items())
    ck.close()
    # and the other way round
    ours = str(tmp_path / "ours.safetensors")
    write_safetensors(ours, list(tensors.items()))
    with safe_open(ours, framework="pt") as fh:
        assert sorted(fh.keys()) == sorted(tensors)
        for name, t in tensors.items():
            assert torch.equal(fh.get_tensor(name), t)
    assert all(torch.equal(v, tensors[k]) for k, v in st.load_file(ours).items())


def test_a_model_folder_written_here_loads_in_the_package(model_folders):
    st = pytest.importorskip("safetensors.torch")
    folder = model_folders["C"]
    theirs = st.load_file(os.path.join(folder, "model.safetensors"))
    ck = Checkpoint(folder)
    assert sorted(theirs) == sorted(ck.names())
    assert all(torch.equal(theirs[n], ck.read(n)) for n in ck.names())


def test_run_order_is_checked():
    from dataclasses import replace
    from tiny_llm_infer_amd.config import LayerCall
    arch = lookup_architecture(ARCH)
    spec = arch.make_spec(arch.read_config(config_json("A"), "x"))
    # a call may name a block twice and may read another call's cache ...
    ok = replace(spec, schedule=(LayerCall(0, 0), LayerCall(1, 1), LayerCall(0, 2), LayerCall(1, 1, False)))
    m = Model(ok)
    assert len(m.cache_needs()) == 3
    # ... but not before it is written, and not one that two calls write
    with pytest.raises(ConfigError):
        Model(replace(spec, schedule=(LayerCall(0, 0, False), LayerCall(1, 0))))
    with pytest.raises(ConfigError):
        Model(replace(spec, schedule=(LayerCall(0, 0), LayerCall(1, 0))))
    with pytest.raises(ConfigError):
        Model(replace(spec, schedule=(LayerCall(5, 0),)))
