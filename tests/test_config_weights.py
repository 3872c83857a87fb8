"""Configuration, registry and weight loading: keys and defaults of the reference
(`inferrs-models/src/config.rs:468-502`), and one clear error for a checkpoint that does not fit."""
import json
import os
import struct

import pytest
import torch

from tiny_configs import TINY_A, TINY_B, write_model

from inferrs_amd.config import ConfigError, Qwen3Config, load_config, registered_architectures
from inferrs_amd.config.registry import resolve_architecture
from inferrs_amd.parts import generated_tensors, model_tensors
from inferrs_amd.weights import (SafetensorsError, WeightError, load_weights, random_tensors,
                                 write_random_model, write_safetensors)


def test_defaults_follow_the_reference():
    raw = dict(vocab_size=100, hidden_size=64, intermediate_size=128, num_hidden_layers=2, num_attention_heads=4)
    c = Qwen3Config.from_dict(raw)
    assert c.num_key_value_heads == 4 and c.head_dim == 16
    assert c.rms_norm_eps == 1e-6 and c.rope_theta == 1e6 and c.tie_word_embeddings is True
    assert c.max_position_embeddings == 40960


def test_head_dim_is_decoupled_from_hidden_size():
    c = Qwen3Config.from_dict(TINY_B)
    assert c.head_dim * c.num_attention_heads != c.hidden_size
    spec = c.to_spec()
    expected, optional = model_tensors(spec)
    assert expected["model.layers.0.self_attn.q_proj.weight"].shape == (192, 96)
    assert expected["model.layers.2.self_attn.o_proj.weight"].shape == (96, 192)
    assert expected["model.layers.0.self_attn.k_norm.weight"].shape == (32,)
    assert "lm_head.weight" in expected and optional == {"lm_head.weight"}
    assert "lm_head.weight" in generated_tensors(spec)


def test_the_head_is_optional_by_presence():
    # qwen3.rs:369-372: lm_head.weight is used when the file has it, else the embedding table,
    # whatever tie_word_embeddings says; a random model has the head only when the config unties it
    spec = Qwen3Config.from_dict(TINY_A).to_spec()
    expected, optional = model_tensors(spec)
    assert optional == {"lm_head.weight"} and "lm_head.weight" not in generated_tensors(spec)


@pytest.mark.parametrize("key", ["vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers",
                                 "num_attention_heads"])
def test_missing_size_names_the_key(key):
    raw = dict(TINY_A)
    del raw[key]
    with pytest.raises(ConfigError, match=key):
        Qwen3Config.from_dict(raw)


@pytest.mark.parametrize("patch,word", [
    (dict(num_key_value_heads=3), "num_key_value_heads"), (dict(head_dim=15), "head_dim"),
    (dict(rms_norm_eps=0.0), "rms_norm_eps"), (dict(rope_theta=-1.0), "rope_theta"),
    (dict(hidden_size="64"), "hidden_size"), (dict(num_hidden_layers=0), "num_hidden_layers"),
    (dict(tie_word_embeddings="yes"), "tie_word_embeddings")])
def test_bad_values_name_the_key(patch, word):
    with pytest.raises(ConfigError, match=word):
        Qwen3Config.from_dict(dict(TINY_A, **patch))


def test_registry_is_exact_and_lists_what_it_knows():
    assert "Qwen3ForCausalLM" in registered_architectures()
    assert resolve_architecture({"architectures": ["Qwen3ForCausalLM"]}) is Qwen3Config
    assert resolve_architecture({"architectures": ["Other"], "model_type": "qwen3"}) is Qwen3Config
    # the reference's substring match would take this for Qwen3 (config.rs:343-366); an exact table does not
    with pytest.raises(ConfigError, match="Unsupported model architecture.*Qwen3MoeForCausalLM.*registered"):
        resolve_architecture({"architectures": ["Qwen3MoeForCausalLM"], "model_type": "qwen3_moe"})


def test_config_json_errors(tmp_path):
    with pytest.raises(ConfigError, match="not found"):
        load_config(str(tmp_path))
    (tmp_path / "config.json").write_text("{ not json")
    with pytest.raises(ConfigError, match="parse"):
        load_config(str(tmp_path))


def test_eos_ids_one_or_many():
    assert Qwen3Config.from_dict(dict(TINY_A, eos_token_id=7)).eos_token_ids == (7,)
    assert Qwen3Config.from_dict(dict(TINY_A, eos_token_id=[7, 9])).eos_token_ids == (7, 9)
    assert Qwen3Config.from_dict(TINY_A).to_spec().eos_token_ids == ()


def test_random_folder_round_trip(tmp_path):
    folder = write_model(str(tmp_path / "m"), TINY_B, seed=3)
    cfg = load_config(folder)
    assert cfg == Qwen3Config.from_dict(TINY_B)
    expected, optional = model_tensors(cfg.to_spec())
    got = load_weights(folder, expected, optional)
    again = random_tensors(expected, 3, torch.bfloat16)
    assert set(got) == set(expected)
    for name, t in got.items():
        assert t.dtype == torch.bfloat16 and torch.equal(t, again[name]), name
    # a tensor's values depend on (seed, name) only
    assert torch.equal(random_tensors({"model.norm.weight": expected["model.norm.weight"]}, 3)["model.norm.weight"],
                       again["model.norm.weight"])
    assert not torch.equal(random_tensors(expected, 4)["model.norm.weight"], again["model.norm.weight"])
    # the safetensors package reads what the writer wrote
    from safetensors.torch import load_file
    theirs = load_file(os.path.join(folder, "model.safetensors"))
    assert all(torch.equal(theirs[n], got[n]) for n in got)
    # norm weights are 1 + N(0, 0.1), matrices N(0, 0.02)
    assert abs(float(got["model.norm.weight"].float().mean()) - 1.0) < 0.1
    assert abs(float(got["model.embed_tokens.weight"].float().std()) - 0.02) < 0.003


def test_stored_precision_is_kept(tmp_path):
    expected, optional = model_tensors(Qwen3Config.from_dict(TINY_A).to_spec())
    tensors = random_tensors(generated_tensors(Qwen3Config.from_dict(TINY_A).to_spec()), 1, torch.bfloat16)
    tensors["model.norm.weight"] = tensors["model.norm.weight"].float() + 1e-4        # stored in 32-bit
    tensors["model.layers.0.mlp.up_proj.weight"] = tensors["model.layers.0.mlp.up_proj.weight"].to(torch.float16)
    os.makedirs(tmp_path / "m")
    write_safetensors(str(tmp_path / "m" / "model.safetensors"), tensors)
    got = load_weights(str(tmp_path / "m"), expected, optional)
    assert got["model.norm.weight"].dtype == torch.float32
    assert torch.equal(got["model.norm.weight"], tensors["model.norm.weight"])
    assert got["model.layers.0.mlp.up_proj.weight"].dtype == torch.float32           # half widens exactly
    assert got["model.embed_tokens.weight"].dtype == torch.bfloat16


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    expected, optional = model_tensors(Qwen3Config.from_dict(TINY_B).to_spec())
    tensors = random_tensors(expected, 1, torch.bfloat16)
    del tensors["model.layers.1.mlp.down_proj.weight"]
    del tensors["model.norm.weight"]
    tensors["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(16)
    tensors["model.layers.2.self_attn.q_proj.weight"] = torch.zeros(96, 96, dtype=torch.bfloat16)
    os.makedirs(tmp_path / "m")
    write_safetensors(str(tmp_path / "m" / "model.safetensors"), tensors)
    with pytest.raises(WeightError) as e:
        load_weights(str(tmp_path / "m"), expected, optional)
    err = e.value
    assert err.missing == ["model.layers.1.mlp.down_proj.weight", "model.norm.weight"]
    assert err.unexpected == ["model.layers.0.self_attn.rotary_emb.inv_freq"]
    assert err.wrong_shape == [("model.layers.2.self_attn.q_proj.weight", (192, 96), (96, 96))]
    text = str(err)
    for word in ("missing tensors (2)", "model.norm.weight", "unexpected tensors (1)", "inv_freq",
                 "shape mismatch for model.layers.2.self_attn.q_proj.weight: expected [192, 96], got [96, 96]"):
        assert word in text


def test_unread_tensors_are_a_note_unless_strict(tmp_path):
    """A checkpoint with a tensor that the model does not read loads (the reference reads what it asks for,
    candle-nn/src/var_builder.rs:501-529); the name is handed back, and `strict` makes it the one error."""
    spec = Qwen3Config.from_dict(TINY_A).to_spec()
    expected, optional = model_tensors(spec)
    tensors = random_tensors(generated_tensors(spec), 1, torch.bfloat16)
    tensors["model.layers.0.self_attn.rotary_emb.inv_freq"] = torch.zeros(8)
    os.makedirs(tmp_path / "m")
    write_safetensors(str(tmp_path / "m" / "model.safetensors"), tensors)
    unused = []
    got = load_weights(str(tmp_path / "m"), expected, optional, unused=unused)
    assert unused == ["model.layers.0.self_attn.rotary_emb.inv_freq"] and set(got) == set(generated_tensors(spec))
    with pytest.raises(WeightError, match=r"unexpected tensors \(1\): model.layers.0.self_attn.rotary_emb.inv_freq") as e:
        load_weights(str(tmp_path / "m"), expected, optional, strict=True)
    assert not e.value.missing and not e.value.wrong_shape


def test_truncated_and_malformed_files(tmp_path):
    folder = tmp_path / "m"
    os.makedirs(folder)
    expected, optional = model_tensors(Qwen3Config.from_dict(TINY_A).to_spec())
    with pytest.raises(SafetensorsError, match="No safetensors files"):
        load_weights(str(folder), expected, optional)
    good = tmp_path / "good.safetensors"
    write_safetensors(str(good), random_tensors(generated_tensors(Qwen3Config.from_dict(TINY_A).to_spec()), 1))
    blob = good.read_bytes()
    (folder / "model.safetensors").write_bytes(blob[: len(blob) // 2])
    with pytest.raises(SafetensorsError, match="truncated"):
        load_weights(str(folder), expected, optional)
    (folder / "model.safetensors").write_bytes(struct.pack("<Q", 5) + b"{nope")
    with pytest.raises(SafetensorsError, match="not valid JSON"):
        load_weights(str(folder), expected, optional)
    (folder / "model.safetensors").write_bytes(b"abc")
    with pytest.raises(SafetensorsError, match="truncated"):
        load_weights(str(folder), expected, optional)


def test_sharded_folders_and_last_file_wins(tmp_path):
    expected, optional = model_tensors(Qwen3Config.from_dict(TINY_A).to_spec())
    tensors = random_tensors(generated_tensors(Qwen3Config.from_dict(TINY_A).to_spec()), 1)
    names = sorted(tensors)
    folder = tmp_path / "m"
    os.makedirs(folder)
    write_safetensors(str(folder / "a-00001.safetensors"), {n: tensors[n] for n in names[:5]})
    second = {n: tensors[n] for n in names[5:]}
    second[names[0]] = tensors[names[0]] + 1          # a duplicate: the later file wins (safetensors.rs:461-487)
    write_safetensors(str(folder / "a-00002.safetensors"), second)
    got = load_weights(str(folder), expected, optional)
    assert torch.equal(got[names[0]], tensors[names[0]] + 1) and torch.equal(got[names[7]], tensors[names[7]])
    # an index file names the shards
    (folder / "model.safetensors.index.json").write_text(json.dumps(
        {"weight_map": {n: ("a-00001.safetensors" if i < 5 else "a-00002.safetensors") for i, n in enumerate(names)}}))
    assert set(load_weights(str(folder), expected, optional)) == set(names)


def test_write_random_model_writes_a_loadable_folder(tmp_path):
    folder = write_random_model(str(tmp_path / "m"), Qwen3Config.from_dict(TINY_A), seed=9)
    assert sorted(os.listdir(folder)) == ["config.json", "model.safetensors"]
    raw = json.load(open(os.path.join(folder, "config.json")))
    assert raw["architectures"] == ["Qwen3ForCausalLM"] and raw["head_dim"] == 16


def test_block_arrangements_and_model_ends_are_registered_parts():
    """The tensors of a model follow from its spec through the registered parts: a block of another arrangement
    with its own number of norms, no final norm, and an unknown arrangement named in the error."""
    from dataclasses import replace
    from inferrs_amd.parts import BlockBase, register_block
    from inferrs_amd.parts.block import part_tensors

    @register_block("test_three_norms")
    class ThreeNorms(BlockBase):
        @classmethod
        def tensors(cls, spec):
            return part_tensors(spec, 3)

    spec = Qwen3Config.from_dict(TINY_A).to_spec()
    base, _ = model_tensors(spec)
    layer0 = spec.layers[0]
    wide = replace(layer0, norms=layer0.norms + (layer0.norms[0],), norm_names=layer0.norm_names + ("extra.weight",),
                   arrangement="test_three_norms")
    other = replace(spec, layers=(wide,) + spec.layers[1:], final_norm=None, final_norm_name=None)
    other.validate()
    names, _ = model_tensors(other)
    assert set(names) == (set(base) | {"extra.weight"}) - {"model.norm.weight"}
    from inferrs_amd.config import SpecError
    with pytest.raises(SpecError, match="3 norms"):
        model_tensors(replace(spec, layers=(replace(layer0, arrangement="test_three_norms"),)))
    with pytest.raises(KeyError, match="no block is registered for the arrangement 'sideways'.*pre_norm"):
        model_tensors(replace(spec, layers=(replace(layer0, arrangement="sideways"),)))
    with pytest.raises(SpecError, match="come together"):
        replace(spec, final_norm=None).validate()


def test_stop_ids_of_a_folder(tmp_path):
    """config.json's ids first, then generation_config.json's, the tokenizer's EOS and the well-known end
    markers that the vocabulary holds (inferrs/src/tokenizer.rs:337-353), without repeats."""
    from inferrs_amd.config import folder_stop_ids
    folder = tmp_path / "m"
    os.makedirs(folder)
    assert folder_stop_ids(str(folder), (7,)) == (7,)
    (folder / "generation_config.json").write_text(json.dumps({"eos_token_id": [151645, 151643, 7]}))
    assert folder_stop_ids(str(folder), (7,)) == (7, 151645, 151643)
    (folder / "tokenizer_config.json").write_text(json.dumps({"eos_token": {"content": "<eos>"}}))
    (folder / "tokenizer.json").write_text(json.dumps({
        "model": {"vocab": {"a": 0, "<|end|>": 5, "<eos>": 9}},
        "added_tokens": [{"id": 151643, "content": "<|endoftext|>"}, {"id": 11, "content": "<|im_end|>"}, {"id": 3, "content": "x"}]}))
    assert folder_stop_ids(str(folder), ()) == (151645, 151643, 7, 9, 11, 5)
    (folder / "generation_config.json").write_text(json.dumps({"eos_token_id": "two"}))
    with pytest.raises(ConfigError, match="generation_config.json"):
        folder_stop_ids(str(folder), ())


def test_chat_template_comes_from_the_folder_or_the_architecture(tmp_path):
    from inferrs_amd import chat
    folder = tmp_path / "m"
    os.makedirs(folder)
    assert chat.detect_template(str(folder), Qwen3Config) == "chatml" and chat.detect_template(str(folder)) == "plain"
    (folder / "tokenizer_config.json").write_text(json.dumps({"chat_template": "{% for m in messages %}<|im_start|>..."}))
    assert chat.detect_template(str(folder)) == "chatml"
    assert chat.render("chatml", "hi", "be brief") == ("<|im_start|>system\nbe brief<|im_end|>\n<|im_start|>user\nhi<|im_end|>\n"
                                                      "<|im_start|>assistant\n")
    assert chat.render("plain", "hi") == "hi"


@pytest.mark.parametrize("key,value", [("attention_bias", True), ("rope_scaling", {"rope_type": "yarn", "factor": 4.0}),
                                       ("hidden_act", "gelu"), ("use_sliding_window", True),
                                       ("layer_types", ["full_attention", "sliding_attention"])])
def test_values_that_the_model_does_not_honour_are_refused(tmp_path, key, value):
    """The reference reads these keys and ignores them (`inferrs-models/src/config.rs:291-292`, `qwen3.rs:28-45`): a
    folder that asks for biases, a scaled rotation, a window or another activation would be computed as another model.
    Here the load fails and names key and value; `allow_ignored_keys` gives the reference's silence back."""
    raw = dict(TINY_A, **{key: value})
    with pytest.raises(ConfigError) as err:
        Qwen3Config.from_dict(raw)
    assert f"'{key}'" in str(err.value) and repr(value) in str(err.value)
    assert Qwen3Config.from_dict(raw, allow_ignored_keys=True) == Qwen3Config.from_dict(TINY_A)
    (tmp_path / "config.json").write_text(json.dumps(raw))
    with pytest.raises(ConfigError, match=key):
        load_config(str(tmp_path))
    assert load_config(str(tmp_path), allow_ignored_keys=True) == Qwen3Config.from_dict(TINY_A)


def test_values_that_change_nothing_are_accepted():
    """What real folders of this architecture hold: the keys are there, with the values that the model has anyway."""
    raw = dict(TINY_A, attention_bias=False, rope_scaling=None, hidden_act="silu", use_sliding_window=False,
               sliding_window=4096, max_window_layers=2, layer_types=["full_attention", "full_attention"],
               attention_dropout=0.0, torch_dtype="bfloat16")
    assert Qwen3Config.from_dict(raw) == Qwen3Config.from_dict(TINY_A)


def test_several_unhonoured_values_are_named_together():
    with pytest.raises(ConfigError) as err:
        Qwen3Config.from_dict(dict(TINY_A, attention_bias=True, hidden_act="gelu_pytorch_tanh"))
    assert "'attention_bias' = True" in str(err.value) and "'hidden_act' = 'gelu_pytorch_tanh'" in str(err.value)
