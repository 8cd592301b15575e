"""Safetensors reading, checkpoint validation and random weights (CPU)."""

import json

import pytest
import torch

from llm_runtime_study_amd.config import config_from_dict, spec_for
from llm_runtime_study_amd.errors import CheckpointError, CheckpointValidationError
from llm_runtime_study_amd.models import DecoderModel
from llm_runtime_study_amd.weights import Checkpoint, load, random_tensors, validate, write_model_dir, write_safetensors
from tests.helpers import TINY_A, TINY_B, qwen3_tensor_shapes


def expected_for(raw):
    return DecoderModel(spec_for(config_from_dict(raw))).tensors()


def test_schema_names_and_count():
    # 11 tensors a layer + embedding, final norm, head (reference tests/test_checkpoint.py: 11 L + 3)
    raw = dict(TINY_B, attention_bias=False)
    expected = expected_for(raw)
    assert len(expected) == 11 * raw["num_hidden_layers"] + 3
    assert {k: v.shape for k, v in expected_for(TINY_B).items()} == qwen3_tensor_shapes(TINY_B)
    tied = expected_for(TINY_A)
    assert tied["lm_head.weight"].optional and not tied["model.embed_tokens.weight"].optional


def test_written_folder_reads_back_identically_with_both_readers(tmp_path):
    from safetensors.torch import load_file

    config = config_from_dict(TINY_B)
    write_model_dir(config, 3, tmp_path, init="scaled")
    checkpoint = Checkpoint.from_model_dir(tmp_path)
    theirs = load_file(str(tmp_path / "model.safetensors"))
    assert set(theirs) == set(checkpoint.manifest)
    for name, tensor in theirs.items():
        assert torch.equal(tensor, checkpoint.tensor(name)) and tensor.dtype == torch.bfloat16
    weights = load(checkpoint, expected_for(TINY_B), "qwen3", "cpu")
    assert all(t.dtype == torch.bfloat16 for t in weights.values())
    # same seed, same folder; another seed, other weights
    again = random_tensors(expected_for(TINY_B), 3, torch.bfloat16, "scaled")
    other = random_tensors(expected_for(TINY_B), 4, torch.bfloat16, "scaled")
    assert torch.equal(again["lm_head.weight"], weights["lm_head.weight"])
    assert not torch.equal(other["lm_head.weight"], weights["lm_head.weight"])


def test_all_problems_are_reported_in_one_error(tmp_path):
    expected = expected_for(TINY_A)
    tensors = random_tensors(expected, 0, torch.bfloat16)
    del tensors["model.layers.1.mlp.up_proj.weight"]
    del tensors["model.norm.weight"]
    tensors["model.layers.0.self_attn.rotary.inv_freq"] = torch.zeros(8)
    tensors["model.layers.0.self_attn.q_proj.weight"] = torch.zeros(64, 63, dtype=torch.bfloat16)
    tensors["model.layers.0.input_layernorm.weight"] = torch.zeros(64, dtype=torch.int32)
    tensors["model.layers.1.mlp.down_proj.weight"] = tensors["model.layers.1.mlp.down_proj.weight"].half()
    write_safetensors(tmp_path / "model.safetensors", tensors)
    with pytest.raises(CheckpointValidationError) as info:
        validate(Checkpoint.from_model_dir(tmp_path), expected, "qwen3", "bfloat16")
    text = str(info.value)
    # the configuration's dtype is the one every floating tensor must have (reference checkpoint.py:478-481)
    assert "dtype mismatch for model.layers.1.mlp.down_proj.weight: expected BF16, got F16" in text
    assert "dtype mismatch for model.layers.0.input_layernorm.weight: expected BF16, got I32" in text
    assert text.count("\n  - ") == 5   # one line for each kind of problem and each tensor at fault: nothing is reported twice
    assert text.startswith("checkpoint does not match qwen3 configuration:")
    assert "missing tensors: model.layers.1.mlp.up_proj.weight, model.norm.weight" in text
    assert "unexpected tensors: model.layers.0.self_attn.rotary.inv_freq" in text
    assert "shape mismatch for model.layers.0.self_attn.q_proj.weight: expected (64, 64), got (64, 63)" in text
    assert "dtype mismatch for model.layers.0.input_layernorm.weight" in text


def test_tied_head_is_optional_and_untied_head_is_required(tmp_path):
    tied = expected_for(TINY_A)
    write_safetensors(tmp_path / "model.safetensors", random_tensors(tied, 0, torch.bfloat16))
    validate(Checkpoint.from_model_dir(tmp_path), tied, "qwen3")
    untied = expected_for(dict(TINY_A, tie_word_embeddings=False))
    with pytest.raises(CheckpointValidationError, match="missing tensors: lm_head.weight"):
        validate(Checkpoint.from_model_dir(tmp_path), untied, "qwen3")


def test_dtype_follows_the_configuration(tmp_path):
    """BF16 for torch_dtype bfloat16, F32 for float32, F16 for float16; anything else is named in the error."""
    expected = expected_for(TINY_A)
    for stored, config_dtype, container in ((torch.bfloat16, "bfloat16", "BF16"), (torch.float32, "float32", "F32"), (torch.float16, "float16", "F16")):
        write_safetensors(tmp_path / "model.safetensors", random_tensors(expected, 0, stored))
        checkpoint = Checkpoint.from_model_dir(tmp_path)
        validate(checkpoint, expected, "qwen3", config_dtype)
        for other in {"bfloat16", "float32", "float16"} - {config_dtype}:
            with pytest.raises(CheckpointValidationError, match=f"dtype mismatch for lm_head.weight: expected .*, got {container}|dtype mismatch for model.embed_tokens.weight: expected .*, got {container}"):
                validate(checkpoint, expected, "qwen3", other)
        checkpoint.close()
    with pytest.raises(CheckpointValidationError, match="unsupported checkpoint dtype 'float64'"):
        validate(Checkpoint.from_model_dir(tmp_path), expected, "qwen3", "float64")


def test_a_model_folder_is_checked_against_its_own_torch_dtype(tmp_path):
    """Through the path Engine.from_model_dir takes: a folder whose tensors are not in the configuration's
    dtype is refused, unless the caller asks for the stored precision."""
    from llm_runtime_study_amd.engine.loading import load_model

    config = config_from_dict(TINY_A)
    write_model_dir(config, 1, tmp_path)
    expected = expected_for(TINY_A)
    tensors = random_tensors(expected, 1, torch.bfloat16)
    tensors["model.norm.weight"] = tensors["model.norm.weight"].float()
    write_safetensors(tmp_path / "model.safetensors", tensors)
    with pytest.raises(CheckpointValidationError, match="dtype mismatch for model.norm.weight: expected BF16, got F32"):
        load_model(tmp_path, torch.float32, "cpu")


def test_stored_precision_is_kept_when_asked_for(tmp_path):
    expected = expected_for(TINY_A)
    tensors = random_tensors(expected, 0, torch.bfloat16)
    tensors["model.norm.weight"] = tensors["model.norm.weight"].float() + 1e-4   # stored in 32-bit: stays so
    tensors["model.layers.0.mlp.down_proj.weight"] = tensors["model.layers.0.mlp.down_proj.weight"].half()
    write_safetensors(tmp_path / "model.safetensors", tensors)
    with pytest.raises(CheckpointValidationError, match="expected BF16, got F32"):
        load(Checkpoint.from_model_dir(tmp_path), expected, "qwen3", "cpu", "bfloat16")
    weights = load(Checkpoint.from_model_dir(tmp_path), expected, "qwen3", "cpu", checkpoint_dtype=None)
    assert weights["model.norm.weight"].dtype == torch.float32
    assert torch.equal(weights["model.norm.weight"], tensors["model.norm.weight"])
    assert weights["model.layers.0.mlp.down_proj.weight"].dtype == torch.float32   # float16 is widened
    assert weights["model.embed_tokens.weight"].dtype == torch.bfloat16


def test_sharded_checkpoint_merges_headers(tmp_path):
    expected = expected_for(TINY_A)
    tensors = random_tensors(expected, 5, torch.bfloat16)
    names = sorted(tensors)
    first, second = names[: len(names) // 2], names[len(names) // 2:]
    write_safetensors(tmp_path / "model-00001-of-00002.safetensors", {n: tensors[n] for n in first})
    write_safetensors(tmp_path / "model-00002-of-00002.safetensors", {n: tensors[n] for n in second})
    weight_map = {n: "model-00001-of-00002.safetensors" for n in first}
    weight_map.update({n: "model-00002-of-00002.safetensors" for n in second})
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps({"weight_map": weight_map}))
    checkpoint = Checkpoint.from_model_dir(tmp_path)
    assert list(checkpoint.manifest) == names
    weights = load(checkpoint, expected, "qwen3", "cpu")
    assert all(torch.equal(weights[n], tensors[n]) for n in names)
    (tmp_path / "model-00002-of-00002.safetensors").unlink()
    with pytest.raises(CheckpointError, match="checkpoint shard does not exist"):
        Checkpoint.from_model_dir(tmp_path)


def test_file_errors(tmp_path):
    with pytest.raises(CheckpointError, match="neither model.safetensors nor model.safetensors.index.json"):
        Checkpoint.from_model_dir(tmp_path)
    (tmp_path / "model.safetensors").write_bytes(b"\x05\x00\x00")
    with pytest.raises(CheckpointError, match="too short"):
        Checkpoint.from_model_dir(tmp_path)
    (tmp_path / "model.safetensors").write_bytes((10**9).to_bytes(8, "little") + b"{}")
    with pytest.raises(CheckpointError, match="bad header length"):
        Checkpoint.from_model_dir(tmp_path)
    write_safetensors(tmp_path / "model.safetensors", {"a": torch.zeros(2)})
    with pytest.raises(CheckpointError, match="tensor is not in the checkpoint: b"):
        Checkpoint.from_model_dir(tmp_path).tensor("b")


def test_lazy_load_reads_a_tensor_when_it_is_asked_for(tmp_path, monkeypatch):
    """load(..., lazy=True): validated as a whole at once, the same tensors as the eager load, and no tensor's bytes
    are touched before a part asks for it; views by prefix (what a model hands its parts) keep that."""
    from llm_runtime_study_amd.parts import LazyTensors, under

    config = config_from_dict(TINY_B)
    write_model_dir(config, 3, tmp_path, init="scaled")
    expected = expected_for(TINY_B)
    checkpoint = Checkpoint.from_model_dir(tmp_path)
    eager = load(checkpoint, expected, "qwen3", "cpu")
    read = []
    original = Checkpoint.tensor
    monkeypatch.setattr(Checkpoint, "tensor", lambda self, name: (read.append(name), original(self, name))[1])
    lazy = load(checkpoint, expected, "qwen3", "cpu", lazy=True)
    assert isinstance(lazy, LazyTensors) and read == []
    assert list(lazy) == list(eager) and len(lazy) == len(eager) and "lm_head.weight" in lazy and "nothing" not in lazy
    layer = under(lazy, "model.layers.1.")
    mixer = under(layer, "self_attn.")
    assert read == [] and "q_proj.weight" in mixer and "gate_proj.weight" not in mixer
    assert sorted(mixer) == sorted(n[len("model.layers.1.self_attn."):] for n in eager if n.startswith("model.layers.1.self_attn."))
    assert torch.equal(mixer["q_proj.weight"], eager["model.layers.1.self_attn.q_proj.weight"])
    assert read == ["model.layers.1.self_attn.q_proj.weight"]
    assert mixer.get("nothing") is None and lazy.get("nothing") is None
    with pytest.raises(KeyError):
        lazy["nothing"]
    assert all(torch.equal(lazy[n], eager[n]) for n in eager)
    # a checkpoint that does not fit is refused before anything is read, lazily or not
    read.clear()
    with pytest.raises(CheckpointValidationError):
        load(checkpoint, expected_for(TINY_A), "qwen3", "cpu", lazy=True)
    assert read == []


def test_a_model_binds_lazy_tensors_as_it_binds_a_dictionary(tmp_path):
    """DecoderModel.bind with tensors made on demand: the same bound weights as with all of them in a dictionary."""
    from llm_runtime_study_amd.config import spec_for
    from llm_runtime_study_amd.models import DecoderModel

    config = config_from_dict(TINY_B)
    write_model_dir(config, 7, tmp_path, init="scaled")
    spec = spec_for(config)
    checkpoint = Checkpoint.from_model_dir(tmp_path)
    one, other = DecoderModel(spec), DecoderModel(spec)
    one.bind(load(checkpoint, one.tensors(), "qwen3", "cpu"), torch.bfloat16)
    other.bind(load(checkpoint, other.tensors(), "qwen3", "cpu", lazy=True), torch.bfloat16)
    assert torch.equal(one.embedding, other.embedding) and torch.equal(one.head, other.head)
    for a, b in zip(one.layers, other.layers):
        assert torch.equal(a.mixer.w_qkv, b.mixer.w_qkv) and torch.equal(a.mixer.b_qkv, b.mixer.b_qkv)
        assert torch.equal(a.mixer.w_o, b.mixer.w_o) and torch.equal(a.feed_forward.down, b.feed_forward.down)
        assert torch.equal(a.mixer_norm.weight, b.mixer_norm.weight)
