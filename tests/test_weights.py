"""Weights: loading by name, dtype rules, the one error that lists everything, random mode (no GPU)."""

import json

import pytest
import torch
from safetensors.torch import load_file, save_file

from helpers import TINIES, TINY_A, TINY_B, write_tiny_model
from simple_inference_amd.config import EngineConfig
from simple_inference_amd.engine import build_model
from simple_inference_amd.weights import WeightError, load_weights, random_tensors, write_model_folder


def expected_of(cfg):
    model, _ = build_model(cfg, EngineConfig(device="cpu", dtype="float32", max_seq_len=64), kernels=None)
    return model.expected_tensors()


def test_expected_tensors_have_the_checkpoint_names_and_shapes():
    exp = expected_of(TINY_B)
    assert exp["model.embed_tokens.weight"].shape == (384, 96)
    assert exp["model.layers.2.self_attn.k_proj.weight"].shape == (32, 96)
    assert exp["model.layers.0.mlp.down_proj.weight"].shape == (96, 224)
    assert exp["model.norm.weight"].shape == (96,) and exp["model.norm.weight"].role == "vector"
    assert exp["lm_head.weight"].shape == (384, 96)
    assert "lm_head.weight" not in expected_of(TINY_A)          # tied: the head is the embedding
    assert len(exp) == 1 + 3 * 9 + 1 + 1


def test_random_folder_reads_back_and_is_seeded(tmp_path):
    a = write_tiny_model(tmp_path / "a", TINIES["a"], seed=5)
    b = write_tiny_model(tmp_path / "b", TINIES["a"], seed=5)
    c = write_tiny_model(tmp_path / "c", TINIES["a"], seed=6)
    ta, tb, tc = (load_file(str(p / "model.safetensors")) for p in (a, b, c))
    assert all(torch.equal(ta[k], tb[k]) for k in ta) and any(not torch.equal(ta[k], tc[k]) for k in ta)
    assert all(v.dtype == torch.bfloat16 for v in ta.values())
    gains = ta["model.norm.weight"].float()
    assert abs(gains.mean() - 1.0) < 0.1 and 0.03 < gains.std() < 0.3     # 1 + N(0, 0.1)
    assert abs(ta["model.embed_tokens.weight"].float().std() - 0.02) < 0.005
    assert json.loads((a / "config.json").read_text())["architectures"] == ["LlamaForCausalLM"]
    exp = expected_of(TINY_A)
    loaded = load_weights(a, exp, "cpu", torch.float32)
    assert set(loaded) == set(exp)
    assert torch.equal(loaded["model.embed_tokens.weight"], ta["model.embed_tokens.weight"].float())


def test_dtype_rules(tmp_path):
    exp = expected_of(TINY_A)
    t = random_tensors(exp, 0, storage="bfloat16")
    t["model.layers.0.mlp.up_proj.weight"] = t["model.layers.0.mlp.up_proj.weight"].float()  # stored in 32 bit
    write_model_folder(tmp_path, TINY_A, t)
    bf = load_weights(tmp_path, exp, "cpu", torch.bfloat16)
    assert bf["model.embed_tokens.weight"].dtype == torch.bfloat16          # stays bfloat16
    assert bf["model.layers.0.mlp.up_proj.weight"].dtype == torch.float32   # stored in 32 bit: stays so
    assert bf["model.norm.weight"].dtype == torch.float32                   # small vectors are held in float32
    f32 = load_weights(tmp_path, exp, "cpu", torch.float32)
    assert all(v.dtype == torch.float32 for v in f32.values())
    assert torch.equal(f32["model.embed_tokens.weight"], bf["model.embed_tokens.weight"].float())  # widened exactly


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    exp = expected_of(TINY_A)
    t = random_tensors(exp, 0)
    del t["model.layers.1.self_attn.o_proj.weight"], t["model.norm.weight"]
    t["model.layers.0.mlp.gate_proj.weight"] = torch.zeros(64, 128, dtype=torch.bfloat16)   # transposed
    t["model.layers.7.mlp.gate_proj.weight"] = torch.zeros(2, 2)
    t["lm_head.weight"] = torch.zeros(256, 64)
    write_model_folder(tmp_path, TINY_A, t)
    with pytest.raises(WeightError) as e:
        load_weights(tmp_path, exp, "cpu", torch.float32)
    err = e.value
    assert err.missing == ["model.layers.1.self_attn.o_proj.weight", "model.norm.weight"]
    assert err.unexpected == ["lm_head.weight", "model.layers.7.mlp.gate_proj.weight"]
    assert err.wrong_shape == [("model.layers.0.mlp.gate_proj.weight", (64, 128), (128, 64))]
    text = str(err)
    for word in ("missing (2)", "unexpected (2)", "wrong shape (1)", "o_proj", "lm_head", "[64, 128]", "[128, 64]"):
        assert word in text


def test_sharded_checkpoint_and_missing_files(tmp_path):
    exp = expected_of(TINY_A)
    t = random_tensors(exp, 1)
    names = list(t)
    half = len(names) // 2
    save_file({k: t[k] for k in names[:half]}, str(tmp_path / "model-00001-of-00002.safetensors"))
    save_file({k: t[k] for k in names[half:]}, str(tmp_path / "model-00002-of-00002.safetensors"))
    index = {"weight_map": {k: ("model-00001-of-00002.safetensors" if i < half else "model-00002-of-00002.safetensors")
                            for i, k in enumerate(names)}}
    (tmp_path / "model.safetensors.index.json").write_text(json.dumps(index))
    loaded = load_weights(tmp_path, exp, "cpu", torch.bfloat16)
    assert torch.equal(loaded[names[-1]], t[names[-1]].to(loaded[names[-1]].dtype))
    (tmp_path / "model-00002-of-00002.safetensors").unlink()
    with pytest.raises(FileNotFoundError, match="00002"):
        load_weights(tmp_path, exp, "cpu", torch.bfloat16)
    with pytest.raises(FileNotFoundError, match="model.safetensors"):
        load_weights(tmp_path / "nothing_here", exp, "cpu", torch.bfloat16)


def test_untied_head_is_a_tensor_of_its_own(tmp_path):
    from twins import TwinKernels
    from simple_inference_amd.engine import model_from_folder
    folder = write_tiny_model(tmp_path, TINIES["b"], seed=2)
    model, _ = model_from_folder(folder, EngineConfig(device="cpu", dtype="float32", max_seq_len=64), TwinKernels())
    assert model.head.weight.data_ptr() != model.embedding.weight.data_ptr()
    folder = write_tiny_model(tmp_path / "tied", TINIES["a"], seed=2)
    model, _ = model_from_folder(folder, EngineConfig(device="cpu", dtype="float32", max_seq_len=64), TwinKernels())
    assert model.head.weight.data_ptr() == model.embedding.weight.data_ptr()     # tied: same storage


def test_a_tied_model_stored_with_its_head_is_taken_if_the_head_repeats_the_embedding(tmp_path):
    """The reference reads an ``lm_head.weight`` that a tied checkpoint also stores (``model/llama.py:147-154``).
    Here it is passed over when it repeats the embedding, and refused with both names when it does not: the
    configuration says one matrix, the file holds two."""
    from twins import TwinKernels
    from simple_inference_amd.engine import model_from_folder
    ecfg = EngineConfig(device="cpu", dtype="float32", max_seq_len=64)
    exp = expected_of(TINY_A)
    t = random_tensors(exp, 3)
    t["lm_head.weight"] = t["model.embed_tokens.weight"].clone()
    write_model_folder(tmp_path / "same", TINY_A, t)
    model, _ = model_from_folder(tmp_path / "same", ecfg, TwinKernels())
    assert model.head.weight.data_ptr() == model.embedding.weight.data_ptr()
    t["lm_head.weight"][3, 5] += 1.0
    write_model_folder(tmp_path / "other", TINY_A, t)
    with pytest.raises(WeightError, match="lm_head.weight is not equal to model.embed_tokens.weight") as e:
        model_from_folder(tmp_path / "other", ecfg, TwinKernels())
    assert e.value.differing == [("lm_head.weight", "model.embed_tokens.weight")] and not e.value.unexpected
    t["lm_head.weight"] = torch.zeros(3, 64, dtype=torch.bfloat16)
    write_model_folder(tmp_path / "shape", TINY_A, t)
    with pytest.raises(WeightError) as e:
        model_from_folder(tmp_path / "shape", ecfg, TwinKernels())
    assert e.value.wrong_shape == [("lm_head.weight", (3, 64), (256, 64))]
    # an untied model has a head of its own: nothing there may be stored twice
    model, _ = build_model(TINY_B, ecfg, kernels=None)
    assert model.plan.duplicates == {}


def test_the_parts_hold_as_many_parameters_as_the_configuration_counts():
    """Reference: ``loader.py:301-316`` checks the loaded total against the model's known size."""
    from simple_inference_amd import preset
    from simple_inference_amd.engine.build import count_parameters, describe
    ecfg = EngineConfig(device="cpu", dtype="bfloat16", max_seq_len=64)
    for name, total in (("llama-3.2-3b", 3_212_749_824), ("llama-3.2-1b", 1_235_814_400), ("llama-3.1-8b", 8_030_261_248)):
        model, cfg = build_model(preset(name), ecfg, kernels=None)
        assert count_parameters(model, cfg) == total
    assert "3,212,749,824 parameters" not in describe(model, cfg, ecfg) and "131,072 bytes of cache a token" in describe(model, cfg, ecfg)
    model, cfg = build_model(TINY_B, ecfg, kernels=None)
    object.__setattr__(cfg, "intermediate_size", cfg.intermediate_size + 1)
    with pytest.raises(ValueError, match="formula"):
        count_parameters(model, cfg)
