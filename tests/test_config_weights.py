"""Configuration, registry, weight loading and the random-weights mode (no GPU)."""

from __future__ import annotations

import json

import pytest
import torch
from safetensors.torch import load_file, save_file

from llmserve_amd import ConfigError, Qwen2Config, WeightsError, resolve_architecture
from llmserve_amd.parts import AttentionSpec, PagedKeyValue
from llmserve_amd.registry import ARCHITECTURES
from llmserve_amd.weights import load_model_folder, write_model_folder
from tests.tiny import TINY_A, TINY_B

QWEN_1_5B = {
    "architectures": ["Qwen2ForCausalLM"], "model_type": "qwen2", "hidden_act": "silu",
    "vocab_size": 151936, "hidden_size": 1536, "intermediate_size": 8960, "num_hidden_layers": 28,
    "num_attention_heads": 12, "num_key_value_heads": 2, "max_position_embeddings": 32768,
    "rope_theta": 1000000.0, "rms_norm_eps": 1e-06, "tie_word_embeddings": True,
    "sliding_window": 32768, "max_window_layers": 21, "use_sliding_window": False, "torch_dtype": "bfloat16",
    "transformers_version": "4.43.1",
}


def test_reads_the_architectures_own_keys():
    config = Qwen2Config.from_dict(QWEN_1_5B)
    assert (config.num_layers, config.head_dim, config.attention_bias) == (28, 128, True)
    assert config.rope_pairing == "half" and config.layer_window(27) is None  # a published checkpoint's config
    plain_folder = {k: v for k, v in QWEN_1_5B.items() if k != "transformers_version"}
    assert Qwen2Config.from_dict(plain_folder).rope_pairing == "adjacent"  # the reference's rotation (model.py:39-42)
    assert Qwen2Config.from_dict({**plain_folder, "rope_pairing": "half"}).rope_pairing == "half"
    # the reference's aliases (config.py:46-54)
    aliased = dict(QWEN_1_5B)
    aliased["num_layers"] = aliased.pop("num_hidden_layers")
    aliased["max_seq_len"] = aliased.pop("max_position_embeddings")
    assert Qwen2Config.from_dict(aliased) == config
    assert Qwen2Config.from_dict(config.to_config_json()) == config


def test_no_size_has_a_default():
    for key in ("vocab_size", "hidden_size", "intermediate_size", "num_hidden_layers", "num_attention_heads",
                "num_key_value_heads", "max_position_embeddings", "rope_theta", "rms_norm_eps"):
        values = dict(QWEN_1_5B)
        del values[key]
        with pytest.raises(ConfigError, match=key):
            Qwen2Config.from_dict(values)


def test_rejects_what_it_cannot_run():
    for change in ({"model_type": "llama"}, {"rope_scaling": {"type": "yarn", "factor": 4.0}}, {"hidden_act": "gelu"},
                   {"num_key_value_heads": 5}, {"vocab_size": "many"}, {"rope_pairing": "odd"},
                   {"hidden_size": 1537}, {"use_sliding_window": True, "sliding_window": None}):
        with pytest.raises(ConfigError):
            Qwen2Config.from_dict({**QWEN_1_5B, **change})


def test_window_layers():
    config = Qwen2Config.from_dict({**QWEN_1_5B, "use_sliding_window": True, "sliding_window": 4096})
    assert [config.layer_window(i) for i in (0, 20, 21, 27)] == [None, None, 4096, 4096]


def test_registry_chooses_by_config_json():
    assert resolve_architecture(QWEN_1_5B).name == "Qwen2ForCausalLM"
    assert resolve_architecture({"model_type": "qwen2"}).name == "Qwen2ForCausalLM"  # checkpoint.py:34-36
    with pytest.raises(ConfigError, match="LlamaForCausalLM"):
        resolve_architecture({"architectures": ["LlamaForCausalLM"], "model_type": "llama"})


def test_spec_is_chosen_layer_by_layer():
    spec = ARCHITECTURES["Qwen2ForCausalLM"].build_spec(TINY_B)
    mixers = [layer.block.mixer for layer in spec.layers]
    assert all(isinstance(m, AttentionSpec) for m in mixers)
    assert [m.window for m in mixers] == [None, 24, 24]
    assert spec.cell_need(0) == PagedKeyValue(1, 32, None) and spec.cell_need(2) == PagedKeyValue(1, 32, 24)
    names = spec.tensors()
    assert names["model.layers.2.self_attn.k_proj.bias"].shape == (32,)
    assert names["model.layers.0.mlp.down_proj.weight"].shape == (192, 320)
    assert names["lm_head.weight"].shape == (384, 192)
    tied = ARCHITECTURES["Qwen2ForCausalLM"].build_spec(TINY_A).tensors()
    assert "lm_head.weight" not in tied and len(tied) == 1 + 2 * 12 + 1


def test_random_folder_is_seeded_by_name(tmp_path):
    first = load_file(write_model_folder(tmp_path / "a", TINY_A, seed=4) / "model.safetensors")
    again = load_file(write_model_folder(tmp_path / "b", TINY_A, seed=4) / "model.safetensors")
    other = load_file(write_model_folder(tmp_path / "c", TINY_A, seed=5) / "model.safetensors")
    assert first.keys() == again.keys()
    assert all(torch.equal(first[name], again[name]) for name in first)
    assert not torch.equal(first["model.embed_tokens.weight"], other["model.embed_tokens.weight"])
    assert first["model.embed_tokens.weight"].dtype == torch.bfloat16
    assert torch.equal(first["model.norm.weight"], torch.ones(64, dtype=torch.bfloat16))
    assert first["model.layers.0.self_attn.q_proj.bias"].float().std() > 0.01  # biases are drawn, not zero
    assert json.loads((tmp_path / "a" / "config.json").read_text())["architectures"] == ["Qwen2ForCausalLM"]


def test_loader_keeps_types(model_folders):
    in_half = load_model_folder(model_folders["B"], "bfloat16")
    assert in_half.tensors["model.layers.0.mlp.up_proj.weight"].dtype == torch.bfloat16
    assert in_half.tensors["model.norm.weight"].dtype == torch.float32  # stored in 32-bit, stays so
    in_full = load_model_folder(model_folders["B"], "float32")
    assert {t.dtype for t in in_full.tensors.values()} == {torch.float32}
    torch.testing.assert_close(
        in_full.tensors["model.embed_tokens.weight"], in_half.tensors["model.embed_tokens.weight"].float(), rtol=0, atol=0
    )
    with pytest.raises(ValueError, match="bfloat16 or float32"):
        load_model_folder(model_folders["B"], "float16")


def _rewrite(folder, tmp_path, change):
    tensors = load_file(folder / "model.safetensors")
    change(tensors)
    target = tmp_path / "changed"
    target.mkdir()
    (target / "config.json").write_text((folder / "config.json").read_text())
    save_file(tensors, str(target / "model.safetensors"))
    return target


def test_one_error_lists_everything_wrong(model_folders, tmp_path):
    def change(tensors):
        del tensors["model.layers.1.mlp.up_proj.weight"]
        del tensors["model.norm.weight"]
        tensors["model.layers.0.self_attn.q_proj.weight"] = torch.zeros(64, 63, dtype=torch.bfloat16)
        tensors["model.layers.7.extra.weight"] = torch.zeros(2)
        tensors["model.layers.0.self_attn.k_proj.bias"] = torch.zeros(32, dtype=torch.int32)

    folder = _rewrite(model_folders["A"], tmp_path, change)
    with pytest.raises(WeightsError) as caught:
        load_model_folder(folder, "float32")
    error = caught.value
    assert error.missing == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert error.unexpected == ["model.layers.7.extra.weight"]
    assert error.wrong_shapes == [("model.layers.0.self_attn.q_proj.weight", (64, 63), (64, 64))]
    assert error.wrong_types[0][0] == "model.layers.0.self_attn.k_proj.bias"
    for fragment in ("missing (2)", "unexpected (1)", "[64, 63]", "[64, 64]", "up_proj"):
        assert fragment in str(error)


def test_names_with_or_without_model_prefix_and_a_tied_head(model_folders, tmp_path):
    def change(tensors):
        for name in list(tensors):
            tensors[name.removeprefix("model.")] = tensors.pop(name)  # checkpoint.py:52
        tensors["lm_head.weight"] = tensors["embed_tokens.weight"].clone()  # a tied head that equals the embedding

    loaded = load_model_folder(_rewrite(model_folders["A"], tmp_path, change), "float32")
    assert "lm_head.weight" not in loaded.tensors and "model.embed_tokens.weight" in loaded.tensors


def test_a_tied_head_that_differs_is_unexpected(model_folders, tmp_path):
    def change(tensors):
        tensors["lm_head.weight"] = tensors["model.embed_tokens.weight"] + 1

    with pytest.raises(WeightsError, match="unexpected"):
        load_model_folder(_rewrite(model_folders["A"], tmp_path, change), "float32")


def test_missing_files(tmp_path, model_folders):
    with pytest.raises(FileNotFoundError):
        load_model_folder(tmp_path, "float32")
    (tmp_path / "config.json").write_text((model_folders["A"] / "config.json").read_text())
    with pytest.raises(FileNotFoundError, match="safetensors"):
        load_model_folder(tmp_path, "float32")  # checkpoint.py:47-48


def test_an_architecture_may_adapt_the_files_tensors_to_its_parts(tmp_path):
    """A checkpoint that stores q, k and v as one fused tensor loads through an architecture registered with
    `adapt_tensors`, which cuts it where the attention part expects three; the parts and the loader are
    unchanged, and what does not fit is still reported in one error."""
    import dataclasses
    import json

    from safetensors.torch import load_file, save_file

    from llmserve_amd import WeightsError, load_model_folder, write_model_folder
    from llmserve_amd.models.qwen2 import qwen2_spec
    from llmserve_amd.registry import register_architecture, unregister_architecture
    from tests.tiny import TINY_A

    @dataclasses.dataclass(frozen=True)
    class FusedConfig(type(TINY_A)):
        architecture = "FusedQwen2ForCausalLM"

    def cut(found, config):
        adapted = {}
        q, kv = config.num_attention_heads * config.head_dim, config.num_key_value_heads * config.head_dim
        for name, tensor in found.items():
            if ".qkv_proj." in name:
                for piece, part in zip(("q_proj", "k_proj", "v_proj"), torch.split(tensor, [q, kv, kv])):
                    adapted[name.replace("qkv_proj", piece)] = part
            else:
                adapted[name] = tensor
        return adapted

    register_architecture("FusedQwen2ForCausalLM", FusedConfig, qwen2_spec, adapt_tensors=cut)
    try:
        plain_folder = write_model_folder(tmp_path / "plain", TINY_A, seed=3)
        tensors = load_file(str(plain_folder / "model.safetensors"))
        fused = {}
        for name, tensor in tensors.items():
            if ".q_proj." in name:
                k, v = tensors[name.replace("q_proj", "k_proj")], tensors[name.replace("q_proj", "v_proj")]
                fused[name.replace("q_proj", "qkv_proj")] = torch.cat([tensor, k, v])
            elif ".k_proj." not in name and ".v_proj." not in name:
                fused[name] = tensor
        folder = tmp_path / "fused"
        folder.mkdir()
        values = json.loads((plain_folder / "config.json").read_text())
        values["architectures"] = ["FusedQwen2ForCausalLM"]
        (folder / "config.json").write_text(json.dumps(values))
        save_file(fused, str(folder / "model.safetensors"))
        loaded, reference = load_model_folder(folder, "float32"), load_model_folder(plain_folder, "float32")
        assert loaded.architecture.name == "FusedQwen2ForCausalLM" and set(loaded.tensors) == set(reference.tensors)
        assert all(torch.equal(loaded.tensors[name], reference.tensors[name]) for name in reference.tensors)
        del fused["model.layers.1.self_attn.qkv_proj.bias"]
        save_file(fused, str(folder / "model.safetensors"))
        with pytest.raises(WeightsError, match="q_proj.bias"):
            load_model_folder(folder, "float32")
    finally:
        unregister_architecture("FusedQwen2ForCausalLM")
