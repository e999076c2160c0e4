"""Configuration and the architecture registry."""
import json

import pytest

import helpers
from bare_cuda_4gib_amd.config import (Architecture, LlamaConfig, ModelConfig, architecture_for, load_config,
                                       register_architecture, registered_architectures)
from bare_cuda_4gib_amd.config.registry import unregister_architecture
from bare_cuda_4gib_amd.errors import ConfigError


def test_keys_and_defaults():
    # defaults as the reference's converter applies them (tools/convert/convert_weights.py:35-46)
    cfg = LlamaConfig.from_dict(dict(vocab_size=100, hidden_size=48, num_hidden_layers=2,
                                     num_attention_heads=4, intermediate_size=64))
    assert (cfg.num_kv_heads, cfg.head_dim, cfg.max_seq_len, cfg.rope_theta, cfg.rms_norm_eps) == (4, 12, 2048, 10000.0, 1e-5)
    assert cfg.tie_word_embeddings is False
    cfg = LlamaConfig.from_dict(helpers.TINY_C)
    assert cfg.head_dim == 48 and cfg.hidden_size == 80          # an explicit head_dim is honoured
    assert cfg.to_dict()["num_key_value_heads"] == 2


@pytest.mark.parametrize("change,word", [
    (dict(vocab_size=None), "vocab_size"), (dict(hidden_size="64"), "integer"),
    (dict(num_key_value_heads=3), "multiple"), (dict(head_dim=15), "even"),
    (dict(hidden_act="gelu"), "hidden_act"), (dict(attention_bias=True), "bias"),
    (dict(rope_scaling={"type": "linear", "factor": 2.0}), "rope_scaling"),
    (dict(rope_theta=-1.0), "rope_theta"), (dict(num_hidden_layers=0), "positive"),
    (dict(hidden_size=66), "multiple"), (dict(rms_norm_eps=float("inf")), "finite"),
])
def test_refusals(change, word):
    raw = dict(helpers.TINY_A)
    for k, v in change.items():
        if v is None:
            raw.pop(k)
        else:
            raw[k] = v
    with pytest.raises(ConfigError) as e:
        LlamaConfig.from_dict(raw)
    assert word in str(e.value)


def test_registry_by_name_and_model_type(tmp_path):
    assert "LlamaForCausalLM" in registered_architectures()
    assert architecture_for({"architectures": ["LlamaForCausalLM"]}).config_class is LlamaConfig
    assert architecture_for({"model_type": "llama"}).name == "LlamaForCausalLM"
    with pytest.raises(ConfigError) as e:
        architecture_for({"architectures": ["NoSuchModel"], "model_type": "nosuch"})
    assert "LlamaForCausalLM" in str(e.value) and "NoSuchModel" in str(e.value)
    (tmp_path / "config.json").write_text(json.dumps(helpers.TINY_B))
    arch, cfg = load_config(str(tmp_path))
    assert arch.name == "LlamaForCausalLM" and cfg.tie_word_embeddings and cfg.rope_theta == 500000.0
    with pytest.raises(ConfigError):
        load_config(str(tmp_path / "missing"))
    (tmp_path / "config.json").write_text("{not json")
    with pytest.raises(ConfigError):
        load_config(str(tmp_path))


def test_another_architecture_can_be_registered():
    class Toy(ModelConfig):
        pass
    arch = register_architecture(Architecture("ToyForTests", "toy_for_tests", LlamaConfig, lambda cfg: None))
    try:
        assert architecture_for({"architectures": ["ToyForTests"]}) is arch
        with pytest.raises(ConfigError):
            register_architecture(arch)
    finally:
        unregister_architecture("ToyForTests")


def test_description_is_data():
    arch, cfg = architecture_for(helpers.TINY_A), LlamaConfig.from_dict(helpers.TINY_A)
    spec = arch.describe(cfg)
    assert len(spec.layers) == 2 and [e.layer for e in spec.schedule] == [0, 1]
    assert spec.layers[0].mixer.params["num_kv_heads"] == 2 and spec.layers[0].mixer.params["position"].params["theta"] == 10000.0
    assert spec.layers[1].ffn.params["intermediate_size"] == 176 and spec.final_norm.params["eps"] == 1e-5


def test_working_memory_is_what_the_parts_state():
    """What a step needs beyond weights and cache is added up from the parts (each product's output, attention's
    float partial results), not a constant times the width: it follows the feed-forward's width and the head
    count, and a step limited by memory alone is sized for the longest portion a request may bring."""
    from bare_cuda_4gib_amd.engine.engine import working_memory_estimate
    from bare_cuda_4gib_amd.engine.model import Model
    cfg = LlamaConfig.from_dict(helpers.TINY_A)
    model = Model(architecture_for(helpers.TINY_A).describe(cfg))
    h, q, kv, inter, vocab = 64, 4 * 16, 2 * 16, 176, 256
    attention = (q + 2 * kv + h) * 2 + q * 2 + 8 * (q + 2 * 4) * 4       # products' outputs, attention's output, parts of cut keys
    ffn = (2 * inter + h) * 2
    per_row = h * (4 + 4 + 2) + attention + ffn
    assert model.working_bytes(10, 3, 2) == 10 * per_row + 3 * (h * 2 + 4 * vocab)
    wide = Model(architecture_for(helpers.TINY_A).describe(LlamaConfig.from_dict(dict(helpers.TINY_A, intermediate_size=1760))))
    assert wide.working_bytes(10, 0, 2) - model.working_bytes(10, 0, 2) == 10 * 2 * (1760 - 176) * 2
    limited = working_memory_estimate(model, max_seqs=4, max_batch_tokens=32, graphs=0)
    unlimited = working_memory_estimate(model, max_seqs=4, max_batch_tokens=0, graphs=0, max_tokens=128)
    assert limited == model.working_bytes(32, 4, 2) and unlimited == model.working_bytes(128, 4, 2) > limited
