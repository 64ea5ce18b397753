"""Configuration reading and the architecture registry (no GPU)."""
import pytest

import helpers
import hf_cpu_amd
from hf_cpu_amd.config import Qwen2Config, config_from_dict, read_config
from hf_cpu_amd.status import EngineError


def test_reads_every_field_of_both_tiny_configs():
    a = config_from_dict(helpers.CONFIG_A)
    b = config_from_dict(helpers.CONFIG_B)
    assert isinstance(a, Qwen2Config)
    assert (a.num_hidden_layers, a.hidden_size, a.num_attention_heads, a.num_key_value_heads, a.head_dim,
            a.intermediate_size, a.vocab_size, a.rope_theta, a.rms_norm_eps, a.tie_word_embeddings) == \
        (2, 64, 4, 2, 16, 176, 512, 10000.0, 1e-6, True)
    assert (b.num_hidden_layers, b.hidden_size, b.num_attention_heads, b.num_key_value_heads, b.head_dim,
            b.intermediate_size, b.vocab_size, b.rope_theta, b.rms_norm_eps, b.tie_word_embeddings) == \
        (3, 96, 3, 1, 32, 256, 1000, 1e6, 1e-5, False)
    assert [a.layer_window(l) for l in range(2)] == [0, 0]
    assert [b.layer_window(l) for l in range(3)] == [0, 32, 32]      # layer l is windowed iff l >= max_window_layers
    assert config_from_dict(a.to_dict()) == a and config_from_dict(b.to_dict()) == b


def test_defaults_follow_the_reference():
    cfg = dict(helpers.CONFIG_A)
    del cfg["num_key_value_heads"], cfg["head_dim"]
    c = config_from_dict(cfg)
    assert c.num_key_value_heads == 4 and c.head_dim == 16         # src/model.c:126-131
    wide = config_from_dict(dict(helpers.CONFIG_A, head_dim=48))      # heads x head_dim need not equal hidden
    assert wide.q_size == 192 and wide.kv_size == 96
    newer = dict(helpers.CONFIG_A)
    del newer["rope_theta"]
    newer["rope_parameters"] = {"rope_theta": 5e5, "rope_type": "default"}
    assert config_from_dict(newer).rope_theta == 5e5
    assert config_from_dict(dict(helpers.CONFIG_A, eos_token_id=7)).eos_token_ids == (7,)
    assert config_from_dict(dict(helpers.CONFIG_A, eos_token_id=[7, 9])).eos_token_ids == (7, 9)
    unused = config_from_dict(dict(helpers.CONFIG_A, sliding_window=131072, max_window_layers=1))
    assert [unused.layer_window(l) for l in range(2)] == [0, 0]       # use_sliding_window is false


@pytest.mark.parametrize("change,code,word", [
    ({"hidden_size": None}, "EFORMAT", "hidden_size"),
    ({"rms_norm_eps": None}, "EFORMAT", "rms_norm_eps"),
    ({"num_hidden_layers": 0}, "EFORMAT", "implausible"),
    ({"num_hidden_layers": 10 ** 7}, "EFORMAT", "implausible"),
    ({"vocab_size": "many"}, "EFORMAT", "not an integer"),
    ({"num_key_value_heads": 3}, "EFORMAT", "multiple"),
    ({"head_dim": 15}, "EFORMAT", "even"),
    ({"rms_norm_eps": 2.0}, "EFORMAT", "implausible"),
    ({"hidden_act": "gelu"}, "ENOTSUP", "gelu"),
    ({"rope_scaling": {"rope_type": "yarn", "factor": 4}}, "ENOTSUP", "yarn"),
    ({"use_sliding_window": True}, "EFORMAT", "sliding_window"),
    ({"use_sliding_window": True, "sliding_window": 8, "max_window_layers": 5}, "EFORMAT", "max_window_layers"),
    ({"architectures": ["MysteryForCausalLM"]}, "ENOTSUP", "MysteryForCausalLM"),
    ({"architectures": None}, "EFORMAT", "architectures"),
    ({"eos_token_id": 512}, "EFORMAT", "vocabulary"),
])
def test_refusals_name_the_key(change, code, word):
    cfg = dict(helpers.CONFIG_A)
    for k, v in change.items():
        if v is None:
            cfg.pop(k)
        else:
            cfg[k] = v
    with pytest.raises(EngineError) as e:
        config_from_dict(cfg)
    assert e.value.code == code and word in str(e.value)


def test_file_errors(tmp_path):
    with pytest.raises(EngineError) as e:
        read_config(str(tmp_path))
    assert e.value.code == "EIO" and "config.json" in str(e.value)
    (tmp_path / "config.json").write_text('{"architectures": ["Qwen2ForCausalLM"],\n "hidden_size": }')
    with pytest.raises(EngineError) as e:
        read_config(str(tmp_path))
    assert e.value.code == "EFORMAT" and "line 2" in str(e.value)
    (tmp_path / "config.json").write_text("[1, 2]")
    with pytest.raises(EngineError) as e:
        read_config(str(tmp_path))
    assert e.value.code == "EFORMAT"


def test_plan_is_data_and_registry_is_open():
    from hf_cpu_amd.models.qwen2 import qwen2_plan
    from hf_cpu_amd.plan import ScheduleEntry
    plan = qwen2_plan(config_from_dict(helpers.CONFIG_B))
    assert [e.layer for e in plan.schedule] == [0, 1, 2] and all(e.cache_of is None for e in plan.schedule)
    assert [lp.mixer.args["window"] for lp in plan.layers] == [0, 32, 32]
    assert plan.layers[1].mixer.kind == "attention" and plan.layers[1].feed_forward.kind == "gated_mlp"
    model = hf_cpu_amd.Model(plan)
    names = [s.name for s in model.param_specs()]
    assert "model.layers.2.self_attn.k_proj.bias" in names and "lm_head.weight" in names
    assert len(names) == len(set(names)) == 3 + 3 * 12
    # a schedule may run a layer twice and let an entry read another entry's cache
    import dataclasses
    twice = dataclasses.replace(plan, schedule=(ScheduleEntry(0), ScheduleEntry(1), ScheduleEntry(1),
                                                ScheduleEntry(2, cache_of=1)))
    needs = hf_cpu_amd.Model(twice).cache_needs()
    assert [n is not None for n in needs] == [True, True, True, False]
    with pytest.raises(ValueError):
        dataclasses.replace(plan, schedule=(ScheduleEntry(0, cache_of=0),)).check()
    with pytest.raises(ValueError):
        dataclasses.replace(plan, schedule=(ScheduleEntry(5),)).check()
    with pytest.raises(EngineError) as e:
        hf_cpu_amd.registry.make_part("mixer", hf_cpu_amd.PartSpec("no_such_mixer", {}))
    assert "no_such_mixer" in str(e.value) and "attention" in str(e.value)


def test_allocation_counter_fails_the_nth_once():
    """The allocation choke point's injection (src/mem.c:12-30): the n-th allocation after
    ``fail_after(n)`` fails with ENOMEM, once; the count goes on."""
    from hf_cpu_amd import memory
    from hf_cpu_amd.status import EngineError
    memory.fail_after(3)
    base = memory.allocations()
    memory.note("a")
    memory.note("b")
    with pytest.raises(EngineError) as e:
        memory.note("the third")
    assert e.value.code == "ENOMEM" and "the third" in e.value.msg and "injected" in e.value.msg
    for _ in range(5):
        memory.note("later")
    assert memory.allocations() == base + 8
    memory.fail_after(0)
    memory.note("none fails")


def test_model_options_are_spelled_by_the_configuration_class(tmp_path):
    """A session's model options come in the engine's words (``window``); the architecture's configuration
    class turns them into its own config.json keys, so nothing above it names a key of Qwen2's. An
    architecture whose class has no such method, or does not know the option, refuses it by name."""
    import json
    import hf_cpu_amd
    from hf_cpu_amd.config import apply_model_options, read_config
    from hf_cpu_amd.status import EngineError
    assert apply_model_options(dict(helpers.CONFIG_A), None) == helpers.CONFIG_A
    assert apply_model_options(dict(helpers.CONFIG_A), {"window": None}) == helpers.CONFIG_A
    on = config_from_dict(apply_model_options(dict(helpers.CONFIG_A, max_window_layers=1), {"window": 9}))
    assert [on.layer_window(l) for l in range(2)] == [0, 9]
    off = config_from_dict(apply_model_options(dict(helpers.CONFIG_B), {"window": 0}))
    assert [off.layer_window(l) for l in range(3)] == [0, 0, 0]
    (tmp_path / "config.json").write_text(json.dumps(dict(helpers.CONFIG_B, layer_types=["full_attention"] + 2 * ["sliding_attention"])))
    assert [read_config(str(tmp_path), {"window": 5}).layer_window(l) for l in range(3)] == [0, 5, 5]
    with pytest.raises(EngineError) as e:
        apply_model_options(dict(helpers.CONFIG_A), {"experts": 4})
    assert e.value.code == "ENOTSUP" and "experts" in e.value.msg and "Qwen2ForCausalLM" in e.value.msg

    class Bare:                                 # a configuration class without model options
        @classmethod
        def from_dict(cls, obj, origin="config.json"):
            return cls()
    hf_cpu_amd.register_architecture("BareForTest", Bare, lambda cfg: None)
    assert isinstance(config_from_dict(apply_model_options({"architectures": ["BareForTest"]}, {})), Bare)
    with pytest.raises(EngineError) as e:
        apply_model_options({"architectures": ["BareForTest"]}, {"window": 8})
    assert e.value.code == "ENOTSUP" and "BareForTest" in e.value.msg and "window" in e.value.msg
