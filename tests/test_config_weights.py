"""Configuration, registry and weight loading (no GPU)."""
import json
import os

import pytest
import torch

import tinyinfer_amd as ti
from helpers import CONFIGS
from tinyinfer_amd.config.qwen3 import Qwen3Config
from safetensors.torch import load_file, save_file
from tinyinfer_amd.weights import WeightsError, FileError, load_weights, write_model_folder


def stored(d):
    """{name: tensor} of a folder's model.safetensors, read with the safetensors package."""
    return load_file(os.path.join(d, "model.safetensors"))


def test_config_reads_every_size_from_the_dict():
    for name, d in CONFIGS.items():
        c = Qwen3Config.from_dict(d)
        assert c.num_hidden_layers == d["num_hidden_layers"]
        assert c.hidden_size == d["hidden_size"] and c.head_dim == d["head_dim"]
        assert c.num_attention_heads == d["num_attention_heads"]
        assert c.num_key_value_heads == d["num_key_value_heads"]
        assert c.intermediate_size == d["intermediate_size"] and c.vocab_size == d["vocab_size"]
        assert c.rope_theta == d["rope_theta"] and c.rms_norm_eps == d["rms_norm_eps"]
        assert c.tie_word_embeddings == d["tie_word_embeddings"]
        # the written config reads back as the same configuration
        assert Qwen3Config.from_dict(json.loads(json.dumps(c.to_dict()))) == c


def test_config_defaults_and_windows():
    d = dict(CONFIGS["A"])
    del d["head_dim"], d["rms_norm_eps"], d["rope_theta"], d["num_key_value_heads"]
    c = Qwen3Config.from_dict(d)
    assert c.head_dim == 16 and c.num_key_value_heads == 4
    assert c.rms_norm_eps == 1e-6 and c.rope_theta == 1e6          # the reference's defaults
    c = Qwen3Config.from_dict(CONFIGS["C"])
    assert c.layer_types == ("full_attention", "full_attention", "sliding_attention", "sliding_attention")
    assert c.sliding_window == 20
    d = dict(CONFIGS["C"], use_sliding_window=False)
    assert Qwen3Config.from_dict(d).sliding_window is None        # a window that is switched off is no window
    c = Qwen3Config.from_dict(CONFIGS["D"])
    assert c.layer_types[0] == "full_attention" and c.layer_types[1] == "sliding_attention"


@pytest.mark.parametrize("change,needle", [
    (dict(num_hidden_layers=None), "num_hidden_layers"),
    (dict(hidden_size=0), "hidden_size"),
    (dict(num_attention_heads=5), "num_key_value_heads"),
    (dict(head_dim=15), "head_dim"),
    (dict(head_dim=24), "head_dim"),          # even, but no attention kernel takes it: said before any weight is read
    (dict(head_dim=40), "steps of 16"),
    (dict(head_dim=512), "up to 256"),
    (dict(attention_bias=True), "attention_bias"),
    (dict(hidden_act="gelu"), "hidden_act"),
    (dict(rope_scaling={"rope_type": "yarn", "factor": 4.0}), "rope_scaling"),
    (dict(vocab_size="many"), "vocab_size"),
    (dict(rms_norm_eps=-1.0), "rms_norm_eps"),
    (dict(layer_types=["full_attention"]), "layer_types"),
    (dict(layer_types=["full_attention", "sliding_attention"]), "sliding_window"),
])
def test_config_errors_name_the_key(change, needle):
    d = dict(CONFIGS["A"])
    d.update(change)
    with pytest.raises(ti.ConfigError) as e:
        Qwen3Config.from_dict(d)
    assert needle in str(e.value)


def test_an_attention_part_refuses_a_head_size_no_kernel_takes():
    """Not only through config.json: whoever builds the part (another architecture's spec) hears it at once."""
    for hd in (8, 24, 272):
        with pytest.raises((ti.ConfigError, ValueError)) as e:
            ti.build_part("mixer", ti.PartSpec("attention", dict(hidden=64, heads=2, kv_heads=1, head_dim=hd)), "layer")
        assert "head_dim" in str(e.value) and str(hd) in str(e.value)
    ti.build_part("mixer", ti.PartSpec("attention", dict(hidden=64, heads=2, kv_heads=1, head_dim=48)), "layer")


def test_registry_picks_by_name_and_lists_what_it_has():
    cfg, spec = ti.config_and_spec(CONFIGS["B"])
    assert isinstance(cfg, Qwen3Config) and len(spec.layers) == 3
    cfg, _ = ti.config_and_spec({k: v for k, v in CONFIGS["B"].items() if k != "architectures"})   # model_type
    assert isinstance(cfg, Qwen3Config)
    with pytest.raises(ti.ConfigError) as e:
        ti.config_and_spec(dict(CONFIGS["B"], architectures=["LlamaForCausalLM"], model_type="llama"))
    assert "Qwen3ForCausalLM" in str(e.value) and "LlamaForCausalLM" in str(e.value)


def test_model_is_built_from_the_spec_layer_by_layer():
    _, spec = ti.config_and_spec(CONFIGS["C"])
    m = ti.Model(spec)
    windows = [b.mixer.window for b in m.blocks]
    assert windows == [None, None, 20, 20]
    # layers that read all keys and layers that read a window keep pages of their own
    assert len(m.cache_groups) == 2 and [n for _, n in m.cache_groups] == [2, 2]
    assert m.blocks[0].mixer.scale == pytest.approx(48 ** -0.5)
    assert m.blocks[1].ffn.intermediate == 176 and m.final_norm.eps == 3e-6


def folder(tmp_path, name="A", dtype="bfloat16"):
    d = str(tmp_path / f"m_{name}_{dtype}")
    write_model_folder(d, CONFIGS[name], seed=3, dtype=dtype)
    return d


def test_random_folder_round_trip_and_dtypes(tmp_path):
    d = folder(tmp_path, "B")
    f = stored(d)
    assert "lm_head.weight" in f                                          # untied: a head of its own
    q = f["model.layers.0.self_attn.q_proj.weight"]
    assert (q.dtype, tuple(q.shape)) == (torch.bfloat16, (192, 96))
    qn = f["model.layers.0.self_attn.q_norm.weight"]
    assert (qn.dtype, tuple(qn.shape)) == (torch.float32, (32,))
    _, spec = ti.config_and_spec(ti.read_config_json(d))
    m = ti.Model(spec)
    load_weights(m, d, "bfloat16", "cpu")
    att = m.blocks[0].mixer
    assert att.w_qkv.dtype == torch.bfloat16 and att.w_qkv.shape == (192 + 2 * 64, 96)   # q, k, v fused
    assert att.q_norm_w.dtype == torch.float32                                           # norms stay 32-bit
    assert m.blocks[0].ffn.w_gate_up.shape == (448, 96)
    assert m.head.weight.data_ptr() != m.embedding.weight.data_ptr()
    assert torch.equal(att.w_qkv[:192], q)
    assert torch.equal(att.w_qkv[192:256], f["model.layers.0.self_attn.k_proj.weight"])
    assert torch.equal(att.w_qkv[256:], f["model.layers.0.self_attn.v_proj.weight"])
    assert torch.equal(m.blocks[0].ffn.w_gate_up[224:], f["model.layers.0.mlp.up_proj.weight"])
    # same seed, same bits; another seed, other bits
    d2 = str(tmp_path / "again")
    write_model_folder(d2, CONFIGS["B"], seed=3)
    t2 = stored(d2)
    assert torch.equal(t2["model.norm.weight"], f["model.norm.weight"])
    write_model_folder(str(tmp_path / "other"), CONFIGS["B"], seed=4)
    t3 = stored(str(tmp_path / "other"))
    assert not torch.equal(t3["model.norm.weight"], t2["model.norm.weight"])
    # norm weights are 1 + N(0, 0.1), matrices N(0, 0.02)
    assert abs(t2["model.norm.weight"].mean().item() - 1.0) < 0.05
    assert abs(t2["model.embed_tokens.weight"].float().std().item() - 0.02) < 0.002


def test_float32_engine_widens_and_tied_head_shares(tmp_path):
    d = folder(tmp_path, "A")
    _, spec = ti.config_and_spec(ti.read_config_json(d))
    m = ti.Model(spec)
    load_weights(m, d, "float32", "cpu")
    assert m.embedding.weight.dtype == torch.float32
    assert m.head.weight.data_ptr() == m.embedding.weight.data_ptr()     # tied: one tensor
    f = stored(d)
    assert "lm_head.weight" not in f
    assert torch.equal(m.embedding.weight, f["model.embed_tokens.weight"].float())


def test_one_error_lists_missing_unexpected_and_wrong_shapes(tmp_path):
    d = folder(tmp_path, "A")
    t = stored(d)
    del t["model.layers.1.mlp.up_proj.weight"]
    del t["model.norm.weight"]
    t["model.layers.0.self_attn.q_proj.bias"] = torch.zeros(64)
    t["model.layers.0.self_attn.k_proj.weight"] = t["model.layers.0.self_attn.k_proj.weight"].T.contiguous()
    t["model.layers.1.input_layernorm.weight"] = torch.ones(63)
    save_file(t, os.path.join(d, "model.safetensors"))
    _, spec = ti.config_and_spec(ti.read_config_json(d))
    with pytest.raises(WeightsError) as e:
        load_weights(ti.Model(spec), d, "bfloat16", "cpu")
    err = e.value
    assert sorted(err.missing) == ["model.layers.1.mlp.up_proj.weight", "model.norm.weight"]
    assert err.unexpected == ["model.layers.0.self_attn.q_proj.bias"]
    assert sorted(n for n, _, _ in err.wrong_shape) == ["model.layers.0.self_attn.k_proj.weight",
                                                       "model.layers.1.input_layernorm.weight"]
    text = str(err)
    for needle in ("missing (2)", "unexpected (1)", "wrong shape (2)", "[64, 32]", "expected [32, 64]"):
        assert needle in text, text


def test_untied_without_head_and_open_tying(tmp_path):
    d = folder(tmp_path, "B")
    t = {n: v for n, v in stored(d).items() if n != "lm_head.weight"}
    save_file(t, os.path.join(d, "model.safetensors"))
    _, spec = ti.config_and_spec(ti.read_config_json(d))
    with pytest.raises(WeightsError) as e:
        load_weights(ti.Model(spec), d, "bfloat16", "cpu")
    assert e.value.missing == ["lm_head.weight"]
    # tie_word_embeddings absent: decided by what the file holds
    cfg = ti.read_config_json(d)
    del cfg["tie_word_embeddings"]
    _, spec = ti.config_and_spec(cfg)
    m = ti.Model(spec)
    load_weights(m, d, "bfloat16", "cpu")
    assert m.head.weight.data_ptr() == m.embedding.weight.data_ptr()


def test_broken_files_are_refused(tmp_path):
    d = folder(tmp_path, "A")
    p = os.path.join(d, "model.safetensors")
    raw = open(p, "rb").read()
    open(p, "wb").write(raw[:len(raw) // 2])                 # cut short
    _, spec = ti.config_and_spec(ti.read_config_json(d))
    with pytest.raises(FileError):
        load_weights(ti.Model(spec), d, "bfloat16", "cpu")
    os.remove(p)
    with pytest.raises(FileError):
        load_weights(ti.Model(spec), d, "bfloat16", "cpu")
    with pytest.raises(ti.ConfigError):
        ti.read_config_json(str(tmp_path / "nowhere"))


def test_schedule_may_repeat_a_layer_or_share_a_cache():
    """The run order is data: a layer named twice gets a cache layer per run; a
    layer with `cache_from` keeps none and reads the other's."""
    from tinyinfer_amd.spec import LayerSpec, PartSpec
    _, spec = ti.config_and_spec(CONFIGS["A"])
    spec.schedule = [0, 1, 0]
    m = ti.Model(spec)
    assert m.cache_groups[0][1] == 3
    b0 = m.bindings[0][id(m.blocks[0].mixer)], m.bindings[2][id(m.blocks[0].mixer)]
    assert b0[0] != b0[1]
    _, spec = ti.config_and_spec(CONFIGS["A"])
    spec.layers[1].cache_from = 0
    spec.layers[1].parts["mixer"].params["shares_kv"] = True
    m = ti.Model(spec)
    assert m.cache_groups[0][1] == 1
    assert m.bindings[1][id(m.blocks[1].mixer)] == m.bindings[0][id(m.blocks[0].mixer)]
    assert "model.layers.1.self_attn.k_proj.weight" not in m.tensors()
