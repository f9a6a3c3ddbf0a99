"""The random-weights mode on the device (`Engine.from_config`, what the benchmark, `--random-weights` and
`LLM(random_seed=)` build their models with) against the one on the host (`write_model_folder`): a tensor's
values are a function of the seed, its name and the element's index, the same in both; matrices
~ N(0, 0.02), every norm weight ~ 1 + N(0, 0.1)."""
import numpy as np
import pytest
import torch

from helpers import CONFIGS, random_tokens

pytestmark = pytest.mark.gpu


def _close(dev, host, what):
    """The device draws the bits the host draws (both take the logarithm and cosine in double precision and round
    once; an element in a hundred thousand may sit so close to a rounding boundary that the two libraries' last
    double bit decides it)."""
    dev, host = dev.float().cpu(), host.float().cpu()
    assert dev.shape == host.shape, (what, dev.shape, host.shape)
    diff = (dev - host).abs()
    ulp = host.abs().clamp_min(1e-30) * (2.0 ** -7 if what.endswith("bf16") else 2.0 ** -22)
    off = diff > 0
    assert float(off.float().mean()) < 1e-5, (what, float(off.float().mean()))       # the same bits
    assert bool((diff <= ulp).all()), (what, float((diff / ulp).max()))               # the others: one step apart


@pytest.mark.parametrize("dtype", ["bfloat16", "float32"])
@pytest.mark.parametrize("name", ["B", "D"])
def test_device_draws_what_the_host_writes(tmp_path, name, dtype):
    import tinyinfer_amd as ti
    from safetensors.torch import load_file
    cfg = CONFIGS[name]
    folder = str(tmp_path / "m")
    ti.write_model_folder(folder, cfg, seed=31, dtype=dtype)
    f = load_file(folder + "/model.safetensors")
    drawn = ti.Engine.from_config(cfg, 31, dtype, page_size=16, max_tokens=256, max_requests=2, max_seq=128)
    tag = "bf16" if dtype == "bfloat16" else "f32"
    m = drawn.model
    L = cfg["num_hidden_layers"]
    for i in (0, L - 1):
        att, ffn = m.blocks[i].mixer, m.blocks[i].ffn
        pre = f"model.layers.{i}."
        # q, k and v are drawn straight into their rows of the fused matrix (element i counts within the tensor, not the buffer)
        qkv = torch.cat([f[pre + f"self_attn.{p}_proj.weight"] for p in "qkv"])
        _close(att.w_qkv, qkv, "w_qkv " + tag)
        _close(att.w_o, f[pre + "self_attn.o_proj.weight"], "w_o " + tag)
        _close(ffn.w_gate_up, torch.cat([f[pre + "mlp.gate_proj.weight"], f[pre + "mlp.up_proj.weight"]]), "w_gate_up " + tag)
        _close(ffn.w_down, f[pre + "mlp.down_proj.weight"], "w_down " + tag)
        _close(att.q_norm_w, f[pre + "self_attn.q_norm.weight"], "q_norm f32")
        _close(att.k_norm_w, f[pre + "self_attn.k_norm.weight"], "k_norm f32")
        _close(m.blocks[i].norm1.weight, f[pre + "input_layernorm.weight"], "norm1 f32")
        _close(m.blocks[i].norm2.weight, f[pre + "post_attention_layernorm.weight"], "norm2 f32")
    _close(m.embedding.weight, f["model.embed_tokens.weight"], "embedding " + tag)
    _close(m.final_norm.weight, f["model.norm.weight"], "final norm f32")
    if cfg["tie_word_embeddings"]:
        assert m.head.weight.data_ptr() == m.embedding.weight.data_ptr() and "lm_head.weight" not in f
    else:
        _close(m.head.weight, f["lm_head.weight"], "head " + tag)
    # the same model either way: a prompt's logits from the drawn engine and from the folder's
    loaded = ti.Engine.from_folder(folder, dtype, page_size=16, max_tokens=256, max_requests=2, max_seq=128)
    toks = random_tokens(50, cfg["vocab_size"], 4)
    a = drawn.step([ti.StepEntry("x", toks, [0, 20, 49])]).cpu().numpy()
    b = loaded.step([ti.StepEntry("x", toks, [0, 20, 49])]).cpu().numpy()
    assert np.abs(a - b).max() < (1e-5 if dtype == "float32" else 2e-2) * max(1.0, float(np.abs(b).max()))


def test_drawn_weights_have_the_stated_distributions():
    """N(0, 0.02) for matrices and the embedding, 1 + N(0, 0.1) for every norm weight (what the benchmark
    configurations name), at a size where the sample moments say something."""
    import tinyinfer_amd as ti
    cfg = dict(CONFIGS["E"], num_hidden_layers=1)
    m = ti.Engine.from_config(cfg, 5, "bfloat16", page_size=16, max_tokens=64, max_requests=1, max_seq=64).model
    for what, w in (("w_qkv", m.blocks[0].mixer.w_qkv), ("w_down", m.blocks[0].ffn.w_down), ("embedding", m.embedding.weight)):
        w = w.float()
        n = w.numel()
        assert abs(float(w.mean())) < 5 * 0.02 / n ** 0.5 + 1e-5, (what, float(w.mean()))
        assert abs(float(w.std()) - 0.02) < 0.02 * 0.01, (what, float(w.std()))
        # and a bell: about 4.55 % beyond two standard deviations, nothing beyond seven
        assert abs(float((w.abs() > 0.04).float().mean()) - 0.0455) < 0.004, what
        assert float(w.abs().max()) < 0.14, what
    # rows of the fused matrix are not copies of one another (element i counts within each tensor, but the name differs)
    qkv = m.blocks[0].mixer.w_qkv.float()
    assert not torch.equal(qkv[:1024], qkv[1024:2048]) and not torch.equal(qkv[2048:3072], qkv[3072:4096])
    norms = torch.cat([m.blocks[0].norm1.weight, m.blocks[0].norm2.weight, m.final_norm.weight]).float()
    assert abs(float(norms.mean()) - 1.0) < 5 * 0.1 / norms.numel() ** 0.5, float(norms.mean())
    assert abs(float(norms.std()) - 0.1) < 0.01, float(norms.std())
    heads = torch.cat([m.blocks[0].mixer.q_norm_w, m.blocks[0].mixer.k_norm_w]).float()
    assert abs(float(heads.mean()) - 1.0) < 0.04 and abs(float(heads.std()) - 0.1) < 0.03
