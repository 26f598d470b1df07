"""Writes the golden vectors under tests/golden/ from an INDEPENDENT implementation.

Run once in the build container:  python tests/golden/make_golden.py

Sources of truth used here (none of them is the reference's code):
  * Hugging Face `transformers` attention modules (LlamaAttention, Qwen2Attention,
    Qwen3Attention) with seeded random weights: they fix the half-split RoPE
    convention, the [out,in] -> [in,out] weight transposes, GQA head mapping,
    Qwen2 biases, Qwen3 per-head QK-norm before RoPE, and llama3 rope scaling.
  * The reference's own data fixture spec/test_data/tiny-llama (config.json +
    model.safetensors, read with safetensors, nothing executed from it): the
    hidden states of tokens [1, 42, 100, 7] after each decoder layer, the scenario
    of spec/rope_kv_cache_spec.cr:29-59.
Only small arrays (inputs, weights, expected outputs) are stored.
"""
import json
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
TINY = "/root/reference/spec/test_data/tiny-llama"


def causal_mask(T):
    m = torch.full((T, T), float("-inf"))
    return torch.triu(m, diagonal=1)[None, None]


def attn_fixture(kind, name, seed, T, **cfg_kw):
    from transformers.models.llama.modeling_llama import LlamaAttention, LlamaConfig, LlamaRotaryEmbedding
    from transformers.models.qwen2.modeling_qwen2 import Qwen2Attention, Qwen2Config, Qwen2RotaryEmbedding
    from transformers.models.qwen3.modeling_qwen3 import Qwen3Attention, Qwen3Config, Qwen3RotaryEmbedding

    torch.manual_seed(seed)
    Cfg, Attn, Rot = {"llama": (LlamaConfig, LlamaAttention, LlamaRotaryEmbedding),
                      "qwen2": (Qwen2Config, Qwen2Attention, Qwen2RotaryEmbedding),
                      "qwen3": (Qwen3Config, Qwen3Attention, Qwen3RotaryEmbedding)}[kind]
    cfg = Cfg(vocab_size=32, num_hidden_layers=1, intermediate_size=32, attention_dropout=0.0, **cfg_kw)
    cfg._attn_implementation = "eager"
    attn = Attn(cfg, layer_idx=0).eval().double()
    rot = Rot(cfg)
    with torch.no_grad():
        for p in attn.parameters():
            p.copy_(torch.randn_like(p) * 0.15)
        if hasattr(attn, "q_norm"):
            attn.q_norm.weight.copy_(1.0 + 0.1 * torch.randn_like(attn.q_norm.weight))
            attn.k_norm.weight.copy_(1.0 + 0.1 * torch.randn_like(attn.k_norm.weight))
        for n in ("q_proj", "k_proj", "v_proj"):
            b = getattr(attn, n).bias
            if b is not None:
                b.copy_(0.3 * torch.randn_like(b))
        # weights must be exactly representable in fp32: the oracle stores fp32
        for p in attn.parameters():
            p.copy_(p.float().double())
        x = torch.randn(1, T, cfg.hidden_size).float().double()
        pos = torch.arange(T)[None]
        cos, sin = rot(x.float(), pos)
        out, _ = attn(x, (cos.double(), sin.double()), causal_mask(T).double())
    hd = attn.head_dim
    d = {
        "x": x[0].numpy().astype(np.float32),
        "expected": out[0].numpy().astype(np.float64),
        "w_q": attn.q_proj.weight.T.contiguous().numpy().astype(np.float32),
        "w_k": attn.k_proj.weight.T.contiguous().numpy().astype(np.float32),
        "w_v": attn.v_proj.weight.T.contiguous().numpy().astype(np.float32),
        "w_o": attn.o_proj.weight.T.contiguous().numpy().astype(np.float32),
        "inv_freq": rot.inv_freq.numpy().astype(np.float64),
        "meta": np.array(json.dumps({
            "d_model": cfg.hidden_size, "num_heads": cfg.num_attention_heads,
            "num_kv_heads": cfg.num_key_value_heads, "head_dim": hd,
            "rope_theta": float(cfg.rope_parameters["rope_theta"]) if hasattr(cfg, "rope_parameters") else float(cfg.rope_theta),
            "eps": float(cfg.rms_norm_eps), "T": T,
            "rope_scaling": cfg_kw.get("rope_parameters"),
        })),
    }
    assert attn.o_proj.bias is None
    if attn.q_proj.bias is not None:
        d["b_q"] = attn.q_proj.bias.numpy().astype(np.float32)
        d["b_k"] = attn.k_proj.bias.numpy().astype(np.float32)
        d["b_v"] = attn.v_proj.bias.numpy().astype(np.float32)
    if hasattr(attn, "q_norm"):
        d["q_norm"] = attn.q_norm.weight.numpy().astype(np.float32)
        d["k_norm"] = attn.k_norm.weight.numpy().astype(np.float32)
    np.savez_compressed(os.path.join(HERE, name + ".npz"), **d)
    print("wrote", name, {k: getattr(v, "shape", None) for k, v in d.items()})


def tiny_llama_fixture():
    from safetensors.torch import load_file
    from transformers import LlamaConfig, LlamaModel

    cfg = LlamaConfig.from_pretrained(TINY)
    cfg._attn_implementation = "eager"
    sd = load_file(os.path.join(TINY, "model.safetensors"))
    model = LlamaModel(cfg).eval()
    missing = model.load_state_dict({k[len("model."):]: v for k, v in sd.items() if k.startswith("model.")},
                                    strict=False)
    assert not missing.missing_keys, missing
    model = model.double()
    tokens = [1, 42, 100, 7]
    with torch.no_grad():
        out = model(torch.tensor([tokens]), output_hidden_states=True)
    hs = [h[0].numpy() for h in out.hidden_states]  # embeddings, after layer 0, after layer 1 (pre final norm)
    d = {"tokens": np.array(tokens), "embed": hs[0].astype(np.float32)}
    # transformers applies the final norm to the last hidden state it reports; recompute the raw one
    x = out.hidden_states[0]
    pos = torch.arange(len(tokens))[None]
    cos, sin = model.rotary_emb(x.float(), pos)
    mask = causal_mask(len(tokens)).double()
    with torch.no_grad():
        for li, layer in enumerate(model.layers):
            x = layer(x, attention_mask=mask, position_ids=pos, position_embeddings=(cos.double(), sin.double()))
            if isinstance(x, tuple):
                x = x[0]
            d[f"hidden_after_{li}"] = x[0].numpy().astype(np.float64)
            p = f"layers.{li}."
            g = lambda n: sd["model." + p + n].float().numpy()
            for short, n in (("w_q", "self_attn.q_proj.weight"), ("w_k", "self_attn.k_proj.weight"),
                             ("w_v", "self_attn.v_proj.weight"), ("w_o", "self_attn.o_proj.weight"),
                             ("gate", "mlp.gate_proj.weight"), ("up", "mlp.up_proj.weight"),
                             ("down", "mlp.down_proj.weight")):
                d[f"l{li}_{short}"] = np.ascontiguousarray(g(n).T)  # reference layout [in, out] (hf_loader.cr:326-337)
            d[f"l{li}_norm1"] = g("input_layernorm.weight")
            d[f"l{li}_norm2"] = g("post_attention_layernorm.weight")
    d["meta"] = np.array(json.dumps({"d_model": cfg.hidden_size, "num_heads": cfg.num_attention_heads,
                                     "num_kv_heads": cfg.num_key_value_heads, "eps": cfg.rms_norm_eps,
                                     "rope_theta": 10000.0, "ff_hidden": cfg.intermediate_size}))
    np.savez_compressed(os.path.join(HERE, "tiny_llama_hidden.npz"), **d)
    print("wrote tiny_llama_hidden", {k: getattr(v, "shape", None) for k, v in d.items()})


def tiny_llama_logits_fixture():
    """Logits of the reference's tiny-llama data fixture for the token prefixes that
    spec/llama_loader_spec.cr runs ([1, 42, 100] and one more token), from transformers'
    LlamaForCausalLM in fp64; the safetensors file and its config are copied next to
    this script as data (nothing in them is executed)."""
    import shutil

    from safetensors.torch import load_file
    from transformers import LlamaConfig, LlamaForCausalLM

    dst = os.path.join(HERE, "tiny-llama")
    os.makedirs(dst, exist_ok=True)
    for f in ("config.json", "model.safetensors"):
        shutil.copyfile(os.path.join(TINY, f), os.path.join(dst, f))
    cfg = LlamaConfig.from_pretrained(TINY)
    cfg._attn_implementation = "eager"
    model = LlamaForCausalLM(cfg).eval()
    res = model.load_state_dict(load_file(os.path.join(TINY, "model.safetensors")), strict=False)
    assert not res.missing_keys, res
    model = model.double()
    d = {}
    for name, tokens in (("t3", [1, 42, 100]), ("t4", [1, 42, 100, 7])):
        with torch.no_grad():
            logits = model(torch.tensor([tokens])).logits[0, -1]
        d["tokens_" + name] = np.array(tokens, np.int32)
        d["logits_" + name] = logits.numpy().astype(np.float64)
    np.savez_compressed(os.path.join(HERE, "tiny_llama_logits.npz"), **d)
    print("wrote tiny_llama_logits", {k: getattr(v, "shape", None) for k, v in d.items()})


def rope_freq_fixture():
    """inv_freq of the published Llama-3.2-1B (hd 64, factor 32) and Llama-3.1-8B (hd 128,
    factor 8) rope_scaling blocks, from transformers' llama3 rope initialiser."""
    from transformers import LlamaConfig
    from transformers.modeling_rope_utils import ROPE_INIT_FUNCTIONS

    d = {}
    for name, hd, heads, factor in (("llama32_1b", 64, 32, 32.0), ("llama31_8b", 128, 32, 8.0)):
        rp = {"rope_type": "llama3", "rope_theta": 500000.0, "factor": factor, "low_freq_factor": 1.0,
              "high_freq_factor": 4.0, "original_max_position_embeddings": 8192}
        cfg = LlamaConfig(hidden_size=hd * heads, num_attention_heads=heads, head_dim=hd,
                          max_position_embeddings=131072, rope_parameters=rp)
        inv, _ = ROPE_INIT_FUNCTIONS["llama3"](cfg, "cpu")
        d[name] = inv.double().numpy()
        d[name + "_params"] = np.array(json.dumps(dict(rp, head_dim=hd)))
    np.savez_compressed(os.path.join(HERE, "hf_rope_llama3_freqs.npz"), **d)
    print("wrote hf_rope_llama3_freqs", {k: getattr(v, "shape", None) for k, v in d.items()})


def main():
    torch.set_grad_enabled(False)
    # LLaMA, GQA g=2, theta 5e5 (Llama-3.2 value), head_dim = d_model/heads
    attn_fixture("llama", "hf_llama_attn", 1, 12, hidden_size=64, num_attention_heads=8, num_key_value_heads=4,
                 rope_parameters={"rope_type": "default", "rope_theta": 500000.0}, rms_norm_eps=1e-5)
    # LLaMA-3 rope scaling (published Llama-3.x parameters), g=4
    attn_fixture("llama", "hf_llama3_scaled_attn", 2, 9, hidden_size=128, num_attention_heads=8,
                 num_key_value_heads=2, rms_norm_eps=1e-5, max_position_embeddings=131072,
                 rope_parameters={"rope_type": "llama3", "rope_theta": 500000.0, "factor": 32.0,
                                  "low_freq_factor": 1.0, "high_freq_factor": 4.0,
                                  "original_max_position_embeddings": 8192})
    # Qwen2: q/k/v biases, no o bias
    attn_fixture("qwen2", "hf_qwen2_attn", 3, 7, hidden_size=32, num_attention_heads=4, num_key_value_heads=2,
                 rope_parameters={"rope_type": "default", "rope_theta": 1000000.0}, rms_norm_eps=1e-6)
    # Qwen3: explicit head_dim != d_model/heads, QK-norm, g=4, theta 1e6
    attn_fixture("qwen3", "hf_qwen3_attn", 4, 10, hidden_size=32, num_attention_heads=8, num_key_value_heads=2,
                 head_dim=16, rope_parameters={"rope_type": "default", "rope_theta": 1000000.0},
                 rms_norm_eps=1e-6)
    rope_freq_fixture()
    if os.path.isdir(TINY):
        tiny_llama_fixture()
        tiny_llama_logits_fixture()
    else:
        print("tiny-llama fixture directory not found; skipped", file=sys.stderr)


if __name__ == "__main__":
    main()
