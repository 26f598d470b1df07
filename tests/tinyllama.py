"""The reference's tiny-llama data fixture (spec/test_data/tiny-llama, copied as data to
tests/golden/tiny-llama) as plain numpy weights in the reference's [in, out] layout, plus
the oracle-side model walk (Network#run with use_kv_cache)."""
import json
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
DIR = os.path.join(HERE, "golden", "tiny-llama")


def load():
    from safetensors.numpy import load_file

    cfg = json.load(open(os.path.join(DIR, "config.json")))
    sd = load_file(os.path.join(DIR, "model.safetensors"))
    t = lambda n: np.ascontiguousarray(sd[n].astype(np.float32).T)  # [out, in] -> [in, out] (hf_loader.cr:326-337)
    w = {"cfg": cfg, "embed": sd["model.embed_tokens.weight"].astype(np.float32),
         "final_norm": sd["model.norm.weight"].astype(np.float32), "lm_head": t("lm_head.weight"), "layers": []}
    for li in range(cfg["num_hidden_layers"]):
        p = f"model.layers.{li}."
        w["layers"].append({
            "w_q": t(p + "self_attn.q_proj.weight"), "w_k": t(p + "self_attn.k_proj.weight"),
            "w_v": t(p + "self_attn.v_proj.weight"), "w_o": t(p + "self_attn.o_proj.weight"),
            "gate": t(p + "mlp.gate_proj.weight"), "up": t(p + "mlp.up_proj.weight"),
            "down": t(p + "mlp.down_proj.weight"),
            "norm1": sd[p + "input_layernorm.weight"].astype(np.float32),
            "norm2": sd[p + "post_attention_layernorm.weight"].astype(np.float32)})
    return w


class OracleModel:
    """Network#run(use_kv_cache) composed from the oracle's pieces."""

    def __init__(self, w, orc):
        c = w["cfg"]
        self.w, self.orc, self.eps = w, orc, c["rms_norm_eps"]
        self.blocks = []
        for lw in w["layers"]:
            b = orc.Block(c["hidden_size"], c["num_attention_heads"], c["num_key_value_heads"], None, eps=self.eps,
                          rope_theta=c["rope_theta"])
            b.set_weights(lw["w_q"], lw["w_k"], lw["w_v"], lw["w_o"])
            self.blocks.append(b)

    def clear_cache(self):
        for b in self.blocks:
            b.clear_cache()

    def hidden(self, tokens, cached=True):
        x = self.orc.embed(self.w["embed"], tokens)
        for b, lw in zip(self.blocks, self.w["layers"]):
            x = b.forward(x, lw["norm1"], lw["norm2"], self.eps, lw["gate"], lw["up"], lw["down"], cached)
        return x

    def run(self, tokens):
        return self.orc.logits_last(self.hidden(tokens), self.w["final_norm"], self.eps, self.w["lm_head"])

    def run_full(self, tokens):
        """Network#run with use_kv_cache off: LlamaBlock#forward in every block, caches untouched."""
        return self.orc.logits_last(self.hidden(tokens, cached=False), self.w["final_norm"], self.eps,
                                    self.w["lm_head"])
