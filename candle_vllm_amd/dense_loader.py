"""config.json + model.safetensors of a llama-family checkpoint (Hugging Face tensor names) -> dense_model.DenseLlama, the 16-bit
host layer (the reference builds the same struct from the same names, src/openai/models/llama.rs:203-260)."""
import os
from dataclasses import dataclass

import numpy as np


@dataclass
class DenseDims:
    hidden: int
    n_layers: int
    n_heads: int
    n_kv_heads: int
    head_dim: int
    intermediate: int
    vocab: int
    rms_eps: float = 1e-5
    rope_theta: float = 10000.0
    max_seq: int = 8192
    block_size: int = 64
    qkv_bias: bool = False


def dims_from_config(c, block_size=64):
    heads = int(c["num_attention_heads"])
    return DenseDims(hidden=int(c["hidden_size"]), n_layers=int(c["num_hidden_layers"]), n_heads=heads,
                     n_kv_heads=int(c.get("num_key_value_heads", heads)), head_dim=int(c.get("head_dim", int(c["hidden_size"]) // heads)),
                     intermediate=int(c["intermediate_size"]), vocab=int(c["vocab_size"]), rms_eps=float(c.get("rms_norm_eps", 1e-5)),
                     rope_theta=float(c.get("rope_theta", 10000.0)), max_seq=int(c.get("max_position_embeddings", 8192)),
                     block_size=block_size, qkv_bias=bool(c.get("attention_bias", False)) or "Qwen2ForCausalLM" in c.get("architectures", []))


# checkpoint name -> (layer slot name of DenseLlama.set_weight)
LAYER_NAMES = {"self_attn.q_proj.weight": "wq", "self_attn.k_proj.weight": "wk", "self_attn.v_proj.weight": "wv", "self_attn.o_proj.weight": "wo",
               "mlp.gate_proj.weight": "w1", "mlp.down_proj.weight": "w2", "mlp.up_proj.weight": "w3", "input_layernorm.weight": "attn_norm",
               "post_attention_layernorm.weight": "ffn_norm", "self_attn.q_proj.bias": "bq", "self_attn.k_proj.bias": "bk",
               "self_attn.v_proj.bias": "bv"}
GLOBAL_NAMES = {"model.embed_tokens.weight": "tok_embd", "model.norm.weight": "output_norm", "lm_head.weight": "output"}


def slot_of(name):
    """checkpoint tensor name -> (layer or -1, slot name), None for tensors the host layer does not use"""
    if name in GLOBAL_NAMES:
        return -1, GLOBAL_NAMES[name]
    if name.startswith("model.layers."):
        idx, rest = name[len("model.layers."):].split(".", 1)
        if rest in LAYER_NAMES:
            return int(idx), LAYER_NAMES[rest]
    return None


def load_dense_llama(model_dir, config, dtype="bfloat16", max_batch=8, max_blocks_per_seq=64, block_size=64, **_):
    if dtype not in ("bfloat16", "bf16"):
        raise ValueError("the 16-bit llama host layer serves bfloat16 checkpoints")
    from .dense_model import DenseLlama
    from .hybrid_model import read_safetensors
    dims = dims_from_config(config, block_size)
    m = DenseLlama(dims, max_batch=max_batch, max_blocks_per_seq=max_blocks_per_seq)
    tensors = read_safetensors(os.path.join(model_dir, "model.safetensors"))
    seen = set()
    for name, (bits, _shape) in tensors.items():
        where = slot_of(name)
        if where is None:
            continue
        f32 = (np.asarray(bits, np.uint16).astype(np.uint32) << 16).view(np.float32)
        m.set_weight(where[0], where[1], f32)
        seen.add(where)
    if (-1, "output") not in seen and "model.embed_tokens.weight" in tensors:            # tied embeddings
        bits = tensors["model.embed_tokens.weight"][0]
        m.set_weight(-1, "output", (np.asarray(bits, np.uint16).astype(np.uint32) << 16).view(np.float32))
    return m
