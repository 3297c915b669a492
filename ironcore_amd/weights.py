"""Weights into the generation model: Hugging Face GPT-2 checkpoints
(safetensors or an in-memory state dict).

Successor of ``WeightMapper._hf_gpt2_to_ironcore``
(ironcore/checkpointing/weight_mapping.py:179-305) with its two defects for
this model fixed:

* key names: the reference maps to ``self_attention.linear_q``,
  ``self_attention.output``, ``output_layernorm.weight`` (weight_mapping.py:
  264-285), but the layers are called ``linear_q`` / ``linear_kv`` /
  ``attn_output`` directly under the transformer layer
  (ironcore/models/transformer.py:47,53,62) and the norms keep their scale
  under ``.layernorm``;
* orientation: it transposes the Conv1D matrices to ``[out, in]``
  (weight_mapping.py:264-267, 285), but the parallel linear layers store
  ``[in, out]`` and multiply ``x @ W`` (ironcore/parallel/tensor_parallel/
  layers.py:41), which is the orientation GPT-2's Conv1D already has.

GPT-2's fused ``c_attn`` ([d, 3d], columns q | k | v) splits into ``linear_q``
([d, d]) and ``linear_kv`` ([d, 2d], k | v, the order ``torch.chunk`` undoes
in transformer.py:88-91).  The vocabulary is padded with zero rows to the
model's padded size (ironcore/tokenizer/tokenizer.py:70-75).
"""
from __future__ import annotations

import re
from typing import Dict

import torch

_IGNORED = re.compile(r"(^|\.)(attn\.bias|attn\.masked_bias|lm_head\.weight)$")


def hf_gpt2_to_model_state(hf_state: Dict[str, torch.Tensor], padded_vocab_size: int,
                           untie_embed: bool = False) -> Dict[str, torch.Tensor]:
    """Map a GPT-2 state dict (keys with or without the ``transformer.``
    prefix) to this model's names and shapes.  Raises on keys it cannot place."""
    out: Dict[str, torch.Tensor] = {}

    def pad_vocab(t):
        if t.shape[0] > padded_vocab_size:
            raise ValueError(f"checkpoint vocabulary {t.shape[0]} exceeds the model's {padded_vocab_size}")
        padded = t.new_zeros(padded_vocab_size, t.shape[1])
        padded[:t.shape[0]] = t
        return padded

    for key, tensor in hf_state.items():
        k = key[len("transformer."):] if key.startswith("transformer.") else key
        if k == "wte.weight":
            out["embedding.word_embeddings.weight"] = pad_vocab(tensor)
            continue
        if k == "wpe.weight":
            out["embedding.position_embedding.weight"] = tensor
            continue
        if k in ("ln_f.weight", "ln_f.bias"):
            out["output_layernorm.layernorm." + k.split(".")[1]] = tensor
            continue
        if key == "lm_head.weight":
            if untie_embed:  # [vocab, d] -> the [d, vocab] the output layer multiplies by
                out["output_layer.weight"] = pad_vocab(tensor).t().contiguous()
            continue
        m = re.match(r"h\.(\d+)\.(.*)", k)
        if m is None:
            if _IGNORED.search(key):
                continue
            raise ValueError(f"unmapped checkpoint key {key!r}")
        pre, rest = f"model.layers.{m.group(1)}.", m.group(2)
        part = rest.rsplit(".", 1)[-1]  # weight | bias
        if rest in ("ln_1.weight", "ln_1.bias"):
            out[pre + "input_layernorm.layernorm." + part] = tensor
        elif rest in ("ln_2.weight", "ln_2.bias"):
            out[pre + "post_attn_layernorm.layernorm." + part] = tensor
        elif rest in ("attn.c_attn.weight", "attn.c_attn.bias"):
            d = tensor.shape[-1] // 3
            out[pre + "linear_q." + part] = tensor[..., :d].contiguous()
            out[pre + "linear_kv." + part] = tensor[..., d:].contiguous()
        elif rest in ("attn.c_proj.weight", "attn.c_proj.bias"):
            out[pre + "attn_output." + part] = tensor
        elif rest in ("mlp.c_fc.weight", "mlp.c_fc.bias"):
            out[pre + "mlp.up_proj." + part] = tensor
        elif rest in ("mlp.c_proj.weight", "mlp.c_proj.bias"):
            out[pre + "mlp.down_proj." + part] = tensor
        elif _IGNORED.search(key):
            continue
        else:
            raise ValueError(f"unmapped checkpoint key {key!r}")
    return out


def load_hf_gpt2(model, source) -> None:
    """Load GPT-2 weights into ``generation.LanguageModel`` from a
    ``.safetensors`` file (path) or a state dict.  Strict: every parameter of
    the model must be covered and every checkpoint key placed."""
    if isinstance(source, dict):
        hf_state = source
    else:
        from safetensors.torch import load_file
        hf_state = load_file(str(source))
    state = hf_gpt2_to_model_state(hf_state, model.padded_vocab_size, model.config.model.untie_embed)
    ref = model.state_dict()
    missing = [k for k in ref if k not in state and not k.startswith("rotary_pos_emb.")]
    if missing:
        raise ValueError(f"checkpoint lacks {missing}")
    for k, v in state.items():
        if k not in ref:
            raise ValueError(f"model has no parameter {k!r}")
        if tuple(v.shape) != tuple(ref[k].shape):
            raise ValueError(f"{k}: checkpoint shape {tuple(v.shape)} != model shape {tuple(ref[k].shape)}")
    model.load_state_dict({k: v.to(ref[k].dtype) for k, v in state.items()}, strict=False)
