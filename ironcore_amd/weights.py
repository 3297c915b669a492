"""Weights into the generation model: Hugging Face GPT-2 and Llama-family
checkpoints (safetensors or an in-memory state dict) and the reference's own
checkpoint directories.

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

Llama family (``WeightMapper._hf_llama_to_ironcore``, weight_mapping.py:404-542):
the same two defects, plus the rotary convention.  Hugging Face rotates the
halves of a head (element i with element i + hd/2); the reference's rotary
module rotates neighbouring pairs (2i, 2i+1) (ironcore/layers/
positional_embedding/rotary.py:75-82).  The two agree once the output channels
of ``q_proj`` and ``k_proj`` are re-ordered per head, old channel i -> 2i and
old channel i + hd/2 -> 2i+1: the same permutation on queries and keys leaves
every q.k unchanged, and values are not rotated.  ``gate_proj`` and ``up_proj``
fuse into the doubled up-projection as ``[gate | up]`` (swiglu takes silu of the
first half, activations.py:37-38).

Native checkpoints (ironcore/checkpointing/native.py:103-229, 323-472):
``<model_path>/latest_step.txt`` names the step, ``<model_path>/step_<n>/
pytorch_model.bin`` is a ``torch.save`` of a dict whose ``model_state_dict``
holds the model's ``state_dict()`` by name.
"""
from __future__ import annotations

import re
from pathlib import Path
from typing import Dict, Optional, Union

import torch

_IGNORED = re.compile(r"(^|\.)(attn\.bias|attn\.masked_bias|lm_head\.weight)$")


def hf_gpt2_to_model_state(hf_state: Dict[str, torch.Tensor], padded_vocab_size: int,
                           untie_embed: bool = False) -> Dict[str, torch.Tensor]:
    """Map a GPT-2 state dict (keys with or without the ``transformer.``
    prefix) to this model's names and shapes.  Raises on keys it cannot place."""
    out: Dict[str, torch.Tensor] = {}

    def pad_vocab(t):
        return _pad_vocab(t, padded_vocab_size)

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


def _pad_vocab(t: torch.Tensor, padded_vocab_size: int) -> torch.Tensor:
    if t.shape[0] > padded_vocab_size:
        raise ValueError(f"checkpoint vocabulary {t.shape[0]} exceeds the model's {padded_vocab_size}")
    padded = t.new_zeros(padded_vocab_size, t.shape[1])
    padded[:t.shape[0]] = t
    return padded


def halves_to_pairs(t: torch.Tensor, heads: int, head_dim: int) -> torch.Tensor:
    """Re-order the LAST dim of ``t`` (``heads * head_dim`` output channels)
    from the half-split rotary layout to the neighbouring-pair layout: within
    each head, new channel 2i = old i and new channel 2i+1 = old i + hd/2."""
    lead = t.shape[:-1]
    x = t.reshape(*lead, heads, 2, head_dim // 2)
    return x.transpose(-1, -2).reshape(*lead, heads * head_dim).contiguous()


_LLAMA_IGNORED = re.compile(r"rotary_emb\.inv_freq$")


def hf_llama_to_model_state(hf_state: Dict[str, torch.Tensor], padded_vocab_size: int, num_heads: int,
                            num_groups: int, head_dim: int, untie_embed: bool = True) -> Dict[str, torch.Tensor]:
    """Map a Llama-style state dict (Llama, Mistral, Qwen2 ... :
    ``model.layers.N.self_attn.{q,k,v,o}_proj``, ``mlp.{gate,up,down}_proj``)
    to this model's names, ``[in, out]`` orientation and pair-wise rotary
    channel order.  Raises on keys it cannot place."""
    out: Dict[str, torch.Tensor] = {}
    layers: Dict[str, Dict[str, torch.Tensor]] = {}
    for key, tensor in hf_state.items():
        if key == "model.embed_tokens.weight":
            out["embedding.word_embeddings.weight"] = _pad_vocab(tensor, padded_vocab_size)
        elif key in ("model.norm.weight", "model.norm.bias"):
            out["output_layernorm.layernorm." + key.rsplit(".", 1)[1]] = tensor
        elif key == "lm_head.weight":
            if untie_embed:  # [vocab, d] -> the [d, vocab] the output layer multiplies by
                out["output_layer.weight"] = _pad_vocab(tensor, padded_vocab_size).t().contiguous()
        elif (m := re.match(r"model\.layers\.(\d+)\.(.*)", key)) is not None:
            layers.setdefault(m.group(1), {})[m.group(2)] = tensor
        elif not _LLAMA_IGNORED.search(key):
            raise ValueError(f"unmapped checkpoint key {key!r}")
    if untie_embed and "output_layer.weight" not in out and "embedding.word_embeddings.weight" in out:
        # a checkpoint saved with tied embeddings for a model that keeps its own output matrix
        out["output_layer.weight"] = out["embedding.word_embeddings.weight"].t().contiguous()

    def oriented(t):  # nn.Linear weight [out, in] -> [in, out]; a bias stays as it is
        return t.t() if t.dim() == 2 else t

    for n, entries in layers.items():
        pre = f"model.layers.{n}."
        used = set()

        def take(name):
            used.add(name)
            return entries[name]

        for part in ("weight", "bias"):
            if f"input_layernorm.{part}" in entries:
                out[pre + f"input_layernorm.layernorm.{part}"] = take(f"input_layernorm.{part}")
            if f"post_attention_layernorm.{part}" in entries:
                out[pre + f"post_attn_layernorm.layernorm.{part}"] = take(f"post_attention_layernorm.{part}")
            if f"self_attn.q_proj.{part}" in entries:
                q = oriented(take(f"self_attn.q_proj.{part}"))
                out[pre + f"linear_q.{part}"] = halves_to_pairs(q, num_heads, head_dim)
            if f"self_attn.k_proj.{part}" in entries:
                k = halves_to_pairs(oriented(take(f"self_attn.k_proj.{part}")), num_groups, head_dim)
                v = oriented(take(f"self_attn.v_proj.{part}"))
                out[pre + f"linear_kv.{part}"] = torch.cat([k, v], dim=-1).contiguous()
            if f"self_attn.o_proj.{part}" in entries:
                out[pre + f"attn_output.{part}"] = oriented(take(f"self_attn.o_proj.{part}")).contiguous()
            if f"mlp.gate_proj.{part}" in entries:
                gate, up = oriented(take(f"mlp.gate_proj.{part}")), oriented(take(f"mlp.up_proj.{part}"))
                out[pre + f"mlp.up_proj.{part}"] = torch.cat([gate, up], dim=-1).contiguous()
            elif f"mlp.up_proj.{part}" in entries:
                out[pre + f"mlp.up_proj.{part}"] = oriented(take(f"mlp.up_proj.{part}")).contiguous()
            if f"mlp.down_proj.{part}" in entries:
                out[pre + f"mlp.down_proj.{part}"] = oriented(take(f"mlp.down_proj.{part}")).contiguous()
        left = [k for k in entries if k not in used and not _LLAMA_IGNORED.search(k)]
        if left:
            raise ValueError(f"unmapped checkpoint keys in layer {n}: {left}")
    return out


def _read_state(source) -> Dict[str, torch.Tensor]:
    if isinstance(source, dict):
        return source
    from safetensors.torch import load_file
    return load_file(str(source))


def _install(model, state: Dict[str, torch.Tensor], zero_missing_bias: bool = False) -> None:
    """Strict load: every parameter of the model covered, every mapped key
    placed, shapes equal.  ``zero_missing_bias`` fills biases the checkpoint
    does not carry with zeros (Qwen2-style checkpoints have them on q/k/v only
    while the model's ``no_bias`` switch is all or nothing)."""
    ref = model.state_dict()
    missing = [k for k in ref if k not in state and not k.startswith("rotary_pos_emb.")]
    if zero_missing_bias:
        for k in [k for k in missing if k.endswith(".bias")]:
            state[k] = torch.zeros_like(ref[k])
        missing = [k for k in missing if not k.endswith(".bias")]
    if missing:
        raise ValueError(f"checkpoint lacks {missing}")
    for k, v in state.items():
        if k not in ref:
            raise ValueError(f"model has no parameter {k!r}")
        if tuple(v.shape) != tuple(ref[k].shape):
            raise ValueError(f"{k}: checkpoint shape {tuple(v.shape)} != model shape {tuple(ref[k].shape)}")
    model.load_state_dict({k: v.to(ref[k].dtype) for k, v in state.items()}, strict=False)


def load_hf_gpt2(model, source) -> None:
    """Load GPT-2 weights into ``generation.LanguageModel`` from a
    ``.safetensors`` file (path) or a state dict.  Strict: every parameter of
    the model must be covered and every checkpoint key placed."""
    _install(model, hf_gpt2_to_model_state(_read_state(source), model.padded_vocab_size,
                                           model.config.model.untie_embed))


def load_hf_llama(model, source, zero_missing_bias: bool = False) -> None:
    """Load Llama-family weights into ``generation.LanguageModel`` (configured
    with ``ln_type="rmsnorm"``, ``activation_type="swiglu"``, rotary positions)
    from a ``.safetensors`` file or a state dict."""
    m = model.config.model
    state = hf_llama_to_model_state(_read_state(source), model.padded_vocab_size, m.num_attention_heads,
                                    m.num_attention_groups, m.d_model // m.num_attention_heads, m.untie_embed)
    _install(model, state, zero_missing_bias)


_LATEST_STEP_FILENAME = "latest_step.txt"  # native.py:35-36
_CKPT_FILENAME = "pytorch_model.bin"


def save_native_checkpoint(model, model_path: Union[str, Path], step: int) -> Path:
    """Write ``model.state_dict()`` in the reference's directory layout
    (native.py:343-350, 455-483) at tensor-parallel size 1: no optimizer or
    scheduler state, ``config`` left out (the reference pickles its own config
    classes there, which only its own loader can resolve)."""
    directory = Path(model_path) / f"step_{step}"
    directory.mkdir(parents=True, exist_ok=True)
    checkpoint = {
        "model_state_dict": {k: v.detach().cpu() for k, v in model.state_dict().items()},
        "optimizer_state_dict": None,
        "lr_scheduler": None,
        "step": step,
        "config": None,
        "hf_config": None,
    }
    with open(directory / _CKPT_FILENAME, "wb") as f:
        torch.save(checkpoint, f)
    (Path(model_path) / _LATEST_STEP_FILENAME).write_text(str(step), encoding="utf-8")
    return directory / _CKPT_FILENAME


def load_native_checkpoint(model, model_path: Union[str, Path], step: int = -1) -> int:
    """Restore the model from ``<model_path>/step_<n>/pytorch_model.bin``
    (native.py:103-229 at tensor-parallel size 1; ``step < 0`` reads
    ``latest_step.txt``).  Returns the step, or -1 when there is nothing to
    load, as the reference does.  The file is read with
    ``torch.load(weights_only=True)``: a checkpoint whose ``config`` entry
    holds the reference's pickled config classes is refused by that loader
    and the error says so; tensors are matched by name and, as in the
    reference (native.py:213-221), reshaped to the parameter when the element
    counts agree."""
    root = Path(model_path)
    if str(model_path) == "" or not root.exists():
        return -1
    if step < 0:
        latest = root / _LATEST_STEP_FILENAME
        if not latest.exists():
            return -1
        step = int(latest.read_text(encoding="utf-8").strip())
    directory = root / f"step_{step}"
    path = (directory / "tp0" if (directory / "tp0").exists() else directory) / _CKPT_FILENAME
    if not path.exists():
        return -1
    try:
        checkpoint = torch.load(path, weights_only=True, map_location="cpu")
    except Exception as err:  # the safe unpickler names the class it will not build
        raise RuntimeError(f"{path}: not loadable without executing code from the file "
                           f"(save it without the pickled config objects): {err}") from err
    saved = checkpoint["model_state_dict"]
    state = {}
    for name, target in model.state_dict().items():
        if name not in saved:
            if name.startswith("rotary_pos_emb."):
                continue
            raise ValueError(f"checkpoint lacks {name!r}")
        if saved[name].numel() != target.numel():
            raise ValueError(f"loaded layer [{name}] has {saved[name].numel()} elements, "
                             f"target shape is {tuple(target.shape)}")
        state[name] = saved[name].reshape_as(target).to(target.dtype)
    model.load_state_dict(state, strict=False)
    return step
