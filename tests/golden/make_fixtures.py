"""Writes the golden fixtures of tests/golden/ (run from the repository root:
``python tests/golden/make_fixtures.py``).

The reference's own tests hold no numeric vectors for this path (shape and
finiteness checks only), so the expected values here come from two
implementations that share no code with this repository's oracle or kernels:

* attention_f64.npz      float64 loops written from the definition of masked
                         softmax attention (oracle/brute_force.py);
* gpt2_transformers.npz,
  llama_transformers.npz logits and greedy continuations computed by the
                         transformers package (GPT2LMHeadModel,
                         LlamaForCausalLM) on weights drawn by
                         seeded_weights.py.
"""
import json
import pathlib
import sys

import numpy as np
import torch

HERE = pathlib.Path(__file__).resolve().parent
sys.path.insert(0, str(HERE.parent.parent))
sys.path.insert(0, str(HERE))

import seeded_weights as sw  # noqa: E402
from oracle import brute_force  # noqa: E402


def attention_cases():
    rng = np.random.default_rng(7)
    cases = {}

    def add(name, b, sq, sk, hn, gn, hd, mask):
        q = rng.standard_normal((b, sq, hn, hd)).astype(np.float32)
        k = rng.standard_normal((b, sk, gn, hd)).astype(np.float32)
        v = rng.standard_normal((b, sk, gn, hd)).astype(np.float32)
        cases[name + "_q"], cases[name + "_k"], cases[name + "_v"] = q, k, v
        if mask is not None:
            cases[name + "_mask"] = mask
        cases[name + "_out"] = brute_force.attention_f64(q, k, v, mask)

    causal = np.tril(np.ones((1, 9, 9), dtype=np.uint8))
    add("mha_causal", 2, 9, 9, 2, 2, 64, causal)
    prefix = 13                                                # chunk of 6 new tokens after 13 cached ones
    offset = (np.arange(19)[None, :] <= (prefix + np.arange(6))[:, None]).astype(np.uint8)[None]
    add("gqa_chunk", 1, 6, 19, 4, 2, 64, offset)
    add("decode", 3, 1, 37, 6, 2, 64, None)                   # one query token, no mask, group of 3
    np.savez_compressed(HERE / "attention_f64.npz", **cases)


def gpt2_case(seed):
    import transformers
    c = sw.GPT2
    cfg = transformers.GPT2Config(vocab_size=c["vocab"], n_positions=c["n_pos"], n_embd=c["d"], n_layer=c["layers"],
                                  n_head=c["heads"], activation_function="gelu", resid_pdrop=0.0, embd_pdrop=0.0,
                                  attn_pdrop=0.0, layer_norm_epsilon=c["eps"], bos_token_id=None, eos_token_id=None)
    model = transformers.GPT2LMHeadModel(cfg).eval()
    state = {"transformer." + k: v for k, v in sw.gpt2_state(seed).items()}
    state["lm_head.weight"] = state["transformer.wte.weight"]
    missing = model.load_state_dict(state, strict=False)
    assert not [k for k in missing.missing_keys if not k.endswith(("attn.bias", "attn.masked_bias"))], missing
    ids = torch.from_numpy(np.random.default_rng(seed + 1).integers(0, c["vocab"], size=(2, 21)))
    with torch.no_grad():
        logits = model(ids).logits
        tokens = model.generate(ids[:, :9], attention_mask=torch.ones_like(ids[:, :9]), max_new_tokens=12,
                                do_sample=False, pad_token_id=0)
        top2 = torch.topk(model(tokens).logits[:, 8:-1], 2, dim=-1)[0]
    margin = float((top2[..., 0] - top2[..., 1]).min())
    np.savez_compressed(HERE / "gpt2_transformers.npz", seed=seed, ids=ids.numpy(), logits=logits.numpy(),
                        tokens=tokens.numpy(), min_margin=margin, config=json.dumps(c),
                        transformers=transformers.__version__)
    return margin


def llama_case(seed):
    import transformers
    c = sw.LLAMA
    cfg = transformers.LlamaConfig(vocab_size=c["vocab"], hidden_size=c["d"], intermediate_size=c["ffn"],
                                   num_hidden_layers=c["layers"], num_attention_heads=c["heads"],
                                   num_key_value_heads=c["groups"], max_position_embeddings=c["n_pos"],
                                   rms_norm_eps=c["eps"], tie_word_embeddings=False, attention_bias=False,
                                   mlp_bias=False, attention_dropout=0.0, bos_token_id=None, eos_token_id=None,
                                   pad_token_id=None)
    model = transformers.LlamaForCausalLM(cfg).eval()
    model.load_state_dict(sw.llama_state(seed), strict=True)
    ids = torch.from_numpy(np.random.default_rng(seed + 1).integers(0, c["vocab"], size=(2, 21)))
    with torch.no_grad():
        logits = model(ids).logits
        tokens = model.generate(ids[:, :9], attention_mask=torch.ones_like(ids[:, :9]), max_new_tokens=12,
                                do_sample=False, pad_token_id=0)
        top2 = torch.topk(model(tokens).logits[:, 8:-1], 2, dim=-1)[0]
    margin = float((top2[..., 0] - top2[..., 1]).min())
    np.savez_compressed(HERE / "llama_transformers.npz", seed=seed, ids=ids.numpy(), logits=logits.numpy(),
                        tokens=tokens.numpy(), min_margin=margin, config=json.dumps(c),
                        transformers=transformers.__version__)
    return margin


if __name__ == "__main__":
    attention_cases()
    # Greedy continuations are only a fair test where no step is a near tie:
    # take the first seed whose smallest top-1/top-2 margin is clear of float noise.
    for case in (gpt2_case, llama_case):
        seed = 1
        while case(seed) < 5e-3:
            seed += 1
    for f in sorted(HERE.glob("*.npz")):
        print(f.name, f.stat().st_size, "bytes")
