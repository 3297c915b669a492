"""Weight loading from a Hugging Face GPT-2 checkpoint.  The checker here is
an INDEPENDENT implementation: transformers' GPT2LMHeadModel with random
weights (no download), saved to safetensors, loaded into the generation model.
On the CPU the name/shape mapping is checked; on the GPU the logits of the HIP
path are compared with transformers' and greedy tokens must agree."""
import pytest
import torch

from ironcore_amd import config as ic_config
from ironcore_amd import generation, weights

transformers = pytest.importorskip("transformers")


def _hf_model(seed=0, n_layer=3, n_head=4, n_embd=256, vocab=500, n_pos=96):
    cfg = transformers.GPT2Config(vocab_size=vocab, n_positions=n_pos, n_embd=n_embd, n_layer=n_layer, n_head=n_head,
                                  activation_function="gelu", resid_pdrop=0.0, embd_pdrop=0.0, attn_pdrop=0.0,
                                  layer_norm_epsilon=1e-5)
    torch.manual_seed(seed)
    model = transformers.GPT2LMHeadModel(cfg).eval()
    with torch.no_grad():  # the default init leaves biases at 0 and norms at 1: make them matter
        for name, p in model.named_parameters():
            if name.endswith("bias") or "ln_" in name:
                p.add_(0.1 * torch.randn_like(p))
    return model


def _our_config(hf):
    c = hf.config
    return ic_config.MainConfig(
        model=ic_config.ModelConfig(d_model=c.n_embd, d_ffn=4 * c.n_embd, num_layers=c.n_layer,
                                    num_attention_heads=c.n_head, head_dim=c.n_embd // c.n_head,
                                    max_seq_len=c.n_positions, max_position_embeddings=c.n_positions,
                                    dropout_attn=0.0, dropout_embd=0.0, dropout_mlp=0.0, precision="fp32",
                                    ln_eps=c.layer_norm_epsilon, activation_type="gelu"),
        trainer=ic_config.TrainerConfig(use_flash_attn=False))


def test_mapping_names_shapes_and_split(tmp_path):
    from safetensors.torch import save_file
    hf = _hf_model()
    state = {k: v.contiguous() for k, v in hf.state_dict().items() if not k.endswith("lm_head.weight")}
    path = tmp_path / "model.safetensors"
    save_file(state, str(path))
    model = generation.LanguageModel(_our_config(hf), vocab_size=500)
    weights.load_hf_gpt2(model, path)
    sd = model.state_dict()
    assert sd["embedding.word_embeddings.weight"].shape[0] == 512           # padded to a multiple of 128
    assert torch.equal(sd["embedding.word_embeddings.weight"][:500], hf.transformer.wte.weight)
    assert torch.count_nonzero(sd["embedding.word_embeddings.weight"][500:]) == 0
    c_attn = hf.transformer.h[1].attn.c_attn
    assert torch.equal(sd["model.layers.1.linear_q.weight"], c_attn.weight[:, :256])
    assert torch.equal(sd["model.layers.1.linear_kv.weight"], c_attn.weight[:, 256:])
    assert torch.equal(sd["model.layers.1.linear_kv.bias"], c_attn.bias[256:])
    assert torch.equal(sd["model.layers.2.mlp.down_proj.weight"], hf.transformer.h[2].mlp.c_proj.weight)
    assert torch.equal(sd["output_layernorm.layernorm.bias"], hf.transformer.ln_f.bias)
    with pytest.raises(ValueError):
        weights.hf_gpt2_to_model_state({"transformer.h.0.attn.rotary.weight": torch.zeros(1)}, 512)
    with pytest.raises(ValueError):                                          # a parameter left uncovered
        weights.load_hf_gpt2(model, {k: v for k, v in state.items() if "ln_f" not in k})


@pytest.mark.gpu
def test_logits_and_greedy_tokens_match_transformers(gpu):
    hf = _hf_model(seed=1)
    model = generation.LanguageModel(_our_config(hf), vocab_size=500)
    weights.load_hf_gpt2(model, {k: v for k, v in hf.state_dict().items()})
    model = model.to(gpu).eval()
    ids = torch.randint(0, 500, (3, 40), generator=torch.Generator().manual_seed(2))
    with torch.no_grad():
        want = hf(ids).logits                                                # [3, 40, 500]
        got = model(ids.to(gpu))[..., :500].cpu()
    assert (got - want).abs().max().item() < 2e-4
    with torch.no_grad():
        # an explicit mask: without one, generate() takes prompt tokens equal to pad_token_id for padding
        hf_tokens = hf.generate(ids, attention_mask=torch.ones_like(ids), max_new_tokens=24, do_sample=False,
                                pad_token_id=0)
    ours = generation.generate(model, ids.to(gpu), 24)
    torch.cuda.synchronize()
    assert torch.equal(ours.cpu(), hf_tokens)


def test_cpu_oracle_matches_transformers():
    """The CPU oracle's model forward (oracle/gpt2.py over oracle/dense_attention.py)
    against transformers' GPT-2 on the same weights: a third-party pin of the
    oracle itself."""
    from oracle import gpt2 as oracle_gpt2
    hf = _hf_model(seed=3)
    cfg = _our_config(hf)
    model = generation.LanguageModel(cfg, vocab_size=500)
    weights.load_hf_gpt2(model, dict(hf.state_dict()))
    w = {k: v.detach().clone() for k, v in model.state_dict().items()}
    m = cfg.model
    dims = oracle_gpt2.Dims(m.num_layers, m.num_attention_heads, m.num_attention_groups, m.d_model, m.ln_eps)
    ids = torch.randint(0, 500, (2, 33), generator=torch.Generator().manual_seed(4))
    with torch.no_grad():
        want = hf(ids).logits
    got = oracle_gpt2.forward_full(w, dims, ids)[..., :500]
    assert (got - want).abs().max().item() < 2e-4
    with torch.no_grad():
        hf_tokens = hf.generate(ids[:, :12], attention_mask=torch.ones_like(ids[:, :12]), max_new_tokens=10,
                                 do_sample=False, pad_token_id=0)
    assert torch.equal(oracle_gpt2.generate_paged(w, dims, ids[:, :12], 10), hf_tokens)
