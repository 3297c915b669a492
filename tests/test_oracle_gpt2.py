"""Pins the model-level oracle (oracle/gpt2.py): the block arithmetic against an
independent torch.nn encoder layer carrying the same weights, and the
block-KV-cache generate loop against full recompute (for a causal model the
last-position logits must agree)."""
import pytest
import torch

from ironcore_amd import config as ic_config
from ironcore_amd import generation
from oracle import gpt2 as oracle_gpt2


def _tiny_config(layers=2, heads=4, groups=4, d_model=64, d_ffn=128, max_len=64):
    return ic_config.MainConfig(
        model=ic_config.ModelConfig(d_model=d_model, d_ffn=d_ffn, num_layers=layers, num_attention_heads=heads,
                                    num_attention_groups=groups, head_dim=d_model // heads, max_seq_len=max_len,
                                    max_position_embeddings=max_len, dropout_attn=0.0, dropout_embd=0.0,
                                    dropout_mlp=0.0, precision="fp32"),
        trainer=ic_config.TrainerConfig(use_flash_attn=False),
        init=ic_config.InitConfig(seed=0, init_std=0.2))


def _model_and_weights(cfg, vocab=300, seed=0):
    torch.manual_seed(seed)
    model = generation.LanguageModel(cfg, vocab_size=vocab)
    with torch.no_grad():                       # non-trivial biases and norm scales
        for name, p in model.named_parameters():
            if "bias" in name or "norm" in name:
                p.add_(0.1 * torch.randn_like(p))
    w = {k: v.detach().clone() for k, v in model.state_dict().items()}
    m = cfg.model
    return model, w, oracle_gpt2.Dims(m.num_layers, m.num_attention_heads, m.num_attention_groups, m.d_model, m.ln_eps)


def test_padded_vocab_rows_are_zero_and_score_zero():
    cfg = _tiny_config()
    model, w, dims = _model_and_weights(cfg, vocab=300)
    assert model.padded_vocab_size == 384
    assert torch.count_nonzero(w["embedding.word_embeddings.weight"][300:]) == 0
    logits = oracle_gpt2.forward_full(w, dims, torch.randint(0, 300, (2, 9)))
    assert logits.shape == (2, 9, 384)
    assert torch.count_nonzero(logits[..., 300:]) == 0


def test_block_matches_torch_encoder_layer():
    """One pre-LN block == nn.TransformerEncoderLayer(norm_first=True) with the
    same weights (an implementation that shares no code with the oracle)."""
    cfg = _tiny_config(layers=1)
    _, w, dims = _model_and_weights(cfg, seed=3)
    d = dims.d_model
    ref = torch.nn.TransformerEncoderLayer(d, dims.num_heads, dim_feedforward=128, dropout=0.0,
                                           activation="gelu", batch_first=True, norm_first=True)
    p = "model.layers.0."
    with torch.no_grad():
        wk, wv = torch.chunk(w[p + "linear_kv.weight"], 2, dim=-1)
        bk, bv = torch.chunk(w[p + "linear_kv.bias"], 2, dim=-1)
        ref.self_attn.in_proj_weight.copy_(torch.cat([w[p + "linear_q.weight"].T, wk.T, wv.T]))
        ref.self_attn.in_proj_bias.copy_(torch.cat([w[p + "linear_q.bias"], bk, bv]))
        ref.self_attn.out_proj.weight.copy_(w[p + "attn_output.weight"].T)
        ref.self_attn.out_proj.bias.copy_(w[p + "attn_output.bias"])
        ref.linear1.weight.copy_(w[p + "mlp.up_proj.weight"].T)
        ref.linear1.bias.copy_(w[p + "mlp.up_proj.bias"])
        ref.linear2.weight.copy_(w[p + "mlp.down_proj.weight"].T)
        ref.linear2.bias.copy_(w[p + "mlp.down_proj.bias"])
        ref.norm1.weight.copy_(w[p + "input_layernorm.layernorm.weight"])
        ref.norm1.bias.copy_(w[p + "input_layernorm.layernorm.bias"])
        ref.norm2.weight.copy_(w[p + "post_attn_layernorm.layernorm.weight"])
        ref.norm2.bias.copy_(w[p + "post_attn_layernorm.layernorm.bias"])
    ref.eval()
    x = torch.randn(2, 11, d, generator=torch.Generator().manual_seed(1))
    mask = torch.tril(torch.ones(11, 11)).view(1, 1, 11, 11) > 0.5
    from oracle.dense_attention import dense_attention
    got = oracle_gpt2._layer(x, w, p, dims, lambda q, k, v: dense_attention(q, k, v, mask))
    with torch.no_grad():
        want = ref(x, src_mask=torch.triu(torch.full((11, 11), float("-inf")), diagonal=1))
    torch.testing.assert_close(got, want, rtol=0, atol=2e-5)


@pytest.mark.parametrize("heads,groups", [(4, 4), (4, 2), (4, 1)])
def test_paged_forward_equals_full_forward(heads, groups):
    cfg = _tiny_config(heads=heads, groups=groups)
    _, w, dims = _model_and_weights(cfg, seed=5)
    ids = torch.randint(0, 300, (3, 37), generator=torch.Generator().manual_seed(2))
    full = oracle_gpt2.forward_full(w, dims, ids)
    cache = oracle_gpt2.OracleCache(dims, 3, 64, 16, torch.float32)
    pre = oracle_gpt2.forward_paged(w, dims, cache, ids[:, :20])          # prefill 20 tokens
    torch.testing.assert_close(pre, full[:, :20], rtol=0, atol=2e-5)
    mid = oracle_gpt2.forward_paged(w, dims, cache, ids[:, 20:33])        # a 13-token chunk
    torch.testing.assert_close(mid, full[:, 20:33], rtol=0, atol=2e-5)
    for t in range(33, 37):                                               # single-token steps
        one = oracle_gpt2.forward_paged(w, dims, cache, ids[:, t:t + 1])
        torch.testing.assert_close(one[:, 0], full[:, t], rtol=0, atol=2e-5)


def test_generate_paged_equals_full_recompute():
    cfg = _tiny_config(layers=3)
    _, w, dims = _model_and_weights(cfg, seed=7)
    ids = torch.randint(0, 300, (4, 12), generator=torch.Generator().manual_seed(3))
    full, margins = oracle_gpt2.generate_full_recompute(w, dims, ids, 20, return_margins=True)
    paged = oracle_gpt2.generate_paged(w, dims, ids, 20)
    assert margins.min().item() > 1e-4, "degenerate test: top-1/top-2 nearly tied"
    assert torch.equal(full, paged)
    assert full.shape == (4, 32)


def test_product_model_on_cpu_shares_the_oracle_arithmetic_outside_attention():
    """Embedding, norms, linears and logits of the product model (torch ops) match
    the oracle when attention is taken out of the picture (one token, so the
    softmax is over a single key and attention returns V)."""
    cfg = _tiny_config()
    model, w, dims = _model_and_weights(cfg, seed=9)
    ids = torch.randint(0, 300, (2, 1))
    want = oracle_gpt2.forward_full(w, dims, ids)

    class _Identity(torch.nn.Module):
        def forward(self, q, k, v, mask=None, **kw):
            rep = q.shape[2] // k.shape[2]
            return v.repeat_interleave(rep, dim=2).reshape(q.shape[0], 1, -1)
    for layer in model.model.layers:
        layer.self_attention = _Identity()
    got = model(ids)
    torch.testing.assert_close(got, want, rtol=0, atol=2e-5)


def test_sampler_matches_reference_recipe():
    logits = torch.tensor([[1.0, 3.0, 2.0, -1.0, 0.5]])
    assert generation.sample_next(logits).item() == 1                      # greedy
    g = torch.Generator().manual_seed(0)
    draws = torch.cat([generation.sample_next(logits, temperature=0.7, top_k=2, generator=g) for _ in range(400)])
    assert set(draws.flatten().tolist()) <= {1, 2}                         # only the top-2 survive
    p1 = torch.softmax(torch.tensor([3.0, 2.0]) / 0.7, 0)[0].item()
    assert abs((draws == 1).float().mean().item() - p1) < 0.08


def _rope_dims(cfg):
    from oracle import rope as oracle_rope
    m = cfg.model
    pe = m.positional_embedding
    tables = oracle_rope.rope_tables(m.d_model // m.num_attention_heads, m.max_position_embeddings, pe.base,
                                     pe.scaling_factor, pe.offset)
    return oracle_gpt2.Dims(m.num_layers, m.num_attention_heads, m.num_attention_groups, m.d_model, m.ln_eps,
                            rope=tables)


def test_rotary_model_paged_forward_equals_full_forward_and_generates_alike():
    """With rotary embeddings at the token's index in its sequence, keys rotated
    once when they enter the cache serve every later step: cached passes equal
    the full causal pass, and the rotation really matters (it changes the logits)."""
    cfg = _tiny_config(layers=2, heads=4, groups=2)
    cfg.model.positional_embedding.type = "rope"
    _, w, _ = _model_and_weights(cfg, seed=9)
    assert "embedding.position_embedding.weight" not in w
    dims = _rope_dims(cfg)
    ids = torch.randint(0, 300, (3, 30), generator=torch.Generator().manual_seed(4))
    full = oracle_gpt2.forward_full(w, dims, ids)
    cache = oracle_gpt2.OracleCache(dims, 3, 64, 16, torch.float32)
    pre = oracle_gpt2.forward_paged(w, dims, cache, ids[:, :17])
    torch.testing.assert_close(pre, full[:, :17], rtol=0, atol=2e-5)
    for t in range(17, 30):
        one = oracle_gpt2.forward_paged(w, dims, cache, ids[:, t:t + 1])
        torch.testing.assert_close(one[:, 0], full[:, t], rtol=0, atol=2e-5)
    m = cfg.model
    plain = oracle_gpt2.Dims(m.num_layers, m.num_attention_heads, m.num_attention_groups, m.d_model, m.ln_eps)
    assert (oracle_gpt2.forward_full(w, plain, ids) - full).abs().max().item() > 1e-2
    gen_full, margins = oracle_gpt2.generate_full_recompute(w, dims, ids[:, :10], 16, return_margins=True)
    assert margins.min().item() > 1e-4
    assert torch.equal(gen_full, oracle_gpt2.generate_paged(w, dims, ids[:, :10], 16))
