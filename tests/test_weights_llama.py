"""Llama-family weights and the reference's checkpoint directories.  The
checker for the model arithmetic is an INDEPENDENT implementation:
transformers' LlamaForCausalLM with random weights (no download).  It uses the
half-split rotary layout, RMSNorm and a SwiGLU MLP with separate gate/up
matrices, so agreement pins the channel permutation, the [gate | up] fusion,
the [in, out] orientation, RMSNorm and the rotation at true positions at once.
On the CPU the oracle's forward is compared with it; on the GPU the HIP path."""
import pytest
import torch

from ironcore_amd import config as ic_config
from ironcore_amd import generation, weights

transformers = pytest.importorskip("transformers")

VOCAB = 500


def _hf_model(seed=0, layers=3, heads=4, groups=2, hidden=256, ffn=384, n_pos=128, tie=False):
    cfg = transformers.LlamaConfig(vocab_size=VOCAB, hidden_size=hidden, intermediate_size=ffn,
                                   num_hidden_layers=layers, num_attention_heads=heads, num_key_value_heads=groups,
                                   max_position_embeddings=n_pos, rms_norm_eps=1e-5, tie_word_embeddings=tie,
                                   attention_bias=False, mlp_bias=False, attention_dropout=0.0)
    torch.manual_seed(seed)
    model = transformers.LlamaForCausalLM(cfg).eval()
    with torch.no_grad():  # norm scales start at 1: make them matter
        for name, p in model.named_parameters():
            if "norm" in name:
                p.add_(0.1 * torch.randn_like(p))
    return model


def _our_config(hf, precision="fp32"):
    c = hf.config
    return ic_config.MainConfig(
        model=ic_config.ModelConfig(
            d_model=c.hidden_size, d_ffn=c.intermediate_size, num_layers=c.num_hidden_layers,
            num_attention_heads=c.num_attention_heads, num_attention_groups=c.num_key_value_heads,
            head_dim=c.hidden_size // c.num_attention_heads, max_seq_len=c.max_position_embeddings,
            max_position_embeddings=c.max_position_embeddings, dropout_attn=0.0, dropout_embd=0.0, dropout_mlp=0.0,
            precision=precision, ln_eps=c.rms_norm_eps, ln_type="rmsnorm", activation_type="swiglu", no_bias=True,
            untie_embed=not c.tie_word_embeddings,
            positional_embedding=ic_config.PositionalEmbeddingConfig(type="rope", base=10000)),
        trainer=ic_config.TrainerConfig(use_flash_attn=False))


def _oracle_dims(cfg):
    from oracle import gpt2 as oracle_gpt2
    from oracle.rope import rope_tables
    m = cfg.model
    rope = rope_tables(m.d_model // m.num_attention_heads, m.max_position_embeddings, m.positional_embedding.base)
    return oracle_gpt2.Dims(m.num_layers, m.num_attention_heads, m.num_attention_groups, m.d_model, m.ln_eps,
                            rope=rope, ln_type="rmsnorm", activation="swiglu")


def test_halves_to_pairs_is_the_stated_permutation():
    hd, heads = 8, 3
    t = torch.arange(heads * hd).view(1, -1)
    got = weights.halves_to_pairs(t, heads, hd)[0]
    for h in range(heads):
        for i in range(hd // 2):
            assert got[h * hd + 2 * i] == h * hd + i
            assert got[h * hd + 2 * i + 1] == h * hd + i + hd // 2


def test_mapping_names_shapes_and_fusion(tmp_path):
    from safetensors.torch import save_file
    hf = _hf_model()
    path = tmp_path / "model.safetensors"
    save_file({k: v.contiguous() for k, v in hf.state_dict().items()}, str(path))
    model = generation.LanguageModel(_our_config(hf), vocab_size=VOCAB)
    assert not any(n.endswith(".bias") for n, _ in model.named_parameters())
    weights.load_hf_llama(model, path)
    sd = model.state_dict()
    layer = hf.model.layers[1]
    assert sd["embedding.word_embeddings.weight"].shape == (512, 256)
    assert torch.count_nonzero(sd["embedding.word_embeddings.weight"][VOCAB:]) == 0
    assert torch.equal(sd["output_layer.weight"][:, :VOCAB], hf.lm_head.weight.t())
    assert sd["model.layers.1.linear_q.weight"].shape == (256, 256)
    assert sd["model.layers.1.linear_kv.weight"].shape == (256, 2 * 2 * 64)
    # values are not permuted, keys and queries are (channel 1 of a head was channel hd/2)
    assert torch.equal(sd["model.layers.1.linear_kv.weight"][:, 128:], layer.self_attn.v_proj.weight.t())
    assert torch.equal(sd["model.layers.1.linear_kv.weight"][:, 1], layer.self_attn.k_proj.weight[32])
    assert torch.equal(sd["model.layers.1.linear_q.weight"][:, 64 + 3], layer.self_attn.q_proj.weight[64 + 32 + 1])
    assert torch.equal(sd["model.layers.1.mlp.up_proj.weight"][:, :384], layer.mlp.gate_proj.weight.t())
    assert torch.equal(sd["model.layers.1.mlp.up_proj.weight"][:, 384:], layer.mlp.up_proj.weight.t())
    assert torch.equal(sd["model.layers.1.mlp.down_proj.weight"], layer.mlp.down_proj.weight.t())
    assert torch.equal(sd["model.layers.1.attn_output.weight"], layer.self_attn.o_proj.weight.t())
    assert torch.equal(sd["output_layernorm.layernorm.weight"], hf.model.norm.weight)
    with pytest.raises(ValueError):
        weights.hf_llama_to_model_state({"model.layers.0.self_attn.qkv_proj.weight": torch.zeros(2, 2)}, 512, 4, 2, 64)
    with pytest.raises(ValueError):  # a parameter left uncovered
        weights.load_hf_llama(model, {k: v for k, v in hf.state_dict().items() if "model.norm" not in k})


def test_cpu_oracle_matches_transformers_llama():
    from oracle import gpt2 as oracle_gpt2
    hf = _hf_model(seed=3)
    cfg = _our_config(hf)
    model = generation.LanguageModel(cfg, vocab_size=VOCAB)
    weights.load_hf_llama(model, dict(hf.state_dict()))
    w = {k: v.detach().clone() for k, v in model.state_dict().items() if not k.startswith("rotary_pos_emb.")}
    dims = _oracle_dims(cfg)
    ids = torch.randint(0, VOCAB, (2, 33), generator=torch.Generator().manual_seed(4))
    with torch.no_grad():
        want = hf(ids).logits
    got = oracle_gpt2.forward_full(w, dims, ids)[..., :VOCAB]
    assert (got - want).abs().max().item() < 2e-4
    with torch.no_grad():
        hf_tokens = hf.generate(ids[:, :12], attention_mask=torch.ones_like(ids[:, :12]), max_new_tokens=10,
                                 do_sample=False, pad_token_id=0)
    assert torch.equal(oracle_gpt2.generate_paged(w, dims, ids[:, :12], 10), hf_tokens)


def test_tied_checkpoint_into_untied_model():
    hf = _hf_model(seed=5, tie=True)
    cfg = _our_config(hf)
    cfg.model.untie_embed = True
    model = generation.LanguageModel(cfg, vocab_size=VOCAB)
    state = {k: v for k, v in hf.state_dict().items() if k != "lm_head.weight"}
    weights.load_hf_llama(model, state)
    sd = model.state_dict()
    assert torch.equal(sd["output_layer.weight"], sd["embedding.word_embeddings.weight"].t())


def test_native_checkpoint_round_trip(tmp_path):
    hf = _hf_model(seed=6, layers=2)
    cfg = _our_config(hf)
    a = generation.LanguageModel(cfg, vocab_size=VOCAB)
    weights.load_hf_llama(a, dict(hf.state_dict()))
    assert weights.load_native_checkpoint(a, tmp_path / "absent") == -1
    assert weights.load_native_checkpoint(a, tmp_path) == -1                  # no latest_step.txt yet
    path = weights.save_native_checkpoint(a, tmp_path, 7)
    assert path == tmp_path / "step_7" / "pytorch_model.bin"
    assert (tmp_path / "latest_step.txt").read_text() == "7"
    weights.save_native_checkpoint(a, tmp_path, 9)
    b = generation.LanguageModel(cfg, vocab_size=VOCAB)
    assert weights.load_native_checkpoint(b, tmp_path) == 9                    # latest
    assert weights.load_native_checkpoint(b, tmp_path, step=7) == 7
    assert weights.load_native_checkpoint(b, tmp_path, step=8) == -1
    for (ka, va), (kb, vb) in zip(a.state_dict().items(), b.state_dict().items()):
        assert ka == kb and torch.equal(va, vb)
    # the reference's layout: a dict with the state under "model_state_dict"
    blob = torch.load(path, weights_only=True)
    assert set(blob) >= {"model_state_dict", "optimizer_state_dict", "lr_scheduler", "step", "config"}
    assert blob["step"] == 9 or blob["step"] == 7
    # same element count, other shape: reshaped as the reference does; other count: refused
    blob["model_state_dict"]["model.layers.0.linear_q.weight"] = blob["model_state_dict"][
        "model.layers.0.linear_q.weight"].reshape(-1)
    torch.save(blob, path)
    assert weights.load_native_checkpoint(b, tmp_path, step=7) == 7
    assert torch.equal(b.state_dict()["model.layers.0.linear_q.weight"], a.state_dict()["model.layers.0.linear_q.weight"])
    blob["model_state_dict"]["model.layers.0.linear_q.weight"] = torch.zeros(5)
    torch.save(blob, path)
    with pytest.raises(ValueError):
        weights.load_native_checkpoint(b, tmp_path, step=7)


class _NotATensor:  # stands for the config objects the reference pickles into its checkpoints
    pass


def test_native_checkpoint_with_pickled_objects_is_refused(tmp_path):
    hf = _hf_model(seed=6, layers=1)
    model = generation.LanguageModel(_our_config(hf), vocab_size=VOCAB)
    (tmp_path / "step_1").mkdir()
    torch.save({"model_state_dict": model.state_dict(), "config": _NotATensor()}, tmp_path / "step_1" / "pytorch_model.bin")
    (tmp_path / "latest_step.txt").write_text("1")
    with pytest.raises(RuntimeError, match="without executing code"):
        weights.load_native_checkpoint(model, tmp_path)


@pytest.mark.gpu
def test_logits_and_greedy_tokens_match_transformers_llama(gpu):
    hf = _hf_model(seed=1)
    model = generation.LanguageModel(_our_config(hf), vocab_size=VOCAB)
    weights.load_hf_llama(model, dict(hf.state_dict()))
    model = model.to(gpu).eval()
    ids = torch.randint(0, VOCAB, (3, 40), generator=torch.Generator().manual_seed(2))
    with torch.no_grad():
        want = hf(ids).logits
        got = model(ids.to(gpu))[..., :VOCAB].cpu()
    assert (got - want).abs().max().item() < 2e-4
    with torch.no_grad():
        # an explicit mask: without one, generate() takes prompt tokens equal to pad_token_id for padding
        hf_tokens = hf.generate(ids, attention_mask=torch.ones_like(ids), max_new_tokens=24, do_sample=False,
                                pad_token_id=0)
    ours = generation.generate(model, ids.to(gpu), 24)
    torch.cuda.synchronize()
    assert torch.equal(ours.cpu(), hf_tokens)


@pytest.mark.gpu
def test_bf16_llama_shape_generation_follows_the_oracle(gpu):
    """bf16, head_dim 128, GQA 4:1 (the MFMA decode and prefill kernels):
    greedy tokens of the HIP path equal the CPU oracle's wherever the oracle's
    own top-1/top-2 margin is clear of bf16 noise."""
    from oracle import gpt2 as oracle_gpt2
    hf = _hf_model(seed=8, layers=2, heads=4, groups=1, hidden=512, ffn=768)
    cfg = _our_config(hf, precision="bf16")
    model = generation.LanguageModel(cfg, vocab_size=VOCAB)
    weights.load_hf_llama(model, dict(hf.state_dict()))
    model = model.to(torch.bfloat16)
    w = {k: v.detach().clone() for k, v in model.state_dict().items() if not k.startswith("rotary_pos_emb.")}
    dims = _oracle_dims(cfg)
    ids = torch.randint(0, VOCAB, (2, 24), generator=torch.Generator().manual_seed(9))
    want, margins = oracle_gpt2.generate_paged(w, dims, ids, 12, return_margins=True)
    ours = generation.generate(model.to(gpu).eval(), ids.to(gpu), 12).cpu()
    torch.cuda.synchronize()
    new_want, new_ours = want[:, 24:], ours[:, 24:]
    for b in range(2):
        for t in range(12):
            if new_ours[b, t] != new_want[b, t]:
                assert margins[b, t].item() < 0.15, (b, t, margins[b, t].item())
                break  # after a near-tie the sequences legitimately part ways
