"""End-to-end greedy generation through the block KV cache on the GPU, checked
against the CPU oracle's loops (same weights, same prompts)."""
import pytest
import torch

from ironcore_amd import config as ic_config
from ironcore_amd import generation
from oracle import gpt2 as oracle_gpt2

pytestmark = pytest.mark.gpu


def _dims(cfg):
    m = cfg.model
    return oracle_gpt2.Dims(m.num_layers, m.num_attention_heads, m.num_attention_groups, m.d_model, m.ln_eps)


def _small(precision, groups=4):
    return ic_config.MainConfig(
        model=ic_config.ModelConfig(d_model=256, d_ffn=512, num_layers=3, num_attention_heads=4,
                                    num_attention_groups=groups, head_dim=64, max_seq_len=128,
                                    max_position_embeddings=128, dropout_attn=0.0, dropout_embd=0.0,
                                    dropout_mlp=0.0, precision=precision),
        trainer=ic_config.TrainerConfig(use_flash_attn=False), init=ic_config.InitConfig(seed=0, init_std=0.08))


@pytest.mark.parametrize("groups", [4, 1])
def test_small_fp32_generate_matches_oracle_tokens(gpu, groups):
    cfg = _small("fp32", groups)
    torch.manual_seed(0)
    model = generation.LanguageModel(cfg, vocab_size=1000)
    w = {k: v.detach().clone() for k, v in model.state_dict().items()}
    ids = torch.randint(0, 1000, (3, 21), generator=torch.Generator().manual_seed(1))
    want, margins = oracle_gpt2.generate_paged(w, _dims(cfg), ids, 24, return_margins=True)
    full = oracle_gpt2.generate_full_recompute(w, _dims(cfg), ids, 24)
    assert torch.equal(want, full)
    model = model.to(gpu)
    got, got_margins = generation.generate(model, ids.to(gpu), 24, return_margins=True)
    torch.cuda.synchronize()
    assert margins.min().item() > 1e-4
    assert torch.equal(got.cpu(), want), f"min margin {margins.min().item()}"
    assert (got_margins.cpu() - margins).abs().max().item() < 1e-3
    # the GPU full-recompute loop (dense calls of the layer) agrees too
    assert torch.equal(generation.generate_full_recompute(model, ids.to(gpu), 24).cpu(), want)


def test_rotary_fp32_generate_matches_oracle_tokens(gpu):
    """Rotary embeddings: the cached path fuses the rotation into the KV append
    (keys enter the pool rotated at their index in the sequence), the dense
    path rotates query and key before the call; both pick the oracle's tokens."""
    from oracle import rope as oracle_rope
    cfg = _small("fp32", 2)
    cfg.model.positional_embedding.type = "rope"
    torch.manual_seed(0)
    model = generation.LanguageModel(cfg, vocab_size=1000)
    w = {k: v.detach().clone() for k, v in model.state_dict().items()}
    m = cfg.model
    dims = oracle_gpt2.Dims(m.num_layers, m.num_attention_heads, m.num_attention_groups, m.d_model, m.ln_eps,
                            rope=oracle_rope.rope_tables(m.d_model // m.num_attention_heads,
                                                         m.max_position_embeddings))
    ids = torch.randint(0, 1000, (3, 19), generator=torch.Generator().manual_seed(5))
    want, margins = oracle_gpt2.generate_paged(w, dims, ids, 20, return_margins=True)
    assert torch.equal(want, oracle_gpt2.generate_full_recompute(w, dims, ids, 20))
    assert margins.min().item() > 1e-4
    model = model.to(gpu)
    got, got_margins = generation.generate(model, ids.to(gpu), 20, return_margins=True)
    torch.cuda.synchronize()
    assert torch.equal(got.cpu(), want), f"min margin {margins.min().item()}"
    assert (got_margins.cpu() - margins).abs().max().item() < 1e-3
    assert torch.equal(generation.generate_full_recompute(model, ids.to(gpu), 20).cpu(), want)


def test_small_bf16_generate_paged_equals_recompute_on_gpu(gpu):
    """bf16, like with like: cached decode and full recompute on the same device
    pick the same tokens wherever the top-1/top-2 margin is not a rounding tie."""
    cfg = _small("bf16")
    torch.manual_seed(0)
    model = generation.LanguageModel(cfg, vocab_size=1000).to(gpu).to(torch.bfloat16)
    ids = torch.randint(0, 1000, (4, 33), generator=torch.Generator().manual_seed(2)).to(gpu)
    paged, margins = generation.generate(model, ids, 20, return_margins=True)
    full = generation.generate_full_recompute(model, ids, 20)
    torch.cuda.synchronize()
    same = (paged == full)[:, 33:]
    # after the first disagreement the contexts differ, so compare up to it
    for row in range(4):
        cols = torch.nonzero(~same[row]).flatten()
        if len(cols):
            first = cols[0].item()
            assert margins[row, first].item() < 0.25, "tokens differ at a step with a clear margin"


def test_gpt2_small_fp32_batch4_prompt128_decode64(gpu):
    """The reference-runnable configuration: GPT-2 small (12 layers, 12 heads,
    head_dim 64, vocab 50257), random-init fp32, batch 4, prompts of 128 uniform
    token ids, greedy decode of 64 tokens, KV block size 16, seed 0."""
    cfg = ic_config.gpt2_small_config("fp32")
    torch.manual_seed(0)
    model = generation.LanguageModel(cfg, vocab_size=50257)
    w = {k: v.detach().clone() for k, v in model.state_dict().items()}
    ids = torch.randint(0, 50257, (4, 128), generator=torch.Generator().manual_seed(0))
    want, margins = oracle_gpt2.generate_paged(w, _dims(cfg), ids, 64, return_margins=True)
    model = model.to(gpu)
    got, got_margins = generation.generate(model, ids.to(gpu), 64, return_margins=True)
    torch.cuda.synchronize()
    print(f"min top-1/top-2 margin: oracle {margins.min().item():.3e}, gpu {got_margins.min().item():.3e}")
    assert got.shape == (4, 192)
    assert torch.equal(got.cpu(), want), f"greedy tokens differ (min margin {margins.min().item():.3e})"


@pytest.mark.parametrize("positional", ["absolute", "rope"])
def test_multiple_choice_scoring_matches_oracle(gpu, positional):
    """HellaSwag-style scoring (hellaswag.py:63-88, 144-175): per-sequence mean
    cross-entropy from one causal pass (the prefill kernel at prefix 0), lowest
    loss wins.  Losses agree with the CPU oracle's to 1e-4 in fp32 and pick the
    same endings."""
    import torch.nn.functional as F
    from ironcore_amd import scoring
    from oracle import rope as oracle_rope
    cfg = _small("fp32", 2)
    cfg.model.positional_embedding.type = positional
    torch.manual_seed(3)
    model = generation.LanguageModel(cfg, vocab_size=1000)
    w = {k: v.detach().clone() for k, v in model.state_dict().items()}
    m = cfg.model
    rope = oracle_rope.rope_tables(m.d_model // m.num_attention_heads, m.max_position_embeddings) \
        if positional == "rope" else None
    dims = oracle_gpt2.Dims(m.num_layers, m.num_attention_heads, m.num_attention_groups, m.d_model, m.ln_eps,
                            rope=rope)
    g = torch.Generator().manual_seed(8)
    tokens = torch.randint(0, 1000, (12, 41), generator=g)           # 3 questions x 4 endings, padded length 41
    tokens[::4, 30:] = 999                                            # some padding tails
    logits = oracle_gpt2.forward_full(w, dims, tokens[:, :-1])
    want = torch.stack([F.cross_entropy(logits[i], tokens[i, 1:]) for i in range(12)])
    got = scoring.per_sample_losses(model.to(gpu).eval(), tokens.to(gpu))
    assert (got - want).abs().max().item() < 1e-4
    prompts = [i // 4 for i in range(12)]
    labels = [1 if i % 4 == 2 else 0 for i in range(12)]
    assert scoring.pick_endings(prompts, got.tolist(), labels) == scoring.pick_endings(prompts, want.tolist(), labels)


def test_scoring_batch_of_eighty_sequences_bf16(gpu):
    """A scoring batch wider than one wave's lanes (80 sequences: the prefill
    kernel then finds a workgroup's sequence by direct lookup instead of the
    in-wave ranking).  bf16 model; losses against the fp32 CPU oracle on the
    same weights within bf16's reach, against the same sequences scored 16 at a
    time (the ranked path) tightly, and the same endings picked."""
    import torch.nn.functional as F
    from ironcore_amd import scoring
    cfg = _small("bf16", 2)
    torch.manual_seed(4)
    model = generation.LanguageModel(cfg, vocab_size=1000)
    w = {k: v.detach().clone() for k, v in model.state_dict().items()}
    g = torch.Generator().manual_seed(9)
    tokens = torch.randint(0, 1000, (80, 33), generator=g)
    tokens[::5, 25:] = 999
    logits = oracle_gpt2.forward_full(w, _dims(cfg), tokens[:, :-1])
    want = torch.stack([F.cross_entropy(logits[i], tokens[i, 1:]) for i in range(80)])
    model = model.to(gpu).to(torch.bfloat16).eval()
    got = scoring.per_sample_losses(model, tokens.to(gpu))
    by16 = torch.cat([scoring.per_sample_losses(model, tokens[i:i + 16].to(gpu)) for i in range(0, 80, 16)])
    assert (got - by16).abs().max().item() < 2e-2
    assert (got - want).abs().max().item() < 6e-2
    prompts = [i // 4 for i in range(80)]
    labels = [1 if i % 4 == 1 else 0 for i in range(80)]
    picked, picked16 = scoring.pick_endings(prompts, got.tolist(), labels), scoring.pick_endings(prompts, by16.tolist(), labels)
    assert abs(picked["score"] - picked16["score"]) <= 5.0   # 20 questions: at most one near-tie may flip


@pytest.mark.parametrize("precision,positional,groups", [("fp32", "absolute", 4), ("fp32", "rope", 2),
                                                         ("bf16", "absolute", 1), ("bf16", "rope", 4)])
def test_graph_replay_generate_equals_the_step_by_step_loop(gpu, precision, positional, groups):
    """One captured decode step (device-side cache bookkeeping, attention through
    the C ABI, token selection) replayed for every new token: the tokens and the
    margins of the eager loop, step for step, across block boundaries (prompt
    of 21 with block 16, 40 new tokens); fp32 also against the CPU oracle.
    Two generations in a row reuse nothing of the first one's graph."""
    cfg = _small(precision, groups)
    cfg.model.positional_embedding.type = positional
    torch.manual_seed(0)
    model = generation.LanguageModel(cfg, vocab_size=1000)
    w = {k: v.detach().clone() for k, v in model.state_dict().items()}
    model = model.to(gpu)
    if precision == "bf16":
        model = model.to(torch.bfloat16)
    for seed, (b, s, n) in enumerate([(3, 21, 40), (5, 16, 3), (2, 30, 2), (1, 7, 1)]):
        ids = torch.randint(0, 1000, (b, s), generator=torch.Generator().manual_seed(seed))
        eager, eager_margins = generation.generate(model, ids.to(gpu), n, return_margins=True)
        graphed, margins = generation.generate(model, ids.to(gpu), n, return_margins=True, use_graph=True)
        torch.cuda.synchronize()
        assert graphed.shape == (b, s + n)
        assert torch.equal(graphed, eager), f"case {seed}"
        assert torch.equal(margins, eager_margins), f"case {seed}"
        if precision == "fp32" and positional == "absolute":
            want = oracle_gpt2.generate_paged(w, _dims(cfg), ids, n)
            assert torch.equal(graphed.cpu(), want)


def test_graph_replay_generate_with_eos_and_a_callers_cache(gpu):
    """End-of-sequence handling on the device (finished rows keep emitting the
    EOS id, the result is cut where the step-by-step loop stops) and a cache the
    caller owns: the sequences stay in it with their true lengths."""
    from ironcore_amd.kv_cache import PagedKVCache
    cfg = _small("fp32", 4)
    torch.manual_seed(0)
    model = generation.LanguageModel(cfg, vocab_size=50).to(gpu)
    ids = torch.randint(0, 50, (4, 10), generator=torch.Generator().manual_seed(3)).to(gpu)
    free_run = generation.generate(model, ids, 30)
    # an id that every row emits at some step, so that the loop ends early
    counts = torch.stack([(free_run[:, 10:] == t).any(1) for t in range(50)]).sum(1)
    eos = int(counts.argmax())
    eager = generation.generate(model, ids, 30, eos_token_id=eos)
    graphed = generation.generate(model, ids, 30, eos_token_id=eos, use_graph=True)
    torch.cuda.synchronize()
    assert torch.equal(graphed, eager)
    m = cfg.model
    cache = PagedKVCache(m.num_layers, 64, 16, m.num_attention_groups, m.d_model // m.num_attention_heads,
                         torch.float32, gpu)
    graphed = generation.generate(model, ids, 25, kv_cache=cache, use_graph=True)
    assert torch.equal(graphed, free_run[:, :35])
    assert sorted(cache.length(sid) for sid in range(4)) == [34] * 4    # the last token is never fed back
    with pytest.raises(ValueError):
        generation.generate(model, ids, 4, temperature=0.8, use_graph=True)


@pytest.mark.parametrize("seed", range(8))
def test_random_models_teacher_forced_logits(gpu, seed):
    """Seeded random architectures (layers, heads, KV groups, head dim, norm,
    activation, positional scheme, bias, tied or untied output) in fp32: the
    logits of a prefill chunk, a second chunk behind it and single cached steps
    on the GPU against the oracle's full causal pass over the same tokens
    (teacher forcing, so near ties in the argmax cannot hide or fake a
    difference), and the graph-replay loop against the step-by-step loop."""
    import random
    from ironcore_amd.kv_cache import PagedKVCache
    from oracle import rope as oracle_rope
    rng = random.Random(seed)
    hd = rng.choice([64, 128])
    heads, groups = rng.choice([(2, 1), (2, 2), (4, 1), (4, 2), (6, 3), (8, 2)])
    layers = rng.randint(1, 3)
    positional = rng.choice(["absolute", "rope"])
    ln_type = rng.choice(["layernorm", "rmsnorm"])
    activation = rng.choice(["gelu", "relu", "swiglu", "glu"])
    no_bias = rng.choice([False, True])
    untie = rng.choice([False, True])
    block = rng.choice([16, 32])
    vocab = rng.choice([300, 1000])
    d = heads * hd
    cfg = ic_config.MainConfig(
        model=ic_config.ModelConfig(d_model=d, d_ffn=2 * d, num_layers=layers, num_attention_heads=heads,
                                    num_attention_groups=groups, head_dim=hd, max_seq_len=160,
                                    max_position_embeddings=160, dropout_attn=0.0, dropout_embd=0.0, dropout_mlp=0.0,
                                    precision="fp32", ln_type=ln_type, activation_type=activation, no_bias=no_bias,
                                    untie_embed=untie,
                                    positional_embedding=ic_config.PositionalEmbeddingConfig(type=positional)),
        trainer=ic_config.TrainerConfig(use_flash_attn=False), init=ic_config.InitConfig(seed=seed, init_std=0.05))
    print(f"model {seed}: {layers} layers, {heads}/{groups} heads, hd {hd}, {positional}, {ln_type}, {activation}, "
          f"no_bias {no_bias}, untied {untie}, block {block}, vocab {vocab}", flush=True)
    torch.manual_seed(seed)
    model = generation.LanguageModel(cfg, vocab_size=vocab)
    w = {k: v.detach().clone() for k, v in model.state_dict().items() if not k.startswith("rotary_pos_emb.")}
    m = cfg.model
    rope = None
    if positional == "rope":
        rope = oracle_rope.rope_tables(hd, m.max_position_embeddings, m.positional_embedding.base)
    dims = oracle_gpt2.Dims(layers, heads, groups, d, m.ln_eps, rope=rope, ln_type=ln_type, activation=activation)
    b, first, second, steps = rng.randint(1, 4), rng.randint(1, 60), rng.randint(1, 40), 6
    total = first + second + steps
    ids = torch.randint(0, vocab, (b, total), generator=torch.Generator().manual_seed(seed))
    want = oracle_gpt2.forward_full(w, dims, ids)
    model = model.to(gpu).eval()
    cache = PagedKVCache(layers, b * ((total + block - 1) // block), block, groups, hd, torch.float32, gpu)
    sids = [cache.add_sequence() for _ in range(b)]
    got = []
    with torch.no_grad():
        got.append(model(ids[:, :first].to(gpu), kv_cache=cache, seq_ids=sids))
        got.append(model(ids[:, first:first + second].to(gpu), kv_cache=cache, seq_ids=sids))
        for t in range(first + second, total):
            got.append(model(ids[:, t:t + 1].to(gpu), kv_cache=cache, seq_ids=sids))
    torch.cuda.synchronize()
    got = torch.cat(got, dim=1).cpu()
    scale = want.abs().max().item()
    diff = (got - want).abs().max().item()
    assert diff <= 2e-4 * max(scale, 1.0), f"max|logit diff| {diff} (logits up to {scale})"
    prompt = ids[:, :first].to(gpu)
    eager = generation.generate(model, prompt, 12, block_size=block)
    graphed = generation.generate(model, prompt, 12, block_size=block, use_graph=True)
    torch.cuda.synchronize()
    assert torch.equal(eager, graphed)


@pytest.mark.parametrize("positional", ["absolute", "rope"])
def test_generate_with_prompts_of_unequal_length(gpu, positional):
    """Prompts of 1 to 40 tokens prefilled in one step: every row continues as
    it does when generated alone (the oracle's loop on that prompt), step by
    step and by graph replay."""
    from oracle import rope as oracle_rope
    cfg = _small("fp32", 2)
    cfg.model.positional_embedding.type = positional
    torch.manual_seed(0)
    model = generation.LanguageModel(cfg, vocab_size=1000)
    w = {k: v.detach().clone() for k, v in model.state_dict().items() if not k.startswith("rotary_pos_emb.")}
    m = cfg.model
    rope = None
    if positional == "rope":
        rope = oracle_rope.rope_tables(m.d_model // m.num_attention_heads, m.max_position_embeddings)
    dims = oracle_gpt2.Dims(m.num_layers, m.num_attention_heads, m.num_attention_groups, m.d_model, m.ln_eps,
                            rope=rope)
    lens = [1, 40, 17, 16, 33]
    ids = torch.randint(0, 1000, (len(lens), max(lens)), generator=torch.Generator().manual_seed(4))
    model = model.to(gpu)
    got = generation.generate(model, ids.to(gpu), 20, prompt_lens=lens)
    graphed, margins = generation.generate(model, ids.to(gpu), 20, prompt_lens=lens, use_graph=True,
                                           return_margins=True)
    torch.cuda.synchronize()
    assert margins.shape == (len(lens), 20)
    for i, n in enumerate(lens):
        want, want_margins = oracle_gpt2.generate_paged(w, dims, ids[i:i + 1, :n], 20, return_margins=True)
        assert want_margins.min().item() > 1e-4
        assert torch.equal(got[i].cpu(), want[0]), f"prompt {i} ({n} tokens)"
        assert torch.equal(graphed[i].cpu(), want[0]), f"prompt {i} ({n} tokens), graph replay"
    with pytest.raises(ValueError):
        generation.generate(model, ids.to(gpu), 4, prompt_lens=[1, 2])


@pytest.mark.parametrize("precision", ["fp32", "bf16"])
def test_rollout_samples_share_the_prompt(gpu, precision):
    """n continuations per prompt from ONE prefill: forks that alias the
    prompt's blocks, decoded in cohorts (bf16; fp32 has no cohort kernel and
    decodes them plainly).  At temperature 0 every sample is the greedy
    continuation of its prompt; with sampling the samples differ, stay inside
    the vocabulary and repeat under the same generator seed."""
    cfg = _small(precision, 2)
    torch.manual_seed(0)
    model = generation.LanguageModel(cfg, vocab_size=1000).to(gpu)
    if precision == "bf16":
        model = model.to(torch.bfloat16)
    prompts = torch.randint(0, 1000, (3, 37), generator=torch.Generator().manual_seed(6)).to(gpu)
    greedy = generation.generate(model, prompts, 12)
    same = generation.generate_samples(model, prompts, 5, 12, temperature=0.0)
    torch.cuda.synchronize()
    assert same.shape == (3, 5, 49)
    if precision == "fp32":
        assert torch.equal(same, greedy.unsqueeze(1).expand(3, 5, 49))
    else:
        # cohorts merge partial results in another order than the plain call: a near tie may flip
        agree = (same == greedy.unsqueeze(1)).float().mean().item()
        assert agree > 0.9 and torch.equal(same[:, :, :38], greedy.unsqueeze(1).expand(3, 5, 49)[:, :, :38])
    g = torch.Generator(device=gpu).manual_seed(11)
    drawn = generation.generate_samples(model, prompts, 5, 12, temperature=1.0, top_k=50, generator=g)
    g.manual_seed(11)
    again = generation.generate_samples(model, prompts, 5, 12, temperature=1.0, top_k=50, generator=g)
    torch.cuda.synchronize()
    assert torch.equal(drawn, again)
    assert torch.equal(drawn[:, :, :37], prompts.unsqueeze(1).expand(3, 5, 37))
    assert int(drawn.min()) >= 0 and int(drawn.max()) < 1000
    assert len({tuple(row.tolist()) for row in drawn[0, :, 37:]}) > 1, "samples of one prompt should differ"
