"""Random traffic through the attention layer and the block KV cache together:
prompts of random length prefilled in one or two chunks, batches of decode
steps over random subsets of the live sequences (with cohorts when the batch
is made of forks listed side by side), steps that give every sequence a chunk of
its own length, forks and frees in between.  The host
keeps every sequence's K/V rows; after each call the layer's output must be
the oracle's dense attention over those rows (bars: parity_bars.py)."""
import random

import pytest
import torch

from ironcore_amd import config as ic_config
from ironcore_amd.kv_cache import OutOfBlocks, PagedKVCache
from ironcore_amd.layers import Attention
from oracle.dense_attention import dense_attention
from parity_bars import hold

pytestmark = pytest.mark.gpu


@pytest.mark.parametrize("seed,hn,gn,hd,block", [(0, 4, 2, 64, 16), (1, 8, 8, 128, 16), (2, 14, 2, 128, 32),
                                                  (3, 6, 1, 64, 64)])
def test_random_layer_and_cache_traffic(gpu, seed, hn, gn, hd, block):
    rng = random.Random(seed)
    g = torch.Generator().manual_seed(seed)
    cfg = ic_config.MainConfig(model=ic_config.ModelConfig(
        d_model=hn * hd, num_attention_heads=hn, num_attention_groups=gn, head_dim=hd, dropout_attn=0.0,
        precision="bf16"), trainer=ic_config.TrainerConfig(use_flash_attn=False))
    attn = Attention(cfg).to(gpu).eval()
    cache = PagedKVCache(1, 160, block, gn, hd, torch.bfloat16, gpu)
    rows = {}                                   # sid -> (K [t, gn, hd], V [t, gn, hd]) on the host

    def draw(b, s, heads):
        return torch.randn(b, s, heads, hd, generator=g).bfloat16()

    def step(sids, s, cohort=1):
        """New tokens for each of sids through the layer (s: one count for all, or one per
        sequence: rows a sequence does not have are padding); checks every output row."""
        b = len(sids)
        counts = [s] * b if isinstance(s, int) else list(s)
        width = max(counts)
        q, k, v = draw(b, width, hn), draw(b, width, gn), draw(b, width, gn)
        meta = cache.prepare(sids, s, cohort_size=cohort)
        out = attn(q.to(gpu), k.to(gpu), v.to(gpu), None, kv_cache=cache.layer(0), attn_metadata=meta)
        torch.cuda.synchronize()
        for i, (sid, c) in enumerate(zip(sids, counts)):
            assert torch.count_nonzero(out[i, c:]) == 0, "padding rows must come back as zeros"
            if c == 0:
                continue
            K = torch.cat([rows[sid][0], k[i, :c]]) if sid in rows else k[i, :c]
            V = torch.cat([rows[sid][1], v[i, :c]]) if sid in rows else v[i, :c]
            rows[sid] = (K, V)
            t = K.shape[0]
            causal = (torch.arange(t).unsqueeze(0) <= (t - c) + torch.arange(c).unsqueeze(1)).view(1, 1, c, t)
            ref = dense_attention(q[i:i + 1, :c], K.unsqueeze(0), V.unsqueeze(0), causal)
            truth = dense_attention(q[i:i + 1, :c].double(), K.unsqueeze(0).double(), V.unsqueeze(0).double(), causal)
            hold(out[i:i + 1, :c], ref, truth, torch.bfloat16, t - c + 1, f"sequence {sid} ({t} tokens, {c} new)")

    calls = 0
    for it in range(60):
        live = list(rows)
        op = rng.choice(["prompt", "decode", "decode", "decode", "group", "fork", "free", "ragged"])
        try:
            if op == "prompt" or not live:
                sid = cache.add_sequence()
                n = rng.randint(1, 150)
                cut = rng.randint(0, n - 1)
                if cut:
                    step([sid], cut)             # chunked prefill: the second chunk attends behind the first
                step([sid], n - cut)
                calls += 1
            elif op == "ragged":
                # chunks of unequal length in one step: fresh prompts beside sequences that continue
                sids = rng.sample(live, rng.randint(0, min(len(live), 3))) + \
                    [cache.add_sequence() for _ in range(rng.randint(1, 3))]
                counts = [rng.choice([0, 1, 5, 40, 90]) for _ in sids]
                if max(counts) == 0:
                    counts[-1] = 7
                for sid, c in zip(sids, counts):
                    if sid not in rows and c == 0:
                        rows[sid] = (torch.zeros(0, gn, hd).bfloat16(), torch.zeros(0, gn, hd).bfloat16())
                step(sids, counts)
                calls += 1
            elif op == "decode":
                batch = rng.sample(live, rng.randint(1, min(len(live), 6)))
                step(batch, 1)
                calls += 1
            elif op == "group":
                # samples of one prompt, listed side by side, decoded in cohorts
                root = rng.choice(live)
                members = [root] + [cache.fork(root) for _ in range(rng.randint(1, 5))]
                for m in members[1:]:
                    rows[m] = (rows[root][0].clone(), rows[root][1].clone())
                for _ in range(rng.randint(1, 3)):
                    step(members, 1, cohort=len(members) if hn // gn <= 8 else 1)
                    calls += 1
            elif op == "fork":
                src = rng.choice(live)
                rows[cache.fork(src)] = (rows[src][0].clone(), rows[src][1].clone())
            else:
                sid = rng.choice(live)
                cache.free_sequence(sid)
                del rows[sid]
        except OutOfBlocks:
            for sid in list(rows)[: max(1, len(rows) // 2)]:
                cache.free_sequence(sid)
                del rows[sid]
    assert calls > 15
