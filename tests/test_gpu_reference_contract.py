"""The reference's own attention-layer suite (tests/test_attention.py of the
reference, classes TestAttentionBasics :116-207, TestAttentionWithDifferentConfigs
:209-287, TestAttentionVaryingDimensions :289-379, TestAttentionMemory :880-925,
and the TransformerLayer classes :433-590 further down), case by case, against
the drop-in layers on the GPU.

Same calls: a layer built from a config and NOT put into eval mode, float32
tensors from torch.randn with autograd recording (none of them requires grad),
the float lower-triangular mask expanded to [b, 1, s, s] or no mask.  There the
assertions are shapes and finiteness; here every output is held to the oracle's
dense attention as well.  (The gradient tests :382-431 are training features:
the layer refuses them loudly, tests/test_kv_cache_host.py.)"""
import pytest
import torch

from ironcore_amd import config as ic_config
from ironcore_amd.layers import Attention
from oracle.dense_attention import dense_attention

pytestmark = pytest.mark.gpu

TOL_FP32 = 1e-4


def create_test_config(d_model=512, num_attention_heads=8, num_attention_groups=8, head_dim=64,
                       use_flash_attn=False, dropout_attn=0.0):
    """The reference helper's arguments (tests/test_attention.py:54-102) on the config mirror."""
    return ic_config.MainConfig(
        model=ic_config.ModelConfig(d_model=d_model, num_attention_heads=num_attention_heads,
                                    num_attention_groups=num_attention_groups, head_dim=head_dim,
                                    dropout_attn=dropout_attn, precision="fp32"),
        trainer=ic_config.TrainerConfig(tensor_model_parallel_size=1, use_flash_attn=use_flash_attn),
        init=ic_config.InitConfig(seed=42, init_std=0.02))


def create_causal_mask(batch_size, seq_len, device):
    return torch.tril(torch.ones(seq_len, seq_len, device=device)).unsqueeze(0).unsqueeze(0).expand(batch_size, -1, -1, -1)


def _call(gpu, config, b, s, hn, gn, hd, masked=True, seed=0):
    attention = Attention(config).to(gpu)          # training mode, as in the reference's tests
    torch.manual_seed(seed)
    query = torch.randn(b, s, hn, hd, device=gpu)
    key = torch.randn(b, s, gn, hd, device=gpu)
    value = torch.randn(b, s, gn, hd, device=gpu)
    mask = create_causal_mask(b, s, gpu) if masked else None
    assert torch.is_grad_enabled()
    output = attention(query, key, value, mask) if masked else attention(query, key, value, attention_mask=None)
    torch.cuda.synchronize()
    assert output.shape == (b, s, hn * hd) and output.dtype == torch.float32
    assert torch.isfinite(output).all()
    want = dense_attention(query.cpu(), key.cpu(), value.cpu(), None if mask is None else mask.cpu())
    assert (output.cpu() - want).abs().max().item() <= TOL_FP32
    return attention


class TestAttentionBasics:
    def test_attention_initialization(self, gpu):
        attention = Attention(create_test_config()).to(gpu)
        assert attention.num_attention_heads == 8 and attention.head_dimension == 64
        assert attention.softmax is not None and attention.attn_dropout is not None

    def test_attention_forward_shape(self, gpu):
        _call(gpu, create_test_config(), 2, 64, 8, 8, 64)

    def test_attention_with_causal_mask(self, gpu):
        _call(gpu, create_test_config(), 2, 64, 8, 8, 64, seed=1)

    def test_attention_without_mask(self, gpu):
        _call(gpu, create_test_config(), 2, 64, 8, 8, 64, masked=False, seed=2)


class TestAttentionWithDifferentConfigs:
    def test_attention_mha(self, gpu):
        _call(gpu, create_test_config(num_attention_heads=8, num_attention_groups=8, head_dim=64), 2, 64, 8, 8, 64)

    def test_attention_gqa(self, gpu):
        _call(gpu, create_test_config(num_attention_heads=8, num_attention_groups=2, head_dim=64), 2, 64, 8, 2, 64)

    def test_attention_mqa(self, gpu):
        _call(gpu, create_test_config(num_attention_heads=8, num_attention_groups=1, head_dim=64), 2, 64, 8, 1, 64)


class TestAttentionVaryingDimensions:
    @pytest.mark.parametrize("seq_len", [16, 32, 64, 128])
    def test_different_sequence_lengths(self, gpu, seq_len):
        _call(gpu, create_test_config(), 2, seq_len, 8, 8, 64, seed=seq_len)

    @pytest.mark.parametrize("batch_size", [1, 2, 4])
    def test_different_batch_sizes(self, gpu, batch_size):
        _call(gpu, create_test_config(), batch_size, 64, 8, 8, 64, seed=batch_size)

    @pytest.mark.parametrize("head_dim", [32, 64, 128])
    def test_different_head_dimensions(self, gpu, head_dim):
        num_heads = 8
        config = create_test_config(d_model=num_heads * head_dim, num_attention_heads=num_heads,
                                    num_attention_groups=num_heads, head_dim=head_dim)
        _call(gpu, config, 2, 64, num_heads, num_heads, head_dim, seed=head_dim)


class TestAttentionMemory:
    def test_memory_usage(self, gpu):
        """12 heads of 64, batch 4, 256 tokens: the call may keep less than 1 GB
        (:888-925).  The kernels never materialise the [b, hn, s, s] scores: what
        stays allocated is the output and the classified mask's bookkeeping."""
        num_heads, head_dim, b, s = 12, 64, 4, 256
        config = create_test_config(d_model=num_heads * head_dim, num_attention_heads=num_heads,
                                    num_attention_groups=num_heads, head_dim=head_dim)
        attention = Attention(config).to(gpu)
        query = torch.randn(b, s, num_heads, head_dim, device=gpu)
        key = torch.randn(b, s, num_heads, head_dim, device=gpu)
        value = torch.randn(b, s, num_heads, head_dim, device=gpu)
        mask = create_causal_mask(b, s, gpu)
        attention(query, key, value, mask)   # (library set-up outside the measurement)
        torch.cuda.synchronize()
        torch.cuda.reset_peak_memory_stats()
        before = torch.cuda.memory_allocated()
        output = attention(query, key, value, mask)
        torch.cuda.synchronize()
        used = torch.cuda.memory_allocated() - before
        assert used < 1e9
        assert used <= 2 * output.numel() * 4            # the output, and nothing of the size of the scores
        assert torch.cuda.max_memory_allocated() - before < b * num_heads * s * s * 4


# ---- TransformerLayer (tests/test_attention.py:433-590 of the reference) -------------------------
# Same constructor, same init_weights(), same call layer(hidden_states, attention_mask,
# rotary_pos_emb=...).  The reference's tests run with autograd recording; the projections' weights
# require grad, and the HIP attention is forward only, so the calls here sit under torch.no_grad()
# (the gradient tests :493-520 are refused, as for the bare layer).  Beyond shape and finiteness
# the output is held to the same layer with its attention replaced by the oracle's.

def _layer_config(num_attention_heads=8, num_attention_groups=8, head_dim=64, d_model=512):
    cfg = create_test_config(d_model=d_model, num_attention_heads=num_attention_heads,
                             num_attention_groups=num_attention_groups, head_dim=head_dim)
    cfg.model.max_seq_len = 128
    cfg.model.max_position_embeddings = 128
    cfg.model.no_bias = False
    cfg.model.num_layers = 1
    cfg.model.d_ffn = 2048
    return cfg


def _layer_vs_oracle(gpu, config, rotary=False, seed=0):
    from ironcore_amd.generation import TransformerLayer
    from ironcore_amd.layers.rotary import RotaryPositionalEmbedding
    b, s = 2, 64
    torch.manual_seed(seed)
    layer = TransformerLayer(config).to(gpu)
    layer.init_weights()
    rope = RotaryPositionalEmbedding(head_dim=config.model.head_dim, max_seq_len=config.model.max_seq_len).to(gpu) if rotary else None
    hidden = torch.randn(b, s, config.model.d_model, device=gpu)
    mask = create_causal_mask(b, s, gpu)
    with torch.no_grad():
        output = layer(hidden, mask, rotary_pos_emb=rope)
        # the same layer, attention by the oracle (transformer.py:77-132)
        norm = layer.input_layernorm(hidden)
        q = layer.linear_q(norm).view(b, s, layer.num_local_attention_heads, layer.head_dimension)
        k, v = torch.chunk(layer.linear_kv(norm), 2, dim=-1)
        k = k.view(b, s, layer.num_local_attention_groups, layer.head_dimension)
        v = v.view(b, s, layer.num_local_attention_groups, layer.head_dimension)
        if rope is not None:
            positions = torch.arange(s, device=gpu, dtype=torch.int32).repeat(b)
            q, k = rope(q, positions), rope(k, positions)
        ctx = dense_attention(q.cpu(), k.cpu(), v.cpu(), mask.cpu()).to(gpu)
        x = hidden + layer.attn_output(ctx)
        want = x + layer.mlp(layer.post_attn_layernorm(x))
    torch.cuda.synchronize()
    assert output.shape == hidden.shape and torch.isfinite(output).all()
    assert (output - want).abs().max().item() <= 1e-4
    return layer


class TestTransformerLayerBasics:
    def test_transformer_layer_initialization(self, gpu):
        from ironcore_amd.generation import TransformerLayer
        layer = TransformerLayer(_layer_config()).to(gpu)
        layer.init_weights()
        assert layer.linear_q is not None and layer.linear_kv is not None
        assert layer.attn_output is not None and layer.self_attention is not None
        for name, param in layer.named_parameters():   # BaseModule.init_weights, ironcore/layers/module.py:43-76
            if "bias" in name:
                assert torch.count_nonzero(param) == 0, name
            elif "norm" in name:
                assert torch.equal(param, torch.ones_like(param)), name
            else:
                assert 0.25 * 0.02 < param.std().item() < 1.5 * 0.02, name

    def test_gpt_layer_forward_shape(self, gpu):
        _layer_vs_oracle(gpu, _layer_config())

    def test_gpt_layer_with_rope(self, gpu):
        _layer_vs_oracle(gpu, _layer_config(), rotary=True, seed=1)


class TestTransformerLayerWithDifferentConfigs:
    def test_gpt_layer_mha(self, gpu):
        _layer_vs_oracle(gpu, _layer_config(num_attention_heads=8, num_attention_groups=8), seed=2)

    def test_gpt_layer_gqa(self, gpu):
        _layer_vs_oracle(gpu, _layer_config(num_attention_heads=8, num_attention_groups=2), seed=3)

    def test_gpt_layer_mqa(self, gpu):
        _layer_vs_oracle(gpu, _layer_config(num_attention_heads=8, num_attention_groups=1), seed=4)
