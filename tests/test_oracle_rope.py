"""Pins oracle/rope.py (rotary.py:31-83 restated) by mathematics: the
reference's own tests hold shape checks only for its rotary embedding."""
import math

import torch

from oracle import rope


def test_tables_match_float64_closed_form():
    cos, sin = rope.rope_tables(64, 50, base=10000, scale=0.5, offset=3)
    assert cos.shape == sin.shape == (50, 32) and cos.dtype == torch.float32
    for p in (0, 1, 17, 49):
        for i in (0, 5, 31):
            ang = (3 + p) * 0.5 * 10000.0 ** (-2.0 * i / 64)
            assert abs(cos[p, i].item() - math.cos(ang)) < 2e-6 * max(1.0, abs(ang))
            assert abs(sin[p, i].item() - math.sin(ang)) < 2e-6 * max(1.0, abs(ang))


def test_rotate_is_complex_multiplication():
    g = torch.Generator().manual_seed(0)
    x = torch.randn(7, 3, 16, generator=g)
    pos = torch.tensor([0, 1, 2, 5, 9, 30, 63], dtype=torch.int32)
    cos, sin = rope.rope_tables(16, 64)
    got = rope.rope_rotate(x, pos, cos, sin)
    assert got.dtype == torch.float32 and got.shape == x.shape
    theta = 10000.0 ** (-torch.arange(0, 16, 2, dtype=torch.float64) / 16)
    ang = pos.double()[:, None] * theta[None, :]
    z = torch.complex(x[..., ::2].double(), x[..., 1::2].double()) * torch.polar(torch.ones_like(ang), ang)[:, None, :]
    want = torch.stack([z.real, z.imag], dim=-1).flatten(-2)
    assert (got.double() - want).abs().max().item() < 1e-5


def test_position_zero_is_the_identity_bit_for_bit():
    g = torch.Generator().manual_seed(1)
    x = torch.randn(4, 2, 32, generator=g).bfloat16()
    cos, sin = rope.rope_tables(32, 8)
    got = rope.rope_rotate(x, torch.zeros(4, dtype=torch.int32), cos, sin)
    assert torch.equal(got, x.float())


def test_pair_norms_are_preserved_and_scores_depend_on_distance_only():
    g = torch.Generator().manual_seed(2)
    q = torch.randn(1, 1, 64, generator=g)
    k = torch.randn(1, 1, 64, generator=g)
    cos, sin = rope.rope_tables(64, 256)
    rq = rope.rope_rotate(q.expand(200, 1, 64), torch.arange(20, 220, dtype=torch.int32), cos, sin)
    assert torch.allclose(rq.view(200, 32, 2).norm(dim=-1), q.view(1, 32, 2).norm(dim=-1).expand(200, 32), atol=1e-5)
    rk = rope.rope_rotate(k.expand(200, 1, 64), torch.arange(13, 213, dtype=torch.int32), cos, sin)
    scores = (rq * rk).sum(-1).squeeze(1)          # every pair is 7 positions apart
    assert (scores - scores[0]).abs().max().item() < 2e-3
    other = (rope.rope_rotate(q, torch.tensor([20], dtype=torch.int32), cos, sin) *
             rope.rope_rotate(k, torch.tensor([12], dtype=torch.int32), cos, sin)).sum()
    assert abs(other.item() - scores[0].item()) > 1e-3  # a different distance gives a different score


def test_positions_select_rows_per_token_not_per_batch_index():
    g = torch.Generator().manual_seed(3)
    x = torch.randn(3, 2, 8, generator=g)
    cos, sin = rope.rope_tables(8, 16)
    a = rope.rope_rotate(x, torch.tensor([4, 4, 4], dtype=torch.int32), cos, sin)
    b = rope.rope_rotate(x[1:2], torch.tensor([4], dtype=torch.int32), cos, sin)
    assert torch.equal(a[1:2], b)


def test_against_transformers_gptj_rotary():
    """A third-party implementation of the same interleaved-pair rotation:
    transformers' GPT-J helpers (read as a library, not part of any reference)."""
    import pytest
    gptj = pytest.importorskip("transformers.models.gptj.modeling_gptj")
    g = torch.Generator().manual_seed(7)
    b, s, h, d = 2, 9, 3, 32
    x = torch.randn(b, s, h, d, generator=g)
    pos = torch.randint(0, 100, (b, s), generator=g)
    table = gptj.create_sinusoidal_positions(100, d)                  # [100, d]: sin | cos
    sincos = table[pos]                                               # [b, s, d]
    sin, cos = torch.split(sincos, d // 2, dim=-1)
    want = gptj.apply_rotary_pos_emb(x, sin, cos)
    cos_t, sin_t = rope.rope_tables(d, 100)
    got = rope.rope_rotate(x.reshape(b * s, h, d), pos.reshape(-1), cos_t, sin_t).view(b, s, h, d)
    assert (got - want).abs().max().item() < 1e-5


def test_module_tables_stay_fp32_through_a_dtype_change():
    """``model.to(bfloat16)`` must not round the sin/cos tables."""
    from ironcore_amd.layers.rotary import RotaryPositionalEmbedding
    rope = RotaryPositionalEmbedding(64, 96, base=10000, offset=3)
    sin, cos, theta = rope.sin_emb.clone(), rope.cos_emb.clone(), rope.theta.clone()
    torch.nn.ModuleList([rope]).to(torch.bfloat16)
    assert rope.sin_emb.dtype == torch.float32 and rope.theta.dtype == torch.float32
    assert torch.equal(rope.sin_emb, sin) and torch.equal(rope.cos_emb, cos) and torch.equal(rope.theta, theta)
