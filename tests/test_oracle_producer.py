"""Pins the CPU oracle of the producer step (QK norm + RoPE) against library routines, closed
forms and invariants, and checks the product's host-side table builder against it."""
import math

import pytest
import torch
import torch.nn.functional as F

from oracle import producer as P


def _x(B=2, S=7, H=3, D=64, seed=0, scale=1.0):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(B, S, H, D, generator=g) * scale).to(torch.bfloat16)


def _angles(S, D, seed=1):
    g = torch.Generator().manual_seed(seed)
    return torch.rand(S, D // 2, generator=g) * 2 * math.pi


def test_rms_norm_is_the_library_routine():
    x = _x(seed=3, scale=3.0)
    w = torch.rand(64) + 0.5
    ref = F.rms_norm(x.float(), (64,), weight=w, eps=1e-6)
    torch.testing.assert_close(P.rms_norm(x, w, 1e-6, False), ref, rtol=1e-6, atol=1e-6)
    y = P.rms_norm(x, None, 0.0, False)
    torch.testing.assert_close(y.pow(2).mean(-1), torch.ones(2, 7, 3), rtol=1e-5, atol=1e-5)


def test_layer_norm_is_the_library_routine():
    x = _x(seed=4, scale=2.0)
    w, b = torch.rand(64) + 0.5, torch.randn(64)
    ref = F.layer_norm(x.float(), (64,), w, b, 1e-5)
    torch.testing.assert_close(P.layer_norm(x, w, b, 1e-5, False), ref, rtol=1e-5, atol=1e-5)


def test_interleaved_rope_is_complex_multiplication():
    x = _x(D=64, seed=5).float()
    th = _angles(7, 64)
    cos = th.cos().repeat_interleave(2, dim=-1)
    sin = th.sin().repeat_interleave(2, dim=-1)
    got = P.rope(x, cos, sin, P.ROPE_INTERLEAVED)
    xc = torch.view_as_complex(x.reshape(2, 7, 3, 32, 2).contiguous())
    ref = torch.view_as_real(xc * torch.polar(torch.ones_like(th), th)[None, :, None, :]).flatten(-2)
    torch.testing.assert_close(got, ref, rtol=1e-5, atol=1e-5)


def test_rotate_half_rope_is_a_rotation_of_pairs_half_apart():
    D = 64
    x = _x(D=D, seed=6).float()
    th = _angles(7, D)
    cos, sin = torch.cat((th.cos(), th.cos()), -1), torch.cat((th.sin(), th.sin()), -1)
    got = P.rope(x, cos, sin, P.ROPE_HALVES)
    a, b = x[..., : D // 2], x[..., D // 2:]
    c, s = th.cos()[None, :, None, :], th.sin()[None, :, None, :]
    ref = torch.cat((a * c - b * s, b * c + a * s), -1)  # [a'; b'] = R(theta) [a; b]
    torch.testing.assert_close(got, ref, rtol=1e-5, atol=1e-5)
    torch.testing.assert_close(got.norm(dim=-1), x.norm(dim=-1), rtol=1e-5, atol=1e-5)


def test_sections_rotate_independently():
    x = _x(D=128, seed=7).float()
    secs = [64, 32, 32]
    th = [_angles(7, d, seed=10 + i) for i, d in enumerate(secs)]
    cos = torch.cat([torch.cat((t.cos(), t.cos()), -1) for t in th], -1)
    sin = torch.cat([torch.cat((t.sin(), t.sin()), -1) for t in th], -1)
    got = P.rope(x, cos, sin, P.ROPE_HALVES, secs)
    parts, o = [], 0
    for d, t in zip(secs, th):
        parts.append(P.rope(x[..., o:o + d], torch.cat((t.cos(), t.cos()), -1), torch.cat((t.sin(), t.sin()), -1), P.ROPE_HALVES))
        o += d
    torch.testing.assert_close(got, torch.cat(parts, -1), rtol=0, atol=0)


@pytest.mark.parametrize("kind", [P.ROPE_INTERLEAVED, P.ROPE_HALVES])
def test_relative_position_property(kind):
    """<rope(q, p), rope(k, p')> depends on p - p' only."""
    D = 64
    g = torch.Generator().manual_seed(8)
    q, k = torch.randn(1, 1, 1, D, generator=g), torch.randn(1, 1, 1, D, generator=g)
    inv = 1.0 / (1e4 ** (torch.arange(0, D, 2).float() / D))

    def tab(p):
        a = (p * inv)[None]
        a = a.repeat_interleave(2, -1) if kind == P.ROPE_INTERLEAVED else torch.cat((a, a), -1)
        return a.cos(), a.sin()

    def dot(p, pp):
        return float((P.rope(q, *tab(p), kind) * P.rope(k, *tab(pp), kind)).sum())

    assert abs(dot(3.0, 1.0) - dot(12.0, 10.0)) < 1e-4
    assert abs(dot(3.0, 1.0) - dot(1.0, 3.0)) > 1e-3  # and it is not symmetric


def test_bf16_math_matches_eager_bf16_ops():
    """executor/step/rope.py:30-35 evaluated by torch in bf16 == the oracle's rounding model."""
    x = _x(D=128, seed=9)
    cos, sin = P.rope3d_tables(1, 1, 7, [64, 32, 32], torch.bfloat16)
    eager = x * cos[None, :, None, :] + torch.cat([P.rotate_half(p) for p in torch.split(x, [64, 32, 32], -1)], -1) * sin[None, :, None, :]
    got = P.qk_norm_rope(x, rope_kind=P.ROPE_HALVES, cos=cos.float(), sin=sin.float(), sections=[64, 32, 32],
                         rounding=P.ROUND_ROPE_BF16).to(torch.bfloat16)
    assert torch.equal(got, eager)


def test_norm_rounding_matches_eager_bf16_module():
    """RMSNorm written the way the callers' modules are: float math, cast back, times the bf16 weight."""
    x = _x(D=128, seed=10, scale=2.0)
    w = (torch.rand(128) + 0.5).to(torch.bfloat16)
    xf = x.float()
    eager = (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + 1e-6)).type_as(x) * w
    got = P.qk_norm_rope(x, norm=P.NORM_RMS, weight=w.float(), eps=1e-6, rounding=P.ROUND_NORM_BF16).to(torch.bfloat16)
    assert torch.equal(got, eager)


def test_rope3d_tables_follow_the_mesh():
    f, h, w = 2, 3, 4
    cos, sin = P.rope3d_tables(f, h, w, [64, 32, 32], torch.float32)
    assert cos.shape == (24, 128)
    n = 1 * 12 + 2 * 4 + 3  # token (1, 2, 3)
    for sec, (d, pos) in enumerate(zip([64, 32, 32], [1, 2, 3])):
        o = [0, 64, 96][sec]
        for j in (0, 5, d // 2 - 1):
            ang = pos / (1e4 ** (2 * j / d))
            assert abs(float(cos[n, o + j]) - math.cos(ang)) < 1e-5
            assert abs(float(sin[n, o + d // 2 + j]) - math.sin(ang)) < 1e-5


def test_product_table_builder_equals_the_oracle():
    from ditango_amd.producer import rope3d_tables
    for dtype in (torch.bfloat16, torch.float32):
        c0, s0 = P.rope3d_tables(3, 4, 5, [64, 32, 32], dtype)
        c1, s1 = rope3d_tables(3, 4, 5, (64, 32, 32), dtype)
        assert torch.equal(c0.float(), c1) and torch.equal(s0.float(), s1)


def test_rope_row_range_and_identity():
    x = _x(D=64, seed=11)
    th = _angles(4, 64)
    cos, sin = th.cos().repeat_interleave(2, -1), th.sin().repeat_interleave(2, -1)
    y = P.qk_norm_rope(x, rope_kind=P.ROPE_INTERLEAVED, cos=cos, sin=sin, rope_begin=3, rope_end=7)
    assert torch.equal(y[:, :3], x[:, :3].float())
    assert not torch.equal(y[:, 3:], x[:, 3:].float())
    z = P.qk_norm_rope(x, rope_kind=P.ROPE_INTERLEAVED, cos=torch.ones(7, 64), sin=torch.zeros(7, 64))
    assert torch.equal(z, x.float())
