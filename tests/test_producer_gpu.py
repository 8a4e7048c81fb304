"""Parity of ``dt_qk_norm_rope`` (through the C ABI) against the CPU oracle.

Bar: the kernel computes in fp32 and rounds once, so every output element must lie within one
rounding of the oracle's fp32 value: |y - o| <= 2^-8 |o| (half a bf16 ulp at worst) plus a
small absolute term for the different fp32 summation order (cancellation in LayerNorm / RoPE).
With the eager-rounding flags the result is compared with torch's own bf16 ops; elements may
differ by one bf16 ulp where a reduction-order difference flips a rounding.
"""
import math

import pytest
import torch

from oracle import producer as P

pytestmark = pytest.mark.gpu

DEV = "cuda:0"


def _close(y, o, atol=3e-5):
    y = y.float().cpu()
    err = (y - o).abs()
    bound = o.abs() * (2.0 ** -8) * 1.001 + atol
    bad = err > bound
    assert not bool(bad.any()), f"{int(bad.sum())} elements off; worst {float((err - bound).max()):.3e}"


def _tables(kind, S, D, sections=(), seed=1, batch=None):
    g = torch.Generator().manual_seed(seed)
    lead = (S,) if batch is None else (batch, S)
    if kind == P.ROPE_INTERLEAVED:
        th = torch.rand(*lead, D // 2, generator=g) * 2 * math.pi
        return th.cos().repeat_interleave(2, -1).contiguous(), th.sin().repeat_interleave(2, -1).contiguous()
    secs = list(sections) if sections else [D]
    cs, sn = [], []
    for d in secs:
        th = torch.rand(*lead, d // 2, generator=g) * 2 * math.pi
        cs.append(torch.cat((th.cos(), th.cos()), -1))
        sn.append(torch.cat((th.sin(), th.sin()), -1))
    return torch.cat(cs, -1).contiguous(), torch.cat(sn, -1).contiguous()


def _run(hip, x, **kw):
    d = {}
    for k in ("weight", "bias", "cos", "sin"):
        if kw.get(k) is not None:
            d[k] = kw[k].to(DEV)
    kw = {**kw, **d}
    y = hip.qk_norm_rope(x, **kw)
    torch.cuda.synchronize()
    return y


@pytest.mark.parametrize("D", [64, 128])
@pytest.mark.parametrize("H", [5, 8])
@pytest.mark.parametrize("norm", [P.NORM_NONE, P.NORM_RMS, P.NORM_LAYER])
@pytest.mark.parametrize("rope", ["none", "interleaved", "halves", "sections"])
def test_norm_rope_matches_oracle(hip, D, H, norm, rope):
    B, S = 2, 37
    g = torch.Generator().manual_seed(D + H)
    x = (torch.randn(B, S, H, D, generator=g) * 2.0 + 0.3).to(torch.bfloat16)
    w = torch.rand(D, generator=g) + 0.5
    b = torch.randn(D, generator=g) * 0.1
    kind = {"none": P.ROPE_NONE, "interleaved": P.ROPE_INTERLEAVED}.get(rope, P.ROPE_HALVES)
    sections = () if rope != "sections" else ((64, 32, 32) if D == 128 else (32, 16, 16))
    cos = sin = None
    if kind != P.ROPE_NONE:
        cos, sin = _tables(kind, S, D, sections)
    o = P.qk_norm_rope(x, norm, w, b, 1e-6, kind, cos, sin, 0, S, sections, 0)
    y = _run(hip, x.to(DEV), norm=norm, weight=w, bias=b, eps=1e-6, rope=kind, cos=cos, sin=sin, sections=sections)
    assert y.shape == (B, S, H, D) and y.dtype == torch.bfloat16 and y.is_contiguous()
    _close(y, o)


def test_reads_q_k_v_in_place_from_fused_projections(hip):
    """HunyuanVideo's "B L (K H D)" and Step-Video's "[..., H, 3*D]" layouts, no copy in front."""
    B, S, H, D = 1, 50, 6, 128
    g = torch.Generator().manual_seed(3)
    w = torch.rand(D, generator=g) + 0.5
    cos, sin = _tables(P.ROPE_INTERLEAVED, S, D)
    qkv = torch.randn(B, S, 3 * H * D, generator=g).to(torch.bfloat16)
    dev = qkv.to(DEV)
    hv = dev.view(B, S, 3, H, D)
    for i in range(2):
        o = P.qk_norm_rope(qkv.view(B, S, 3, H, D)[:, :, i], P.NORM_RMS, w, None, 1e-6, P.ROPE_INTERLEAVED, cos, sin)
        y = _run(hip, hv[:, :, i], norm=P.NORM_RMS, weight=w, rope=P.ROPE_INTERLEAVED, cos=cos, sin=sin)
        _close(y, o)
    v = _run(hip, hv[:, :, 2])  # plain strided -> contiguous copy
    assert torch.equal(v.cpu(), qkv.view(B, S, 3, H, D)[:, :, 2])
    sv = dev.view(B, S, H, 3 * D)
    c3, s3 = _tables(P.ROPE_HALVES, S, D, (64, 32, 32))
    for i in range(2):
        xs = qkv.view(B, S, H, 3 * D)[..., i * D:(i + 1) * D]
        o = P.qk_norm_rope(xs, P.NORM_RMS, w, None, 1e-6, P.ROPE_HALVES, c3, s3, 0, S, (64, 32, 32))
        y = _run(hip, sv[..., i * D:(i + 1) * D], norm=P.NORM_RMS, weight=w, rope=P.ROPE_HALVES, cos=c3, sin=s3,
                 sections=(64, 32, 32))
        _close(y, o)


def test_rope_on_video_tokens_only_and_batched_tables(hip):
    """CogVideoX rotates query[:, :, text_seqlen:] only (attention_processor.py:64-67)."""
    B, S, H, D, text = 2, 61, 4, 64, 17
    g = torch.Generator().manual_seed(4)
    x = torch.randn(B, S, H, D, generator=g).to(torch.bfloat16)
    w, b = torch.rand(D, generator=g) + 0.5, torch.randn(D, generator=g) * 0.1
    cos, sin = _tables(P.ROPE_INTERLEAVED, S - text, D)
    o = P.qk_norm_rope(x, P.NORM_LAYER, w, b, 1e-6, P.ROPE_INTERLEAVED, cos, sin, text, S)
    y = _run(hip, x.to(DEV), norm=P.NORM_LAYER, weight=w, bias=b, rope=P.ROPE_INTERLEAVED, cos=cos, sin=sin,
             rope_begin=text, rope_end=S)
    _close(y, o)
    cb, sb = _tables(P.ROPE_INTERLEAVED, S - text, D, batch=B, seed=9)
    ob = P.qk_norm_rope(x, P.NORM_NONE, None, None, 0.0, P.ROPE_INTERLEAVED, cb, sb, text, S)
    yb = _run(hip, x.to(DEV), rope=P.ROPE_INTERLEAVED, cos=cb, sin=sb, rope_begin=text, rope_end=S)
    _close(yb, ob)
    assert torch.equal(yb[:, :text].cpu(), x[:, :text])


def test_in_place_on_a_contiguous_tensor(hip):
    B, S, H, D = 1, 33, 7, 128
    g = torch.Generator().manual_seed(5)
    x = torch.randn(B, S, H, D, generator=g).to(torch.bfloat16)
    cos, sin = _tables(P.ROPE_HALVES, S, D)
    o = P.qk_norm_rope(x, P.NORM_RMS, None, None, 1e-6, P.ROPE_HALVES, cos, sin)
    xd = x.to(DEV)
    y = hip.qk_norm_rope(xd, norm=P.NORM_RMS, rope=P.ROPE_HALVES, cos=cos.to(DEV), sin=sin.to(DEV), out=xd)
    torch.cuda.synchronize()
    assert y.data_ptr() == xd.data_ptr()
    _close(xd, o)


@pytest.mark.parametrize("model", ["hunyuan", "step"])
def test_eager_rounding_modes(hip, model):
    """With the rounding flags the kernel follows the bf16 roundings of the callers' eager modules."""
    B, S, H, D = 1, 64, 8, 128
    g = torch.Generator().manual_seed(6)
    x = (torch.randn(B, S, H, D, generator=g) * 1.5).to(torch.bfloat16)
    w = (torch.rand(D, generator=g) + 0.5).to(torch.bfloat16).float()
    if model == "hunyuan":
        cos, sin = _tables(P.ROPE_INTERLEAVED, S, D)
        kind, secs, rounding = P.ROPE_INTERLEAVED, (), P.ROUND_NORM_BF16
    else:
        cos, sin = P.rope3d_tables(4, 4, 4, [64, 32, 32], torch.bfloat16)
        cos, sin = cos.float(), sin.float()
        kind, secs, rounding = P.ROPE_HALVES, (64, 32, 32), P.ROUND_NORM_BF16 | P.ROUND_ROPE_BF16
    o = P.qk_norm_rope(x, P.NORM_RMS, w, None, 1e-6, kind, cos, sin, 0, S, secs, rounding).to(torch.bfloat16)
    y = _run(hip, x.to(DEV), norm=P.NORM_RMS, weight=w, eps=1e-6, rope=kind, cos=cos, sin=sin, sections=secs,
             rounding=rounding).cpu()
    same = (y == o).float().mean().item()
    assert same > 0.995, f"only {same:.4f} of the elements bit-identical"
    # where they differ an intermediate rounding flipped: at most one bf16 ulp of the largest operand
    diff = (y.float() - o.float()).abs()
    assert float(diff.max()) <= 2.0 ** -7 * float(o.float().abs().max())


def test_full_size_hunyuan_share_properties(hip):
    """HunyuanVideo per-rank share (14882 tokens x 24 heads x 128): unit RMS after the norm, row norms
    preserved by the rotation, and rotating by theta then by -theta returns the input."""
    B, S, H, D = 1, 14882, 24, 128
    g = torch.Generator(device=DEV).manual_seed(7)
    qkv = torch.randn(B, S, 3, H, D, generator=g, device=DEV, dtype=torch.float32).to(torch.bfloat16)
    th = torch.rand(S, D // 2, generator=g, device=DEV) * 2 * math.pi
    cos, sin = th.cos().repeat_interleave(2, -1).contiguous(), th.sin().repeat_interleave(2, -1).contiguous()
    n = hip.qk_norm_rope(qkv[:, :, 0], norm=P.NORM_RMS, eps=1e-6)
    rms = n.float().pow(2).mean(-1).sqrt()
    assert float((rms - 1).abs().max()) < 4e-3
    r = hip.qk_norm_rope(n, rope=P.ROPE_INTERLEAVED, cos=cos, sin=sin)
    assert float((r.float().norm(dim=-1) - n.float().norm(dim=-1)).abs().max()) < 0.05
    back = hip.qk_norm_rope(r, rope=P.ROPE_INTERLEAVED, cos=cos, sin=(-sin).contiguous())
    assert float((back.float() - n.float()).abs().max()) <= 2.0 ** -6 * float(n.float().abs().max())
    # a sample of rows against the oracle
    rows = torch.randint(0, S, (64,), generator=torch.Generator().manual_seed(8))
    xs = qkv[:, rows.to(DEV), 0].cpu()
    o = P.qk_norm_rope(xs, P.NORM_RMS, None, None, 1e-6, P.ROPE_INTERLEAVED, cos[rows.to(DEV)].cpu(), sin[rows.to(DEV)].cpu())
    full = hip.qk_norm_rope(qkv[:, :, 0], norm=P.NORM_RMS, eps=1e-6, rope=P.ROPE_INTERLEAVED, cos=cos, sin=sin)
    _close(full[:, rows.to(DEV)], o)


def test_rejects_bad_arguments(hip):
    x = torch.zeros(1, 4, 2, 128, dtype=torch.bfloat16, device=DEV)
    t = torch.zeros(4, 128, device=DEV)
    with pytest.raises(hip.DitangoHipError):
        hip.qk_norm_rope(x, rope=P.ROPE_HALVES, cos=t, sin=t, sections=(64, 32))          # do not sum to D
    with pytest.raises(hip.DitangoHipError):
        hip.qk_norm_rope(x, rope=P.ROPE_HALVES, cos=t, sin=t, sections=(120, 8))          # not multiples of 16
    with pytest.raises(hip.DitangoHipError):
        hip.qk_norm_rope(x, rope=P.ROPE_INTERLEAVED, cos=t, sin=t, rope_begin=2, rope_end=9)
    with pytest.raises(hip.DitangoHipError):
        hip.qk_norm_rope(torch.zeros(1, 4, 2, 96, dtype=torch.bfloat16, device=DEV))      # head dim not built
    with pytest.raises(hip.DitangoHipError):
        hip.qk_norm_rope(x, norm=7)
    with pytest.raises(hip.DitangoHipError):
        hip.qk_norm_rope(x.float())


def test_full_kv_sequence_of_the_hunyuan_shape(hip):
    """RMSNorm + interleaved RoPE of K over the whole HunyuanVideo KV sequence (119 056 tokens x 24 heads), read in
    place from a fused "B L (K H D)" projection, the text tokens behind rope_end left unrotated: every output row of
    a seeded sample of 512 tokens against the oracle, and the rows in between untouched by neighbours (finite)."""
    B, S, H, D, n_txt = 1, 119056, 24, 128, 256
    g = torch.Generator(device=DEV).manual_seed(21)
    qkv = (torch.randn(B, S, 3, H, D, generator=g, device=DEV) * 1.5).to(torch.bfloat16)
    x = qkv[:, :, 1]                                   # K, strided view
    gc = torch.Generator().manual_seed(22)
    w = torch.rand(D, generator=gc) + 0.5
    cos, sin = _tables(P.ROPE_INTERLEAVED, S - n_txt, D, seed=23)
    y = hip.qk_norm_rope(x, norm=P.NORM_RMS, weight=w.to(DEV), eps=1e-6, rope=P.ROPE_INTERLEAVED, cos=cos.to(DEV),
                         sin=sin.to(DEV), rope_begin=0, rope_end=S - n_txt)
    torch.cuda.synchronize()
    assert y.shape == (B, S, H, D) and y.is_contiguous() and bool(torch.isfinite(y.float()).all())
    rows = torch.sort(torch.cat([torch.randperm(S - n_txt, generator=gc)[:448], torch.arange(S - n_txt - 32, S - n_txt + 32)])).values
    xs = x[:, rows.to(DEV)].cpu()
    for lo, hi, rot in ((0, int((rows < S - n_txt).sum()), True), (int((rows < S - n_txt).sum()), len(rows), False)):
        if hi <= lo:
            continue
        r = rows[lo:hi]
        o = P.qk_norm_rope(xs[:, lo:hi], P.NORM_RMS, w, None, 1e-6, P.ROPE_INTERLEAVED if rot else P.ROPE_NONE,
                           cos[r] if rot else None, sin[r] if rot else None, 0, hi - lo, (), 0)
        _close(y[:, r.to(DEV)], o)
