"""Size-independent properties of the chunk attention at the full per-rank sizes, where the host oracle only
reaches a sample of rows: every row, head and key of the CogVideoX (d = 64) and HunyuanVideo (d = 128) shares.

* softmax rows sum to one: with V = 1 every output element is 1 (to the rounding of P);
* duplicated keys: the job over the chunk listed twice has the same output and lse + ln 2;
* permuting the keys (K and V rows together) changes nothing but the summation order;
* linearity in V: attention of a v1 + b v2 is a out1 + b out2 with the lse untouched.

A mistake in the key-range bookkeeping (a dropped or doubly counted tile, a wrong chunk boundary, a stale buffer) breaks
at least one of them on some row; all of them hold for bf16 and fp16 tensors.
"""
import math

import pytest
import torch

pytestmark = pytest.mark.gpu

SHAPES = {
    "cogvideox": (1, 48, 64, 2222, 2222, "layer"),
    "hunyuanvideo": (1, 24, 128, 14882, 14882, "rms"),
}
DEV = "cuda"


def _draw(B, n, H, D, g, norm, dtype):
    x = torch.randn(B, n, H, D, generator=g, device=DEV)
    if norm == "rms":
        x = x / x.pow(2).mean(-1, keepdim=True).sqrt()
    elif norm == "layer":
        x = torch.nn.functional.layer_norm(x, (D,))
    return x.to(dtype)


def _state(hip, q, chunks, job, workspace=True):
    """(out, lse) of q against the chunk list ``job`` of the table ``chunks`` = [(k, v), ...]."""
    B, Sq, H, D = q.shape
    table = hip.ChunkTable([k for k, _ in chunks], [v for _, v in chunks])
    out = torch.empty(B, Sq, H, D, dtype=q.dtype, device=DEV)
    lse = torch.empty(B, H, Sq, dtype=torch.float32, device=DEV)
    hip.attn_jobs_fwd(q, table, [job], [out], [lse], workspace=hip.attn_workspace(DEV) if workspace else None)
    torch.cuda.synchronize()
    return out, lse


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("name", ["cogvideox", "hunyuanvideo"])
def test_properties_hold_on_every_row_at_full_size(hip, name, dtype):
    B, H, D, Sq, Sk, norm = SHAPES[name]
    print(f"case properties {name} {dtype}: H={H} D={D} Sq={Sq} Sk={Sk}", flush=True)
    g = torch.Generator(device=DEV).manual_seed(19)
    q, k = _draw(B, Sq, H, D, g, norm, dtype), _draw(B, Sk, H, D, g, norm, dtype)
    v1, v2 = _draw(B, Sk, H, D, g, None, dtype), _draw(B, Sk, H, D, g, None, dtype)
    ulp = 2.0 ** -8 if dtype == torch.bfloat16 else 2.0 ** -11      # half a unit in the last place, relative

    out1, lse1 = _state(hip, q, [(k, v1)], [0])
    assert torch.isfinite(out1).all() and torch.isfinite(lse1).all()

    # rows of the softmax sum to one
    ones, _ = _state(hip, q, [(k, torch.ones_like(v1))], [0])
    dev1 = (ones.float() - 1).abs().max().item()
    print(f"  V = 1: max |out - 1| = {dev1:.3e}", flush=True)
    assert dev1 <= 2 * ulp

    # the chunk listed twice in one job: same output, lse + ln 2
    out_d, lse_d = _state(hip, q, [(k, v1)], [0, 0])
    e_out = (out_d.float() - out1.float()).abs().max().item()
    e_lse = (lse_d - lse1 - math.log(2.0)).abs().max().item()
    print(f"  duplicated keys: out {e_out:.3e}, lse - ln 2 {e_lse:.3e}", flush=True)
    assert e_out <= 4 * ulp * out1.float().abs().max().item() and e_lse <= 2e-5

    # the same keys in another order
    perm = torch.randperm(Sk, generator=g, device=DEV)
    out_p, lse_p = _state(hip, q, [(k[:, perm].contiguous(), v1[:, perm].contiguous())], [0])
    e_out = (out_p.float() - out1.float()).abs().max().item()
    e_lse = (lse_p - lse1).abs().max().item()
    print(f"  permuted keys: out {e_out:.3e}, lse {e_lse:.3e}", flush=True)
    assert e_out <= 4 * ulp * out1.float().abs().max().item() and e_lse <= 2e-5

    # linear in V (the combination is rounded to the tensors' dtype, so is each output: a few roundings of slack)
    a, b = 0.75, -1.5
    out2, lse2 = _state(hip, q, [(k, v2)], [0])
    v3 = (a * v1.float() + b * v2.float()).to(dtype)
    out3, lse3 = _state(hip, q, [(k, v3)], [0])
    want = a * out1.float() + b * out2.float()
    e_out = (out3.float() - want).abs().max().item()
    print(f"  linear in V: out {e_out:.3e}", flush=True)
    assert torch.equal(lse2, lse1) and torch.equal(lse3, lse1)
    scale = max(out1.float().abs().max().item(), out2.float().abs().max().item(), want.abs().max().item())
    assert e_out <= 8 * ulp * scale
