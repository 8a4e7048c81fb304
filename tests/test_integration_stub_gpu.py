"""The reference-side binding that the integration guide shows a maintainer (``flash_attn_func`` and
``flash_attn_varlen_func`` as ctypes stubs over the C ABI) is executed as written -- only the library's path is
filled in -- and checked against the oracle, so the guide cannot drift from the ABI."""
import os
import re

import pytest
import torch

from oracle import attention_math as om

pytestmark = pytest.mark.gpu
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GUIDE = os.path.join(ROOT, "INTEGRATION.md")


def _stub_namespace(hip):
    text = open(GUIDE).read()
    section = text[text.index("## B."):text.index("## C.")]
    blocks = re.findall(r"```python\n(.*?)```", section, flags=re.S)
    assert len(blocks) == 2 and "def flash_attn_func" in blocks[0] and "def flash_attn_varlen_func" in blocks[1]
    code = "\n".join(blocks).replace('ctypes.CDLL("libditango_hip.so")', f'ctypes.CDLL("{hip.LIB_PATH}")')
    ns = {}
    exec(compile(code, "binding stubs of the integration guide", "exec"), ns)
    return ns


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_documented_flash_attn_stubs_run_and_match_the_oracle(hip, dtype):
    ns = _stub_namespace(hip)
    g = torch.Generator().manual_seed(2)
    B, Sq, Sk, H, D = 2, 150, 170, 3, 128
    q = torch.randn(B, Sq, H, D, generator=g).to(dtype)
    k = torch.randn(B, Sk, H, D, generator=g).to(dtype)
    v = torch.randn(B, Sk, H, D, generator=g).to(dtype)
    out, lse, _ = ns["flash_attn_func"](q.cuda(), k.cuda(), v.cuda(), dropout_p=0.0, return_attn_probs=True)
    torch.cuda.synchronize()
    ref_o, ref_l = om.chunk_attention(q, k, v)
    assert out.dtype == dtype and tuple(lse.shape) == (B, H, Sq)
    assert (out.float().cpu() - ref_o).abs().max() <= 2e-2 and (lse.cpu() - ref_l).abs().max() <= 1e-3
    # the packed twin: two segments, boundaries on the GPU, rows behind the last boundary zeroed
    total_q, total_k = 300, 333
    cu_q, cu_k = [0, 200, 290], [0, 250, 333]
    qp = torch.randn(total_q, H, D, generator=g).to(dtype)
    kp = torch.randn(total_k, H, D, generator=g).to(dtype)
    vp = torch.randn(total_k, H, D, generator=g).to(dtype)
    dev = lambda c: torch.tensor(c, dtype=torch.int32, device="cuda")
    out, lse, _ = ns["flash_attn_varlen_func"](qp.cuda(), kp.cuda(), vp.cuda(), dev(cu_q), dev(cu_k), 200, 250)
    torch.cuda.synchronize()
    ref_o, ref_l = om.varlen_chunk_attention(qp, kp, vp, cu_q, cu_k)
    assert tuple(out.shape) == (total_q, H, D) and tuple(lse.shape) == (H, total_q) and out.dtype == dtype
    assert (out.float().cpu()[:290] - ref_o[:290]).abs().max() <= 2e-2
    assert (lse.cpu()[:, :290] - ref_l[:, :290]).abs().max() <= 1e-3
    assert int(torch.count_nonzero(out[290:])) == 0
