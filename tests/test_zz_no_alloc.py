"""The allocation-free attention entry point (``dt_attn_seg_jobs_noalloc_fwd``) against the entry point
it is a variant of (``dt_attn_seg_jobs_ws_fwd`` with a caller workspace of the same size), through the
C ABI: two calls in a row, the second on a smaller input, bit for bit (same kernels, same split)."""
import pytest
import torch

pytestmark = pytest.mark.gpu


def _inputs(B, H, D, Sq, lens, seed):
    g = torch.Generator(device="cuda").manual_seed(seed)
    q = torch.randn(B, Sq, H, D, generator=g, device="cuda").bfloat16()
    ks = [torch.randn(B, n, H, D, generator=g, device="cuda").bfloat16() for n in lens]
    vs = [torch.randn(B, n, H, D, generator=g, device="cuda").bfloat16() for n in lens]
    return q, ks, vs


def _states(n, B, Sq, H, D):
    # poisoned, so that rows a launch leaves unwritten cannot compare equal by accident
    outs = [torch.full((B, Sq, H, D), float("nan"), dtype=torch.bfloat16, device="cuda") for _ in range(n)]
    lses = [torch.full((B, H, Sq), float("nan"), dtype=torch.float32, device="cuda") for _ in range(n)]
    return outs, lses


def test_noalloc_entry_matches_workspace_entry_twice(hip):
    scratch_bytes = hip.DT_NOALLOC_TAIL_SLOTS * (256 * 128 * 2 + 256 * 4)
    ws = torch.empty(scratch_bytes, dtype=torch.uint8, device="cuda")
    # (B, H, D, Sq, chunk lengths, jobs): 288 work items (tail of 32 on 256 CUs), then 2 x 160 (tail of 64)
    cases = [(1, 24, 128, 3000, [4000], [[0]]),
             (1, 16, 128, 2500, [2000, 1500], [[0], [1]]),
             (1, 36, 64, 2000, [2100], [[0]])]
    for i, (B, H, D, Sq, lens, jobs) in enumerate(cases):
        print(f"no-alloc case {i}: B={B} H={H} D={D} Sq={Sq} lens={lens} jobs={jobs}", flush=True)
        q, ks, vs = _inputs(B, H, D, Sq, lens, seed=100 + i)
        table = hip.ChunkTable(ks, vs)
        ref_o, ref_l = _states(len(jobs), B, Sq, H, D)
        hip.attn_jobs_fwd(q, table, jobs, ref_o, ref_l, workspace=ws)
        got_o, got_l = _states(len(jobs), B, Sq, H, D)
        hip.attn_jobs_fwd(q, table, jobs, got_o, got_l, no_alloc=True)
        plain_o, plain_l = _states(len(jobs), B, Sq, H, D)
        hip.attn_jobs_fwd(q, table, jobs, plain_o, plain_l)
        torch.cuda.synchronize()
        for j in range(len(jobs)):
            assert torch.isfinite(got_l[j]).all() and torch.isfinite(got_o[j].float()).all()
            assert torch.equal(got_o[j], ref_o[j]) and torch.equal(got_l[j], ref_l[j]), f"case {i} job {j}"
            # and it is the same attention as the launch without any scratch (parts are rounded once more)
            assert (got_o[j].float() - plain_o[j].float()).abs().max().item() <= 2e-2
            assert (got_l[j] - plain_l[j]).abs().max().item() <= 1e-4
        # the split really ran: the tail rows went through bf16 partial states, which shows in the last bits
        assert any(not torch.equal(got_o[j], plain_o[j]) for j in range(len(jobs))), f"case {i}: tail was not split"
