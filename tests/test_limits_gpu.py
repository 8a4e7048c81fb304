"""The per-launch limits of the C ABI (40 chunks, 40 states, 64 chunk references, 64-way merge),
the splitting of larger requests on the host side (launch groups, chunk windows, merge rounds), tile counts around the pairing of iterations,
and the error behaviour at the boundary (return code + message, never a launch)."""
import ctypes

import pytest
import torch

from oracle import attention_math as om

pytestmark = pytest.mark.gpu

OUT_TOL, LSE_TOL = 2e-2, 1e-3


def _check(out, lse, ref_out, ref_lse, what):
    err = (out.float().cpu() - ref_out).abs().max().item()
    lerr = (lse.cpu() - ref_lse).abs().max().item()
    assert err <= OUT_TOL and lerr <= LSE_TOL, f"{what}: out {err:.3e} lse {lerr:.3e}"


def _rand(shape, g):
    return torch.randn(*shape, generator=g).bfloat16()


def test_forty_chunks_in_one_job(hip):
    B, Sq, H, D, C = 1, 70, 2, 128, hip.DT_MAX_CHUNKS
    g = torch.Generator().manual_seed(1)
    lens = [1 + (7 * i) % 50 for i in range(C)]
    q = _rand((B, Sq, H, D), g)
    ks = [_rand((B, n, H, D), g) for n in lens]
    vs = [_rand((B, n, H, D), g) for n in lens]
    ref_out, ref_lse = om.full_attention(q, ks, vs)
    table = hip.ChunkTable([k.cuda() for k in ks], [v.cuda() for v in vs])
    out = torch.empty(B, Sq, H, D, dtype=torch.bfloat16, device="cuda")
    lse = torch.empty(B, H, Sq, dtype=torch.float32, device="cuda")
    hip.attn_jobs_fwd(q.cuda(), table, [list(range(C))], [out], [lse])
    torch.cuda.synchronize()
    _check(out, lse, ref_out, ref_lse, "40 chunks, one job")
    # the C ABI itself turns a 41st chunk down ...
    big = hip.ChunkTable([k.cuda() for k in ks] + [ks[0].cuda()], [v.cuda() for v in vs] + [vs[0].cuda()])
    with pytest.raises(hip.DitangoHipError):
        big.whole()
    # ... and so does a single job over 41 distinct chunks (the caller splits such a job and merges)
    with pytest.raises(hip.DitangoHipError):
        hip.attn_jobs_fwd(q.cuda(), big, [list(range(C + 1))], [out], [lse])


def test_table_of_more_chunks_than_a_launch_addresses(hip):
    """70 chunks, 70 single-chunk jobs and two jobs of 35 chunks each: the binding groups jobs into
    launches whose sub-table holds at most 40 distinct chunks."""
    B, Sq, H, D, C = 1, 40, 2, 64, 70
    g = torch.Generator().manual_seed(8)
    lens = [5 + (11 * i) % 40 for i in range(C)]
    q = _rand((B, Sq, H, D), g)
    ks = [_rand((B, n, H, D), g) for n in lens]
    vs = [_rand((B, n, H, D), g) for n in lens]
    table = hip.ChunkTable([k.cuda() for k in ks], [v.cuda() for v in vs])
    jobs = [[c] for c in range(C)] + [list(range(0, C, 2)), list(range(1, C, 2))]
    outs = [torch.empty(B, Sq, H, D, dtype=torch.bfloat16, device="cuda") for _ in jobs]
    lses = [torch.empty(B, H, Sq, dtype=torch.float32, device="cuda") for _ in jobs]
    hip.attn_jobs_fwd(q.cuda(), table, jobs, outs, lses)
    torch.cuda.synchronize()
    for j, chunks in enumerate(jobs):
        ref = om.full_attention(q, [ks[c] for c in chunks], [vs[c] for c in chunks])
        _check(outs[j], lses[j], *ref, f"job {j}")
    # everything merged = attention over all 70 chunks (a 70-way merge: more than one merge launch holds)
    o, l = hip.merge_states(outs[:C], lses[:C])
    torch.cuda.synchronize()
    ref_out, ref_lse = om.full_attention(q, ks, vs)
    _check(o, l, ref_out, ref_lse, "70-way merge of the chunk states")


def test_more_jobs_than_one_launch_holds(hip):
    """45 single-chunk states and then jobs whose chunk references exceed 64: the binding splits launches."""
    B, Sq, H, D, C = 1, 40, 1, 64, 9
    g = torch.Generator().manual_seed(2)
    q = _rand((B, Sq, H, D), g)
    ks = [_rand((B, 30 + i, H, D), g) for i in range(C)]
    vs = [_rand((B, 30 + i, H, D), g) for i in range(C)]
    refs = [om.chunk_attention(q, k, v) for k, v in zip(ks, vs)]
    table = hip.ChunkTable([k.cuda() for k in ks], [v.cuda() for v in vs])
    dq = q.cuda()
    jobs = [[j % C] for j in range(45)]
    outs = [torch.empty(B, Sq, H, D, dtype=torch.bfloat16, device="cuda") for _ in jobs]
    lses = [torch.empty(B, H, Sq, dtype=torch.float32, device="cuda") for _ in jobs]
    hip.attn_jobs_fwd(dq, table, jobs, outs, lses)
    torch.cuda.synchronize()
    for j in range(45):
        _check(outs[j], lses[j], *refs[j % C], f"job {j}")
    # 12 jobs of 9 references each = 108 references > 64 per launch
    jobs = [list(range(C)) for _ in range(12)]
    full = om.full_attention(q, ks, vs)
    hip.attn_jobs_fwd(dq, table, jobs, outs[:12], lses[:12])
    torch.cuda.synchronize()
    for j in range(12):
        _check(outs[j], lses[j], *full, f"full job {j}")


@pytest.mark.parametrize("n", [64, 65, 100, 127, 200])
@pytest.mark.parametrize("D,dst_dtype", [(128, torch.float32), (64, torch.bfloat16)])
def test_many_way_merge_in_rounds(hip, n, D, dst_dtype):
    """One launch folds up to 64 states; more go through a running fp32 state in rounds of 63.  Against
    the closed form, with -inf states, a repeated pointer and mixed dtypes / lse layouts among them."""
    assert hip.DT_MAX_MERGE == 64
    B, Sq, H = 1, 50, 3
    g = torch.Generator().manual_seed(3 + n)
    outs = [_rand((B, Sq, H, D), g) for _ in range(n)]
    lses = [torch.randn(B, H, Sq, generator=g) * 3 for _ in range(n)]
    lses[7].fill_(float("-inf"))
    lses[n - 2].fill_(float("-inf"))
    outs[n - 1], lses[n - 1] = outs[3], lses[3]                      # the same state twice
    d_outs = [x.cuda() for x in outs]
    d_lses = [x.cuda() for x in lses]
    d_outs[n // 2] = d_outs[n // 2].float()                          # one fp32 state ...
    d_lses[n // 3] = d_lses[n // 3].transpose(1, 2).contiguous().unsqueeze(-1)   # ... one lse stored [B,S,H,1]
    ref_out, ref_lse = om.merge_states_closed_form([o.float() for o in outs], lses)
    o, l = hip.merge_states(d_outs, d_lses, dst_dtype=dst_dtype)
    torch.cuda.synchronize()
    tol = 1e-5 if dst_dtype == torch.float32 else 2.0 ** -8 * float(ref_out.abs().max())
    assert o.dtype == dst_dtype
    assert (o.float().cpu() - ref_out).abs().max() <= tol and (l.cpu() - ref_lse).abs().max() <= 1e-5
    # in place over the first input (cache coarsening writes over its first member)
    first_o, first_l = d_outs[0].clone(), d_lses[0].clone()
    hip.merge_states([first_o] + d_outs[1:], [first_l] + d_lses[1:], dst_out=first_o, dst_lse=first_l)
    torch.cuda.synchronize()
    assert (first_o.float().cpu() - ref_out).abs().max() <= 2.0 ** -8 * float(ref_out.abs().max())
    assert (first_l.cpu() - ref_lse).abs().max() <= 1e-5


@pytest.mark.parametrize("Sk", [63, 64, 65, 127, 128, 129, 191, 193, 256, 257, 320, 449, 512, 513, 577])
@pytest.mark.parametrize("D", [64, 128])
def test_tile_counts_around_the_unrolled_iterations(hip, Sk, D):
    """1 to 10 key tiles, full and ragged: the loop runs four tiles per trip (one per LDS buffer) and
    leaves the last trip after the last tile."""
    B, Sq, H = 1, 96, 1
    g = torch.Generator().manual_seed(Sk)
    q, k, v = _rand((B, Sq, H, D), g), _rand((B, Sk, H, D), g), _rand((B, Sk, H, D), g)
    ref = om.chunk_attention(q, k, v)
    out, lse = hip.attn_chunk_fwd(q.cuda(), k.cuda(), v.cuda())
    torch.cuda.synchronize()
    _check(out, lse, *ref, f"Sk={Sk} D={D}")


def test_c_abi_rejects_without_launching(hip):
    lib = hip.load_library()
    q = torch.zeros(1, 8, 1, 128, dtype=torch.bfloat16, device="cuda")
    out = torch.full((1, 8, 1, 128), 7.0, dtype=torch.bfloat16, device="cuda")
    lse = torch.zeros(1, 1, 8, device="cuda")

    def call(qp, D=128, Sk=8, stride_s=128):
        return lib.dt_attn_chunk_fwd(qp, q.data_ptr(), q.data_ptr(), out.data_ptr(), lse.data_ptr(), 1, 8, Sk, 1, D,
                                     8 * 128, stride_s, 128, 8 * 128, 128, 128, ctypes.c_float(0.0), None)

    assert call(q.data_ptr() + 2) == -1 and b"aligned" in lib.dt_last_error()       # DT_ERR_INVALID
    assert call(q.data_ptr(), D=96) == -2 and b"96" in lib.dt_last_error()           # DT_ERR_UNSUPPORTED
    assert call(q.data_ptr(), Sk=-1) == -1
    assert call(q.data_ptr(), stride_s=130) == -1
    assert call(None) == -1
    torch.cuda.synchronize()
    assert (out.float() == 7.0).all()                                                # nothing ran
    assert call(q.data_ptr()) == 0


@pytest.mark.parametrize("D,H,nq,lens,jobs", [
    (128, 8, 40, [2610], [[0]]),                       # 320 items: 64 left over -> cut in parts; odd part sizes
    (64, 8, 36, [2600, 2500], [[0], [1]]),             # two jobs of 288 items, 64 left over in the last
    (128, 8, 43, [2000, 0, 1900], [[0, 1, 2]]),        # one job over several chunks (an empty one among them)
    (128, 8, 33, [2000], [[0]]),                       # 264 items: 8 left over
])
def test_tail_balancing_matches_plain_launch_and_oracle(hip, D, H, nq, lens, jobs):
    """With a workspace the last round of workgroups runs as key-range parts folded by a second
    kernel: same states as the plain launch up to the extra bf16 rounding of the parts."""
    B, Sq = 1, 256 * nq - 19
    g = torch.Generator().manual_seed(D + nq)
    q = (torch.randn(B, Sq, H, D, generator=g) * 1.3).bfloat16()
    ks = [torch.randn(B, n, H, D, generator=g).bfloat16() for n in lens]
    vs = [torch.randn(B, n, H, D, generator=g).bfloat16() for n in lens]
    live = [c for c, n in enumerate(lens) if n > 0]
    table = hip.ChunkTable([k.cuda() for k in ks], [v.cuda() for v in vs])
    ws = hip.attn_workspace("cuda")
    dq = q.cuda()

    def run(workspace):
        outs = [torch.zeros(B, Sq, H, D, dtype=torch.bfloat16, device="cuda") for _ in jobs]
        lses = [torch.zeros(B, H, Sq, dtype=torch.float32, device="cuda") for _ in jobs]
        hip.attn_jobs_fwd(dq, table, jobs, outs, lses, workspace=workspace)
        torch.cuda.synchronize()
        return outs, lses

    po, pl = run(None)
    bo, bl = run(ws)
    changed = 0
    for j in range(len(jobs)):
        changed += int((po[j] != bo[j]).any())
        assert (po[j].float() - bo[j].float()).abs().max() <= 2.0 ** -7 * po[j].float().abs().max()
        assert (pl[j] - bl[j]).abs().max() <= 1e-5
    assert changed > 0, "the balanced launch was expected to take the split path for this shape"
    # a sample of query rows, the tail items (last rows of the last heads) included, against the oracle
    rows = torch.cat([torch.arange(0, 64), torch.arange(Sq - 300, Sq)])
    for j, chunks in enumerate(jobs):
        cs = [c for c in chunks if c in live]
        ref_out, ref_lse = om.full_attention(q[:, rows], [ks[c] for c in cs], [vs[c] for c in cs])
        _check(bo[j][:, rows.cuda()], bl[j][:, :, rows.cuda()], ref_out, ref_lse, f"balanced job {j}")


def test_tail_balancing_in_the_device_scheduled_launch(hip):
    B, H, D, C = 1, 8, 128, 3
    Sq = 256 * 36
    g = torch.Generator().manual_seed(77)
    q = torch.randn(B, Sq, H, D, generator=g).bfloat16().cuda()
    ks = [torch.randn(B, 4000, H, D, generator=g).bfloat16().cuda() for _ in range(C)]
    vs = [torch.randn(B, 4000, H, D, generator=g).bfloat16().cuda() for _ in range(C)]
    table = hip.ChunkTable(ks, vs)
    ids = torch.tensor([1, 2, 0], dtype=torch.int32, device="cuda")
    cnt = torch.tensor([2], dtype=torch.int32, device="cuda")

    def run(workspace, max_jobs):
        ao = torch.zeros(C, B, Sq, H, D, dtype=torch.bfloat16, device="cuda")
        al = torch.zeros(C, B, H, Sq, device="cuda")
        do = torch.zeros(B, Sq, H, D, dtype=torch.bfloat16, device="cuda")
        dl = torch.zeros(B, H, Sq, device="cuda")
        hip.attn_sched_fwd(q, table, ids, cnt, max_jobs, ao, al, 2, do, dl, workspace=workspace)
        torch.cuda.synchronize()
        return ao, al, do, dl

    plain = run(None, 2)
    for max_jobs in (2, 3):   # 3: the tail belongs to a job the device list leaves idle
        bal = run(hip.attn_workspace("cuda"), max_jobs)
        for p, b in zip(plain, bal):
            assert (p.float() - b.float()).abs().max() <= max(1e-5, 2.0 ** -7 * float(p.float().abs().max()))
        assert (bal[0][0] == 0).all()      # chunk 0 was not scheduled
        if max_jobs == 2:
            # 2 x 288 items leave 64 for the last round: the split path ran (its parts round differently)
            assert any(bool((p != b).any()) for p, b in zip(plain, bal))


@pytest.mark.parametrize("seed", range(8))
def test_tail_balancing_random_launches_match_plain(hip, seed):
    """Random launches big enough to leave a partial last round: balanced == plain up to the parts' rounding."""
    import random
    rng = random.Random(seed)
    D = rng.choice([64, 128])
    H = rng.choice([8, 16])
    nq = rng.randrange(17, 49) if H == 16 else rng.randrange(33, 60)
    B, Sq = 1, 256 * nq - rng.randrange(0, 200)
    C = rng.choice([1, 2, 3])
    lens = [rng.randrange(1200, 3500) for _ in range(C)]
    jobs = [[c] for c in range(C)] if rng.random() < 0.5 else [list(range(C))] + [[rng.randrange(C)]]
    g = torch.Generator(device="cuda").manual_seed(seed)
    q = torch.randn(B, Sq, H, D, generator=g, device="cuda").bfloat16()
    ks = [torch.randn(B, n, H, D, generator=g, device="cuda").bfloat16() for n in lens]
    vs = [torch.randn(B, n, H, D, generator=g, device="cuda").bfloat16() for n in lens]
    table = hip.ChunkTable(ks, vs)
    print(f"case seed={seed} D={D} H={H} Sq={Sq} lens={lens} jobs={jobs} items={H * nq}", flush=True)
    res = []
    for ws in (None, hip.attn_workspace("cuda")):
        outs = [torch.zeros(B, Sq, H, D, dtype=torch.bfloat16, device="cuda") for _ in jobs]
        lses = [torch.zeros(B, H, Sq, dtype=torch.float32, device="cuda") for _ in jobs]
        hip.attn_jobs_fwd(q, table, jobs, outs, lses, workspace=ws)
        torch.cuda.synchronize()
        res.append((outs, lses))
    for j in range(len(jobs)):
        po, bo = res[0][0][j].float(), res[1][0][j].float()
        assert torch.isfinite(bo).all()
        assert (po - bo).abs().max() <= 2.0 ** -7 * po.abs().max()
        assert (res[0][1][j] - res[1][1][j]).abs().max() <= 1e-5


def test_attention_workspace_is_per_stream(hip):
    """Launches on different streams must not share the tail-balancing workspace (they would race on it)."""
    a = hip.attn_workspace("cuda")
    assert hip.attn_workspace("cuda").data_ptr() == a.data_ptr()
    side = torch.cuda.Stream()
    with torch.cuda.stream(side):
        b = hip.attn_workspace("cuda")
        assert hip.attn_workspace("cuda").data_ptr() == b.data_ptr()
    assert a.data_ptr() != b.data_ptr() and a.numel() == b.numel()
    assert hip.attn_workspace("cuda").data_ptr() == a.data_ptr()
    # the table is bounded: streams beyond MAX_WORKSPACES push the least recently used entry out
    streams = [torch.cuda.Stream() for _ in range(hip.MAX_WORKSPACES + 2)]
    for st in streams:
        with torch.cuda.stream(st):
            hip.attn_workspace("cuda")
            hip.attn_workspace("cuda")          # a repeated request must not grow the table
        assert len(hip._workspaces) <= hip.MAX_WORKSPACES
    assert len(hip._workspaces) == hip.MAX_WORKSPACES
    with torch.cuda.stream(streams[-1]):
        last = hip.attn_workspace("cuda")
    assert hip.attn_workspace("cuda").data_ptr() != last.data_ptr()     # the default stream's entry was re-created
    hip.release_workspaces()
    assert len(hip._workspaces) == 0


def test_cache_load_into_given_tensors(hip):
    B, S, H, D = 1, 70, 2, 64
    g = torch.Generator().manual_seed(9)
    o = _rand((B, S, H, D), g).cuda()
    l = torch.randn(B, H, S, generator=g).cuda()
    dst_o = torch.empty(B, S, H, D, dtype=torch.float32, device="cuda")
    dst_l = torch.empty(B, S, H, 1, dtype=torch.float32, device="cuda")
    ro, rl = hip.cache_load(o, l, dst_out=dst_o, dst_lse=dst_l)
    torch.cuda.synchronize()
    assert ro is dst_o and rl is dst_l
    assert torch.equal(dst_o, o.float()) and torch.equal(dst_l.squeeze(-1).transpose(1, 2), l)
