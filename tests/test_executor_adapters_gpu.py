"""The attention adapters of the three model executors (the call sites of the cached block attention), with the
reference's class names, against a restatement of what the reference adapter computes: eager torch ops for the
stretch around the attention (projections, norm modules, rotary embedding, layouts, casts -- followed line by line
from executor/cogvideox/attention_processor.py:39-86, executor/hunyuanvideo/attention_hunyuan.py:29-63,
executor/step/attentions.py:85-100) and the oracle for the attention itself.  A ring of two ranks: the other rank's
K/V are what the same adapter produces from that rank's shard."""
import pytest
import torch

from oracle import attention_math as om

pytestmark = pytest.mark.gpu
OUT_TOL, LSE_TOL = 2e-2, 1e-3


@pytest.fixture
def env(hip):
    from ditango_amd.core import config, parallel_state, redundancy_map as rmod
    from ditango_amd import utils

    def make(N, rank, T=2, L=1):
        parallel_state.init_local_groups(N, rank)
        config.init_config(None, num_inference_steps=T, num_layers=L)
        rmod.destroy_redundancy_map()
        rmod._redundancy_map = rmod.RedundancyMap(config.get_config())
        return parallel_state.get_usp_group()

    yield make
    from ditango_amd.core import parallel_state, redundancy_map as rmod
    rmod.destroy_redundancy_map()
    parallel_state.destroy_local_groups()
    utils.update_timestep(0)


class _DiffusersLikeAttention(torch.nn.Module):
    """The fields of diffusers' ``Attention`` that the CogVideoX processor touches (qk_norm="layer_norm")."""

    def __init__(self, channels, heads, head_dim):
        super().__init__()
        self.heads = heads
        self.is_cross_attention = False
        self.to_q = torch.nn.Linear(channels, heads * head_dim)
        self.to_k = torch.nn.Linear(channels, heads * head_dim)
        self.to_v = torch.nn.Linear(channels, heads * head_dim)
        self.norm_q = torch.nn.LayerNorm(head_dim, eps=1e-6)
        self.norm_k = torch.nn.LayerNorm(head_dim, eps=1e-6)
        self.to_out = torch.nn.ModuleList([torch.nn.Linear(heads * head_dim, channels), torch.nn.Dropout(0.0)])


def _apply_rotary_emb_real(x, freqs_cis):
    """diffusers 0.31 ``apply_rotary_emb(x, (cos, sin))`` with ``use_real=True``, ``use_real_unbind_dim=-1``:
    x ``[B,H,S,D]``, pairs (2i, 2i+1) rotate together, fp32 math, cast back."""
    cos, sin = freqs_cis
    cos, sin = cos[None, None].to(x.device), sin[None, None].to(x.device)
    x_real, x_imag = x.reshape(*x.shape[:-1], -1, 2).unbind(-1)
    x_rotated = torch.stack([-x_imag, x_real], dim=-1).flatten(3)
    return (x.float() * cos + x_rotated.float() * sin).to(x.dtype)


def _reference_cvx_qkv(attn, hidden_states, encoder_hidden_states, image_rotary_emb):
    """executor/cogvideox/attention_processor.py:39-71, eager, as written there."""
    text_seqlen = encoder_hidden_states.size(1)
    batch_size = hidden_states.shape[0]
    x = torch.cat([encoder_hidden_states, hidden_states], dim=1)
    query, key, value = attn.to_q(x), attn.to_k(x), attn.to_v(x)
    head_num = attn.heads
    head_dim = key.shape[-1] // head_num
    query = query.view(batch_size, -1, head_num, head_dim).transpose(1, 2)
    key = key.view(batch_size, -1, head_num, head_dim).transpose(1, 2)
    value = value.view(batch_size, -1, head_num, head_dim).transpose(1, 2)
    query, key = attn.norm_q(query), attn.norm_k(key)
    query[:, :, text_seqlen:] = _apply_rotary_emb_real(query[:, :, text_seqlen:], image_rotary_emb)
    key[:, :, text_seqlen:] = _apply_rotary_emb_real(key[:, :, text_seqlen:], image_rotary_emb)
    return query.transpose(1, 2).contiguous(), key.transpose(1, 2).contiguous(), value.transpose(1, 2).contiguous()


@pytest.mark.parametrize("D,H,dtype", [(64, 6, torch.bfloat16), (128, 3, torch.bfloat16), (64, 6, torch.float16)])
def test_cogvideox_processor_matches_the_reference_adapter(env, D, H, dtype):
    from ditango.executor.cogvideox.attention_processor import CVX_oCacheAttnProcessor      # the reference's import path
    from ditango_amd.utils import update_timestep
    N, rank, B, C, n_text, n_video = 2, 0, 1, 192, 26, 170
    group = env(N, rank)
    torch.manual_seed(3)
    attn = _DiffusersLikeAttention(C, H, D).cuda().to(dtype)      # the model's dtype: bf16, or fp16
    with torch.no_grad():
        for ln in (attn.norm_q, attn.norm_k):            # a trained affine, not the identity
            ln.weight.add_(0.1 * torch.randn_like(ln.weight))
            ln.bias.add_(0.1 * torch.randn_like(ln.bias))
    g = torch.Generator().manual_seed(5)
    shards = [(torch.randn(B, n_video, C, generator=g).to(dtype).cuda(), torch.randn(B, n_text, C, generator=g).to(dtype).cuda())
              for _ in range(N)]
    ang = torch.rand(n_video, D // 2, generator=g) * 6.28
    rope = (ang.cos().repeat_interleave(2, -1).contiguous().cuda(), ang.sin().repeat_interleave(2, -1).contiguous().cuda())
    proc = CVX_oCacheAttnProcessor(0)
    with torch.no_grad():
        # the other rank's K/V: the same adapter on that rank's shard
        _, k1, v1 = proc.project_qkv(attn, *shards[1], rope)
        group.set_kv_chunks([None, k1], [None, v1])
        update_timestep(0)
        hidden, enc = proc(attn, *shards[0], attention_mask=None, image_rotary_emb=rope)
        torch.cuda.synchronize()
        assert hidden.dtype == dtype and tuple(hidden.shape) == (B, n_video, C) and tuple(enc.shape) == (B, n_text, C)
        # 1. the producer: q / k / v against the reference's eager chain, to one rounding of the model's dtype
        q_a, k_a, v_a = proc.project_qkv(attn, *shards[0], rope)
        q_r, k_r, v_r = _reference_cvx_qkv(attn, *shards[0], rope)
        _, k1_r, v1_r = _reference_cvx_qkv(attn, *shards[1], rope)
        for a, r, what in ((q_a, q_r, "q"), (k_a, k_r, "k"), (v_a, v_r, "v"), (k1, k1_r, "k of the other rank")):
            err = (a.float() - r.float()).abs().max().item()
            print(f"cogvideox adapter D={D}: {what} max-abs vs eager {err:.3e}", flush=True)
            assert err <= 2.0 ** -6 * max(1.0, r.float().abs().max().item()), what
        assert torch.equal(v_a, v_r)
        # 2. the whole call: the reference's eager q / k / v, the oracle's attention over both ranks' chunks, cast, out-projection
        ref_o, ref_l = om.full_attention(q_r.cpu(), [k_r.cpu(), k1_r.cpu()], [v_r.cpu(), v1_r.cpu()])
        lse = proc.oAttn.last_lse.cpu().squeeze(-1).transpose(1, 2)
        assert (lse - ref_l).abs().max() <= 5e-3          # q / k differ from the eager ones by up to one rounding
        ref_h = ref_o.to(dtype).cuda().reshape(B, -1, H * D)
        ref_h = attn.to_out[1](attn.to_out[0](ref_h))
        ref_enc, ref_hidden = ref_h.split([n_text, n_video], dim=1)
        for a, r, what in ((hidden, ref_hidden, "hidden_states"), (enc, ref_enc, "encoder_hidden_states")):
            rel = ((a.float() - r.float()).norm() / r.float().norm()).item()
            print(f"cogvideox adapter D={D}: {what} rel-l2 {rel:.3e}", flush=True)
            assert rel <= 1e-2, what


def test_hunyuan_processor_matches_the_varlen_oracle(env):
    from ditango.executor.hunyuanvideo.attention_hunyuan import Hunyuan_DiTangoProcessor
    from ditango_amd.utils import update_timestep
    N, rank, B, H, D, S = 2, 1, 1, 3, 128, 300
    group = env(N, rank)
    g = torch.Generator().manual_seed(9)
    q = torch.randn(B, S, H, D, generator=g).bfloat16()
    ks = [torch.randn(B, S, H, D, generator=g).bfloat16() for _ in range(N)]
    vs = [torch.randn(B, S, H, D, generator=g).bfloat16() for _ in range(N)]
    cu_q = [0, 270, 300]                          # valid tokens | padded text, as get_cu_seqlens builds them
    cu_k = [[0, 250, 300], [0, 270, 300]]
    dev_cu = lambda c: torch.tensor(c, dtype=torch.int32, device="cuda")
    group.set_kv_chunks([k[0].cuda() for k in ks], [v[0].cuda() for v in vs], cu_seqlens_kv=[dev_cu(c) for c in cu_k])
    proc = Hunyuan_DiTangoProcessor(0)
    update_timestep(0)
    out = proc.ringfusion_attn(q.cuda(), ks[rank].cuda(), vs[rank].cuda(), cu_seqlens_q=dev_cu(cu_q), cu_seqlens_kv=dev_cu(cu_k[rank]),
                               max_seqlen_q=S, max_seqlen_kv=S, batch_size=B)
    torch.cuda.synchronize()
    assert out.dtype == torch.float32 and tuple(out.shape) == (B, S, H * D)      # fed onward in fp32 under autocast (:58-63)
    states = [om.varlen_chunk_attention(q[0], ks[c][0], vs[c][0], cu_q, cu_k[c]) for c in range(N)]
    ref_o, ref_l = om.merge_states_closed_form([s[0][None] for s in states], [s[1][None] for s in states])
    err = (out.cpu().view(B, S, H, D) - ref_o).abs().max().item()
    lerr = (proc.oAttn.last_lse.cpu().squeeze(-1).transpose(1, 2) - ref_l).abs().max().item()
    print(f"hunyuan adapter: out max-abs {err:.3e} lse {lerr:.3e}", flush=True)
    assert err <= OUT_TOL and lerr <= LSE_TOL


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
def test_step_attention_o_attn_func_matches_the_oracle(env, dtype):
    from ditango.executor.step.attentions import Attention
    from ditango_amd.utils import update_timestep
    N, rank, B, H, D, S = 2, 0, 1, 4, 128, 210
    group = env(N, rank)
    g = torch.Generator().manual_seed(13)
    q = torch.randn(B, S, H, D, generator=g).to(dtype)
    ks = [torch.randn(B, S, H, D, generator=g).to(dtype) for _ in range(N)]
    vs = [torch.randn(B, S, H, D, generator=g).to(dtype) for _ in range(N)]
    group.set_kv_chunks([k.cuda() for k in ks], [v.cuda() for v in vs])
    module = Attention(layer_id=0)
    update_timestep(0)
    x = module.attn_processor("oattn")(q.cuda(), ks[rank].cuda(), vs[rank].cuda())
    torch.cuda.synchronize()
    assert x.dtype == dtype and tuple(x.shape) == (B, S, H, D)                   # ``x.to(q.dtype)`` of :98
    ref_o, ref_l = om.full_attention(q, ks, vs)
    err = (x.float().cpu() - ref_o).abs().max().item()
    lerr = (module.oAttn.last_lse.cpu().squeeze(-1).transpose(1, 2) - ref_l).abs().max().item()
    print(f"step adapter: out max-abs {err:.3e} lse {lerr:.3e}", flush=True)
    assert err <= OUT_TOL and lerr <= LSE_TOL
    for baseline in ("torch", "parallel"):
        with pytest.raises(NotImplementedError):
            module.attn_processor(baseline)
