"""The reference's import names resolve to this package: a call site written against
``ditango.*`` (executor/cogvideox/attention_processor.py:8-11,27-29,
executor/hunyuanvideo/attention_hunyuan.py:2-3,25-27, executor/step/attentions.py:6-12) runs
unchanged.  Host-only: the attention objects plan and book-keep in dry-run mode."""
import sys

import pytest
import torch


def test_reference_import_lines_resolve_to_the_same_modules():
    from ditango.core.attention import proAttention
    from ditango.core.parallel_state import get_isp_group, get_usp_group, get_world_group
    from ditango.utils import get_timestep, update_timestep, split_tensor_uneven, remove_padding_after_gather
    from ditango.utils import update_out_and_lse, _update_out_and_lse, rel_l1
    from ditango.timer import get_timer, enable_timing, print_time_statistics, is_timing_enabled
    from ditango.core.config import get_config
    from ditango.logger import init_logger
    from ditango.core.cache import proCache
    from ditango.core.redundancy_map import (redundancy_preprocess, is_preprocessing, get_redundancy_map,
                                             init_redundancy_map)
    import ditango
    import ditango_amd.core.attention as impl_attention
    import ditango_amd.utils as impl_utils
    assert proAttention is impl_attention.proAttention
    assert sys.modules["ditango.utils"] is impl_utils and ditango.utils is impl_utils
    assert sys.modules["ditango.core"].attention is impl_attention
    # one step counter, not two
    update_timestep(7)
    assert impl_utils.get_timestep() == 7 == get_timestep()
    update_timestep(0)
    assert callable(get_timer("x").__enter__) and init_logger("t") is not None
    # the three attention adapters resolve under the reference's paths; the model forks, the comparison
    # baselines and the multi-process bootstrap are not part of the package
    from ditango.executor.cogvideox.attention_processor import CVX_oCacheAttnProcessor
    from ditango.executor.hunyuanvideo.attention_hunyuan import Hunyuan_DiTangoProcessor, MEMORY_LAYOUT
    from ditango.executor.step.attentions import Attention
    import ditango_amd.executor.step.attentions as impl_step
    assert Attention is impl_step.Attention and callable(CVX_oCacheAttnProcessor) and callable(Hunyuan_DiTangoProcessor)
    assert set(MEMORY_LAYOUT) == {"flash", "torch", "vanilla", "oAttn"}
    for missing in ("ditango.baseline", "ditango.core.initialize", "ditango.executor.cogvideox.pipeline_cogvideox"):
        with pytest.raises(ImportError):
            __import__(missing)


def test_call_site_shape_drives_attn_and_varlen_attn_in_dry_run():
    """What CVX_oCacheAttnProcessor.__init__ / __call__ and Hunyuan_DiTangoProcessor do, reduced to
    the calls into this package: build the per-layer object from the ISP group, step the counter,
    call attn / varlen_attn.  In dry-run mode the calls return None and leave the plan behind."""
    from ditango.core import config, parallel_state, redundancy_map
    from ditango.core.attention import proAttention
    from ditango.core.parallel_state import get_isp_group
    from ditango.utils import update_timestep, get_timestep

    N, T, L = 8, 6, 2
    parallel_state.init_local_groups(N, 3)
    try:
        config.init_config(None, num_inference_steps=T, num_layers=L)
        redundancy_map.destroy_redundancy_map()
        redundancy_map._redundancy_map = redundancy_map.RedundancyMap(config.get_config())
        rm = redundancy_map.get_redundancy_map()
        rm.divider_map[:, :] = torch.tensor([[1, 1], [1, 1], [1, 1], [4, 2], [2, 2], [1, 1]])
        layers = [proAttention(l, get_isp_group(), dry_run=True) for l in range(L)]
        assert layers[0].isp_size == N and layers[0].local_chunk_id == 3 and layers[0].target_chunk_id == 0
        for t in range(T):
            update_timestep(t)
            assert get_timestep() == t
            assert layers[0].attn(None, None, None) is None
            # no sequence lengths: varlen_attn is attn (core/attention.py:252-254)
            assert layers[1].varlen_attn(None, None, None) is None
            for l in range(L):
                p = layers[l].last_plan
                assert p.timestep == t and p.layer_id == l
                assert p.curr_stride == rm.get_curr_isp_stride(t, l) and len(p.computed) >= 1
        # a full-stride step computes every chunk once; a stride-2 step the local chunk and one block
        assert sorted(c for c, _ in layers[0].last_plan.computed) == list(range(N))
    finally:
        redundancy_map.destroy_redundancy_map()
        parallel_state.destroy_local_groups()
        update_timestep(0)
