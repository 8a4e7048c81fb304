"""CPU oracle for DiTango's cached block attention.

TEST INFRASTRUCTURE ONLY.  Nothing under ``oracle/`` is part of the product:
only ``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import it, and only as the checker.  The product package
``ditango_amd`` never imports this package and has no CPU fallback.

Modules (each function cites the reference file:line it restates):

* ``attention_math``  chunk attention closed form and the LSE merge
  (reference: ``utils.py:24-84`` and the public contract of
  ``flash_attn_func`` as called at ``core/attention.py:137-143,185-191``).
* ``state_machine``   ``proCache`` / ``proAttention.attn`` restated with a
  literal lock-step simulation of all ring ranks
  (``core/cache.py:9-128``, ``core/attention.py:21-237``).
* ``divider_map``     redundancy map -> divider map -> strides
  (``core/redundancy_map.py:49-87,199-326``) and ``rel_l1``
  (``utils.py:202-267``).
* ``mask_schedule``   the explicit per-chunk mask mode (a generalisation the
  reference cannot express; semantics documented in that module).
* ``producer``        QK normalisation + rotary embedding in front of the
  attention call (``executor/cogvideox/attention_processor.py:55-71``,
  ``executor/hunyuanvideo/hunyuan_transformer.py:177-191``,
  ``executor/step/blocks.py:66-75``, ``executor/step/rope.py:13-90``).

Pinning status (what fixes each function besides "it restates the source"):

* chunk attention: pinned against ``torch.nn.functional.scaled_dot_product_attention``
  and ``torch.logsumexp`` (library routines), softmax row-sum, key-permutation
  invariance and the identity full attention == merge of per-chunk states.
  The bf16 rounding behaviour inside the third-party ``flash_attn==2.7.0.post2``
  kernels (absent from the reference tree) is **parity unpinned**; tolerances
  are therefore against this fp32 closed form.
* LSE merge: pinned against ``torch.logaddexp`` / weighted average closed form,
  associativity, commutativity, identity for an empty (-inf) state.
* state machine: pinned by brute force over all legal divider sequences for
  N in {2,4,8} and random ones for N=16: send/recv pairing of the simulated
  ring, every chunk contributing exactly once per call (except the documented
  double count), constant-input steps reproducing full attention.
* divider map: pinned bit-exact against the REFERENCE'S OWN OUTPUT on the three
  redundancy maps it ships (``configs/*/redundancy_map_50_*.pt`` with the
  percentiles and dividers of its ``config.yaml`` files) for ring sizes 2, 4, 8
  and 16: ``tests/golden/divider_maps.npz``, written by
  ``tests/golden/make_divider_fixtures.py``, which imports the two functions from
  the reference tree; and by the structural rules of ``_refine_divider_map``.
* producer: RMSNorm / LayerNorm pinned against ``torch.nn.functional.rms_norm``
  / ``layer_norm``; interleaved RoPE against complex multiplication
  (``torch.view_as_complex``); rotate-half RoPE against explicit 2x2 rotations,
  norm preservation and the relative-position property; the Step-Video tables
  against a direct evaluation of cos/sin at the mesh positions.  Where the
  third-party modules (diffusers 0.31.0, hyvideo, stepvideo) place their
  intermediate bf16 roundings is **parity unpinned**.
"""
