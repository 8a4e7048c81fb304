"""``ditango`` -- the import name of the reference package, resolved to ``ditango_amd``.

The reference's call sites import the hot path as ``ditango.*``
(executor/cogvideox/attention_processor.py:8-11, executor/hunyuanvideo/attention_hunyuan.py:2-3,
executor/step/attentions.py:6-12).  With this directory on ``sys.path`` those imports work
unchanged: every name below is the SAME module object as its ``ditango_amd`` counterpart (one
step counter, one redundancy map, one set of groups), not a copy.  Only the modules of the
cached block attention path and its three call-site adapters (``ditango.executor.*``: the attention
processors only, not the model forks) exist; ``ditango.baseline`` and ``ditango.core.initialize`` of the
reference are not part of this build and raise ImportError.
"""
import importlib
import sys

import ditango_amd as _impl

_ALIASED = ("logger", "timer", "utils", "producer", "core", "core.config", "core.parallel_state",
            "core.redundancy_map", "core.cache", "core.attention", "executor", "executor.cogvideox",
            "executor.cogvideox.attention_processor", "executor.hunyuanvideo", "executor.hunyuanvideo.attention_hunyuan",
            "executor.step", "executor.step.attentions")

for _name in _ALIASED:
    _mod = importlib.import_module("ditango_amd." + _name)
    sys.modules[__name__ + "." + _name] = _mod
    if "." not in _name:
        globals()[_name] = _mod

__version__ = _impl.__version__
__all__ = ["logger", "timer", "utils", "producer", "core", "executor"]
