"""The three call sites of the cached block attention: the attention adapters of the reference's model
executors (executor/cogvideox/attention_processor.py, executor/hunyuanvideo/attention_hunyuan.py,
executor/step/attentions.py), with the reference's class and method names.  The models themselves
(diffusers / hyvideo / stepvideo forks, weights, pipelines) are not part of this package: the adapters
take the projection modules they are handed (duck-typed) and own only what happens between the QKV
projection and the output projection."""
