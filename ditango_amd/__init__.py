"""ditango_amd -- MI355X-native cached block attention (the hot path of chen-yy20/ditango).

Module paths mirror the reference package (``ditango.core.attention`` ->
``ditango_amd.core.attention`` and so on).  All arithmetic runs in hand-written
gfx950 HIP kernels reached through the C ABI of ``libditango_hip.so``; there
is no non-HIP fallback.
"""
__version__ = "0.1.0"
