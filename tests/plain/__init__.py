"""Plain, slow implementation of the Qwen2 decoder and of the sampler.

Whole sequences, no cache, one function per part, NumPy only. It shares no
code with the ``alofa_amd`` package: it exists so that the engine has
something independent to be compared with. Every function cites the lines of
the reference (paths relative to the reference checkout) that fix its formula.
"""
