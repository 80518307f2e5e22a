"""Plain, slow, whole-sequence implementation of the LFM2 hybrid decoder.

Written from the formulas of System64fumo/kappai (every function cites the file and
lines it was read from).  It works on whole sequences, keeps no cache, has one function
per part and shares no code with the ``kappai_amd`` package: it is what the engine is
compared with.
"""
