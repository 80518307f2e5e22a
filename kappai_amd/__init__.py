"""kappai_amd: a small, whole inference engine for one MI355X, built from what
System64fumo/kappai shows for the LFM2 hybrid decoder."""
__version__ = "0.1.0"
