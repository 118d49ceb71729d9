"""A plain, slow implementation of the architecture, written from the reference's formulas.

Whole sequences, no cache, one function per part, float32 (or float64) on the
CPU.  It shares no code with the engine: it reads the model folder with the
safetensors library and ``json``, and computes with elementary torch operations.
"""
