"""Plain, slow reading of the reference's Qwen3 formulas: whole sequences, no cache.

Nothing here imports the engine package; the engine's tests compare against it.
"""
