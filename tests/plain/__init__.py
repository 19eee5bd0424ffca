"""Plain, slow Qwen2 implementation used only as the tests' oracle.

Whole sequences, no cache, one function per part, numpy only.  It shares no
code with the engine: it reads checkpoints through the `safetensors` library
and keeps its own notion of the configuration (a plain dict of config.json).
"""
