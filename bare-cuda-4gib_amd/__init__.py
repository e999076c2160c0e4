"""A small, whole inference engine for one GPU (AMD MI355X, gfx950).

Sub-packages, by what they own:

config    typed configurations read from config.json, and the registry that
          maps an architecture's name to its configuration class and builder
weights   safetensors reading and writing, loading by tensor name, random models
parts     norms, position encodings, mixers, feed-forwards, blocks
cache     page pools, block tables, per-request state slots
engine    the model (layers plus a schedule), the step function, the scheduler,
          the Engine entry point
sampling  greedy / temperature / top-k / top-p
csrc      hand-written HIP kernels and their loader
cli       command-line programs
"""

__all__ = ["config", "weights", "parts", "cache", "engine", "sampling", "csrc"]
