"""Hand-written HIP kernels for gfx950 and their loader.

``kernels/`` holds the sources, ``build.py`` compiles them with hipcc into
``libbc4g.so`` beside this file, ``library.py`` loads that library through
ctypes, and ``ops.py`` wraps each entry point for torch tensors (shape checks
on the host, then the launch on torch's current stream).
"""
