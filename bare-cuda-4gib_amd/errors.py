"""The framework's exception types."""


class EngineError(RuntimeError):
    """Any failure the framework reports on purpose (reference: llm::Error,
    engine/include/llm/error.h:10-19)."""


class ConfigError(EngineError):
    """config.json is missing a key, has a wrong type, or asks for what the
    architecture cannot express."""


class WeightError(EngineError):
    """Tensors are missing, unexpected, or of the wrong shape or dtype."""


class OutOfPages(EngineError):
    """A reservation needs more cache pages than are free.  Raised before
    anything was changed, so the caller can wait, preempt or refuse."""


class KernelError(EngineError):
    """A kernel refuses the sizes it was given, or the kernel library is
    missing."""
