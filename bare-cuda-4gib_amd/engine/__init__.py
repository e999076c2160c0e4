from .spec import ModelSpec, LayerSpec, PartSpec, ScheduleEntry  # noqa: F401
from .runtime import Runtime, parse_dtype  # noqa: F401
from .batch import StepContext  # noqa: F401
from .model import Model, load_model, expected_weights  # noqa: F401
from .executor import Executor, StepEntry  # noqa: F401
from . import generate  # noqa: F401
from .scheduler import Scheduler, Request, TokenEvent, SchedulerStats, EngineLimits  # noqa: F401
from .engine import Engine, generate_batch  # noqa: F401
