from .params import SamplingParams, check_sampling, seed_for  # noqa: F401
from .mt19937_64 import MT19937_64  # noqa: F401
from .host import sample_token, sample_weights  # noqa: F401
from .device import DevicePicker  # noqa: F401
