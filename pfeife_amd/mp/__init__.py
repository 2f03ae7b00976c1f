from ..option import PipeOption  # noqa: F401
from .net_states import check_initialized, get_device, get_state, initialize_pfeife  # noqa: F401
from .partial import PartialModule, PartialRunner, partial_compiler  # noqa: F401
