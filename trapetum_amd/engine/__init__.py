from .batch import StepContext, StepError   # noqa: F401
from .engine import Engine, load_model, read_stop_ids   # noqa: F401
from .generate import Finished, generate, plan_batch   # noqa: F401
from .model import Model   # noqa: F401
from .runtime import Runtime   # noqa: F401
