from .batch import StepEntry  # noqa: F401
from .request import Phase, Request, StopRule  # noqa: F401
from .scheduler import Scheduler  # noqa: F401
