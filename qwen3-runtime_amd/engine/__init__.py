from .batch import StepEntry  # noqa: F401
from .request import Request, RequestStatus  # noqa: F401
from .scheduler import Scheduler  # noqa: F401
