from .batch import StepContext, StepEntry, Workspace  # noqa: F401
from .engine import Engine, build_model  # noqa: F401
from .request import FinishReason, Request, RequestStatus  # noqa: F401
from .runner import ModelRunner, decode_buckets  # noqa: F401
from .scheduler import Portion, Scheduler, SchedulerConfig, StepPlan  # noqa: F401
