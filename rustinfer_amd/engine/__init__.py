from .context import StepContext, Workspace
from .step import Engine, StepEntry, StepError
from .factory import build_engine, make_runtime
