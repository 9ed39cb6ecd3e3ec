from .context import StepContext, Workspace
from .step import Engine, StepEntry, StepError, pick_graph_bucket
from .factory import build_engine, make_runtime
