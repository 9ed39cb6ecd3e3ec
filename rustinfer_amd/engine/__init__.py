from .context import StepContext, Workspace
from .step import Engine, StepEntry, StepError, device_token, pick_graph_bucket
from .factory import build_engine, make_runtime
