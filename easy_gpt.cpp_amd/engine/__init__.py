from .context import GroupTables, StepContext
from .engine import DTYPES, Engine, StepEntry, load_model

__all__ = ["DTYPES", "Engine", "GroupTables", "StepContext", "StepEntry", "load_model"]
