from .batch import KVStepTables, Scratch, StepContext, StepEntry
from .engine import Engine
