"""Step function, scheduler, serving loop and trace replay."""
from .batch import StepEntry, StepContext
from .step import ModelRunner
from .scheduler import Scheduler, Request, Work, Phase
from .engine import Engine

__all__ = ['StepEntry', 'StepContext', 'ModelRunner', 'Scheduler', 'Request', 'Work', 'Phase', 'Engine']
