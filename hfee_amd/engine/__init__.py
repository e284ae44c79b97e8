from .model import Model, EngineInfo, load_model, random_model, declared_tensors
from .step import Engine, StepEntry, StepPlan, StepError
from .scheduler import Scheduler, Request, Stats, Finished, PromptTooLong
