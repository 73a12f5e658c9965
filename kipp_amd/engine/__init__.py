from .batch import StepBatch, StepEntry
from .engine import Engine
from .model import Model, load_model, model_params, random_model
