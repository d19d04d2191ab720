from .generate import Request, Result, generate, plan_batches
from .model import DecoderModel
from .plan import LayerPlan, ModelPlan, ScheduleEntry
from .step import Engine, StepContext, StepEntry, StepError
