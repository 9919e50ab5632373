from .step import ModelRunner, StepEntry, StepError

__all__ = ["ModelRunner", "StepEntry", "StepError"]
from .request import GenerationResult, Request, SeqDecodingParams  # noqa: E402
from .scheduler import Scheduler, is_stop_signal  # noqa: E402
from .engine import InferenceEngine  # noqa: E402

__all__ += ["GenerationResult", "Request", "SeqDecodingParams", "Scheduler", "is_stop_signal", "InferenceEngine"]
