from .config import EngineConfig  # noqa: F401
from .llm import ZipageEngine  # noqa: F401
from .pages import PagePool  # noqa: F401
from .qwen3 import QWEN3_0_6B, QWEN3_8B, Qwen3, Qwen3Shape, StepContext  # noqa: F401
from .scheduler import Scheduler  # noqa: F401
from .sequence import SamplingParams, Sequence  # noqa: F401
