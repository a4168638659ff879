"""atoma_infer_amd: a single-GPU Llama inference engine for AMD MI355X (gfx950)."""
__version__ = "0.1.0"

from . import models as _models  # noqa: F401  (registers the architectures)
from .config import EngineConfig, LlamaConfig, load_model_config, register_architecture  # noqa: F401
from .sampling import GenerateParameters  # noqa: F401
from .weights import write_random_model  # noqa: F401


def __getattr__(name):
    # the engine imports torch.cuda machinery; load it on first use
    if name in ("LlmEngine", "generate"):
        from .engine import engine as _e
        return getattr(_e, name)
    raise AttributeError(name)
