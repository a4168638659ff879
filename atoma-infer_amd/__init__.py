"""atoma_infer_amd: a single-GPU Llama inference engine for AMD MI355X (gfx950)."""
__version__ = "0.1.0"

from . import models as _models  # noqa: F401  (registers the architectures)
