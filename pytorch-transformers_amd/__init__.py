"""A small MI355X-native model library with generation: configuration, weights, parts, cache,
step function, generation loop and sampling for the Falcon architecture, on hand-written gfx950
HIP kernels.  Import name: ``pytorch_transformers_amd``."""
from .config import AutoConfig, ConfigError, BimepelConfig, FalconConfig, GenerationConfig, KekapelConfig, PavodraConfig, register
from .engine import falcon as _falcon  # registers model_type "falcon"  # noqa: F401
from .engine import pavodra as _pavodra  # registers model_type "pavodra"  # noqa: F401
from .engine import bimepel as _bimepel  # registers model_type "bimepel"  # noqa: F401
from .engine import kekapel as _kekapel  # registers model_type "kekapel"  # noqa: F401
from .engine import nopuzen as _nopuzen  # registers model_type "nopuzen"  # noqa: F401
from .auto import AutoModelForCausalLM
from .pipeline import TextGenerationPipeline, pipeline
from .sampling.custom import LogitsProcessor, LogitsProcessorList, StoppingCriteria, StoppingCriteriaList
from .streaming import BaseStreamer, TextIteratorStreamer, TextStreamer

__version__ = "0.1.0"
__all__ = ["BimepelConfig", "KekapelConfig", "AutoConfig", "AutoModelForCausalLM", "BaseStreamer", "ConfigError", "FalconConfig", "GenerationConfig", "PavodraConfig",
           "LogitsProcessor", "LogitsProcessorList", "StoppingCriteria", "StoppingCriteriaList", "TextGenerationPipeline",
           "TextIteratorStreamer", "TextStreamer", "pipeline", "register"]
