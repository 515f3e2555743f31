"""MI355X-native recurrent-core decode path of the Huginn/Raven model.

The directory name carries a hyphen, so the package is imported under the name
`recurrent_pretraining_amd` through `__graft_entry__.import_package()` (or any importlib call that
registers this directory under that name).
"""

from . import hip  # noqa: F401
from . import adaptive  # noqa: F401
from . import vllm_binding  # noqa: F401
from .adaptive import (  # noqa: F401
    ArgmaxStabilityExitEvaluator,
    CosineExitEvaluator,
    EntropyDiffExitEvaluator,
    KLExitEvaluator,
    LatentDiffExitEvaluator,
    MinKLExitEvaluator,
    NoOpExitEvaluator,
    NumStepsGenerator,
    PerIterationExitEvaluator,
    get_adaptive_exit_evaluator,
)
from .cache import HuginnDynamicCache, HuginnStaticCache, remap_step  # noqa: F401
from .config import RavenConfig  # noqa: F401
from .modeling import (  # noqa: F401
    CausalLMOutputRecurrentLatents,
    DecodeRunner,
    GenerationSettings,
    RavenForCausalLM,
    precompute_freqs_cis,
)
from .paged import PagedDecoder  # noqa: F401

__all__ = [
    "hip", "HuginnDynamicCache", "HuginnStaticCache", "remap_step", "RavenConfig", "RavenForCausalLM", "DecodeRunner",
    "CausalLMOutputRecurrentLatents", "GenerationSettings", "precompute_freqs_cis", "adaptive", "vllm_binding",
    "PerIterationExitEvaluator", "NoOpExitEvaluator", "EntropyDiffExitEvaluator", "LatentDiffExitEvaluator",
    "KLExitEvaluator", "MinKLExitEvaluator", "ArgmaxStabilityExitEvaluator", "CosineExitEvaluator", "NumStepsGenerator",
    "get_adaptive_exit_evaluator", "PagedDecoder",
]
