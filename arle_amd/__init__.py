"""arle_amd: a small, whole inference engine for one AMD MI355X (gfx950).

Model folder (config.json + safetensors) or a configuration and a seed -> generated tokens:
typed configuration and architecture registry (`config`), weights (`weights`), layers put
together from parts (`parts`, `models`), a paged cache with state slots (`cache`), one step
function and a scheduler above it (`engine`), sampling (`sampling`), hand-written HIP
kernels (`csrc`, `kernels`).
"""

__version__ = "0.1.0"


def __getattr__(name):
    # heavy imports (torch) happen only when the entry points are asked for
    if name in ("LLM", "generate", "CompletionOutput", "CompletionStreamDelta"):
        from .engine import api
        return getattr(api, name)
    if name in ("Engine", "StepEntry", "DeviceToken"):
        from . import engine
        return getattr(engine, name)
    if name in ("PRIORITY_LOW", "PRIORITY_NORMAL", "PRIORITY_HIGH"):
        from .engine import scheduler
        return getattr(scheduler, name)
    if name == "SamplingParams":
        from .sampling import SamplingParams
        return SamplingParams
    raise AttributeError(name)
