"""tempura_amd: a small, whole Llama 3 inference engine for one AMD MI355X (gfx950).

The names a user starts from (the reference's ``InferenceModel`` and ``inspect``,
/root/reference/engine/src/model.rs:305-448, /root/reference/model/src/inspect.rs:84-135)::

    import tempura_amd as tempura
    eng = tempura.Engine(model_dir, dtype="bfloat16")
    outs = eng.generate([[1, 2, 3]], tempura.SamplingParams(temperature=0.0, max_new_tokens=16))
    tempura.inspect(model_dir)
"""
__version__ = "0.1.0"

from .config import PRESETS, LlamaConfig, load_config          # noqa: E402,F401
from .sampling import SamplingParams                           # noqa: E402,F401
from .engine import Engine                                     # noqa: E402,F401
from .inspect import inspect                                   # noqa: E402,F401  (the function, which now hides the module of its name)

__all__ = ["Engine", "SamplingParams", "LlamaConfig", "PRESETS", "load_config", "inspect", "__version__"]
