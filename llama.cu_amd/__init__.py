"""llama.cu_amd: a small, whole inference engine for one MI355X (gfx950).

One architecture (the Llama dense decoder), everything between a request's tokens and
its next token: configuration and registry, weights, parts, paged cache, one step
function, scheduler, sampling, and hand-written HIP kernels.
"""
from . import config, parts, models, weights  # noqa: F401
from .config import LlamaConfig, register_architecture
from .parts import register_part

from .sampling import SamplingParams
from .engine.config import EngineConfig

import os

_engines: dict = {}


def _folder_stamp(folder: str):
    """Sizes and modification times of the folder's configuration and weight files: a folder that was written
    again is another model."""
    stamp = []
    try:
        for name in sorted(os.listdir(folder)):
            if name == "config.json" or name.endswith(".safetensors") or name.endswith(".safetensors.index.json"):
                st = os.stat(os.path.join(folder, name))
                stamp.append((name, st.st_size, st.st_mtime_ns))
    except OSError:
        pass
    return tuple(stamp)


def Engine(model: str, config: EngineConfig = None, **fields):
    """The engine for the model folder ``model`` (see engine.engine.Engine); ``config`` holds the engine's
    constants, ``fields`` replace single ones (``dtype="float32", max_seqs=4, ...``)."""
    from .engine.engine import Engine as _Engine
    return _Engine.from_folder(model, config, **fields)


def generate(model: str, prompts, sampling: SamplingParams = SamplingParams(), max_steps: int = 1000,
             dtype: str = "bfloat16", device: str = "cuda:0", **kw):
    """Generate for ``prompts`` (lists of token ids, or strings that the folder's tokenizer
    encodes) with the model of the folder ``model``; returns token ids, or strings for
    string prompts."""
    from . import text
    # a model is loaded once per process, folder as it is on the disk (its files' sizes and times) and set of
    # options; the engine is idle between calls, and a call's draws do not depend on the calls before it
    key = (os.path.abspath(model), _folder_stamp(model), dtype, str(device), repr(sorted(kw.items())))
    engine = _engines.get(key)
    if engine is None:
        _engines.clear()
        engine = _engines[key] = Engine(model, dtype=dtype, device=device, **kw)
    as_text = len(prompts) > 0 and isinstance(prompts[0], str)
    tok = text.load_tokenizer(model, engine.runner.spec.vocab_size) if as_text else None
    ids = [tok.encode(p) for p in prompts] if as_text else [list(p) for p in prompts]
    out = engine.generate(ids, sampling, max_steps)
    return [tok.decode(o) for o in out] if as_text else out


__all__ = ["config", "parts", "models", "weights", "LlamaConfig", "register_architecture", "register_part",
           "SamplingParams", "EngineConfig", "Engine", "generate"]

# modules of the user's that register further architectures or parts (LLAMA_CU_AMD_PLUGINS=module[,module]): imported
# last, when everything they may import from here is there
config.load_plugins_from_env()
