"""Model registry: the architecture a checkpoint's config.json names -> how to build and load it (the role of
ModelRegistry, aphrodite/modeling/models/__init__.py:160-230, for the models this package runs itself).  An entry is a
loader ``(model_dir, config_dict, dtype=, device=, **options) -> model``; every model it returns offers the engine's
interface: ``vocab_size``, ``make_caches(num_blocks, block_size, num_slots, device)`` and ``step(batch, caches, rows)``."""
from typing import Any, Callable, Dict, List, Optional

_LOADERS: Dict[str, Callable] = {}


def register_model(architecture: str, loader: Callable) -> None:
    _LOADERS[architecture] = loader


def architecture_of(config: Dict[str, Any]) -> Optional[str]:
    """``architectures[0]`` of a transformers-style config, else the plain ``architecture`` key."""
    archs = config.get("architectures")
    if isinstance(archs, (list, tuple)) and archs:
        return str(archs[0])
    a = config.get("architecture")
    if a is None and config.get("model_type") in ("llama", "mistral", "mixtral"):
        return "LlamaForCausalLM"          # exports that name only the model type
    return None if a is None else str(a)


def supported_architectures() -> List[str]:
    _register_builtin()
    return sorted(_LOADERS)


def resolve(config: Dict[str, Any]) -> Callable:
    _register_builtin()
    arch = architecture_of(config)
    if arch not in _LOADERS:
        raise ValueError(f"Model architecture {arch!r} is not supported; supported: {sorted(_LOADERS)}")
    return _LOADERS[arch]


_builtin_done = False


def _register_builtin() -> None:
    global _builtin_done
    if _builtin_done:
        return
    _builtin_done = True

    def llama(model_dir, config, **kw):
        from .loader import load_llama_model
        return load_llama_model(model_dir, config, **kw)

    def fatudra(model_dir, config, **kw):
        from .fatudra import load_fatudra
        return load_fatudra(model_dir, config, **kw)

    def gipozen(model_dir, config, **kw):
        from .gipozen import load_gipozen
        return load_gipozen(model_dir, config, **kw)

    def fekotar(model_dir, config, **kw):
        from .fekotar import load_fekotar
        return load_fekotar(model_dir, config, **kw)

    def pagulix(model_dir, config, **kw):
        from .pagulix import load_pagulix
        return load_pagulix(model_dir, config, **kw)

    for arch in ("LlamaForCausalLM", "MistralForCausalLM", "MixtralForCausalLM"):
        _LOADERS.setdefault(arch, llama)
    _LOADERS.setdefault("Fatudra", fatudra)
    _LOADERS.setdefault("Gipozen", gipozen)
    _LOADERS.setdefault("Fekotar", fekotar)
    _LOADERS.setdefault("Pagulix", pagulix)
