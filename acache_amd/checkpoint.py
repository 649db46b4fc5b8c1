"""From the model object a caller of the reference holds to the model the paged engine runs.

The reference's entry points are handed the checkpoint's own model class (llada/eval_ACache.py:100-107, 189 and
dream/eval_ACache.py for the HF path; nano-vdllm's ``ModelRunner(model, config)``, model_runner.py:15-19, for the
engine).  Those classes carry their own attention; the engine needs this package's blocks.  ``engine_model_for``
bridges the two; ``llada.adopt_state`` says which tensors are shared with the checkpoint object and which are
merged copies."""
from __future__ import annotations

import weakref

_ADOPTED = weakref.WeakKeyDictionary()   # checkpoint model object -> the engine model built around its weights


def engine_model_for(model):
    """``model`` itself when it is one of this package's models; for the checkpoint model object the HF path
    passes (llada/eval_ACache.py:100-107, 189; dream/eval_ACache.py likewise), the engine model built around the
    same parameter tensors, made once per object."""
    inner = getattr(model, "model", None)
    if (inner is not None and hasattr(model, "config")
            and any(hasattr(m, "k_cache") and hasattr(m, "probe") for m in model.modules())):
        return model
    try:
        cached = _ADOPTED.get(model)
    except TypeError:        # not weakly referenceable / not hashable: adopt without remembering
        cached = None
    if cached is not None:
        return cached
    cfg = getattr(model, "config", None)
    if cfg is None or not hasattr(model, "state_dict"):
        raise TypeError(
            f"this engine needs an acache_amd model, a ready acache_amd.ModelRunner or a "
            f"LLaDA / Dream checkpoint model object (with .config and .state_dict()), got {type(model).__name__}")
    if hasattr(cfg, "d_model"):
        from .llada import engine_model_from_checkpoint
    elif hasattr(cfg, "hidden_size"):
        from .dream import engine_model_from_checkpoint
    else:
        raise TypeError(f"{type(cfg).__name__} is neither a LLaDA nor a Dream configuration")
    engine = engine_model_from_checkpoint(model)   # TypeError for settings the engine's decoder does not implement
    try:
        _ADOPTED[model] = engine
    except TypeError:
        pass
    return engine
