"""Engine factory.

Contract of the reference (umbrella/speculation/auto_engine.py:12-22) kept verbatim:
``AutoEngine.from_config(device, engine="static"|"dynamic", model=<target>, draft_model=<draft>, **engine_kwargs)``
returns a constructed (not yet initialised) engine; an unknown engine raises ``ValueError``, a missing model name
fails an ``assert``.  ``_ENGINE_MAPPING`` stays a plain dict so callers can register their own engines.
``engine="batch"`` is the autoregressive batch engine of the sequence-mixer models (no draft model: ``draft_model`` may
be left out for engines whose class says ``NEEDS_DRAFT = False``)."""
from .batch_engine import BatchEngine as _Batch
from .dynamic_speculation_engine import DynamicSpeculationEngine as _Dynamic
from .static_speculation_engine import StaticSpeculationEngine as _Static


def _pop_required(config: dict, key: str):
    value = config.pop(key, None)
    assert value is not None, f"engine config lacks '{key}'"
    return value


class AutoEngine:
    _ENGINE_MAPPING = {"static": _Static, "dynamic": _Dynamic, "batch": _Batch}

    @classmethod
    def from_config(cls, device: str, **config):
        kind = config.pop("engine", "dynamic")
        engine_cls = cls._ENGINE_MAPPING.get(kind)
        if engine_cls is None:
            raise ValueError(f"Engine type '{kind}' is not supported. Supported types: {sorted(cls._ENGINE_MAPPING)}")
        if getattr(engine_cls, "NEEDS_DRAFT", True):
            draft = _pop_required(config, "draft_model")
        else:
            draft = config.pop("draft_model", None)
        target = _pop_required(config, "model")
        return engine_cls(draft, target, device=device, **config)
