"""Name -> graph-builder registry (reference: python/mirage/mpk/model_registry.py)."""
_MODEL_BUILDERS = {}


def register_model_builder(*names):
    """Class decorator: register a builder under one or several model names."""
    flat = list(names[0]) if len(names) == 1 and isinstance(names[0], (list, tuple, set)) else list(names)

    def decorator(cls):
        for n in flat:
            _MODEL_BUILDERS[n] = cls
        return cls

    return decorator


def get_builder(name: str):
    builder = _MODEL_BUILDERS.get(name)
    if builder is None:
        raise ValueError(f"Unknown builder: {name}. Registered: {list(_MODEL_BUILDERS.keys())}")
    return builder
