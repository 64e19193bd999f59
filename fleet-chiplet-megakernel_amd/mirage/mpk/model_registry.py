"""Which graph-builder class serves which model name (reference: python/mirage/mpk/model_registry.py)."""
_MODEL_BUILDERS = {}


def register_model_builder(*names):
    """Class decorator.  Takes the model names one by one or as a single list / tuple / set of them."""
    if len(names) == 1 and not isinstance(names[0], str):
        names = tuple(names[0])

    def bind(builder_cls):
        _MODEL_BUILDERS.update(dict.fromkeys(names, builder_cls))
        return builder_cls

    return bind


def get_builder(name: str):
    try:
        return _MODEL_BUILDERS[name]
    except KeyError:
        raise ValueError(f"no graph builder is registered for model {name!r} (known: {sorted(_MODEL_BUILDERS)})") from None
