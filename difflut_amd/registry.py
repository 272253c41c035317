"""Name -> component registry with the reference's API (difflut/registry.py:11-458):
REGISTRY.register_*/get_*/list_*/build_* for nodes, layers, convolutional layers, encoders,
initializers and regularizers, plus the module-level decorator aliases."""
import warnings

_KINDS = {  # attribute suffix -> (plural used by list_*, label used in messages)
    "node": ("nodes", "Node"),
    "layer": ("layers", "Layer"),
    "convolutional_layer": ("convolutional_layers", "Convolutional layer"),
    "encoder": ("encoders", "Encoder"),
    "initializer": ("initializers", "Initializer"),
    "regularizer": ("regularizers", "Regularizer"),
}


class Registry:
    def __init__(self):
        self._tables = {kind: {} for kind in _KINDS}

    # one implementation, exposed under the per-kind method names below
    def _register(self, kind, name=None):
        table, label = self._tables[kind], _KINDS[kind][1]

        def decorator(obj):
            key = name if name is not None else obj.__name__
            if key in table:
                warnings.warn(f"{label} '{key}' is already registered and will be overwritten.", UserWarning,
                              stacklevel=2)
            table[key] = obj
            return obj

        return decorator

    def _get(self, kind, name):
        table, (plural, label) = self._tables[kind], _KINDS[kind]
        if name not in table:
            raise ValueError(f"{label} '{name}' not found. Available {plural}: {list(table.keys())}")
        return table[name]

    def list_all(self):
        return {plural: list(self._tables[kind].keys()) for kind, (plural, _) in _KINDS.items()}

    def __repr__(self):
        body = ",\n".join(f"  {plural}={len(self._tables[kind])}" for kind, (plural, _) in _KINDS.items())
        return f"Registry(\n{body}\n)"


def _install(kind, plural):
    setattr(Registry, f"register_{kind}", lambda self, name=None: self._register(kind, name))
    setattr(Registry, f"get_{kind}", lambda self, name: self._get(kind, name))
    setattr(Registry, f"list_{plural}", lambda self: list(self._tables[kind].keys()))
    if kind not in ("initializer", "regularizer"):
        setattr(Registry, f"build_{kind}", lambda self, name, **kwargs: self._get(kind, name)(**kwargs))


for _kind, (_plural, _) in _KINDS.items():
    _install(_kind, _plural)

REGISTRY = Registry()
register_node = REGISTRY.register_node
register_layer = REGISTRY.register_layer
register_convolutional_layer = REGISTRY.register_convolutional_layer
register_encoder = REGISTRY.register_encoder
register_initializer = REGISTRY.register_initializer
register_regularizer = REGISTRY.register_regularizer
