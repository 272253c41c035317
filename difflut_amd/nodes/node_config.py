"""Typed carrier of node constructor arguments (difflut/nodes/node_config.py:13-158)."""
from dataclasses import dataclass, field
from typing import Any, Callable, Dict, Optional


@dataclass
class NodeConfig:
    input_dim: Optional[int] = None
    output_dim: Optional[int] = None
    regularizers: Optional[Dict[str, Any]] = None
    init_fn: Optional[Callable] = None
    init_kwargs: Optional[Dict[str, Any]] = None
    extra_params: Dict[str, Any] = field(default_factory=dict)  # node-specific keyword arguments

    def __post_init__(self):
        self.regularizers = {} if self.regularizers is None else self.regularizers
        self.init_kwargs = {} if self.init_kwargs is None else self.init_kwargs

    def to_dict(self):
        """Keyword arguments for the node constructor: set fields only, then extra_params."""
        out = {}
        for name in ("input_dim", "output_dim"):
            if getattr(self, name) is not None:
                out[name] = getattr(self, name)
        if self.regularizers:
            out["regularizers"] = self.regularizers
        if self.init_fn is not None:
            out["init_fn"] = self.init_fn
        if self.init_kwargs:
            out["init_kwargs"] = self.init_kwargs
        out.update(self.extra_params)
        return out

    def copy(self):
        return NodeConfig(self.input_dim, self.output_dim, dict(self.regularizers) or None, self.init_fn,
                          dict(self.init_kwargs) or None, dict(self.extra_params))

    def __repr__(self):
        parts = [f"{n}={getattr(self, n)}" for n in ("input_dim", "output_dim") if getattr(self, n) is not None]
        if self.init_fn is not None:
            parts.append(f"init_fn={self.init_fn.__name__}")
        parts += [f"{k}={v}" for k, v in self.extra_params.items()]
        return f"NodeConfig({', '.join(parts)})"
