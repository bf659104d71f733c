"""One registry from the architecture name in config.json to everything that builds
its model: the typed configuration, the layer plan and the checkpoint's tensor names.

The reference accepts exactly one name through a constant (atomserve/config.py:11,
34-38); here the same check is a table lookup, so another architecture is one more
`register_architecture` call and no change elsewhere.
"""

import json
import os
from dataclasses import dataclass
from typing import Any, Callable

from atomserve_amd.config.model_config import ConfigError


@dataclass(frozen=True)
class Architecture:
    """name:           the string in config.json's `architectures`
    parse_config:   raw config.json dict -> typed configuration (validates)
    build_plan:     typed configuration -> parts.plan.ModelPlan (layers as data)
    checkpoint_map: typed configuration -> {plan tensor name: [checkpoint names to stack]}
    checkpoint_shapes: typed configuration -> {checkpoint name: (shape, role)}, in the order in which
                    random weights are drawn; roles: "matrix", "vector" (gains around 1), "bias" and
                    "log_rate" (small values around 0), "near_identity" (a square matrix around the
                    identity), "fraction" (values between 0 and 1), "depth_weights" (mostly on the last entry), "expert_table:<experts>" (int32 rows of distinct expert numbers)
    ignored:        typed configuration -> checkpoint names that may be present and unused
    complete:       (typed configuration, shape_of) -> the configuration with the sizes that config.json leaves to
                    the tensors' shapes (shape_of(checkpoint name) -> shape, or None for a name the folder lacks);
                    None: config.json tells every size
    """

    name: str
    parse_config: Callable[[dict], Any]
    build_plan: Callable[[Any], Any]
    checkpoint_map: Callable[[Any], dict]
    checkpoint_shapes: Callable[[Any], dict]
    ignored: Callable[[Any], set] = lambda config: set()
    complete: Any = None


_ARCHITECTURES: dict[str, Architecture] = {}


def register_architecture(arch: Architecture, replace: bool = False) -> Architecture:
    if arch.name in _ARCHITECTURES and not replace:
        raise ValueError(f"architecture {arch.name!r} is already registered")
    _ARCHITECTURES[arch.name] = arch
    return arch


def supported_architectures() -> list[str]:
    _load_builtin()
    return sorted(_ARCHITECTURES)


def architecture_for(raw: dict) -> Architecture:
    """The registered architecture that config.json names, or a ConfigError listing what is."""
    _load_builtin()
    names = raw.get("architectures") or []
    if not names and isinstance(raw.get("architecture"), str):  # some configurations name theirs in the singular
        names = [raw["architecture"]]
    if len(names) != 1 or names[0] not in _ARCHITECTURES:
        raise ConfigError(
            f"atomserve_amd only supports {', '.join(sorted(_ARCHITECTURES))}; "
            f"config.json names {names}"
        )
    return _ARCHITECTURES[names[0]]


def load_model_config(model_dir: str) -> tuple[Architecture, Any]:
    """Read `<model_dir>/config.json`; returns (architecture, typed configuration)."""
    path = os.path.join(model_dir, "config.json")
    if not os.path.isfile(path):
        raise FileNotFoundError(f"no config.json in {model_dir}")
    with open(path) as f:
        raw = json.load(f)
    arch = architecture_for(raw)
    config = arch.parse_config(raw)
    if arch.complete is not None:
        from atomserve_amd.weights.loader import checkpoint_shapes_of

        config = arch.complete(config, checkpoint_shapes_of(model_dir))
    return arch, config


def _load_builtin() -> None:
    # Imported lazily: the model modules import parts, which import this package.
    import atomserve_amd.models.dozusun  # noqa: F401
    import atomserve_amd.models.koravik  # noqa: F401
    import atomserve_amd.models.mumizen  # noqa: F401
    import atomserve_amd.models.natatar  # noqa: F401
    import atomserve_amd.models.qwen3  # noqa: F401
