"""Import name of the library whose sources live in the folder ``palm-infra_amd/`` beside this one.

A folder name with a hyphen cannot be imported, so this package only points its search path at that
folder: ``palm_infra_amd.config`` is ``palm-infra_amd/config`` and so on.
"""
import os as _os

_SOURCE_ROOT = _os.path.join(_os.path.dirname(_os.path.dirname(_os.path.abspath(__file__))), "palm-infra_amd")
if not _os.path.isdir(_SOURCE_ROOT):  # pragma: no cover - a broken checkout
    raise ImportError(f"palm_infra_amd: source folder not found: {_SOURCE_ROOT}")
__path__.insert(0, _SOURCE_ROOT)

__version__ = "0.1.0"


def load(model_dir, dtype="bfloat16", max_tokens=None, device="cuda:0", **options):
    """Load a model folder (config.json + model.safetensors) and return an engine ready to step and
    generate.  See ``palm_infra_amd.engine.Engine``."""
    from palm_infra_amd.engine import Engine
    return Engine.from_dir(model_dir, dtype=dtype, max_tokens=max_tokens, device=device, **options)
