"""MI355X (gfx950) execution path for HTR-W1 packed linears.

    from htr_amd import ops
    y = ops.linear(x, qweight, scales, su, sv, bias)      # same call as htr.ops.linear of the reference
"""
from . import wire  # noqa: F401

__all__ = ["wire", "ops"]


def __getattr__(name):
    if name == "ops":
        import importlib
        return importlib.import_module(".ops", __name__)
    raise AttributeError(name)
