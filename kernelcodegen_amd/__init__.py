"""MI355X-native kernels behind KernelCodeGen's operator interface.

`ops` holds the device entry points (torch tensors in, HIP kernels underneath,
through the C-ABI of include/kcg.h); `inputs` the deterministic workload
generator.  The C++ mirror of the reference's Frontend / Optimizer / facade
lives in `host/`.
"""
from . import inputs, lib  # noqa: F401

__all__ = ["inputs", "lib", "ops"]


def __getattr__(name):
    if name == "ops":
        import importlib
        return importlib.import_module(".ops", __name__)
    raise AttributeError(name)
