"""MI355X (gfx950) int8-KV dynamic-batching attention path, pmx-compatible.

The directory name carries dots, so it is loaded by path (see
``__graft_entry__.load_package``) under the module name ``pmx_amd``.

    ops        host-side mirror of the operator interface over the C ABI
    harness    device-side set-up of a synthetic batch (cache pool, index arrays)
    workloads  the benchmark configurations (numpy only)
    build      compiles libpmx_hip.so from csrc/
"""
from . import workloads  # noqa: F401  (numpy only; safe without the library)

__all__ = ["workloads", "ops", "harness", "build"]


def __getattr__(name):
    # ops / harness need torch and the built library: import them on first use
    if name in ("ops", "harness", "build", "_lib"):
        import importlib
        return importlib.import_module("." + name, __name__)
    raise AttributeError(name)
