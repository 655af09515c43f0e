"""Module layout of the reference's Python extension ``pccl.engine_c``
(``csrc/python_api.cc:10-28``): class ``Engine`` and submodule ``utils`` with
``LaunchEnvironments``; here backed by the C ABI of ``libpccl_engine.so``."""
import types

from .engine import Engine, EngineError, LaunchEnvironments  # noqa: F401

utils = types.SimpleNamespace(LaunchEnvironments=LaunchEnvironments)

__all__ = ["Engine", "EngineError", "utils"]
