"""A small, whole Llama inference engine for one MI355X."""

from tokasaurus_amd.config import EngineConfig  # noqa: F401
from tokasaurus_amd.sampling import SamplingParams  # noqa: F401


def __getattr__(name: str):
    if name in ("Engine", "Completion"):
        from tokasaurus_amd.engine import engine

        return getattr(engine, name)
    raise AttributeError(name)
