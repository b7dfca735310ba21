"""return_amd: a one-GPU inference engine for MI355X (gfx950), built after the rollout
engine of wenhaoli-xmu/ReTurn for the Qwen3 dense decoder."""
from .config import EngineConfig, load_config, register_architecture
from .sampling import SamplingParams

__all__ = ["EngineConfig", "SamplingParams", "load_config", "register_architecture", "Engine"]


def __getattr__(name):
    if name == "Engine":
        from .engine import Engine
        return Engine
    raise AttributeError(name)
