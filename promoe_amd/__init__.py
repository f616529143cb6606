"""MI355X-native MoE layer engine with the promoe (sparse_llm_cache) cache boundary."""
from . import layout  # noqa: F401

__all__ = ["layout"]
