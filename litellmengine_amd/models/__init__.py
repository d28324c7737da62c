from . import qwen3  # noqa: F401  (registers Qwen3ForCausalLM)
from .build import expected_tensors, load_model, make_context, parse_dtype, random_model
from .decoder import DecoderLM, PlanEntry

__all__ = ["DecoderLM", "PlanEntry", "expected_tensors", "load_model", "make_context", "parse_dtype", "random_model"]
