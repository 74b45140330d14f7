from . import qwen3  # noqa: F401  (registers Qwen3ForCausalLM)
from . import visadra  # noqa: F401  (registers Visadra)
from . import kezasun  # noqa: F401  (registers Kezasun)
from . import malilorn  # noqa: F401  (registers Malilorn)
from . import birelix  # noqa: F401  (registers Birelix)
from .build import expected_tensors, load_model, make_context, parse_dtype, random_model
from .decoder import DecoderLM, PlanEntry

__all__ = ["DecoderLM", "PlanEntry", "expected_tensors", "load_model", "make_context", "parse_dtype", "random_model"]
