from . import gpt2  # noqa: F401  (registers GPT2LMHeadModel)
from . import virudra  # noqa: F401  (registers Virudra)
from . import pedatar  # noqa: F401  (registers Pedatar)
from . import pafolorn  # noqa: F401  (registers Pafolorn)
from . import salivik  # noqa: F401  (registers Salivik)
from .causal_lm import CausalLM, load_model

__all__ = ["CausalLM", "load_model"]
