from . import llama, lufazen  # noqa: F401  (register LlamaForCausalLM, Lufazen)
from .decoder import Decoder
