from . import llama, lufazen, fofapel  # noqa: F401  (register LlamaForCausalLM, Lufazen, Fofapel)
from .decoder import Decoder
