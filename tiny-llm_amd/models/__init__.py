from . import llama, lufazen, fofapel, gesutar  # noqa: F401  (register LlamaForCausalLM, Lufazen, Fofapel, Gesutar)
from .decoder import Decoder
