from . import llama, lufazen, fofapel, gesutar, vevapel  # noqa: F401  (register LlamaForCausalLM, Lufazen, Fofapel, Gesutar, Vevapel)
from .decoder import Decoder
