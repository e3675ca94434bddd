from . import llama  # noqa: F401  (registers LlamaForCausalLM)
from .decoder import Decoder
from .llama import build_llama
