from . import llama  # noqa: F401  (registers LlamaForCausalLM)
from . import zifelorn  # noqa: F401  (registers Zifelorn)
from .decoder import Decoder
from .llama import build_llama
from .zifelorn import build_zifelorn
