from . import llama  # noqa: F401  (registers LlamaForCausalLM)
from . import zifelorn  # noqa: F401  (registers Zifelorn)
from . import vezodra  # noqa: F401  (registers Vezodra)
from .decoder import Decoder
from .llama import build_llama
from .zifelorn import build_zifelorn
from .vezodra import build_vezodra
