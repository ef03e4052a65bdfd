from . import llama  # noqa: F401  (registers LlamaForCausalLM)
from . import zifelorn  # noqa: F401  (registers Zifelorn)
from . import vezodra  # noqa: F401  (registers Vezodra)
from . import mutusun  # noqa: F401  (registers Mutusun)
from . import labirax  # noqa: F401  (registers Labirax)
from .decoder import Decoder
from .llama import build_llama
from .zifelorn import build_zifelorn
from .vezodra import build_vezodra
from .mutusun import build_mutusun
from .labirax import build_labirax
