from . import llama  # registers "LlamaForCausalLM"
from . import nusilix  # registers "Nusilix"
from . import ribovik  # registers "Ribovik"

__all__ = ["llama", "nusilix", "ribovik"]
