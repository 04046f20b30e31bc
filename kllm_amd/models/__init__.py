from . import llama  # registers "LlamaForCausalLM"
from . import nusilix  # registers "Nusilix"

__all__ = ["llama", "nusilix"]
