from .config import ModelConfig, get_config, list_models, from_hf_config
from .base import AttnMeta
from .llama import LlamaForCausalLM
from .gpt2 import GPT2ForCausalLM
from .dofivik import DofivikForCausalLM
from .loluzen import LoluzenForCausalLM
from .lotelix import LotelixForCausalLM
from .vizonex import VizonexForCausalLM
from .loader import build_model, load_checkpoint, save_checkpoint

__all__ = ["ModelConfig", "get_config", "list_models", "from_hf_config", "AttnMeta", "LlamaForCausalLM",
           "GPT2ForCausalLM", "DofivikForCausalLM", "VizonexForCausalLM", "LoluzenForCausalLM", "LotelixForCausalLM", "build_model", "load_checkpoint", "save_checkpoint"]
