"""Model definitions (Llama-3 / Mixtral / GPT-2, layer-list hybrids) and architecture presets."""
from .config import PRESETS, ModelConfig, get_config  # noqa: F401
from .llama import AttnMeta, CausalLM  # noqa: F401
from .checkpoint import config_from_hf, load_checkpoint, save_checkpoint  # noqa: F401
from .hybrid import HybridLM  # noqa: F401
from .registry import MODEL_CLASSES, build_model, config_from_dir  # noqa: F401
