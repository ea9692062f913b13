"""Model families: Llama-3 (8B/70B), Mistral-7B, GPT-2-small, Mupulorn, Goganex (+ tiny test presets)."""
from .config import ARCHITECTURES, ModelConfig, PRESETS, config_from_dir, get_config
from .gpt2 import build_model
