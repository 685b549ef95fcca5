"""Architecture name -> model class (reference: nanovllm/models/models_map.py).
The decoder families of the reference that share the paged-KV decode path: Qwen3 / Qwen2 (one class,
qwen3.py:70-72 switches between q/k norm and qkv bias), Llama (models/llama.py) and Qwen3-MoE
(models/qwen3_moe.py).  MiniCPM and Qwen3-VL are outside this package's scope."""
from nanovllm.models.felolorn import FelolornConfig, FelolornForCausalLM
from nanovllm.models.gazutar import GazutarConfig, GazutarForCausalLM
from nanovllm.models.llama import LlamaForCausalLM
from nanovllm.models.qwen3 import Qwen3ForCausalLM
from nanovllm.models.qwen3_moe import Qwen3MoeForCausalLM
from nanovllm.models.sanevik import SanevikConfig, SanevikForCausalLM
from nanovllm.models.zedirax import ZediraxConfig, ZediraxForCausalLM

model_dict = {
    "Qwen3ForCausalLM": Qwen3ForCausalLM,
    "Qwen2ForCausalLM": Qwen3ForCausalLM,
    "LlamaForCausalLM": LlamaForCausalLM,
    "Qwen3MoeForCausalLM": Qwen3MoeForCausalLM,
    "Gazutar": GazutarForCausalLM,
    "Zedirax": ZediraxForCausalLM,
    "Felolorn": FelolornForCausalLM,
    "Sanevik": SanevikForCausalLM,
}

# designs whose config.json is not a transformers configuration: {"architecture": <name>, ...} -> the reader of it
native_configs = {
    "Gazutar": GazutarConfig,
    "Zedirax": ZediraxConfig,
    "Felolorn": FelolornConfig,
    "Sanevik": SanevikConfig,
}


def native_config(model_dir: str, dtype: str = "bfloat16"):
    """The configuration object of a native design, or None when config.json is a transformers one."""
    import json
    import os

    with open(os.path.join(model_dir, "config.json")) as f:
        raw = json.load(f)
    reader = native_configs.get(raw.get("architecture")) if isinstance(raw, dict) else None
    return reader.from_dir(model_dir, dtype) if reader is not None else None
