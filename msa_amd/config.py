"""Configuration dataclasses, named and shaped like the reference's (src/config/memory_config.py:6-55
and the msa_config block of the checkpoint's config.json, src/utils/resave_model.py:33-50)."""
from __future__ import annotations

from dataclasses import dataclass, field
from typing import Dict, List, Union

QWEN3_TEMPLATE = {"prompt": "<|im_start|>user\n{prompt}<|im_end|>\n",
                  "response": "<|im_start|>assistant\n<think>\n{think_content}\n</think>\n\n{output}<|im_end|>"}
QWEN3_INSTRUCT_TEMPLATE = {"prompt": "<|im_start|>user\n{prompt}<|im_end|>\n",
                           "response": "<|im_start|>assistant\n{output}<|im_end|>"}
_TEMPLATES = {"QWEN3_TEMPLATE": QWEN3_TEMPLATE, "QWEN3_INSTRUCT_TEMPLATE": QWEN3_INSTRUCT_TEMPLATE}


@dataclass
class GenerateConfig:
    devices: List[int] = None
    template: Union[str, Dict] = None
    max_generate_tokens: int = 256
    max_seq_len: int = 0
    max_query_seq_len: int = 0
    max_batch_size: int = 0
    top_p: float = 0.9
    temperature: float = 0.0
    qa_mode: bool = False

    def __post_init__(self):
        if isinstance(self.template, str):
            if self.template not in _TEMPLATES:
                raise ValueError(f"unknown template {self.template!r}")
            self.template = _TEMPLATES[self.template]
        if self.template is not None and not isinstance(self.template, dict):
            raise TypeError("template must be a dict or a known template name")

    @property
    def world(self) -> int:
        return len(self.devices) if self.devices else 0


@dataclass
class ModelConfig:
    model_path: str = "EverMind-AI/MSA-4B"
    doc_top_k: int = 16
    pooling_kernel_size: int = 64
    router_layer_idx: str = "all"
    template_token_id: int = -2
    template_id_num: int = 3


@dataclass
class MemoryConfig:
    block_size: int = 16000
    slice_chunk_size: int = 16 * 1024
    pooling_kernel_size: int = 64
    memory_file_path: str = ""
    socket_ip: str = ""
    socket_port: int = 0


class DotDict(dict):
    """dict with attribute access (src/msa/configuration_msa.py:6-16)."""
    __setattr__ = dict.__setitem__
    __delattr__ = dict.__delitem__

    def __getattr__(self, name):
        if name.startswith("__"):             # keep copy / pickle protocol lookups honest
            raise AttributeError(name)
        return self.get(name)


def default_msa_config() -> DotDict:
    """The shipped hyper-parameters (scripts/resave_model.sh:2-33)."""
    return DotDict(pooling_kernel_size=64, top_k_docs=16, router_layer_idx=",".join(str(i) for i in range(18, 36)),
                   head_reduce_method="mean", query_reduce_method="max", chunk_reduce_method="max",
                   decouple_pooling_mode="mean", aux_loss_method="INFONCE", decouple_router=True)


@dataclass
class MSAConfig:
    """The Qwen3 fields the layer reads plus ``msa_config`` (src/msa/configuration_msa.py:19-53).
    Defaults are Qwen3-4B's."""
    hidden_size: int = 2560
    num_hidden_layers: int = 36
    num_attention_heads: int = 32
    num_key_value_heads: int = 8
    head_dim: int = 128
    intermediate_size: int = 9728
    vocab_size: int = 151936
    rms_norm_eps: float = 1e-6
    rope_theta: float = 1_000_000.0
    max_position_embeddings: int = 40960
    attention_bias: bool = False
    attention_dropout: float = 0.0
    msa_config: DotDict = field(default_factory=default_msa_config)

    def __post_init__(self):
        if isinstance(self.msa_config, dict) and not isinstance(self.msa_config, DotDict):
            self.msa_config = DotDict(self.msa_config)
