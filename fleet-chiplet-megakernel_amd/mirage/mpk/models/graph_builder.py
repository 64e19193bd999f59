"""What a model hands to its graph builder (reference: python/mirage/mpk/models/graph_builder.py:8-51)."""
import abc
from dataclasses import dataclass
from typing import Any, Dict, List, Optional, Tuple

import torch


@dataclass
class MirageModelConfig:
    # model architecture
    hidden_size: int = None
    intermediate_size: int = None
    vocab_size: int = None
    local_num_q_heads: int = None
    local_num_kv_heads: int = None
    head_dim: int = None
    num_layers: int = None
    # kv cache: per layer [max_num_pages, page_size, kv_heads, head_dim] (a list, or one tensor with a leading layer dimension)
    k_cache: List[torch.Tensor] = None
    v_cache: List[torch.Tensor] = None
    # position embeddings (cos, sin), each [1, positions, head_dim] as the library's rotary module returns them
    position_embeddings: Tuple[torch.Tensor, torch.Tensor] = None
    # model weights under the checkpoint's names ("model.layers.0.self_attn.q_proj.weight", ...)
    state_dict: Optional[dict] = None
    with_lm_head: bool = True

    def info_as_string(self):
        fields = [("Hidden size", self.hidden_size), ("Intermediate size", self.intermediate_size), ("Vocab size", self.vocab_size),
                  ("Num q heads", self.local_num_q_heads), ("Num kv heads", self.local_num_kv_heads), ("Head dim", self.head_dim),
                  ("Num layers", self.num_layers),
                  ("K cache [0]", None if self.k_cache is None else tuple(self.k_cache[0].shape)),
                  ("V cache [0]", None if self.v_cache is None else tuple(self.v_cache[0].shape)),
                  ("Position embeddings cos", None if self.position_embeddings is None else tuple(self.position_embeddings[0].shape)),
                  ("Position embeddings sin", None if self.position_embeddings is None else tuple(self.position_embeddings[1].shape)),
                  ("State dict len", 0 if self.state_dict is None else len(self.state_dict))]
        return "".join(f"{k}: {v}\n" for k, v in fields) + "-------------------------------------------\n"


class GraphBuilder(abc.ABC):
    def __init__(self, mpk, weights: Optional[Dict[str, Any]] = None):
        self.mpk = mpk
        self.weights = weights or {}

    @abc.abstractmethod
    def build_from_model(self, model_name: str = None, model_path: str = None):
        raise NotImplementedError("build_from_model is not implemented")
