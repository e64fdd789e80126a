"""Boundary dataclasses with the reference's field names.

CacheConfig / RolloutConfig: tunix/common/configs.py:61-121.
SamplerOutput: tunix/generate/base_sampler.py:30-56.
RolloutOutput: tunix/rl/rollout/base_rollout.py:36-67.
"""
import dataclasses
from typing import Any, Optional

import numpy as np


@dataclasses.dataclass(frozen=True)
class CacheConfig:
  cache_size: int
  num_layers: int
  num_kv_heads: int
  head_dim: int


@dataclasses.dataclass
class RolloutConfig:
  max_tokens_to_generate: int = 64
  temperature: float = 0.9
  top_p: Optional[float] = 1.0
  top_k: Optional[int] = None
  seed: Any = None
  max_prompt_length: int = 64
  kv_cache_size: int = 1024
  data_type: Any = None
  eos_tokens: Optional[list] = None
  rollout_mapping_config: Any = None
  tensor_parallel_size: int = -1
  data_parallel_size: int = -1
  expert_parallel_size: int = 1
  return_logprobs: bool = False


@dataclasses.dataclass
class SamplerOutput:
  text: list
  logits: Any
  tokens: Any
  padded_prompt_tokens: np.ndarray
  logprobs: Optional[list]
  routed_experts: Optional[list] = None
  prompt_lengths: Optional[np.ndarray] = None


@dataclasses.dataclass
class RolloutOutput:
  text: list
  logits: Any
  tokens: list
  left_padded_prompt_tokens: np.ndarray
  logprobs: Optional[list]
  routed_experts: Optional[list] = None
  prompt_lengths: Optional[np.ndarray] = None
