"""Rollout plugin: a drop-in for ``ClusterConfig.rollout_engine`` (a class is
instantiated as engine(rollout_actor=..., tokenizer=..., mesh=..., rollout_config=...),
tunix/rl/rl_cluster.py:388-410).  Mirrors tunix/rl/rollout/base_rollout.py:70-112
(BaseRollout) and tunix/rl/rollout/vanilla_rollout.py:28-106 (VanillaRollout).
"""
import abc
import dataclasses

from tunix_amd.configs import CacheConfig, RolloutConfig, RolloutOutput
from tunix_amd.sampler import Sampler


class BaseRollout(abc.ABC):
  """Same abstract surface as the reference's BaseRollout."""

  @abc.abstractmethod
  def generate(self, prompts, rollout_config, **kwargs):
    ...

  @abc.abstractmethod
  def get_per_token_logps(self, prompt_tokens, completion_tokens):
    ...

  @abc.abstractmethod
  def update_params(self, params, filter_types=None):
    ...

  @abc.abstractmethod
  def pad_id(self):
    ...

  @abc.abstractmethod
  def eos_id(self):
    ...

  @abc.abstractmethod
  def model(self):
    ...


class TmxRollout(BaseRollout):
  """Rollout worker backed by the MI355X Sampler.

  Accepts both construction styles of the reference: positional
  (model, tokenizer, cache_config) like VanillaRollout, or the engine keywords
  (rollout_actor, tokenizer, mesh, rollout_config) of a user-defined engine
  (tunix/rl/rl_cluster.py:388-410 hands over the nnx actor itself).  The actor may be a
  QLoRAModel, a (reference ModelConfig, state tree) pair, or the reference's LoRA-wrapped nnx
  module (needs flax importable to read its state); the latter two are quantised here, once,
  with `group` / `lora_alpha` / `quant_bound` (bind them with functools.partial).
  """

  @staticmethod
  def _as_policy(actor, group, lora_alpha, quant_bound):
    from tunix_amd.model import ModelConfig, QLoRAModel
    if isinstance(actor, QLoRAModel) or isinstance(getattr(actor, 'config', None), ModelConfig):
      return actor  # already a policy of this package (its config is this package's ModelConfig)
    if isinstance(actor, tuple) and len(actor) == 2:
      cfg, tree = actor
    elif hasattr(actor, 'config'):
      try:
        from flax import nnx
      except ImportError as e:
        raise TypeError('rollout_actor is an nnx module but flax is not importable to read its state: pass a '
                        'QLoRAModel (QLoRAModel.from_state_tree) or a (config, state tree) pair') from e
      cfg, tree = actor.config, nnx.state(actor)
    else:
      raise TypeError(f'rollout_actor of type {type(actor).__name__}: expected a QLoRAModel, a (config, state tree) '
                      'pair or an nnx module with .config')
    if not isinstance(cfg, ModelConfig):
      cfg = ModelConfig.from_reference(cfg)
    return QLoRAModel.from_state_tree(cfg, tree, group=group, lora_alpha=0.0 if lora_alpha is None else lora_alpha,
                                      bound=quant_bound)

  def __init__(self, model=None, tokenizer=None, cache_config_or_size=None, *, rollout_actor=None,
               mesh=None, rollout_config: RolloutConfig = None, group=64, lora_alpha=None, quant_bound=7.5):
    del mesh  # one GPU: nothing to shard
    actor = model if model is not None else rollout_actor
    if actor is None or tokenizer is None:
      raise ValueError('a model (rollout_actor) and a tokenizer are required')
    actor = self._as_policy(actor, group, lora_alpha, quant_bound)
    if cache_config_or_size is None:
      if rollout_config is None:
        raise ValueError('either cache_config_or_size or rollout_config is required')
      c = actor.config
      cache_config_or_size = CacheConfig(rollout_config.kv_cache_size, c.num_layers,
                                         c.num_kv_heads, c.head_dim)
    self._sampler = Sampler(actor, tokenizer, CacheConfig(**dataclasses.asdict(cache_config_or_size)))

  def generate(self, prompts, rollout_config, *, prompt_token_ids=None, **kwargs):
    out = self._sampler(
        input_strings=prompts,
        max_generation_steps=rollout_config.max_tokens_to_generate,
        max_prompt_length=rollout_config.max_prompt_length,
        echo=False,
        temperature=rollout_config.temperature,
        top_p=rollout_config.top_p,
        top_k=rollout_config.top_k,
        seed=rollout_config.seed,
        pad_output=False,
        eos_tokens=rollout_config.eos_tokens,
        return_logprobs=rollout_config.return_logprobs,
        prompt_token_ids=prompt_token_ids,
    )
    return RolloutOutput(
        text=out.text, logits=out.logits, tokens=out.tokens,
        left_padded_prompt_tokens=out.padded_prompt_tokens, logprobs=out.logprobs,
        prompt_lengths=out.prompt_lengths)

  def get_per_token_logps(self, prompt_tokens, completion_tokens):
    """vanilla_rollout.py:75-88: compute_per_token_logps with this rollout's pad id."""
    return self._sampler.per_token_logps(prompt_tokens, completion_tokens, pad_id=self.pad_id())

  def update_params(self, params, filter_types=None):
    self._sampler.update_params(params, filter_types)

  def pad_id(self):
    return self._sampler.tokenizer.pad_id()

  def eos_id(self):
    return self._sampler.tokenizer.eos_id()

  def model(self):
    return self._sampler.transformer
