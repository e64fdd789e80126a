"""MI355X-native decode path for tunix's Sampler running an int4 QLoRA policy."""
__all__ = ['configs', 'quant', 'model', 'sampler', 'rollout', 'checkpoint', 'utils']
