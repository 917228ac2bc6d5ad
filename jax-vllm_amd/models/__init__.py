from . import qwen3  # noqa: F401  (registers Qwen3ForCausalLM)
