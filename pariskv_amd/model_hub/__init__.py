from .qwen import QwenConfig, QwenLayer, QwenModel  # noqa: F401
