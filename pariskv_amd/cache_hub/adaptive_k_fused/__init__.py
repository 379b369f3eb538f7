from .adaptive_topk import adaptive_topk_cuda  # noqa: F401
