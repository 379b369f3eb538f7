from .trans_h2d import h2d_gather_kv  # noqa: F401
