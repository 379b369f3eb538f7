from .collison_interface import update_cache_cnt_cuda_interface, load_kernel_module  # noqa: F401
