from .compressed_tensors_utils import modify_save_pretrained

__all__ = ["modify_save_pretrained"]
