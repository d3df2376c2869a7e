from .flash_attention_impl import get_flash_attention, get_flash_attention_grad

__all__ = ["get_flash_attention", "get_flash_attention_grad"]
