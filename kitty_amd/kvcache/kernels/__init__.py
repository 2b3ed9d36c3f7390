from .kitty_attention import kitty_attention_forward
from .kitty_quant_pack import quantize_pack_k, quantize_pack_v, select_boost_k

__all__ = ["kitty_attention_forward", "quantize_pack_k", "quantize_pack_v", "select_boost_k"]
