from .kitty_attention import kitty_attention_forward, kitty_prefill_attention
from .kitty_quant_pack import quantize_pack_k, quantize_pack_v, select_boost_k

__all__ = ["kitty_attention_forward", "kitty_prefill_attention", "quantize_pack_k", "quantize_pack_v", "select_boost_k"]
