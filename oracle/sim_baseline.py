"""CPU baseline: the reference's CPU-capable "dequantize-then-attend" path.  TEST/BENCH INFRASTRUCTURE.

A PyTorch restatement of the reference's fake-quant simulator and eager attention, used only as the
timed ``cpu_baseline`` of ``bench.py`` (and nowhere in the product):

* ``fake_quant_groupwise_lastdim`` / ``build_promote_mask`` follow src/kitty_sim/utils_quant.py:64-114
  and :12-61 (magnitude-based selection, clamp-then-round-half-even, range floored at 1e-4 for fp16);
* the prefill schedule follows src/kitty_sim/kitty_simulate.py:196-215 (K in 128-token groups from
  the sink on, V per token for all but the newest 128 tokens);
* ``eager_attention`` follows src/kitty/models/qwen3/modeling_qwen3.py:132-167 (repeat_kv, matmul,
  fp32 softmax, matmul).

Its numerics differ from the packed path on purpose (different epsilon, rounding and boost count
in the reference itself); it is a speed baseline, not a parity oracle - "parity unpinned".
"""
import torch


def build_promote_mask(key_states: torch.Tensor, promote_ratio: float) -> torch.Tensor:
    B, nh, D, _ = key_states.shape
    k_chan = max(0, min(int(D * promote_ratio + 1e-6), D))
    mask = torch.zeros((B, nh, D), dtype=torch.bool)
    if k_chan == 0:
        return mask
    score = key_states.abs().mean(dim=-1)
    _, top = score.topk(k_chan, dim=-1)
    mask.scatter_(-1, top, True)
    return mask


def fake_quant_groupwise_lastdim(data, group_size, bit, promote_mask=None, promote_bit=4):
    B, nh, D, T = data.shape
    assert T % group_size == 0
    G = T // group_size
    x = data.contiguous().view(B, nh, D, G, group_size)
    mn = x.min(dim=-1, keepdim=True).values
    mx = x.max(dim=-1, keepdim=True).values
    eps = 1e-4 if data.dtype in (torch.float16, torch.bfloat16) else 1e-6
    rng = (mx - mn).clamp(min=eps)
    if promote_mask is not None:
        pm = promote_mask.view(B, nh, D, 1, 1)
        scale = torch.where(pm, rng / (2 ** promote_bit - 1), rng / (2 ** bit - 1))
        max_val = torch.where(pm, torch.full_like(scale, 2 ** promote_bit - 1), torch.full_like(scale, 2 ** bit - 1))
    else:
        scale = rng / (2 ** bit - 1)
        max_val = torch.full_like(scale, 2 ** bit - 1)
    q = ((x - mn) / scale).clamp(torch.zeros_like(max_val), max_val).round()
    return (q * scale + mn).view(B, nh, D, T).to(data.dtype)


def simulate_prefill(K, V, sink=32, buf=128, group=128, kbits=2, vbits=2, promote_ratio=0.25, promote_bit=4):
    """In-place fake quantization of dense fp16 K, V [B, H, T, D] as the simulator's prefill does."""
    T = K.shape[-2]
    if T > sink + buf:
        n = T - sink
        end = sink + (n - n % buf)
        for i in range(sink, end, buf):
            ks = K[:, :, i:i + buf, :].transpose(2, 3).contiguous()
            pm = build_promote_mask(ks, promote_ratio)
            K[:, :, i:i + buf, :] = fake_quant_groupwise_lastdim(ks, group, kbits, pm, promote_bit).transpose(2, 3)
        vend = sink + (n - buf)
        V[:, :, sink:vend, :] = fake_quant_groupwise_lastdim(V[:, :, sink:vend, :], group, vbits)
    return K, V


def eager_attention(query, key, value, scaling, n_rep):
    """query [B, H_Q, 1, D]; key/value [B, H_KV, T, D] -> [B, 1, H_Q, D]."""
    B, H, T, D = key.shape
    key = key[:, :, None].expand(B, H, n_rep, T, D).reshape(B, H * n_rep, T, D)
    value = value[:, :, None].expand(B, H, n_rep, T, D).reshape(B, H * n_rep, T, D)
    w = torch.matmul(query, key.transpose(2, 3)) * scaling
    w = torch.nn.functional.softmax(w, dim=-1, dtype=torch.float32).to(query.dtype)
    return torch.matmul(w, value).transpose(1, 2).contiguous()
