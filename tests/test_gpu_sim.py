"""GPU parity of the accuracy simulator (kitty_amd/sim.py, kernel kitty_fake_quant) with its CPU
oracle (oracle/sim_oracle.py; reference: src/kitty_sim/utils_quant.py, kitty_simulate.py:170-252)
and with the reference's operator chain evaluated by torch on the same device.  Bit-exact."""
import numpy as np
import pytest
import torch

from oracle import sim_baseline as SB
from oracle import sim_oracle as SO

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def S():
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    from kitty_amd import _lib, sim
    _lib.lib()                                   # raises if the HIP library is not built
    return sim


def _kv(shape, seed, student_t=False):
    g = np.random.default_rng(seed)
    x = (g.standard_t(3, shape) if student_t else g.standard_normal(shape)).astype(np.float32)
    x[..., [5, 77]] *= 10.0                   # outlier channels
    return x.astype(np.float16)


def _bits(t):
    return t.detach().cpu().numpy().view(np.uint16)


@pytest.mark.parametrize("group", [32, 64, 128])
@pytest.mark.parametrize("bit,pbit", [(2, 4), (1, 2), (3, 8), (4, 4), (8, 8)])
def test_keys_in_place_bit_exact(S, group, bit, pbit):
    """Groups along the tokens with one promote mask per 128-token block, on a token range inside
    a larger strided tensor; everything outside the range stays as it was."""
    B, H, T, lo, n = 2, 3, 700, 32, 128 * 4 + (group if group < 128 else 0)
    x = _kv((B, H, T, 128), seed=bit * 10 + group, student_t=(bit == 3))
    tiles = -(-n // 128)
    mask = np.random.default_rng(1).random((B, H, tiles, 128)) < 0.2
    want = x.copy()
    for i in range(tiles):
        hi = min(lo + 128 * (i + 1), lo + n)
        ks = np.ascontiguousarray(x[:, :, lo + 128 * i:hi].transpose(0, 1, 3, 2))
        want[:, :, lo + 128 * i:hi] = SO.fake_quant_groupwise_lastdim(ks, group, bit, mask[:, :, i], pbit).transpose(0, 1, 3, 2)
    big = torch.zeros((B, H, T + 9, 128 + 64), dtype=torch.float16, device="cuda")[:, :, :T, :128]
    big.copy_(torch.from_numpy(x))
    assert S.fake_quant_tokens_(big, lo, n, 0, group, bit, torch.from_numpy(mask).cuda(), pbit) is big
    assert np.array_equal(_bits(big.contiguous()), want.view(np.uint16))
    assert not np.array_equal(want[:, :, lo:lo + n], x[:, :, lo:lo + n])


@pytest.mark.parametrize("group", [32, 64, 128])
@pytest.mark.parametrize("bit", [1, 2, 4, 8])
def test_values_in_place_bit_exact(S, group, bit):
    B, H, T, lo, n = 2, 2, 500, 32, 333                  # any number of tokens
    x = _kv((B, H, T, 128), seed=bit + group)
    x[0, 0, 40] = 0.25                                    # a constant row
    want = x.copy()
    want[:, :, lo:lo + n] = SO.fake_quant_groupwise_lastdim(x[:, :, lo:lo + n], group, bit)
    t = torch.from_numpy(x).cuda()
    S.fake_quant_tokens_(t, lo, n, 1, group, bit)
    assert np.array_equal(_bits(t), want.view(np.uint16))


def test_reference_signature_equals_torch_operators_on_the_device(S):
    """The reference's chain, operator by operator, run by torch on the same GPU: what the
    reference computes there.  A million elements per case, so that a difference in the rounding of
    the divisions would show."""
    g = torch.Generator(device="cuda").manual_seed(11)
    for bit, pbit, group in ((2, 4, 128), (2, 4, 32), (4, 8, 64), (3, 4, 128)):
        k = torch.randn((4, 8, 256, 128), generator=g, device="cuda").mul_(1.7).half()      # [B, nh, T, D]
        kt = k.transpose(2, 3)                                                                 # the reference's key layout
        mask = S.build_promote_mask(kt, 0.2, 1)
        assert mask.shape == (4, 8, 128) and int(mask.sum()) == 4 * 8 * 25
        got = S.fake_quant_groupwise_lastdim(kt, group, bit, mask, pbit)
        want = SB.fake_quant_groupwise_lastdim(kt.contiguous(), group, bit, mask, pbit)
        assert got.shape == want.shape and torch.equal(got.contiguous().view(torch.int16), want.view(torch.int16)), (bit, group)
        assert torch.equal(kt, k.transpose(2, 3))                                             # out of place
        v = torch.randn((4, 8, 256, 128), generator=g, device="cuda").half()
        got = S.fake_quant_groupwise_lastdim(v, group, bit)
        want = SB.fake_quant_groupwise_lastdim(v, group, bit)
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), (bit, group)
    assert S.fake_quant_groupwise_lastdim(v, 128, 16) is v
    with pytest.raises(ValueError):
        S.fake_quant_groupwise_lastdim(v[..., :64], 32, 2)
    with pytest.raises(ValueError):
        S.fake_quant_tokens_(v, 0, 100, 0, 128, 2)                                           # not whole groups
    with pytest.raises(ValueError):
        S.fake_quant_tokens_(v, 0, 128, 0, 16, 2)                                            # group size


@pytest.mark.parametrize("sel", [1, 2])
def test_promote_mask_equals_the_oracle(S, sel):
    for seed in range(20):
        ks = _kv((2, 2, 128, 128), seed=seed).transpose(0, 1, 3, 2).copy()                    # [B, nh, D, T]
        if SO.selection_is_tie_free(ks, 0.1, sel):
            break
    got = S.build_promote_mask(torch.from_numpy(ks).cuda(), 0.1, sel)
    assert np.array_equal(got.cpu().numpy(), SO.build_promote_mask(ks, 0.1, sel))
    r = S.build_promote_mask(torch.from_numpy(ks).cuda(), 0.1, 0)                              # random: counts only
    assert r.shape == (2, 2, 128) and bool((r.sum(-1) == 12).all()) and bool((r[0] == r[1]).all())
    assert not S.build_promote_mask(torch.from_numpy(ks).cuda(), 0.0, sel).any()
    assert S.build_promote_mask(torch.from_numpy(ks).cuda(), 1.0, sel).all()


@pytest.mark.parametrize("post,bitdec,sel,group", [(True, False, 1, 128), (False, False, 2, 32), (True, True, 1, 64),
                                                   (False, True, 1, 128)])
def test_cache_steps_like_the_oracle(S, post, bitdec, sel, group):
    """Prefill and 300 decode steps, two layers: what update() returns at every step and the final
    buffers equal the oracle's, whose schedule is the reference's cat-and-clone one."""
    B, nh, T0, steps = 2, 2, 32 + 128 * 2 + 77, 300
    cfg = S.KittyKVCacheConfig(group_size=group, promote_ratio=0.2, channel_selection=sel, VCache_BitDecoding=bitdec,
                               PostQuant=post)
    cache = S.KittyKVCache(cfg, max_length=T0 + steps)
    kv = [(_kv((B, nh, T0 + steps, 128), seed=50 + l), _kv((B, nh, T0 + steps, 128), seed=60 + l)) for l in range(2)]
    for l, (k, v) in enumerate(kv):                        # 25 loud channels per head: the top 25 are never a tie
        for b in range(B):
            for h in range(nh):
                loud = np.random.default_rng(l * 100 + b * 10 + h).permutation(128)[:25]
                k[b, h][:, loud] = (k[b, h][:, loud].astype(np.float32) * 4.0).astype(np.float16)
    for l, (k, v) in enumerate(kv):
        for blk in range((T0 + steps - 32) // 128):        # the data must not tie at the selection boundary
            ks = np.ascontiguousarray(k[:, :, 32 + 128 * blk:32 + 128 * (blk + 1)].transpose(0, 1, 3, 2))
            assert SO.selection_is_tie_free(ks, 0.2, sel), (l, blk)
    ocs = [SO.SimCache(group_size=group, promote_ratio=0.2, channel_selection=sel, VCache_BitDecoding=bitdec,
                       PostQuant=post) for _ in range(2)]
    for l, (k, v) in enumerate(kv):
        kr, vr = cache.update(torch.from_numpy(k[:, :, :T0]).cuda(), torch.from_numpy(v[:, :, :T0]).cuda(), l)
        ko, vo = ocs[l].update(k[:, :, :T0], v[:, :, :T0])
        assert np.array_equal(_bits(kr.contiguous()), ko.view(np.uint16)) and np.array_equal(_bits(vr.contiguous()), vo.view(np.uint16))
    for s in range(steps):
        L = T0 + s + 1
        for l, (k, v) in enumerate(kv):
            kr, vr = cache.update(torch.from_numpy(k[:, :, L - 1:L]).cuda(), torch.from_numpy(v[:, :, L - 1:L]).cuda(), l)
            ko, vo = ocs[l].update(k[:, :, L - 1:L], v[:, :, L - 1:L])
            if s % 16 == 0 or (L - 32 - 128) % 128 in (0, 1, 2):
                assert kr.shape == ko.shape and np.array_equal(_bits(kr.contiguous()), ko.view(np.uint16)), (s, l, "K")
                assert np.array_equal(_bits(vr.contiguous()), vo.view(np.uint16)), (s, l, "V")
        assert cache.get_seq_length(0) == L
    cache.flush_pending()
    for l in range(2):
        assert np.array_equal(_bits(cache.key_cache[l][:, :, :T0 + steps].contiguous()), ocs[l].K.view(np.uint16))
        assert np.array_equal(_bits(cache.value_cache[l][:, :, :T0 + steps].contiguous()), ocs[l].V.view(np.uint16))
    with pytest.raises(ValueError):
        cache.update(torch.zeros(B, nh, 1, 128, dtype=torch.float16, device="cuda"),
                     torch.zeros(B, nh, 1, 128, dtype=torch.float16, device="cuda"), 0)      # full
    with pytest.raises(ValueError):
        S.KittyKVCacheConfig(buffer_length=64)
    with pytest.raises(ValueError):
        S.KittyKVCacheConfig(kbits=12)


def _tiny_llama():
    from transformers import LlamaConfig, LlamaForCausalLM
    cfg = LlamaConfig(vocab_size=256, hidden_size=256, intermediate_size=512, num_hidden_layers=2,
                      num_attention_heads=2, num_key_value_heads=1, head_dim=128, max_position_embeddings=4096,
                      attn_implementation="sdpa")
    torch.manual_seed(0)
    return LlamaForCausalLM(cfg).cuda().half().eval()


def test_stock_model_takes_the_simulator_cache(S):
    """A stock transformers Llama (torch's dense attention) with the simulator's cache as
    past_key_values, as the reference's evaluation runs it: at 16 bits the logits are those of
    transformers' own DynamicCache; at 2 bits generate() runs and the layer buffers end up equal to
    the oracle's, fed the keys and values the model handed to update()."""
    pytest.importorskip("transformers")
    from transformers import DynamicCache
    model = _tiny_llama()
    B, T0, steps = 2, 32 + 128 + 30, 140
    ids = torch.randint(0, 256, (B, T0), generator=torch.Generator().manual_seed(2)).cuda()
    plain = S.KittyKVCache(S.KittyKVCacheConfig(kbits=16, vbits=16, promote_ratio=0.0), max_length=T0 + 8)
    ref = DynamicCache()
    with torch.no_grad():
        cur = ids
        for s in range(6):
            a = model(input_ids=cur, past_key_values=ref, use_cache=True).logits[:, -1].float()
            b = model(input_ids=cur, past_key_values=plain, use_cache=True).logits[:, -1].float()
            assert (a - b).abs().max().item() <= 2e-2, s
            cur = a.argmax(-1, keepdim=True)
    assert plain.get_seq_length() == T0 + 5

    cache = S.KittyKVCache(S.KittyKVCacheConfig(promote_ratio=0.2), max_length=T0 + steps)
    seen = [[], []]
    inner = cache.update

    def recording_update(k, v, layer_idx, cache_kwargs=None):
        seen[layer_idx].append((k.detach().cpu().numpy().copy(), v.detach().cpu().numpy().copy()))
        return inner(k, v, layer_idx, cache_kwargs)

    cache.update = recording_update
    # topk's order among equal scores is not pinned: the oracle takes the masks the product chose
    # (selection itself is checked in test_promote_mask_equals_the_oracle), block by block in order
    masks, last = [[], []], []
    inner_mask, inner_quant_k = S.build_promote_mask, cache._quant_k

    def recording_mask(*a):
        last.append(inner_mask(*a))
        return last[-1]

    def recording_quant_k(layer, lo, hi):
        inner_quant_k(layer, lo, hi)
        m = last.pop().cpu().numpy()                     # [B, nh, blocks, D]
        masks[layer].extend(m[:, :, i] for i in range(m.shape[2]))

    S.build_promote_mask, cache._quant_k = recording_mask, recording_quant_k
    try:
        with torch.no_grad():
            out = model.generate(ids, past_key_values=cache, max_new_tokens=steps, do_sample=False, use_cache=True,
                                 pad_token_id=0, eos_token_id=None)
        cache.flush_pending()
    finally:
        S.build_promote_mask = inner_mask
    assert out.shape == (B, T0 + steps)
    n = len(seen[0])
    assert n == len(seen[1]) and cache.get_seq_length(0) == T0 + n - 1 >= T0 + steps - 1
    for l in range(2):
        assert len(masks[l]) == (T0 + n - 1 - 32 - 1) // 128 and all(int(m.sum()) == B * 25 for m in masks[l])
        feed = iter(masks[l])
        oc = SO.SimCache(promote_ratio=0.2, mask_fn=lambda ks: next(feed))
        assert seen[l][0][0].shape[2] == T0
        for k, v in seen[l]:
            oc.update(k, v)
        L = oc.K.shape[2]
        assert np.array_equal(_bits(cache.key_cache[l][:, :, :L].contiguous()), oc.K.view(np.uint16)), l
        assert np.array_equal(_bits(cache.value_cache[l][:, :, :L].contiguous()), oc.V.view(np.uint16)), l
    quantized = (cache.key_cache[0][:, :, 32:32 + 128] != torch.from_numpy(seen[0][0][0][:, :, 32:32 + 128]).cuda()).any()
    assert bool(quantized)
