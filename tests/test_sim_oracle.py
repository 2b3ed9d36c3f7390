"""The oracle of the accuracy simulator (oracle/sim_oracle.py; reference: src/kitty_sim/utils_quant.py,
kitty_simulate.py:170-252), pinned without a GPU: against torch's own fp16 operators evaluating the
reference's chain, against a scalar loop in numpy float16 arithmetic, and by closed forms."""
import numpy as np
import pytest
import torch

from oracle import sim_baseline as SB
from oracle import sim_oracle as SO


def _data(shape, seed, scale=1.0):
    g = np.random.default_rng(seed)
    x = g.standard_normal(shape).astype(np.float32) * scale
    x[..., 3, :] *= 10.0                      # an outlier row
    return x.astype(np.float16)


@pytest.mark.parametrize("bit,group,use_mask", [(2, 128, True), (2, 32, False), (4, 64, True), (1, 128, False),
                                                (3, 32, True), (8, 128, False)])
def test_fake_quant_equals_torch_fp16_operators(bit, group, use_mask):
    """The reference's operator chain run by torch on fp16 CPU tensors (true division by the scalar)."""
    x = _data((2, 3, 16, 256), seed=bit * 100 + group)
    mask = None
    if use_mask:
        mask = np.zeros((2, 3, 16), dtype=bool)
        mask[:, :, [1, 3, 8]] = True
    got = SO.fake_quant_groupwise_lastdim(x, group, bit, mask, 4 if bit <= 4 else 8, scalar_div="true")
    want = SB.fake_quant_groupwise_lastdim(torch.from_numpy(x), group, bit,
                                           None if mask is None else torch.from_numpy(mask), 4 if bit <= 4 else 8)
    assert np.array_equal(got.view(np.uint16), want.numpy().view(np.uint16))
    # the device flavour (reciprocal of the scalar) is the same function up to the scale's last bit
    dev = SO.fake_quant_groupwise_lastdim(x, group, bit, mask, 4 if bit <= 4 else 8)
    assert np.abs(dev.astype(np.float32) - got.astype(np.float32)).max() <= 0.05


def test_fake_quant_equals_a_scalar_loop_in_float16_arithmetic():
    x = _data((1, 2, 4, 64), seed=5)
    mask = np.array([[[True, False, False, True], [False, False, True, False]]])
    got = SO.fake_quant_groupwise_lastdim(x, 32, 2, mask, 4, scalar_div="true")
    h = np.float16
    for n in range(2):
        for d in range(4):
            levels = 15 if mask[0, n, d] else 3
            for g in range(2):
                grp = x[0, n, d, 32 * g:32 * g + 32]
                mn, mx = grp.min(), grp.max()
                rng = max(h(mx - mn), h(1e-4))
                scale = h(rng / h(levels))
                for t in range(32):
                    q = h(h(grp[t] - mn) / scale)
                    q = h(np.rint(min(max(q, h(0)), h(levels))))
                    assert got[0, n, d, 32 * g + t] == h(h(q * scale) + mn), (n, d, g, t)


def test_fake_quant_closed_forms():
    # values on the levels of an exactly representable grid come back unchanged
    lv = np.array([0.0, 1.0, 2.0, 3.0], dtype=np.float16)
    x = np.tile(lv, 32).reshape(1, 1, 1, 128) - np.float16(1.0)
    assert np.array_equal(SO.fake_quant_groupwise_lastdim(x, 128, 2, scalar_div="true"), x)
    # a constant group: range floored at 1e-4, code 0, value = the minimum itself
    c = np.full((1, 1, 2, 128), 0.3337, dtype=np.float16)
    assert np.array_equal(SO.fake_quant_groupwise_lastdim(c, 128, 2), c)
    # clamp before round: the maximum maps to the top code, never above
    x = _data((1, 1, 8, 128), seed=9)
    for bit in (1, 2, 4):
        dq = SO.fake_quant_groupwise_lastdim(x, 128, bit).astype(np.float32)
        xs = x.astype(np.float32)
        mn, mx = xs.min(-1, keepdims=True), xs.max(-1, keepdims=True)
        scale = (mx - mn) / (2 ** bit - 1)
        assert np.unique(np.round((dq - mn) / scale)[0, 0, 0]).size <= 2 ** bit
        assert (np.abs(dq - xs) <= scale * 0.5 + 0.02 * np.abs(xs).max()).all()
        assert (dq.min(-1) >= mn[..., 0] - 1e-2).all() and (dq.max(-1) <= mx[..., 0] + 2e-2 * np.abs(mx[..., 0]) + 1e-2).all()
    # half to even after the clamp: codes 0.5 -> 0, 1.5 -> 2, 2.5 -> 2 on a grid with scale 1
    x = np.zeros((1, 1, 1, 32), dtype=np.float16)
    x[0, 0, 0, :6] = [0.0, 3.0, 0.5, 1.5, 2.5, 3.0]
    dq = SO.fake_quant_groupwise_lastdim(x, 32, 2, scalar_div="true")
    assert list(dq[0, 0, 0, :6]) == [0.0, 3.0, 0.0, 2.0, 2.0, 3.0]
    assert SO.fake_quant_groupwise_lastdim(x, 32, 16) is x                      # 16 bit: untouched


@pytest.mark.parametrize("sel", [1, 2])
def test_promote_mask_equals_torch_operators(sel):
    for seed in range(20):
        ks = _data((2, 2, 128, 128), seed=seed)
        if SO.selection_is_tie_free(ks, 0.1, sel):
            break
    t = torch.from_numpy(ks)
    score = t.abs().mean(dim=-1) if sel == 1 else (t - t.mean(dim=-1, keepdim=True)).pow(2).mean(dim=-1)
    assert np.array_equal(SO.promote_scores(ks, sel).astype(np.float16).view(np.uint16), score.numpy().view(np.uint16))
    want = torch.zeros((2, 2, 128), dtype=torch.bool).scatter_(-1, score.topk(12, dim=-1).indices, True)
    got = SO.build_promote_mask(ks, 0.1, sel)
    assert got.sum() == 2 * 2 * 12 and np.array_equal(got, want.numpy())
    assert SO.promote_count(128, 0.2) == 25 and SO.promote_count(128, 0.25) == 32 and SO.promote_count(128, 0.0) == 0
    assert not SO.build_promote_mask(ks, 0.0, sel).any() and SO.build_promote_mask(ks, 1.0, sel).all()
    with pytest.raises(ValueError):
        SO.build_promote_mask(ks, 0.1, 7)


@pytest.mark.parametrize("post,bitdec", [(True, False), (False, False), (True, True), (False, True)])
def test_sim_cache_schedule(post, bitdec):
    """Which tokens are quantized when (kitty_simulate.py:196-247): keys in whole 128-token blocks
    from the sink on, one step after the block is complete; values per token once 128 newer
    tokens exist (or with the keys' blocks, in BitDecoding mode); PostQuant returns the state
    before the step's quantization."""
    B, nh, D, T0, steps = 1, 1, 128, 32 + 128 + 40, 230
    g = np.random.default_rng(3)
    k = g.standard_normal((B, nh, T0 + steps, D)).astype(np.float16)
    v = g.standard_normal((B, nh, T0 + steps, D)).astype(np.float16)
    c = SO.SimCache(PostQuant=post, VCache_BitDecoding=bitdec)
    kr, vr = c.update(k[:, :, :T0], v[:, :, :T0])
    if post:
        assert np.array_equal(kr, k[:, :, :T0]) and np.array_equal(vr, v[:, :, :T0])
    for s in range(steps):
        before_k, before_v = c.K.copy(), c.V.copy()
        L = T0 + s + 1
        kr, vr = c.update(k[:, :, L - 1:L], v[:, :, L - 1:L])
        assert kr.shape[-2] == L
        if post:                                    # what attention sees: last state + the new token
            assert np.array_equal(kr[:, :, :L - 1], before_k) and np.array_equal(kr[:, :, L - 1:], k[:, :, L - 1:L])
            assert np.array_equal(vr[:, :, :L - 1], before_v)
        else:
            assert kr is c.K and vr is c.V
        changed_k = np.flatnonzero((c.K[0, 0, :L - 1] != before_k[0, 0]).any(-1))
        n = L - 32 - 128
        if n > 0 and n % 128 == 1:
            assert changed_k.size > 100 and changed_k.min() >= L - 129 and changed_k.max() == L - 2
        else:
            assert changed_k.size == 0
    L = T0 + steps
    qk = np.flatnonzero((c.K[0, 0] != k[0, 0, :L]).any(-1))
    blocks = (L - 32 - 1) // 128                    # blocks complete one step ago
    assert qk.min() >= 32 and qk.max() == 32 + 128 * blocks - 1 and qk.size > 128 * blocks - 5
    qv = np.flatnonzero((c.V[0, 0] != v[0, 0, :L]).any(-1))
    assert qv.min() >= 32 and qv.max() == (32 + 128 * blocks - 1 if bitdec else L - 129)
    assert np.array_equal(c.K[0, 0, :32], k[0, 0, :32]) and np.array_equal(c.K[0, 0, 32 + 128 * blocks:], k[0, 0, 32 + 128 * blocks:L])
