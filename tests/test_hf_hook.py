"""The hook for stock transformers attention modules (kitty_amd/hf.py)."""
import numpy as np
import pytest
import torch

transformers = pytest.importorskip("transformers")


def _tiny_llama(attn, head_dim=128):
    from transformers import LlamaConfig, LlamaForCausalLM
    cfg = LlamaConfig(vocab_size=256, hidden_size=256, intermediate_size=512, num_hidden_layers=2,
                      num_attention_heads=2, num_key_value_heads=1, head_dim=head_dim, max_position_embeddings=4096,
                      attn_implementation=attn)
    torch.manual_seed(0)
    return LlamaForCausalLM(cfg)


def _tiny_qwen3(attn):
    from transformers import Qwen3Config, Qwen3ForCausalLM
    cfg = Qwen3Config(vocab_size=256, hidden_size=256, intermediate_size=512, num_hidden_layers=2,
                      num_attention_heads=4, num_key_value_heads=1, head_dim=128, max_position_embeddings=4096,
                      attn_implementation=attn)
    torch.manual_seed(0)
    return Qwen3ForCausalLM(cfg)


class _DecodeCapture:
    """Stands in for the decode-attention call of the hook and checks every call it sees against the
    CPU oracle: the layer's bytes at that moment (after update, before quantize_decode) are copied
    into an oracle layer, and the kernel's output for the query the model really produced is held to
    the contract of tests/test_gpu_parity.py (max-abs 2e-3 against dequantize-then-attend)."""

    def __init__(self, hf, max_len, every=1):
        self.hf, self.max_len, self.every, self.calls, self.worst = hf, max_len, every, 0, 0.0

    def __enter__(self):
        from tests import gpu_util
        from tests.test_gpu_parity import _check_attn
        self.orig = self.hf.kitty_attention_forward

        def checked(module, query, layer, scaling, **kw):
            out, w = self.orig(module, query, layer, scaling, **kw)
            self.calls += 1
            if self.calls % self.every == 0:
                assert abs(scaling - 128 ** -0.5) < 1e-9
                ol = gpu_util.oracle_from_layer(layer, self.max_len)
                got = out.detach().cpu().numpy().astype(np.float64)
                self.worst = max(self.worst, _check_attn(got, ol, query.detach().cpu().numpy(), what=f"call {self.calls}"))
            return out, w

        self.hf.kitty_attention_forward = checked
        return self

    def __exit__(self, *exc):
        self.hf.kitty_attention_forward = self.orig
        return False


def test_register_and_cache_adapter_on_cpu():
    from kitty_amd import hf
    hf.register()
    hf.register()                                   # idempotent
    from transformers.modeling_utils import ALL_ATTENTION_FUNCTIONS
    assert ALL_ATTENTION_FUNCTIONS[hf.NAME] is hf.kitty_attention
    model = _tiny_llama("kitty")                    # the name is accepted by a stock model
    assert model.config._attn_implementation == "kitty"
    cache = hf.KittyHFCache(model.config, 1, 256, device="cpu")
    k = torch.randn(1, 1, 40, 128, dtype=torch.float16)
    v = torch.randn(1, 1, 40, 128, dtype=torch.float16)
    rk, rv = cache.update(k, v, 0)
    assert rk is k and rv is v and hf._current.phase == "prefill" and hf._current.cache is cache
    assert cache.get_mask_sizes(40, 0) == (40, 0)
    assert cache.get_seq_length(0) == 0             # nothing is counted before quantize_prefill, as in the reference


@pytest.mark.gpu
def test_stock_llama_matches_dense_attention_while_everything_is_fp16():
    """Prompt of 20 tokens and 60 decode steps: 80 tokens fit the sink and the fp16 windows, nothing
    is quantized, so the logits must agree with the same model on torch's dense attention."""
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    from transformers import DynamicCache
    from kitty_amd import hf
    hf.register()
    dev = torch.device("cuda")
    ref = _tiny_llama("sdpa").to(dev).half().eval()
    mod = _tiny_llama("kitty").to(dev).half().eval()
    mod.load_state_dict(ref.state_dict())
    B, T0, steps = 2, 20, 60
    ids = torch.randint(0, 256, (B, T0), generator=torch.Generator().manual_seed(1)).to(dev)
    c_ref, c_mod = DynamicCache(), hf.KittyHFCache(mod.config, B, 512, device=dev)
    with torch.no_grad():
        cur = ids
        for s in range(steps + 1):
            a = ref(input_ids=cur, past_key_values=c_ref, use_cache=True).logits[:, -1].float()
            b = mod(input_ids=cur, past_key_values=c_mod, use_cache=True).logits[:, -1].float()
            assert torch.isfinite(b).all()
            assert (a - b).abs().max().item() <= 3e-2, (s, (a - b).abs().max().item())
            cur = a.argmax(-1, keepdim=True)
    assert c_mod.get_seq_length(0) == T0 + steps
    L = c_mod.kv_cache[1]
    assert (L.Sink_Count, L.PageCount_K, L.Q_Buffer_Count_K) == (32, 0, T0 + steps - 32)
    # generate() drives the same cache (greedy tokens are not compared: with random weights the top
    # two logits are often closer than fp16 attention kernels agree)
    with torch.no_grad():
        gen_cache = hf.KittyHFCache(mod.config, B, 512, device=dev)
        got = mod.generate(ids, past_key_values=gen_cache, max_new_tokens=12, do_sample=False, pad_token_id=0)
    assert tuple(got.shape) == (B, T0 + 12) and torch.equal(got[:, :T0], ids)
    assert gen_cache.get_seq_length(0) == T0 + 11          # the last token is returned, not fed back


@pytest.mark.gpu
def test_stock_llama_long_prompt_decode_and_chunk():
    """A prompt that is packed, decode steps across flushes, then a chunk of new tokens: the cache
    goes through the reference's state machine and the logits stay close to dense attention."""
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    from transformers import DynamicCache
    from kitty_amd import hf
    from oracle import kitty_oracle as O
    hf.register()
    dev = torch.device("cuda")
    ref = _tiny_llama("sdpa").to(dev).half().eval()
    mod = _tiny_llama("kitty").to(dev).half().eval()
    mod.load_state_dict(ref.state_dict())
    B, T0, steps, chunk = 1, 300, 150, 70
    g = torch.Generator().manual_seed(2)
    ids = torch.randint(0, 256, (B, T0), generator=g).to(dev)
    c_ref, c_mod = DynamicCache(), hf.KittyHFCache(mod.config, B, 1024, device=dev)
    ol = O.OracleLayer(B, 1024, 1)                                  # counters only: the state machine
    zeros = lambda n: np.zeros((B, 1, n, 128), np.float16)
    # every 7th decode-attention call of the model (both layers, across the flushes) against the oracle
    with torch.no_grad(), _DecodeCapture(hf, 1024, every=7) as cap:
        cur, cos = ids, []
        for s in range(steps + 1):
            a = ref(input_ids=cur, past_key_values=c_ref, use_cache=True).logits[:, -1].float()
            b = mod(input_ids=cur, past_key_values=c_mod, use_cache=True).logits[:, -1].float()
            assert torch.isfinite(b).all()
            cos.append(torch.nn.functional.cosine_similarity(a, b, dim=-1).min().item())
            n = cur.shape[1]
            if s == 0:
                ol.update(zeros(n), zeros(n)); ol.quantize_prefill()
            else:
                ol.update(zeros(1), zeros(1)); ol.quantize_decode()
            cur = a.argmax(-1, keepdim=True)
        L = c_mod.kv_cache[0]
        for f in ("Sink_Count", "PageCount_K", "PageCount_V", "Q_Buffer_Count_K", "Q_Buffer_Count_V", "Local_Count_V",
                  "Write_Offset_Local_V"):
            assert getattr(L, f) == getattr(ol, f), f
        more = torch.randint(0, 256, (B, chunk), generator=g).to(dev)
        b = mod(input_ids=more, past_key_values=c_mod, use_cache=True).logits.float()
        a = ref(input_ids=more, past_key_values=c_ref, use_cache=True).logits.float()
        assert torch.isfinite(b).all() and b.shape == a.shape
        assert c_mod.get_seq_length(0) == T0 + steps + chunk
    # 2-bit pages disturb the logits only a little: every step's logit vector points the same way as
    # dense attention's (random weights leave the argmax itself nearly tied, so it is not compared)
    print("cosine similarity of the logits: min %.4f mean %.4f" % (min(cos), sum(cos) / len(cos)))
    assert min(cos) >= 0.97, min(cos)
    assert cap.calls == 2 * steps and cap.worst <= 2e-3
    print("decode attention inside the model vs oracle: worst max-abs error %.2e over %d checked calls"
          % (cap.worst, cap.calls // 7))


@pytest.mark.gpu
def test_stock_qwen3_on_the_hook():
    """The reference's own model family (per-head q/k RMS norm before the rotation,
    modeling_qwen3.py:214-215) as the stock transformers module: dense agreement while everything is
    fp16, then a packed prompt with decode steps whose attention calls are checked against the oracle
    on the queries and caches the model really produced, and generate() as the reference's benchmark
    drives it (fresh cache, greedy, no early stop: benchmark_kitty.py:131-149)."""
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    from transformers import DynamicCache
    from kitty_amd import hf
    hf.register()
    dev = torch.device("cuda")
    ref = _tiny_qwen3("sdpa").to(dev).half().eval()
    mod = _tiny_qwen3("kitty").to(dev).half().eval()
    mod.load_state_dict(ref.state_dict())
    g = torch.Generator().manual_seed(5)
    with torch.no_grad():
        # (i) 20 + 40 tokens: nothing is quantized
        B = 2
        ids = torch.randint(0, 256, (B, 20), generator=g).to(dev)
        c_ref, c_mod = DynamicCache(), hf.KittyHFCache(mod.config, B, 512, device=dev)
        cur = ids
        for s in range(41):
            a = ref(input_ids=cur, past_key_values=c_ref, use_cache=True).logits[:, -1].float()
            b = mod(input_ids=cur, past_key_values=c_mod, use_cache=True).logits[:, -1].float()
            assert torch.isfinite(b).all() and (a - b).abs().max().item() <= 3e-2, (s, (a - b).abs().max().item())
            cur = a.argmax(-1, keepdim=True)
        # (ii) a packed prompt, decode across a K flush, every 5th attention call against the oracle
        ids = torch.randint(0, 256, (B, 32 + 128 * 2 + 100), generator=g).to(dev)
        cache = hf.KittyHFCache(mod.config, B, 1024, device=dev)
        with _DecodeCapture(hf, 1024, every=5) as cap:
            cur = mod(input_ids=ids, past_key_values=cache, use_cache=True).logits[:, -1].float().argmax(-1, keepdim=True)
            for s in range(60):
                out = mod(input_ids=cur, past_key_values=cache, use_cache=True).logits[:, -1].float()
                assert torch.isfinite(out).all()
                cur = out.argmax(-1, keepdim=True)
        L = cache.kv_cache[1]
        assert cap.calls == 2 * 60 and cap.worst <= 2e-3
        assert (L.PageCount_K, L.Q_Buffer_Count_K, L.PageCount_V) == (3, 32, 2)
        # (iii) generate() with a fresh cache, as the reference's benchmark calls it
        gen_cache = hf.KittyHFCache(mod.config, B, 1024, device=dev)
        got = mod.generate(input_ids=ids, max_length=ids.shape[1] + 40, max_new_tokens=None, do_sample=False,
                           temperature=None, top_p=None, top_k=None, past_key_values=gen_cache, eos_token_id=None,
                           pad_token_id=0, disable_compile=True)
        assert tuple(got.shape) == (B, ids.shape[1] + 40) and torch.equal(got[:, :ids.shape[1]], ids)
        assert gen_cache.get_seq_length(0) == ids.shape[1] + 39
        gen_cache.check_status()


@pytest.mark.gpu
def test_chunk_through_the_hook_with_device_counters():
    """Several new tokens per sequence over a packed cache with the counters on the device: chunk
    attention, then the device-side chunk append; the logits are those of the host-counter cache."""
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    from kitty_amd import hf
    hf.register()
    dev = torch.device("cuda")
    mod = _tiny_llama("kitty").to(dev).half().eval()
    B, T0 = 2, 32 + 128 + 90
    g = torch.Generator().manual_seed(6)
    ids = torch.randint(0, 256, (B, T0), generator=g).to(dev)
    host, devc = (hf.KittyHFCache(mod.config, B, 1024, device=dev) for _ in range(2))
    with torch.no_grad():
        mod(input_ids=ids, past_key_values=host, use_cache=True)
        mod(input_ids=ids, past_key_values=devc, use_cache=True)
        devc.enable_device_counters()
        for n in (50, 1, 200):
            more = torch.randint(0, 256, (B, n), generator=g).to(dev)
            a = mod(input_ids=more, past_key_values=host, use_cache=True).logits
            b = mod(input_ids=more, past_key_values=devc, use_cache=True).logits
            assert torch.equal(a, b), n
    torch.cuda.synchronize()
    assert devc.get_seq_length(0) == host.get_seq_length(0) == T0 + 251
    for lh, ld in zip(host.kv_cache, devc.kv_cache):
        assert ld.seq_counts.cpu().tolist() == [lh.counts()] * B
        assert torch.equal(lh.KeyCache, ld.KeyCache) and torch.equal(lh.ValueCache, ld.ValueCache)
    devc.check_status()


@pytest.mark.gpu
def test_stock_llama_with_device_side_counters():
    """After the prompt the cache can keep its counters on the device (one append launch, one flush
    launch pair per layer and step): the logits are those of the host-counter mode, bit for bit."""
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    from kitty_amd import hf
    hf.register()
    dev = torch.device("cuda")
    mod = _tiny_llama("kitty").to(dev).half().eval()
    B, T0, steps = 2, 32 + 128 + 100, 60                       # the K Q-buffer fills and is flushed on the way
    ids = torch.randint(0, 256, (B, T0), generator=torch.Generator().manual_seed(3)).to(dev)
    host, devc = (hf.KittyHFCache(mod.config, B, 1024, device=dev) for _ in range(2))
    with torch.no_grad():
        a = mod(input_ids=ids, past_key_values=host, use_cache=True).logits[:, -1]
        b = mod(input_ids=ids, past_key_values=devc, use_cache=True).logits[:, -1]
        assert torch.equal(a, b)
        devc.enable_device_counters()
        cur = a.float().argmax(-1, keepdim=True)
        for s in range(steps):
            a = mod(input_ids=cur, past_key_values=host, use_cache=True).logits[:, -1]
            b = mod(input_ids=cur, past_key_values=devc, use_cache=True).logits[:, -1]
            assert torch.equal(a, b), s
            cur = a.float().argmax(-1, keepdim=True)
    torch.cuda.synchronize()
    assert devc.kv_cache[0].seq_counts.cpu().tolist() == [host.kv_cache[0].counts()] * B


@pytest.mark.gpu
def test_stock_llama_on_the_paged_cache():
    """Two prompts of different lengths admitted into slots 0 and 2 of three, decoded together with
    per-row positions; slot 0 is released and a third prompt admitted while slot 2 keeps decoding.
    Every sequence's logits agree with the same model serving that sequence alone on a KittyHFCache
    (same kernels, other split counts: 3e-2 on fp16 logits)."""
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    from kitty_amd import hf
    hf.register()
    dev = torch.device("cuda")
    mod = _tiny_llama("kitty").to(dev).half().eval()
    g = torch.Generator().manual_seed(4)
    prompts = {0: torch.randint(0, 256, (1, 32 + 128 + 70), generator=g).to(dev),
               2: torch.randint(0, 256, (1, 45), generator=g).to(dev)}
    late = torch.randint(0, 256, (1, 32 + 128 * 2 + 9), generator=g).to(dev)
    paged = hf.PagedKittyHFCache(mod.config, 3, 1024, pool_pages=10, device=dev)
    solo, cur = {}, torch.zeros(3, 1, dtype=torch.long, device=dev)

    def admit(slot, ids):
        solo[slot] = hf.KittyHFCache(mod.config, 1, 1024, device=dev)
        with paged.admitting(slot):
            a = mod(input_ids=ids, past_key_values=paged, use_cache=True).logits[:, -1].float()
        b = mod(input_ids=ids, past_key_values=solo[slot], use_cache=True).logits[:, -1].float()
        assert (a - b).abs().max().item() <= 3e-2
        cur[slot] = b.argmax(-1)

    def decode(steps):
        for s in range(steps):
            pos = paged.position_ids()
            a = mod(input_ids=cur, position_ids=pos, past_key_values=paged, use_cache=True).logits[:, -1].float()
            for slot in paged.active_slots():
                b = mod(input_ids=cur[slot:slot + 1], past_key_values=solo[slot], use_cache=True).logits[:, -1].float()
                assert int(pos[slot]) == solo[slot].get_seq_length(0) - 1
                assert (a[slot:slot + 1] - b).abs().max().item() <= 3e-2, (s, slot)
                cur[slot] = b.argmax(-1)

    with torch.no_grad():
        for slot, ids in prompts.items():
            admit(slot, ids)
        assert paged.active_slots() == [0, 2] and list(paged.seq_lengths()) == [230, 0, 45]
        decode(70)                                   # slot 0 flushes keys, slot 2 leaves the sink behind
        paged.release(0)
        admit(1, late)
        decode(40)
    paged.check_tables()
    assert paged.active_slots() == [1, 2] and list(paged.seq_lengths()) == [0, 297 + 40, 45 + 110]


@pytest.mark.gpu
@pytest.mark.parametrize("head_dim", [64, 256])
def test_stock_llama_with_another_head_dimension(head_dim):
    """The reference takes ``config.head_dim`` (kitty.py:39-44); head dimensions 64 and 256 go through the
    same hook onto the kernels for other head dimensions.  While everything is fp16 (80 tokens) the logits
    agree with torch's dense attention; a longer ``generate()`` crosses prefill quantization and both
    flushes and leaves the counters the state machine predicts."""
    if not torch.cuda.is_available():
        pytest.skip("needs a GPU")
    from transformers import DynamicCache
    from kitty_amd import hf
    hf.register()
    dev = torch.device("cuda")
    ref = _tiny_llama("sdpa", head_dim).to(dev).half().eval()
    mod = _tiny_llama("kitty", head_dim).to(dev).half().eval()
    mod.load_state_dict(ref.state_dict())
    B, T0, steps = 2, 20, 60
    ids = torch.randint(0, 256, (B, T0), generator=torch.Generator().manual_seed(3)).to(dev)
    c_ref, c_mod = DynamicCache(), hf.KittyHFCache(mod.config, B, 1024, device=dev)
    assert c_mod.kv_cache[0].D == head_dim and c_mod.kv_cache[0].D_BOOSTED == head_dim // 4
    with torch.no_grad():
        cur = ids
        for s in range(steps + 1):
            a = ref(input_ids=cur, past_key_values=c_ref, use_cache=True).logits[:, -1].float()
            b = mod(input_ids=cur, past_key_values=c_mod, use_cache=True).logits[:, -1].float()
            assert torch.isfinite(b).all()
            assert (a - b).abs().max().item() <= 3e-2, (s, (a - b).abs().max().item())
            cur = a.argmax(-1, keepdim=True)
    T1, new = 32 + 128 + 100, 170
    ids = torch.randint(0, 256, (B, T1), generator=torch.Generator().manual_seed(4)).to(dev)
    with torch.no_grad():
        cache = hf.KittyHFCache(mod.config, B, 1024, device=dev)
        got = mod.generate(ids, past_key_values=cache, max_new_tokens=new, do_sample=False, pad_token_id=0,
                           eos_token_id=None)
    assert tuple(got.shape) == (B, T1 + new) and torch.equal(got[:, :T1], ids)
    n = T1 + new - 1 - 32
    for L in cache.kv_cache:
        assert (L.Sink_Count, L.PageCount_K, L.Q_Buffer_Count_K) == (32, n // 128, n % 128)
        assert (L.PageCount_V, L.Q_Buffer_Count_V, L.Local_Count_V) == ((n - 128) // 128, (n - 128) % 128, 128)
    cache.check_status()
