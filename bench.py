#!/usr/bin/env python3
"""Benchmark of the packed-KV decode attention hot path on one MI355X.

A step = one layer's decode attention (split pass + merge pass) over one batch of synthetic,
already-packed KV resident in HBM.  Default workload: Llama-3.1-8B-shaped decode, 32 Q / 8 KV
heads, head_dim 128, batch 16, 32k context (BASELINE.json configs[1]).  Steps rotate over several
independent copies of the cache so that every step streams from HBM rather than from the 256 MB
Infinity Cache.  Prints ONE JSON line.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload c1|c0|c2|c4] [--copies N]

``--workload e2e`` times a whole 32-layer decoder step around the cache (tokens/s).
``--workload fq`` times the accuracy simulator's fake-quantization kernel on the configs[1] shape.
``--workload c3`` measures the other kernel family instead (BASELINE.json configs[3]): a 2048-token
chunk attending a 30720-token packed prefix, bound by the matrix cores, plus the append of the chunk.
"""
import argparse
import json
import os
import sys
import time
import types

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

WORKLOADS = {
    # name: (B, H_Q, H_KV, T, description)
    "c0": (1, 32, 8, 4096, "decode B=1 32Q/8KV D=128 ctx=4096 (configs[0])"),
    "c1": (16, 32, 8, 32768, "Llama-3.1-8B-shaped decode B=16 32Q/8KV D=128 ctx=32768, 2-bit Kitty KV (configs[1])"),
    "c4": (1, 64, 8, 131072, "long-context decode B=1 64Q/8KV D=128 ctx=131072 (configs[4])"),
    # per-sequence contexts uniform in [1k, 16k] and residual fill uniform in [0, 128): T below is the allocation
    "c2": (64, 32, 8, 16543, "Qwen3-8B-shaped ragged decode B=64 32Q/8KV D=128 ctx~U[1k,16k] (configs[2])"),
}
C3 = dict(B=4, H_Q=32, H_KV=8, T0=30720, Tq=2048,
          desc="chunked prefill B=4 32Q/8KV D=128: 2048-token chunk over a 30720-token packed prefix, "
               "Student-t(3) keys, then append of the chunk (configs[3])")
HBM_PEAK_GBPS = 8000.0
MFMA_F16_PEAK_TFLOPS = 2500.0
TRAFFIC_FILE = os.path.join(ROOT, "profiles", "decode_split_pmc_traffic.txt")


def measured_traffic(workload, splits):
    """HBM bytes per launch of the split pass as measured with rocprofv3 --pmc FETCH_SIZE /
    WRITE_SIZE on this workload in a run of its own (counters cannot be read from inside this
    process): the figure of the summary committed under profiles/, not a measurement of this run.
    None when there is no such summary for this workload."""
    try:
        with open(TRAFFIC_FILE) as f:
            rec = json.load(f).get(workload)
        return None if rec is None else rec["fetch_bytes"] + rec["write_bytes"]
    except (OSError, ValueError, KeyError):
        return None



class HipEvents:
    """hipEvent_t handles from the HIP runtime this process already has loaded (torch's)."""

    def __init__(self):
        import ctypes
        self.ct = ctypes
        self.hip = ctypes.CDLL("libamdhip64.so")
        self.hip.hipEventCreate.argtypes = [ctypes.POINTER(ctypes.c_void_p)]
        self.hip.hipEventElapsedTime.argtypes = [ctypes.POINTER(ctypes.c_float), ctypes.c_void_p, ctypes.c_void_p]
        self.hip.hipEventSynchronize.argtypes = [ctypes.c_void_p]

    def create(self):
        ev = self.ct.c_void_p()
        rc = self.hip.hipEventCreate(self.ct.byref(ev))
        if rc != 0:
            raise RuntimeError(f"hipEventCreate failed ({rc})")
        return ev

    def synchronize(self, ev) -> None:
        rc = self.hip.hipEventSynchronize(ev)
        if rc != 0:
            raise RuntimeError(f"hipEventSynchronize failed ({rc})")

    def elapsed_us(self, a, b) -> float:
        ms = self.ct.c_float()
        rc = self.hip.hipEventElapsedTime(self.ct.byref(ms), a, b)
        if rc != 0:
            raise RuntimeError(f"hipEventElapsedTime failed ({rc})")
        return ms.value * 1e3


def synth_kv(B, H, T, D, seed, device, student_t=False):
    """K ~ N(0,1) (or Student-t, nu=3) with 8 fixed outlier channels per head scaled x10, V ~ N(0,1);
    fp16 [B,H,T,D]."""
    import torch
    g = torch.Generator(device=device).manual_seed(seed)
    K = torch.empty((B, H, T, D), dtype=torch.float16, device=device)
    V = torch.empty((B, H, T, D), dtype=torch.float16, device=device)
    mult = torch.ones((H, 1, D), dtype=torch.float32, device=device)
    pg = torch.Generator().manual_seed(seed)
    for h in range(H):
        mult[h, 0, torch.randperm(D, generator=pg)[:8].to(device)] = 10.0
    for b in range(B):
        x = torch.randn((H, T, D), generator=g, device=device, dtype=torch.float32)
        if student_t:   # Student-t with 3 degrees of freedom: normal / sqrt(chi2_3 / 3)
            chi = torch.randn((H, T, D, 3), generator=g, device=device, dtype=torch.float32).square_().sum(-1)
            x = x / (chi / 3).sqrt_()
        K[b] = (x * mult).clamp_(-6e4, 6e4).half()
        V[b] = torch.randn((H, T, D), generator=g, device=device, dtype=torch.float32).half()
    return K, V


def algorithmic_bytes(B, H_Q, H_KV, layer):
    """Bytes one decode step has to move: packed pages + metadata + fp16 windows + Q and O."""
    pk, pv = layer.PageCount_K, layer.PageCount_V
    D, DB = layer.D, layer.D_BOOSTED
    k_page = 32 * (D + DB) + D + 4 * D          # planes, slot map, (scale, zero) pairs: 5760 at D = 128
    v_page = 32 * D + 512                       # codes, (scale, zero) pairs: 4608 at D = 128
    per_head_packed = k_page * pk + v_page * pv
    per_head_fp16 = 2 * D * (2 * layer.Sink_Count + layer.Q_Buffer_Count_K + layer.Q_Buffer_Count_V + layer.Local_Count_V)
    qo = 2 * H_Q * D * 2
    return B * (H_KV * (per_head_packed + per_head_fp16) + qo), B * H_KV * per_head_packed


def cpu_baseline(K, V, q, H_Q, H_KV):
    """The reference's CPU path (fake-quant simulator + eager attention) on the whole workload - every
    sequence, full context - on the host cores; few repetitions rather than a smaller shape.  `value`
    is the attention step (what the metric measures); the one-time fake quantization of the context is
    reported beside it."""
    import torch
    from oracle import sim_baseline as S
    cores = os.cpu_count() or 1
    threads = min(cores, 16)
    torch.set_num_threads(threads)
    K, V = K.clone(), V.clone()
    t0 = time.perf_counter()
    S.simulate_prefill(K, V)
    t_quant = time.perf_counter() - t0
    n_rep = H_Q // H_KV
    S.eager_attention(q, K, V, 128 ** -0.5, n_rep)          # warm-up
    reps, t_att = 0, 0.0
    while reps < 2 or (t_att < 10.0 and reps < 10):
        t0 = time.perf_counter()
        S.eager_attention(q, K, V, 128 ** -0.5, n_rep)
        t_att += time.perf_counter() - t0
        reps += 1
    return {
        "value": t_att / reps * 1e6, "unit": "us/step", "cores": threads, "kind": "port",
        "sample": (f"the whole workload ({K.shape[0]} sequences x {K.shape[2]} tokens, dense fake-quantized fp16 KV, eager "
                   f"GQA attention with fp32 softmax), 1 warm-up + {reps} timed steps, torch {threads} threads; the "
                   f"fake quantization of the context took {t_quant:.2f} s once and is not part of the step"),
        "fake_quant_s_once": t_quant,
    }


def bench_chunked_prefill(args):
    print(json.dumps(chunked_prefill_result(args)))


def chunked_prefill_result(args):
    """configs[3]: a step = chunked-prefill attention of one layer; the append is timed beside it."""
    import torch
    import kitty_amd
    from kitty_amd import _lib
    from kitty_amd.kvcache.kernels import kitty_prefill_attention
    _lib.lib()
    dev = torch.device("cuda:0")
    B, H_Q, H_KV, T0, Tq, D = C3["B"], C3["H_Q"], C3["H_KV"], C3["T0"], C3["Tq"], 128
    cfg = types.SimpleNamespace(num_hidden_layers=1, head_dim=D, num_key_value_heads=H_KV,
                                num_attention_heads=H_Q, hidden_size=H_Q * D)
    mod = types.SimpleNamespace(num_attention_heads=H_Q, num_key_value_heads=H_KV)
    K, V = synth_kv(B, H_KV, T0 + Tq, D, 1003, dev, student_t=True)
    q = torch.randn((B, H_Q, Tq, D), generator=torch.Generator(device=dev).manual_seed(7), device=dev).half()
    cache = kitty_amd.KittyCache(cfg, B, T0 + Tq + 256, device=dev)
    cache.update(K[:, :, :T0], V[:, :, :T0], 0)
    cache.quantize_prefill(0)
    L = cache.kv_cache[0]
    kc, vc = K[:, :, T0:], V[:, :, T0:]
    scaling = D ** -0.5
    for _ in range(args.warmup):
        kitty_prefill_attention(mod, q, kc, vc, L, scaling)
    torch.cuda.synchronize()
    ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(args.steps)]
    t0 = time.perf_counter()
    for a, b in ev:
        a.record()
        kitty_prefill_attention(mod, q, kc, vc, L, scaling)
        b.record()
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) / args.steps * 1e3
    kern_ms = sum(a.elapsed_time(b) for a, b in ev) / len(ev)
    flops = 4.0 * B * H_Q * Tq * (T0 + Tq / 2) * D
    tflops = flops / (kern_ms * 1e-3) / 1e12
    # the append: restore the counters after each one so that every repetition does the same work
    fields = ("Sink_Count", "PageCount_K", "PageCount_V", "Q_Buffer_Count_K", "Q_Buffer_Count_V", "Local_Count_V",
              "Write_Offset_Local_V")
    saved = {f: getattr(L, f) for f in fields}
    app_ms = []
    for _ in range(5):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        cache.append(kc, vc, 0)
        e1.record()
        torch.cuda.synchronize()
        app_ms.append(e0.elapsed_time(e1))
        for f, x in saved.items():
            setattr(L, f, x)
    result = {
        "metric": "chunked_prefill_attention_ms_per_step", "value": ms_per_step, "unit": "ms/step", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": ms_per_step, "higher_is_better": False,
        "scaling": "weak", "vs_baseline": None, "dtype": "f16 operands (pages dequantized to f16), f32 accumulate",
        "data": "synthetic (seeded Student-t(3) K with 8 outlier channels/head x10, N(0,1) V and Q)",
        "config": {"workload": C3["desc"], "batch": B, "q_heads": H_Q, "kv_heads": H_KV, "head_dim": D,
                   "prefix": T0, "chunk": Tq},
        "roofline": {"bound": "mfma", "achieved": tflops, "peak": MFMA_F16_PEAK_TFLOPS, "unit": "TFLOP/s",
                     "frac": tflops / MFMA_F16_PEAK_TFLOPS, "traffic": None, "kernel": "prefill_attn_kernel",
                     "kernel_avg_us": kern_ms * 1e3, "algorithmic_flops_per_launch": flops},
        "append": {"ms": min(app_ms), "input_bytes": 2 * B * H_KV * Tq * D * 2,
                   "gbps_in": 2 * B * H_KV * Tq * D * 2 / (min(app_ms) * 1e-3) / 1e9,
                   "what": "KittyCache.append of the 2048-token chunk (16 K + 16 V pages per head, host logic included)"},
    }
    if not args.no_cpu_baseline:
        import torch.nn.functional as F
        torch.set_num_threads(min(16, os.cpu_count() or 1))
        kk, vv = K[:1, :1].float().cpu(), V[:1, :1].float().cpu()
        G = H_Q // H_KV
        qq = q[:1, :G].float().cpu()
        mask = torch.ones(Tq, T0 + Tq, dtype=torch.bool).tril_(T0)
        t1 = time.perf_counter()
        F.scaled_dot_product_attention(qq, kk.expand(1, G, -1, -1), vv.expand(1, G, -1, -1), attn_mask=mask, scale=scaling)
        dt = time.perf_counter() - t1
        result["cpu_baseline"] = {"value": dt * B * H_KV * 1e3, "unit": "ms/step", "cores": torch.get_num_threads(),
                                  "kind": "port", "sample": f"dense fp32 causal attention of 1 of {B * H_KV} "
                                  f"(sequence, KV head) units, {dt:.2f} s, scaled x{B * H_KV}"}
    return result


def bench_fake_quant(args):
    """The accuracy simulator's kernel: a step = fake quantization of one layer's dense fp16 K and V
    of the configs[1] shape as the simulator's prefill does it (keys in 128-token groups per
    channel with 25 promoted channels per block, values per token), in place."""
    import torch
    from kitty_amd import _lib, sim
    _lib.lib()
    dev = torch.device("cuda:0")
    B, H_Q, H_KV, T, desc = WORKLOADS["c1"]
    D, sink = 128, 32
    n = (T - sink) // 128 * 128
    K, V = synth_kv(B, H_KV, T, D, 1001, dev)
    blocks = K[:, :, sink:sink + n].unflatten(2, (-1, 128)).transpose(-1, -2)
    mask = sim.build_promote_mask(blocks, 0.2, 1)
    src = [(K.clone(), V.clone()) for _ in range(2)]       # 4 x 1 GiB: nothing stays in the Infinity Cache
    steps, warmup = min(args.steps, 200), min(args.warmup, 20)

    def step(i, ev=None):
        k, v = src[i % 2]
        if ev is not None:
            ev[0].record()
        sim.fake_quant_tokens_(k, sink, n, 0, 128, 2, mask, 4)
        if ev is not None:
            ev[1].record()
        sim.fake_quant_tokens_(v, sink, n, 1, 128, 2)
        if ev is not None:
            ev[2].record()

    for i in range(warmup):
        step(i)
    torch.cuda.synchronize()
    evs = [[torch.cuda.Event(enable_timing=True) for _ in range(3)] for _ in range(steps)]
    t0 = time.perf_counter()
    for i in range(steps):
        step(i, evs[i])
    torch.cuda.synchronize()
    ms_per_step = (time.perf_counter() - t0) / steps * 1e3
    k_us = sum(e[0].elapsed_time(e[1]) for e in evs) / steps * 1e3
    v_us = sum(e[1].elapsed_time(e[2]) for e in evs) / steps * 1e3
    nbytes = 2 * B * H_KV * n * D * 2                        # read + write, per tensor
    result = {
        "metric": "fake_quant_ms_per_step", "value": ms_per_step, "unit": "ms/step", "n_gpus": 1, "steps": steps,
        "warmup": warmup, "ms_per_step": ms_per_step, "higher_is_better": False, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16 (every operator of the reference's chain rounded to f16)", "data": "synthetic (as configs[1])",
        "config": {"workload": "accuracy simulator: fake quantization of one layer's dense K and V, " + desc,
                   "kbits": 2, "vbits": 2, "promote_bit": 4, "promote_ratio": 0.2, "group_size": 128},
        "roofline": {"bound": "hbm", "achieved": nbytes / (k_us * 1e-6) / 1e9, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": nbytes / (k_us * 1e-6) / 1e9 / HBM_PEAK_GBPS, "traffic": None,
                     "kernel": "fake_quant_kernel<0> (keys)", "kernel_avg_us": k_us,
                     "algorithmic_bytes_per_launch": nbytes,
                     "values_kernel": {"kernel": "fake_quant_kernel<1>", "kernel_avg_us": v_us,
                                       "achieved": nbytes / (v_us * 1e-6) / 1e9,
                                       "frac": nbytes / (v_us * 1e-6) / 1e9 / HBM_PEAK_GBPS}},
    }
    if not args.no_cpu_baseline:
        from oracle import sim_baseline as SB
        threads = min(os.cpu_count() or 1, 16)
        torch.set_num_threads(threads)
        kc, vc = K[:1].cpu(), V[:1].cpu()
        SB.simulate_prefill(kc[:, :, :sink + 1024].clone(), vc[:, :, :sink + 1024].clone(), promote_ratio=0.2)   # warm-up
        t1 = time.perf_counter()
        SB.simulate_prefill(kc, vc, promote_ratio=0.2)
        dt = time.perf_counter() - t1
        result["cpu_baseline"] = {"value": dt * B * 1e3, "unit": "ms/step", "cores": threads, "kind": "port",
                                  "sample": f"the reference's torch operators (fp16 CPU tensors) on 1 of {B} sequences "
                                            f"of the workload ({dt:.2f} s), scaled x{B}"}
    print(json.dumps(result))


def bench_generate(args):
    print(json.dumps(generate_result(args)))


def generate_result(args):
    """End-to-end as the reference measures it (latency_benchmarking/benchmark_kitty.py:127-197): a stock
    transformers model - random-init Llama-3.1-8B or Qwen3-8B shapes from a local config, nothing is
    downloaded - with ``attn_implementation="kitty"`` and a fresh ``KittyHFCache`` per run, ``generate()``
    greedy to ``max_length`` with early stopping disabled; warm-up runs, then a synchronised wall clock
    over the repeat runs."""
    import torch
    import transformers
    from kitty_amd import _lib, hf
    _lib.lib()
    hf.register()
    dev = torch.device("cuda:0")
    B, T0, max_len = args.e2e_batch, args.e2e_prompt, args.e2e_max_len
    common = dict(hidden_size=4096, num_hidden_layers=32, num_attention_heads=32, num_key_value_heads=8, head_dim=128,
                  max_position_embeddings=131072, attn_implementation="kitty")
    if args.e2e_model == "qwen3":
        cfg = transformers.Qwen3Config(vocab_size=151936, intermediate_size=12288, rope_theta=1000000.0, **common)
        cls, name = transformers.Qwen3ForCausalLM, "Qwen3-8B"
    else:
        cfg = transformers.LlamaConfig(vocab_size=128256, intermediate_size=14336, rope_theta=500000.0, **common)
        cls, name = transformers.LlamaForCausalLM, "Llama-3.1-8B"
    torch.manual_seed(0)
    old = torch.get_default_dtype()
    torch.set_default_dtype(torch.float16)
    try:
        with torch.device(dev):
            model = cls(cfg)
    finally:
        torch.set_default_dtype(old)
    model.eval()
    ids = torch.randint(0, cfg.vocab_size, (B, T0), generator=torch.Generator().manual_seed(1)).to(dev)

    def run():
        cache = hf.KittyHFCache(cfg, B, max_len, device=dev)
        out = model.generate(input_ids=ids, max_length=max_len, max_new_tokens=None, return_dict_in_generate=False,
                             do_sample=False, temperature=None, top_p=None, top_k=None, past_key_values=cache,
                             eos_token_id=None, pad_token_id=0, disable_compile=True)
        return out, cache

    with torch.no_grad():
        for _ in range(args.e2e_warmup_runs):
            run()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.e2e_repeat_runs):
            out, cache = run()
        torch.cuda.synchronize()
        dt = (time.perf_counter() - t0) / args.e2e_repeat_runs
    assert tuple(out.shape) == (B, max_len) and cache.get_seq_length(0) == max_len - 1
    cache.check_status()
    new = max_len - T0
    return {
        "metric": "end_to_end_generate_tokens_per_s", "value": B * new / dt, "unit": "tokens/s", "n_gpus": 1,
        "steps": args.e2e_repeat_runs, "warmup": args.e2e_warmup_runs, "ms_per_step": dt * 1e3 / new,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f16 model, 2/4-bit packed KV",
        "data": f"synthetic (random-init {name} shapes, random prompt tokens)",
        "config": {"workload": f"stock transformers {cls.__name__} ({name} shapes, 32 layers) through the attention hook: "
                               f"generate() of batch {B}, prompt {T0}, to max_length {max_len}, greedy, fresh cache per run",
                   "batch": B, "prompt": T0, "max_length": max_len, "layers": 32, "mode": "generate",
                   "transformers": transformers.__version__},
        "generate_s_per_run": dt, "new_tokens_per_sequence": new,
        "note": "one step = one decode iteration of generate(); the host-side launch sequence of the stock model's "
                "dense layers is inside the timed region, as in the reference's benchmark",
    }


def bench_end_to_end(args):
    if args.e2e_mode == "generate":
        return bench_generate(args)
    return bench_decode_loop(args)


def bench_decode_loop(args):
    """The side number of configs[4]: decode tokens/s of a full 32-layer Llama-3.1-8B-shaped model
    with random weights, every layer's KV in the packed cache.  The dense parts (projections, MLP,
    norms, RoPE, LM head) are plain torch; attention and the cache are this library, driven in the
    reference's call order (update -> attend -> quantize_decode, modeling_qwen3.py:225-251)."""
    import torch
    import torch.nn.functional as F
    import kitty_amd
    from kitty_amd import _lib
    from kitty_amd.kvcache.kernels import kitty_attention_forward
    _lib.lib()
    dev = torch.device("cuda:0")
    B, T0 = args.e2e_batch, args.e2e_context
    LAYERS, HID, H_Q, H_KV, D, FF, VOCAB = 32, 4096, 32, 8, 128, 14336, 128256
    cfg = types.SimpleNamespace(num_hidden_layers=LAYERS, head_dim=D, num_key_value_heads=H_KV,
                                num_attention_heads=H_Q, hidden_size=HID)
    mod = types.SimpleNamespace(num_attention_heads=H_Q, num_key_value_heads=H_KV)
    g = torch.Generator(device=dev).manual_seed(8)
    rnd = lambda *shape, std=0.02: (torch.randn(*shape, generator=g, device=dev, dtype=torch.float32) * std).half()
    layers = [dict(wqkv=rnd((H_Q + 2 * H_KV) * D, HID), wo=rnd(HID, HID), wgu=rnd(2 * FF, HID), wd=rnd(HID, FF),
                   n1=torch.ones(HID, device=dev, dtype=torch.float16),
                   n2=torch.ones(HID, device=dev, dtype=torch.float16)) for _ in range(LAYERS)]
    emb, head = rnd(VOCAB, HID), rnd(VOCAB, HID)
    nf = torch.ones(HID, device=dev, dtype=torch.float16)
    mode = args.e2e_mode
    CHECK = 6 if mode == "graph" else 0   # steps of an eager twin the graph's tokens are checked against
    steps = args.warmup + args.steps + CHECK + 4

    def make_cache():
        cache = kitty_amd.KittyCache(cfg, B, T0 + steps + 256, device=dev)
        K, V = synth_kv(B, H_KV, T0, D, 1004, dev)
        for li in range(LAYERS):          # a context of T0 tokens in every layer (same synthetic K/V)
            cache.update(K, V, li)
            cache.quantize_prefill(li)
        if mode != "host":
            cache.enable_device_counters()
        return cache

    inv_freq = 1.0 / (500000.0 ** (torch.arange(0, D, 2, device=dev, dtype=torch.float32) / D))

    def rope_table(pos):                  # pos: float or 0-d tensor -> (cos, sin), fp16 [1, D]
        ang = pos * inv_freq
        return (torch.cat([ang.cos(), ang.cos()]).half().view(1, D), torch.cat([ang.sin(), ang.sin()]).half().view(1, D))

    def rope(x, cos, sin):                # x [B, H, 1, D], rotate-half convention
        x1, x2 = x[..., : D // 2], x[..., D // 2:]
        return x * cos + torch.cat([-x2, x1], dim=-1) * sin

    def rms(x, w):
        xf = x.float()
        return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + 1e-5)).half() * w

    @torch.no_grad()
    def step(cache, tok, pos):
        x = emb[tok]                      # [B, HID]: 2-D activations keep the GEMM launches cheap
        cos, sin = rope_table(pos)
        for li, w in enumerate(layers):
            h = rms(x, w["n1"])
            qkv = F.linear(h, w["wqkv"]).view(B, 1, H_Q + 2 * H_KV, D).transpose(1, 2)
            q, k, v = qkv[:, :H_Q], qkv[:, H_Q:H_Q + H_KV], qkv[:, H_Q + H_KV:]
            q = rope(q, cos, sin).contiguous()
            if mode == "host":
                cache.update(rope(k, cos, sin), v, li)
            else:                         # the append kernel rotates the key itself (same bits)
                cache.update_with_rope(k, v, cos, sin, li)
            a, _ = kitty_attention_forward(mod, q, cache.kv_cache[li], D ** -0.5)
            cache.quantize_decode(li)
            x = x + F.linear(a.view(B, HID), w["wo"])
            h = rms(x, w["n2"])
            gu = F.linear(h, w["wgu"])
            x = x + F.linear(F.silu(gu[..., :FF]) * gu[..., FF:], w["wd"])
        return F.linear(rms(x, nf), head).argmax(-1).view(B)

    cache = make_cache()
    tok = torch.zeros(B, dtype=torch.long, device=dev)
    graph_ok = None
    if mode == "graph":
        # Device counters make the launch sequence of a step independent of the sequence lengths, so one
        # captured graph serves every step; position and token live in device buffers it updates itself.
        pos_t = torch.full((), float(T0), device=dev, dtype=torch.float32)
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):     # eager steps first: workspaces exist, libraries are initialised
            for _ in range(3):
                tok.copy_(step(cache, tok, pos_t))
                pos_t += 1
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        saved = cache.host_counters()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph):
            tok.copy_(step(cache, tok, pos_t))
            pos_t += 1
        cache.restore_host_counters(saved)   # capture ran the host bookkeeping of a step that did not execute

        def run_step(i):
            graph.replay()
            cache.step_host_counters()

        # every replay against an eager twin started from the same state, with eager work in between
        twin = make_cache()
        ttok = torch.zeros(B, dtype=torch.long, device=dev)
        for i in range(3):
            ttok = step(twin, ttok, float(T0 + i))
        graph_ok = True
        for i in range(CHECK):
            run_step(i)
            ttok = step(twin, ttok, float(T0 + 3 + i))
            torch.cuda.synchronize()
            graph_ok = graph_ok and bool(torch.equal(tok, ttok))
        graph_ok = graph_ok and twin.host_counters() == cache.host_counters() and all(
            torch.equal(a.seq_counts, b.seq_counts) for a, b in zip(cache.kv_cache, twin.kv_cache))
        del twin
        done = 3 + CHECK
    else:
        done = 0

        def run_step(i):
            nonlocal tok
            tok = step(cache, tok, float(T0 + done + i))

    for i in range(args.warmup):
        run_step(i)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(args.steps):
        run_step(args.warmup + i)
    torch.cuda.synchronize()
    dt = (time.perf_counter() - t0) / args.steps
    notes = {"host": "dense layers are torch (hipBLASLt); one Python-driven launch sequence per layer, host counters "
                     "(the reference's mode), not graph-captured",
             "device": "as host mode, but per-sequence counters on the device (append fused with the key's rotary "
                       "embedding, flush launches)",
             "graph": "per-sequence counters on the device; the whole step captured once in a HIP graph and replayed"}
    print(json.dumps({
        "metric": "end_to_end_decode_tokens_per_s", "value": B / dt, "unit": "tokens/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": dt * 1e3, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "f16 model, 2/4-bit packed KV",
        "data": "synthetic (random-init Llama-3.1-8B shapes, synthetic KV context in every layer)",
        "config": {"workload": f"32-layer Llama-3.1-8B-shaped decode, batch {B}, context {T0}, greedy (configs[4] side number)",
                   "batch": B, "context": T0, "layers": LAYERS, "mode": mode},
        "graph_tokens_match_eager": graph_ok, "final_length": cache.get_seq_length(0),
        "note": notes[mode],
    }))


def lib_check():
    import torch
    from kitty_amd import _lib
    _lib.lib()                           # raises when the HIP library is not built: no fallback
    assert torch.cuda.is_available(), "bench.py needs a GPU"


class DecodeBench:
    """One decode workload resident in HBM: the packed caches (made by the quantizer under test, enough
    independent copies to rotate over more than 3x the Infinity Cache), q, the workspace, and the
    byte counts a step has to move."""

    def __init__(self, workload, variant, args):
        import torch
        import kitty_amd
        from kitty_amd import _lib
        self.lib, self._lib, self.torch = _lib.lib(), _lib, torch
        dev = self.dev = torch.device("cuda:0")
        self.workload, self.variant = workload, variant
        B, H_Q, H_KV, T, self.desc = WORKLOADS[workload]
        self.B, self.H_Q, self.H_KV, self.T = B, H_Q, H_KV, T
        D = self.D = getattr(args, "head_dim", 128)
        if D != 128:
            self.desc = self.desc.replace("D=128", f"D={D}") + " - the plain kernels for other head dimensions"
            if workload == "c2":
                raise ValueError("per-sequence counters on the device (c2) are built for head_dim 128")
        cfg = types.SimpleNamespace(num_hidden_layers=1, head_dim=D, num_key_value_heads=H_KV,
                                    num_attention_heads=H_Q, hidden_size=H_Q * D)
        max_len = T + 256
        K, V = self.K, self.V = synth_kv(B, H_KV, T, D, 1000 + int(workload[1]), dev)
        probe = kitty_amd.KittyCache(cfg, B, max_len, device=dev)
        probe.update(K, V, 0)
        probe.quantize_prefill(0)
        seq_counts = None
        if workload == "c2":
            import numpy as np
            rng = np.random.default_rng(1002)
            rows = []
            for _ in range(B):
                Ti, Ri = int(rng.integers(1024, 16385)), int(rng.integers(0, 128))
                pk = (Ti - 32 - Ri) // 128
                rows.append([32, pk, Ri, pk - 1, Ri, 128, int(rng.integers(0, 128)), 0])
            seq_counts = torch.tensor(rows, dtype=torch.int32, device=dev)
            self.total_bytes = sum(H_KV * (5760 * r[1] + 4608 * r[3] + 256 * (2 * r[0] + r[2] + r[4] + r[5]))
                                   + 2 * H_Q * 128 * 2 for r in rows)
            self.packed_bytes = sum(H_KV * (5760 * r[1] + 4608 * r[3]) for r in rows)
        else:
            self.total_bytes, self.packed_bytes = algorithmic_bytes(B, H_Q, H_KV, probe.kv_cache[0])
        copies = args.copies or max(2, -(-3 * 256 * 2 ** 20 // self.total_bytes))      # > 3x the Infinity Cache
        copies = min(copies, 256)
        caches = [probe]
        quant_ms = []
        for i in range(1, copies + 2):       # the extra rounds only time the quantizer
            c = caches[i] if i < len(caches) else kitty_amd.KittyCache(cfg, B, max_len, device=dev)
            c.update(K, V, 0)
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            c.quantize_prefill(0)
            e1.record()
            torch.cuda.synchronize()
            quant_ms.append(e0.elapsed_time(e1))
            if i < copies:
                caches.append(c)
        if args.scatter_pages:
            gen = torch.Generator(device=dev).manual_seed(5)
            for c in caches:
                L = c.kv_cache[0]
                for codes, meta, table in ((L.KeyCache, L.KeyCache_metadata, L.PageTable_K),
                                           (L.ValueCache, L.ValueCache_metadata, L.PageTable_V)):
                    perm = torch.randperm(codes.shape[0], generator=gen, device=dev)
                    for t in (codes, meta):
                        moved = torch.empty_like(t)
                        moved[perm] = t
                        t.copy_(moved)
                    table.copy_(perm[table])
            del moved
        self.caches = caches
        L0 = self.L0 = probe.kv_cache[0]
        self.quant_ms = min(quant_ms)
        self.quant_in_bytes = 2 * B * H_KV * (L0.PageCount_K + L0.PageCount_V) * 128 * D
        self.quant_kernels = self.quantizer_kernels(K, V, L0)
        self.q = torch.randn((B, H_Q, 1, D), generator=torch.Generator(device=dev).manual_seed(7), device=dev,
                             dtype=torch.float32).half()
        self.out = torch.empty((B, 1, H_Q, D), dtype=torch.float16, device=dev)
        max_tiles = (2 + L0.MAX_PAGE) if seq_counts is not None else 1 + (T - L0.Sink_Count + 127) // 128
        self.splits = args.splits or self.lib.kitty_decode_attn_default_splits(B, H_KV, max_tiles,
                                                                               int(seq_counts is not None))
        self.ws_bytes = self.lib.kitty_decode_attn_workspace_bytes(B, H_Q, D, self.splits)
        self.ws = torch.empty(self.ws_bytes, dtype=torch.uint8, device=dev)
        if seq_counts is not None:
            for c in caches:
                c.kv_cache[0].seq_counts = seq_counts
        self.descs = [c.kv_cache[0].descriptor() for c in caches]
        self.stream = torch.cuda.current_stream(dev).cuda_stream
        self.scaling = D ** -0.5
        self.hip = HipEvents()

    def quantizer_kernels(self, K, V, L, rounds=40):
        """The K and the V quantizer alone, each launched `rounds` times back to back over the first
        cache's own pages (same input, so the same bytes again) with an event pair around every launch:
        the median of the second half is the level the kernel holds; a launch after a synchronisation
        (as `ms` of the whole call is timed) starts on an idle device."""
        torch = self.torch
        from kitty_amd.kvcache.kernels import quantize_pack_k, quantize_pack_v
        P, S, out = L.PAGE_SIZE, L.Sink_Count, {}
        calls = {"k": lambda: quantize_pack_k(K, S, L.PageCount_K, L.PageTable_K, 0, L.KeyCache, L.KeyCache_metadata,
                                              P, L.D_BOOSTED),
                 "v": lambda: quantize_pack_v(V, S, L.PageCount_V, L.PageTable_V, 0, L.ValueCache,
                                              L.ValueCache_metadata, P)}
        for name, call in calls.items():
            pages = L.PageCount_K if name == "k" else L.PageCount_V
            if pages == 0:
                continue
            ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(rounds)]
            for a, b in ev:
                a.record()
                call()
                b.record()
            torch.cuda.synchronize()
            us = sorted(a.elapsed_time(b) * 1e3 for a, b in ev[rounds // 2:])
            head = self.B * self.H_KV * pages
            in_bytes = head * P * self.D * 2
            out_bytes = head * ((32 * (self.D + L.D_BOOSTED) + self.D + 4 * self.D) if name == "k" else (32 * self.D + 512))
            med = us[len(us) // 2]
            out[name] = {"median_us": med, "min_us": us[0], "gbps_in": in_bytes / med / 1e3,
                         "hbm_frac": (in_bytes + out_bytes) / med / 1e3 / HBM_PEAK_GBPS,
                         "bytes_in": in_bytes, "bytes_out": out_bytes, "launches": rounds}
        return out

    def step(self, i, ev=None, variant=None):
        lib, _lib = self.lib, self._lib
        d = self.descs[i % len(self.descs)]
        if ev is not None:     # the events ride on the split kernel's own dispatch: its duration on the device
            _lib.check(lib.kitty_profile_next_split(ev[0], ev[1]), "profile")
        rc = lib.kitty_decode_attn_split(d, self.q.data_ptr(), self.B, self.H_Q, self.scaling, self.ws.data_ptr(),
                                         self.ws_bytes, self.splits, self.variant if variant is None else variant,
                                         self.stream)
        _lib.check(rc, "split")
        _lib.check(lib.kitty_decode_attn_merge(self.ws.data_ptr(), self.ws_bytes, self.B, self.H_Q, self.D, self.splits,
                                               self.out.data_ptr(), self.stream), "merge")

    def settle(self, variant=None, max_windows=150):
        """Untimed launches until the kernel's duration has reached its SUSTAINED level.  After idle the
        clocks first rise (the first ~100 launches run 5-8 % slower) and then, under a load that keeps
        the package at its power limit, come down again over some thousand launches to the level they
        hold for good; a window that is separated from the next by a host synchronisation reads the
        level in between.  So the windows run back to back, 100 launches each with the events on every
        fifth launch, and the run counts as settled once the median of a window stays within 1 % of
        the previous one for three windows in a row after at least 10 windows (1000 launches)."""
        hip = self.hip
        n_win, every = 100, 5
        sets = [[(hip.create(), hip.create()) for _ in range(n_win // every)] for _ in range(2)]
        settle = {"windows": 0, "launches": 0, "median_us": None, "settled": False, "window_medians_us": []}
        prev, stable, pending = None, 0, None
        for w in range(max_windows):
            cur = sets[w % 2]
            for j in range(n_win):
                self.step(self.n_done, cur[j // every] if j % every == 0 else None, variant)
                self.n_done += 1
            if pending is not None:   # read window w - 1 while window w runs: the device is never idle in between
                hip.synchronize(pending[-1][1])
                med = sorted(hip.elapsed_us(a, b) for a, b in pending)[len(pending) // 2]
                settle["window_medians_us"].append(round(med, 2))
                stable = stable + 1 if prev is not None and abs(med - prev) <= 0.01 * prev else 0
                prev = med
                settle.update(windows=w, launches=w * n_win, median_us=med)
                if stable >= 3 and w >= 10:
                    settle["settled"] = True
                    break
            pending = cur
        return settle

    def timed(self, steps, warmup, variant=None):
        """`steps` steps as a caller runs them (wall clock, synchronised on both sides), then the same
        steps twice more with events on the split kernel's dispatch: once right after the
        synchronisation, as the wall clock saw them, and once behind `warmup` + 20 untimed steps
        with no wait in between.  The first launch after a blocking synchronisation reads 15-20 us
        long and the next ones up to 5 us, on some boxes; the kernel's own duration is the second
        figure, which is also what a kernel trace of the run averages to."""
        torch, hip = self.torch, self.hip
        events = [(hip.create(), hip.create()) for _ in range(2 * steps)]   # before the warm-up: no host work (and
        for i in range(warmup):                                              # no idle device) between it and the timed steps
            self.step(self.n_done + i, None, variant)
        self.n_done += warmup
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(steps):
            self.step(self.n_done + i, None, variant)
        torch.cuda.synchronize()
        us_per_step = (time.perf_counter() - t0) / steps * 1e6
        t0 = time.perf_counter()
        for i in range(steps):
            self.step(self.n_done + i, events[i], variant)
        torch.cuda.synchronize()
        us_per_step_events = (time.perf_counter() - t0) / steps * 1e6
        self.n_done += 2 * steps
        for i in range(warmup + 20):
            self.step(self.n_done + i, None, variant)
        self.n_done += warmup + 20
        for i in range(steps):
            self.step(self.n_done + i, events[steps + i], variant)
        torch.cuda.synchronize()
        self.n_done += steps
        self.kern_us_after_sync = sorted(hip.elapsed_us(a, b) for a, b in events[:steps])
        kern_us = sorted(hip.elapsed_us(a, b) for a, b in events[steps:])
        return us_per_step, us_per_step_events, kern_us

    n_done = 0

    def summary(self, steps, warmup, variant=None, max_windows=30):
        """The fields of the headline for a side workload: settled briefly, then timed."""
        settle = self.settle(variant, max_windows=max_windows)
        us_per_step, _, kern_us = self.timed(steps, warmup, variant)
        avg = sum(kern_us) / len(kern_us)
        gbps = self.total_bytes / (avg * 1e-6) / 1e9
        return {"workload": self.desc, "variant": self.variant if variant is None else variant,
                "num_splits": self.splits, "value": us_per_step, "unit": "us/step", "steps": steps,
                "kernel": "decode split pass" + (" (one round of flat shares)" if self.workload == "c2" else ""),
                "kernel_avg_us": avg, "kernel_median_us": kern_us[len(kern_us) // 2],
                "algorithmic_bytes_per_launch": self.total_bytes, "packed_bytes_per_launch": self.packed_bytes,
                "achieved_gbps": gbps, "frac": gbps / HBM_PEAK_GBPS,
                "packed_frac": self.packed_bytes / (avg * 1e-6) / 1e9 / HBM_PEAK_GBPS,
                "kernel_avg_us_after_sync": sum(self.kern_us_after_sync) / len(self.kern_us_after_sync),
                "settled_after_launches": settle["launches"], "settled": settle["settled"]}

    def headline(self, args):
        torch, hip = self.torch, self.hip
        settle = self.settle()
        us_per_step, us_per_step_events, kern_us = self.timed(args.steps, args.warmup)
        kern_avg_us = sum(kern_us) / len(kern_us)
        achieved = self.total_bytes / (kern_avg_us * 1e-6) / 1e9
        # cache-hot figure (same copy every step), reported separately
        win = [(hip.create(), hip.create()) for _ in range(20)]
        for i in range(20):
            self.step(0, win[i])
        torch.cuda.synchronize()
        hot_us = sorted(hip.elapsed_us(a, b) for a, b in win)[len(win) // 2]
        if args.copy_calibration:
            src = torch.empty(1 << 30, dtype=torch.uint8, device=self.dev).fill_(3)
            dst = torch.empty_like(src)
            for _ in range(5):
                dst.copy_(src)
            torch.cuda.synchronize()
        L0 = self.L0
        return {
            "metric": "packed_kv_decode_attention_us_per_step",
            "value": us_per_step,
            "unit": "us/step",
            "n_gpus": 1,
            "steps": args.steps,
            "warmup": args.warmup,
            "ms_per_step": us_per_step * 1e-3,
            "higher_is_better": False,
            "scaling": "weak",
            "vs_baseline": None,
            "dtype": "u8 codes + f16 scales/zeros, f32 accumulate",
            "data": "synthetic (seeded N(0,1) K with 8 outlier channels/head x10, N(0,1) V, random-init)",
            "config": {"workload": self.desc, "batch": self.B, "q_heads": self.H_Q, "kv_heads": self.H_KV,
                       "head_dim": self.D, "context": self.T, "pages_k": L0.PageCount_K, "pages_v": L0.PageCount_V,
                       "num_splits": self.splits, "variant": self.variant, "cache_copies_rotated": len(self.caches),
                       "page_placement": "scattered" if args.scatter_pages else "identity"},
            "roofline": {
                "bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                "frac": achieved / HBM_PEAK_GBPS, "traffic": measured_traffic(self.workload, self.splits),
                "kernel": "decode split pass", "kernel_avg_us": kern_avg_us,
                "kernel_median_us": kern_us[len(kern_us) // 2],
                "algorithmic_bytes_per_launch": self.total_bytes, "packed_bytes_per_launch": self.packed_bytes,
                "packed_gbps": self.packed_bytes / (kern_avg_us * 1e-6) / 1e9,
                "packed_frac": self.packed_bytes / (kern_avg_us * 1e-6) / 1e9 / HBM_PEAK_GBPS,
                "cache_hot_kernel_us": hot_us,
                "timing": "HIP events attached to the split kernel's dispatch on the launch stream (kernel begin to "
                          "end), averaged over the timed steps run again with the events attached (their marker "
                          "packets cost a step about 5 us, so `value` is timed without them) behind untimed steps "
                          "with no wait in between; `kernel_avg_us_after_sync`: the same steps right after a "
                          "synchronisation, as `value` runs them (the first launch after a blocking wait reads "
                          "15-20 us long, the next ones up to 5 us on some boxes)",
                "kernel_avg_us_after_sync": sum(self.kern_us_after_sync) / len(self.kern_us_after_sync),
                "kernel_median_us_after_sync": self.kern_us_after_sync[len(self.kern_us_after_sync) // 2],
                "us_per_step_with_events": us_per_step_events,
                "traffic_source": "rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE summary committed under profiles/ (a run "
                                  "of its own, calibrated by a 1 GiB copy), not measured in this run",
                "clock_settling": settle,
            },
            "quantizer": {"gbps_in": self.quant_in_bytes / (self.quant_ms * 1e-3) / 1e9, "ms": self.quant_ms,
                          "input_bytes": self.quant_in_bytes,
                          "what": "quantize_prefill of the whole context (K select+quantize+pack, V quantize+pack) "
                                  "after a synchronisation; `kernels`: each kernel alone, launched back to back",
                          "kernels": self.quant_kernels},
        }


def other_workloads(headline, args):
    """The other BASELINE configs and the plain kernel, measured in this process after the headline so
    that one run of the default command holds a figure for each: same fields as the headline's
    roofline, fewer steps.  A workload that fails leaves its error text instead of stopping the run."""
    import gc
    import torch
    out = {}

    def guarded(name, fn):
        try:
            out[name] = fn()
        except Exception as e:                       # noqa: BLE001 - the headline must survive a side workload
            out[name] = {"error": f"{type(e).__name__}: {e}"[:300]}
        gc.collect()
        torch.cuda.empty_cache()

    side = types.SimpleNamespace(copies=0, splits=0, scatter_pages=False, head_dim=128)
    guarded("c1_variant1", lambda: headline.summary(10, 3, variant=1, max_windows=4))
    for name in ("c0", "c2", "c4"):
        guarded(name, lambda name=name: DecodeBench(name, 0, side).summary(40, 5))
    c3_args = types.SimpleNamespace(steps=5, warmup=2, no_cpu_baseline=True)
    guarded("c3", lambda: chunked_prefill_result(c3_args))
    e2e = types.SimpleNamespace(e2e_batch=16, e2e_prompt=64, e2e_max_len=192, e2e_model="llama", e2e_warmup_runs=1,
                                e2e_repeat_runs=1)
    guarded("e2e_generate", lambda: generate_result(e2e))
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    # the defaults are long enough for the clocks to settle: the first ~100 launches after idle run 5-8 % slower
    ap.add_argument("--steps", type=int, default=2000)
    ap.add_argument("--warmup", type=int, default=500)
    ap.add_argument("--workload", default="c1", choices=sorted(WORKLOADS) + ["c3", "e2e", "fq"])
    ap.add_argument("--e2e-batch", type=int, default=16)
    ap.add_argument("--e2e-context", type=int, default=32768)
    ap.add_argument("--e2e-mode", default="generate", choices=["generate", "host", "device", "graph"],
                    help="generate: a stock transformers model through the attention hook, generate() as the "
                         "reference's benchmark runs it; the others drive hand-written dense layers around the cache "
                         "over a long synthetic context - host: the reference's shared host counters; device: "
                         "per-sequence counters on the device; graph: device counters and the whole step replayed "
                         "from one captured HIP graph")
    ap.add_argument("--e2e-model", default="llama", choices=["llama", "qwen3"])
    ap.add_argument("--e2e-prompt", type=int, default=64)
    ap.add_argument("--e2e-max-len", type=int, default=1024)
    ap.add_argument("--e2e-warmup-runs", type=int, default=1)
    ap.add_argument("--e2e-repeat-runs", type=int, default=2)
    ap.add_argument("--copies", type=int, default=0, help="independent cache copies to rotate over (0 = auto)")
    ap.add_argument("--splits", type=int, default=0)
    ap.add_argument("--variant", type=int, default=0)
    ap.add_argument("--head-dim", type=int, default=128, choices=[64, 128, 256],
                    help="c0 / c1 / c4 with another head dimension (the untuned kernels for 64 and 256)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-other-workloads", action="store_true",
                    help="default workload only: leave out the `workloads` key (configs[0], [2], [3], [4], the plain "
                         "kernel on configs[1] and a short generate() run, each measured after the headline)")
    ap.add_argument("--scatter-pages", action="store_true",
                    help="place every packed page at a random position of the page arrays (page tables to match), "
                         "as a page pool leaves them after sequences have come and gone; default: the reference's "
                         "identity tables")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 1 GiB device copy a few times, so that a counter run of this command "
                         "holds a kernel of known traffic to scale FETCH_SIZE / WRITE_SIZE by")
    args = ap.parse_args()
    if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
        print("bench.py: this build measures the one-GPU kernel path only; run with --gpus 1 "
              "(no collectives, sharding or multi-rank code exists in this path)", file=sys.stderr)
        sys.exit(2)

    if args.workload == "c3":
        return bench_chunked_prefill(args)
    if args.workload == "e2e":
        return bench_end_to_end(args)
    if args.workload == "fq":
        return bench_fake_quant(args)
    lib_check()
    headline = DecodeBench(args.workload, args.variant, args)
    result = headline.headline(args)
    if args.head_dim != 128:     # a side measurement of the plain kernels: neither the host baseline nor the other configs
        args.no_cpu_baseline = args.no_other_workloads = True
        result["roofline"]["traffic"] = None
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(headline.K.cpu(), headline.V.cpu(), headline.q.cpu(), headline.H_Q,
                                              headline.H_KV)
    if args.workload == "c1" and not args.no_other_workloads:
        result["workloads"] = other_workloads(headline, args)
    print(json.dumps(result))


if __name__ == "__main__":
    main()
