"""Writes the quantizer golden vectors under tests/golden/.

Runs the reference's own ``quantize_pack_k`` / ``quantize_pack_v``
(src/kitty/kvcache/kernels/kitty_quant_pack.py:253-356) on CPU tensors through
Triton's CPU interpreter and stores inputs and outputs as ``.npz`` data.  The
reference file is loaded by path (it imports only torch and triton); nothing
from it is copied.  Only this container has the reference mounted, so the
vectors are committed and the tests read the ``.npz`` files, never the
reference.

    TRITON_INTERPRET=1 python tests/golden/make_quant_golden.py [case name ...]

Without names every case is written; with names only those (the cases for head dimensions 64 and 256
were added later than the others).
"""
import importlib.util
import os
import sys

os.environ.setdefault("TRITON_INTERPRET", "1")
sys.dont_write_bytecode = True      # the reference checkout is read-only: leave no __pycache__ beside its file

import numpy as np
import torch

REF = "/root/reference/src/kitty/kvcache/kernels/kitty_quant_pack.py"
OUT = os.path.dirname(os.path.abspath(__file__))


def load_reference():
    spec = importlib.util.spec_from_file_location("ref_kitty_quant_pack", REF)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def make_inputs(case, seed):
    g = torch.Generator().manual_seed(seed)
    B, H, T, D = case["B"], case["H"], case["T"], case.get("D", 128)
    kind = case["kind"]
    if kind == "normal_outlier":
        x = torch.randn(B, H, T, D, generator=g)
        for h in range(H):
            ch = torch.randperm(D, generator=g)[:8]
            x[:, h, :, ch] *= 10.0
    elif kind == "student_t":
        z = torch.randn(B, H, T, D, generator=g)
        chi = torch.randn(B, H, T, D, 3, generator=g).pow(2).sum(-1) / 3.0
        x = z / chi.sqrt()
        for h in range(H):
            ch = torch.randperm(D, generator=g)[:8]
            x[:, h, :, ch] *= 10.0
    elif kind == "spread":
        # every channel gets its own magnitude so that the boost scores are far apart:
        # any correct top-k then returns the same slot map (no ties to break)
        x = torch.randn(B, H, T, D, generator=g)
        for h in range(H):
            mult = 1.06 ** (torch.randperm(D, generator=g).float() * (128.0 / D))   # same spread of magnitudes for every D
            x[:, h] *= mult.view(1, 1, D)
    elif kind == "edge":
        # constant groups, tiny ranges, large magnitudes, subnormals, exact .5 ties
        x = torch.randn(B, H, T, D, generator=g)
        x[:, :, :, 0] = 0.0                       # constant zero channel
        x[:, :, :, 1] = 3.25                      # constant non-zero channel
        x[:, :, :, 2] = 1.0 + 1e-3 * torch.randn(B, H, T, generator=g)   # tiny range
        x[:, :, :, 3] *= 6e-6                     # fp16 subnormal range
        x[:, :, :, 4] *= 2000.0                   # large values
        x[:, :, :, 5] = (torch.arange(T) % 16).float().view(1, 1, T) * 0.5      # exact ramp
        x[:, :, :, 6] = (torch.arange(T) % 4).float().view(1, 1, T)             # 4 exact levels
        x[:, :, :, 7] = (torch.arange(T) % 7).float().view(1, 1, T) * 0.5       # .5 rounding ties
        x[:, :, 5, :] = 0.0                       # constant token (V side)
        x[:, :, 6, :] = -7.5                      # constant token (V side)
        x[:, :, 7, :] = (torch.arange(D) % 4).float() * 0.25                    # V KAT: codes 0..3
        x[:, :, 8, :] = (torch.arange(D) % 7).float() * 0.5                     # V ties
    else:
        raise ValueError(kind)
    return x.to(torch.float16)


CASES = [
    dict(name="k_v_normal", kind="normal_outlier", B=2, H=2, T=32 + 2 * 128 + 5, t_offset=32, pages=2,
         max_page=3, page_offset=0, seed=11),
    dict(name="k_v_student", kind="student_t", B=1, H=2, T=128, t_offset=0, pages=1,
         max_page=4, page_offset=2, seed=12),
    dict(name="k_v_spread", kind="spread", B=1, H=2, T=2 * 128, t_offset=0, pages=2,
         max_page=2, page_offset=0, seed=14),
    dict(name="k_v_edge", kind="edge", B=1, H=1, T=128, t_offset=0, pages=1,
         max_page=2, page_offset=1, seed=13),
    # other head dimensions (the reference boosts head_dim // 4 channels, kitty.py:44); tie-free scores
    dict(name="k_v_d64", kind="spread", D=64, B=1, H=2, T=32 + 2 * 128, t_offset=32, pages=2,
         max_page=3, page_offset=1, seed=15),
    dict(name="k_v_d256", kind="spread", D=256, B=1, H=1, T=128, t_offset=0, pages=1,
         max_page=2, page_offset=1, seed=16),
]


def tie_free(x, case, d_boost):
    """True when, on every page-head, the top-(d_boost+1) fp16 scores are pairwise distinct."""
    t0, P = case["t_offset"], case["pages"]
    B, H, _, D = x.shape
    pages = x[:, :, t0: t0 + 128 * P].reshape(B, H, P, 128, D)
    score = pages.abs().mean(dim=-2).double()
    top = score.sort(dim=-1, descending=True).values[..., : d_boost + 1]
    return bool((top[..., 1:] < top[..., :-1]).all())


def main():
    ref = load_reference()
    PAGE = 128
    only = set(sys.argv[1:])
    for case in CASES:
        if only and case["name"] not in only:
            continue
        D = case.get("D", 128)
        DB = D // 4
        x = make_inputs(case, case["seed"])
        if case["kind"] == "spread":
            seed = case["seed"]
            while not tie_free(x, case, DB):
                seed += 1000
                x = make_inputs(case, seed)
            print("spread case uses seed", seed)
        B, H = case["B"], case["H"]
        MAXP = case["max_page"]
        bytes_k = H * (PAGE // 4 * (D + DB) + D)
        bytes_v = H * PAGE * D // 4
        # a permuted (non-identity) page table exercises the page indirection
        perm = torch.randperm(B * MAXP, generator=torch.Generator().manual_seed(case["seed"] + 100))
        page_table = perm.view(B, MAXP).to(torch.int64)
        kc = torch.zeros(B * MAXP, bytes_k, dtype=torch.uint8)
        km = torch.zeros(B * MAXP, H, D, 2, dtype=torch.float16)
        vc = torch.zeros(B * MAXP, bytes_v, dtype=torch.uint8)
        vm = torch.zeros(B * MAXP, H, PAGE, 2, dtype=torch.float16)
        ref.quantize_pack_k(x, case["t_offset"], case["pages"], page_table, case["page_offset"], kc, km, PAGE, DB)
        ref.quantize_pack_v(x, case["t_offset"], case["pages"], page_table, case["page_offset"], vc, vm, PAGE)
        path = os.path.join(OUT, f"quant_{case['name']}.npz")
        np.savez_compressed(
            path,
            x=x.numpy(), t_offset=case["t_offset"], pages=case["pages"], page_offset=case["page_offset"],
            page_table=page_table.numpy(), d_boost=DB, page_size=PAGE,
            key_cache=kc.numpy(), key_meta=km.numpy(), value_cache=vc.numpy(), value_meta=vm.numpy(),
        )
        print("wrote", path, "K bytes nonzero:", int((kc != 0).sum()), "V bytes nonzero:", int((vc != 0).sum()))


if __name__ == "__main__":
    sys.exit(main())
