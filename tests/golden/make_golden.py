"""Writes tests/golden/quantize_helpers_golden.npz.

Runs in the build container only (needs the reference checkout; the GPU box
has none).  It loads ONE reference file, quantize/quantize_helpers.py (numpy
and torch only, no compiled extension), by path, feeds it small seeded inputs
and stores inputs and outputs as plain arrays.  No reference text or object is
stored: only numbers.

The vectors pin what reading alone cannot: which code the reference's fp16
CPU quantiser picks at rounding boundaries, its permutation tables, and its
pack / unpack pair.

    python tests/golden/make_golden.py [/root/reference]
"""
import importlib.util
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))


def load_reference_helpers(root):
    path = os.path.join(root, "quantize", "quantize_helpers.py")
    spec = importlib.util.spec_from_file_location("_ref_quantize_helpers", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def main():
    root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    ref = load_reference_helpers(root)
    out = {}

    out["weight_perm"] = ref.get_w4a16_weight_perms().numpy().astype(np.int64)
    sp, sp1 = ref.get_scale_perms()
    out["scale_perm"] = np.asarray(sp, dtype=np.int64)
    out["scale_perm_single"] = np.asarray(sp1, dtype=np.int64)

    # case A: K=256, N=256, no padding.  case B: K=256, N=320 -> pad_out 192.
    # case C: K=200 (not a multiple of 128 -> zero rows appended), N=256,
    #         with an all-zero group column to exercise the 0/0 -> code 8 rule.
    gen = torch.Generator().manual_seed(1234)
    cases = {"A": (256, 256, 0), "B": (256, 320, 192), "C": (200, 256, 0)}
    for name, (k, n, pad_out) in cases.items():
        w = (torch.randn(k, n, generator=gen) * 0.05).to(torch.float16)
        if name == "C":
            w[:128, 7] = 0
        # a few exact ties: element = (j + 0.5) * scale-ish values
        w[0, 0] = w[:128, 0].abs().max() * 0.5
        w_ref, packed, scale = ref.w4a16_quantize(w.clone(), 4, 128, None, pad_out=pad_out)
        out[f"{name}_w"] = w.numpy()
        if name == "A":
            out[f"{name}_w_ref"] = w_ref.numpy()
        out[f"{name}_packed"] = packed.numpy()
        out[f"{name}_scale"] = scale.numpy()
        kp, np_ = w_ref.shape
        perm = ref.get_w4a16_weight_perms()
        q = ref.unpack_w4a16_permute_weights(packed, kp, np_, 4, perm, 128)
        out[f"{name}_codes"] = q.numpy().astype(np.uint8)
        out[f"{name}_scale_unperm"] = ref.w4a16_unpermute_scales(scale, kp, np_, 128).numpy()

    # the GPTQ branch: codes re-derived from given group scales
    k, n = 256, 256
    w = (torch.randn(k, n, generator=gen) * 0.05).to(torch.float16)
    w_fq, _, s = ref.get_fake_quantize_weights(w.clone(), 4, 128)
    w_ref, packed, scale = ref.w4a16_quantize(w_fq.clone(), 4, 128, s.clone(), pad_out=0)
    out["G_w"] = w_fq.numpy()
    out["G_scale_in"] = s.numpy()
    out["G_packed"] = packed.numpy()
    out["G_scale"] = scale.numpy()

    # raw pack of uniform random codes (the benchmark's generator): K=128, N=512
    codes = torch.randint(0, 16, (128, 512), generator=gen, dtype=torch.int32)
    perm = ref.get_w4a16_weight_perms()
    out["P_codes"] = codes.numpy().astype(np.uint8)
    out["P_packed"] = ref.get_w4a16_permute_weights(codes, 128, 512, 4, perm, 128).numpy()

    # scale permutations in both modes on an index ramp
    ramp = torch.arange(2 * 256, dtype=torch.float32).reshape(2, 256).to(torch.float16)
    out["S_ramp"] = ramp.numpy()
    out["S_grouped"] = ref.w4a16_permute_scales(ramp.clone(), 256, 256, 128).numpy()
    ramp1 = torch.arange(256, dtype=torch.float32).reshape(1, 256).to(torch.float16)
    out["S_ramp1"] = ramp1.numpy()
    out["S_single"] = ref.w4a16_permute_scales(ramp1.clone(), 128, 256, 128).numpy()

    dst = os.path.join(HERE, "quantize_helpers_golden.npz")
    np.savez_compressed(dst, **out)
    print("wrote", dst, os.path.getsize(dst), "bytes;", len(out), "arrays")


if __name__ == "__main__":
    main()
