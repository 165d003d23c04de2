"""Writes tests/golden/bcq_shift_reference.npz: (B, alpha) produced by the
ShiftAddLLM checkout's own BCQ-with-power-of-two-scales quantiser on small seeded
inputs.  Runs only where the checkout is present (the build container); the
fixture, not the checkout, travels with the repository.

What is called: the inner CPU functions of quantizers/bcq_quant/bcq_shift.py
(greedy_mean_torch, then `rounds` x refine_mean_torch with use_bst=True,
apot_nums=1) -- the body of quantize_shift (bcq_shift.py:82-129) without its
.cuda() call.  Usage:  python tests/golden/make_bcq_fixture.py [/root/reference]
"""
import importlib.util
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))


def load_reference(root):
    path = os.path.join(root, "quantizers", "bcq_quant", "bcq_shift.py")
    spec = importlib.util.spec_from_file_location("ref_bcq_shift", path)
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)
    return mod


def reference_quantize(ref, w, nb, rounds):
    wf = torch.ones(w.shape, dtype=torch.float32)
    ret, B, alpha = ref.greedy_mean_torch(w.clone(), n_bits=nb, wf=wf)
    if rounds > 0 and nb > 1:
        for _ in range(rounds):
            ret, B, alpha = ref.refine_mean_torch(w, ret, B, alpha, wf=wf, use_bst=True, apot_nums=1)
    return B, alpha


def main():
    root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
    ref = load_reference(root)
    out = {}
    for case, (rows, gs, nb, sigma, seed) in enumerate([(32, 128, 3, 0.02, 0), (32, 128, 2, 0.02, 1),
                                                        (16, 128, 4, 0.015, 2), (8, 64, 3, 1.0, 3)]):
        g = torch.Generator().manual_seed(seed)
        w = torch.randn((rows, gs), generator=g) * sigma
        B, alpha = reference_quantize(ref, w, nb, rounds=5)
        out[f"w{case}"] = w.numpy()
        out[f"B{case}"] = B.numpy().astype(np.int8)
        out[f"alpha{case}"] = alpha.numpy().astype(np.float32)
        out[f"nb{case}"] = np.int32(nb)
    out["cases"] = np.int32(4)
    np.savez_compressed(os.path.join(HERE, "bcq_shift_reference.npz"), **out)
    print("wrote", os.path.join(HERE, "bcq_shift_reference.npz"))


if __name__ == "__main__":
    main()
