"""Writes tests/golden/topk_golden.npz: inputs and expected outputs of the upstream naive `torch_topk`
(flash_nsa/ops/torch_ref.py:64-105), the one function of the path whose conventions (weights, forced-block
marking, per-row valid count) no closed form pins.  Run once in the build container, where the upstream tree is
mounted read-only; the resulting file is plain data and is what the tests read.

    python tests/golden/make_topk_golden.py /root/reference
"""
import importlib.util
import sys

import numpy as np
import torch


def main(ref_root):
    spec = importlib.util.spec_from_file_location("_upstream_torch_ref", f"{ref_root}/flash_nsa/ops/torch_ref.py")
    mod = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(mod)

    cases = [
        # T, QH, KH, D, kernel, stride, block, topn, init, local, seed
        (321, 4, 1, 32, 32, 16, 64, 16, 1, 2, 0),
        (200, 8, 2, 32, 32, 16, 64, 4, 1, 2, 1),
        (1100, 4, 2, 16, 32, 16, 64, 16, 1, 2, 2),
        (48, 4, 1, 32, 32, 16, 64, 16, 1, 2, 3),
        (31, 4, 1, 32, 32, 16, 64, 16, 1, 2, 4),
        (700, 4, 1, 16, 32, 16, 64, 8, 2, 1, 5),
        (520, 4, 2, 16, 64, 32, 128, 4, 1, 1, 6),
        (600, 2, 1, 16, 32, 8, 32, 6, 1, 2, 7),
    ]
    out = {"n_cases": np.array(len(cases))}
    for ci, (T, QH, KH, D, K, S, Bs, N, I, Lc, seed) in enumerate(cases):
        g = torch.Generator().manual_seed(seed)
        q = torch.randn(T, QH, D, generator=g)
        y = max((T - K) // S + 1, 0)
        ck = torch.randn(y, KH, D, generator=g)
        topk = mod.torch_topk(q, ck, K, S, Bs, N, I, Lc, ignore_idx=99999999)
        out[f"c{ci}_params"] = np.array([T, QH, KH, D, K, S, Bs, N, I, Lc, seed])
        out[f"c{ci}_q"] = q.numpy()
        out[f"c{ci}_ck"] = ck.numpy()
        out[f"c{ci}_topk"] = topk.numpy().astype(np.int64)
    np.savez_compressed("tests/golden/topk_golden.npz", **out)
    print("wrote tests/golden/topk_golden.npz")


if __name__ == "__main__":
    main(sys.argv[1] if len(sys.argv) > 1 else "/root/reference")
