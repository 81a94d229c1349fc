"""Writes tests/golden/fused_ops_golden.npz by RUNNING the reference's own Triton kernels
(src/p2/search/fused_cfr_triton.py) under Triton's CPU interpreter (TRITON_INTERPRET=1) in the
build container.  Run once, here only:  python tests/golden/gen_fused_ops_golden.py

Inputs are the seeded ones of tests/fused_op_cases.py (rebuilt by the tests, not stored); the
fixture holds every output restricted to 64 seeded hand columns plus its full float64 row sums.
All kernels are called through the reference's public wrappers, with two exceptions whose
wrappers refuse CPU tensors before launching (``fused_block_and_normalize_beliefs_``, :286-336,
and ``unblocked_mass_triton``, :1110-1160): for these the wrapper's own launch lines are repeated
here verbatim in meaning (same kernel, grid, constants).  What this pins beyond the numpy oracle's
reading of the code: the kernels' own arithmetic order, and the three places where the fused
evaluator departs from the base class — the reach kernel writes child rows only, the belief kernel
skips the roots, the average-value kernel multiplies by 1/(old+new).
"""
from __future__ import annotations

import os
import sys

os.environ["TRITON_INTERPRET"] = "1"          # before triton is imported
os.environ.setdefault("TORCHDYNAMO_DISABLE", "1")

import numpy as np  # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(os.path.dirname(HERE))
sys.path.insert(0, HERE)
sys.path.insert(0, ROOT)
from gen_cfr_golden import REF_SRC, install_stand_ins  # noqa: E402


def main() -> None:
    install_stand_ins()
    sys.path.insert(0, REF_SRC)
    import torch
    from p2.search import fused_cfr_triton as F
    from tests import fused_op_cases as C
    assert F.triton_is_available()

    def block_normalize(target, allowed, prob, eps=1e-5):      # fused_cfr_triton.py:310-336 without the CUDA assert
        if target.dim() == 3:
            n, p, h = target.shape
            rows, stride = n * p, p
        else:
            n, h = target.shape
            rows, stride = n, 1
        F._fused_block_normalize_kernel[(rows,)](target, allowed, prob, stride, h, eps, BLOCK_H=512, num_warps=4)

    def unblocked_mass(target):                                 # :1130-1160 without the CUDA check
        flat = target.reshape(-1, 1326).contiguous()
        b, h = flat.shape
        card_a, card_b = F._get_combo_cards(flat.device)
        s, cardsum = F._preprocess_unblocked_stats(flat)
        out = torch.empty_like(flat)
        F._unblocked_mass_finalize_kernel[(b,)](flat, cardsum.contiguous(), s.contiguous(), card_a, card_b, out, h,
                                                NUM_CARDS=52, BLOCK_H=2048, num_warps=4)
        return out.view(target.shape)

    rng = np.random.default_rng(99)
    cols = np.sort(rng.choice(1326, 64, replace=False))
    out = {"columns": cols, "case_names": np.array(C.NAMES)}
    for name in C.NAMES:
        x = C.inputs(name)
        got = C.torch_ops(name, x, F, torch.device("cpu"), raw={"block_normalize": block_normalize,
                                                               "unblocked_mass": unblocked_mass})
        for key, t in got.items():
            a = t.detach().cpu().numpy()
            out[f"{name}/{key}"] = np.ascontiguousarray(a[..., cols]).astype(np.float32)
            out[f"{name}/{key}_rowsum"] = a.astype(np.float64).sum(-1)
        print(name, {k: tuple(v.shape) for k, v in got.items()}, flush=True)
    path = os.path.join(HERE, "fused_ops_golden.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, os.path.getsize(path) // 1024, "KiB")


if __name__ == "__main__":
    main()
