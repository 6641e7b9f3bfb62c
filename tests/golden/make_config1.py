"""Writes tests/golden/config1.npz: the CPU-plumbing configuration (bf16 A[32,512] ~N(0,1), seed 0;
W[256,512] ~N(0,0.02) block-quantised 128x128; per-token-group FP8 quant of A, group 128; block-FP8
matmul to bf16 C[32,256]) evaluated by the CPU oracle in this repository.

The reference holds no stored vectors for this path (every expected value in its tests is
recomputed by a torch oracle at test time), so these vectors come from the restatement in oracle/;
they freeze it against later edits and give the GPU tests fixed data.

Run from the repository root:  python tests/golden/make_config1.py
"""
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

from oracle import gemm as og  # noqa: E402
from oracle import quant as oq  # noqa: E402


def main():
    torch.manual_seed(0)
    a = torch.randn(32, 512).to(torch.bfloat16)
    w = torch.randn(256, 512) * 0.02
    aq, a_s, _ = oq.group_quant(a, 128, form="divide")
    aq2, a_s2, _ = oq.group_quant(a, 128, form="reciprocal")
    _, _, a_e8 = oq.group_quant(a, 128, form="divide", scale_ue8m0=True)
    wq, w_s = oq.block_quant_weight(w)
    c = og.block_fp8_matmul(aq, wq, a_s, w_s, out_dtype=torch.bfloat16)
    out = os.path.join(os.path.dirname(os.path.abspath(__file__)), "config1.npz")
    np.savez_compressed(
        out,
        a_bf16_bits=a.view(torch.int16).numpy(),
        w_f32=w.numpy(),
        aq_divide=aq, as_divide=a_s, aq_reciprocal=aq2, as_reciprocal=a_s2, a_ue8m0=a_e8,
        wq=wq, ws=w_s,
        c_bf16_bits=c.view(torch.int16).numpy(),
    )
    print("wrote", out, os.path.getsize(out), "bytes")


if __name__ == "__main__":
    main()
