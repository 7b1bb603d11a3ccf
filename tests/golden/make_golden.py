"""Writes the golden fixtures in this directory from the CPU oracle.

The reference stores no vectors for this path (its tests draw inputs on a GPU at
run time), so these are produced by *our* oracle, whose correctness is pinned
separately by tests/test_oracle.py.  They freeze one equal-head-dim case and one
small-value-head case so that the oracle and the HIP path are also checked
against fixed data.  Run from the repository root:

    python tests/golden/make_golden.py

Inputs are drawn in fp32, rounded to bf16 and stored as the raw 16-bit patterns;
expected outputs are fp32 from fp64 arithmetic on the rounded inputs.
"""

import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import naive  # noqa: E402

CASES = {
    "equal_d_b1_h1_n128_d32": (1, 1, 128, 32, 32, 1234),
    "small_v_b1_h1_n128_dqk64_dv16": (1, 1, 128, 64, 16, 4321),
}


def bits(t: torch.Tensor) -> np.ndarray:
    return t.bfloat16().view(torch.int16).numpy().view(np.uint16)


def main() -> None:
    for name, (b, h, n, dqk, dv, seed) in CASES.items():
        g = torch.Generator().manual_seed(seed)
        q = (torch.nn.functional.elu(torch.randn(b, h, n, dqk, generator=g)) + 1).bfloat16()
        k = (torch.nn.functional.elu(torch.randn(b, h, n, dqk, generator=g)) + 1).bfloat16()
        v = torch.randn(b, h, n, dv, generator=g).bfloat16()
        do = torch.randn(b, h, n, dv, generator=g).bfloat16()
        o = naive.causal_dot_product(q.double(), k.double(), v.double())
        dq, dk, dv_ = naive.causal_dot_product_grads(q.double(), k.double(), v.double(), do.double())
        np.savez_compressed(
            os.path.join(HERE, name + ".npz"),
            q_bf16=bits(q), k_bf16=bits(k), v_bf16=bits(v), do_bf16=bits(do),
            o=o.float().numpy(), dq=dq.float().numpy(), dk=dk.float().numpy(), dv=dv_.float().numpy(),
        )
        print("wrote", name)


if __name__ == "__main__":
    main()
