"""Writes tests/golden/tiny_expected.npz: rows of the float64 grid_sample oracle's outputs on
the seeded "tiny" workload (forward and the three gradients).

The reference commits no golden vectors for this operator (its test regenerates unseeded
random inputs and caches nothing in the repository), so these vectors come from this
repository's own oracle, which tests/test_oracle.py pins independently (hand arithmetic,
closed forms, finite differences, agreement of two formulations).  Nothing from the
reference is imported or executed here.

    python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from drivingsdk_amd import workloads  # noqa: E402
from oracle import msda_oracle as orc  # noqa: E402


def main():
    inp = workloads.make_inputs("tiny", with_grad_output=True)
    out, gv, gl, ga = orc.msda_grid_sample_fwd_bwd(inp.value, inp.spatial_shapes, inp.sampling_locations,
                                                   inp.attention_weights, inp.grad_output)
    nq, nk = out.shape[1], gv.shape[1]
    rows_q = np.arange(0, nq, 97)
    rows_k = np.arange(0, nk, 89)
    np.savez_compressed(
        os.path.join(HERE, "tiny_expected.npz"),
        rows_q=rows_q, rows_k=rows_k,
        output=out.numpy()[0, rows_q], grad_value=gv.numpy()[0, rows_k],
        grad_sampling_locations=gl.numpy()[0, rows_q], grad_attention_weights=ga.numpy()[0, rows_q],
        output_sum=np.float64(out.double().sum()),
    )
    print("wrote tiny_expected.npz", len(rows_q), "query rows,", len(rows_k), "key rows")


if __name__ == "__main__":
    main()
