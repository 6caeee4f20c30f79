"""Writes the fixtures in this folder.  Run from the repository root:  python tests/golden/make_golden.py

* `mx_vectors.json`      -- the explicit input/output vectors held by the reference's MX tests
                            (python/triton_kernels/tests/test_mxfp.py:92-141) as plain numbers, plus the e2m1
                            decision thresholds; expected values are the reference's, not computed here.
* `routing_examples.json` -- the worked examples in the reference's docstrings
                            (tensor_details/bitmatrix.py:11-19, tensor_details/ragged_tensor.py:16-29; only
                            the `block_offs` rows of the latter are self-consistent and kept).
* `c1_layer.npz`         -- intermediates of the small bf16 layer (128 tokens, 8 experts, top-2, d 512,
                            hidden 2x1024) computed by the CPU oracle from seeded inputs: router outputs,
                            expert-sorted gate weights, the k-expanded second GEMM output and the layer
                            output (bf16 stored as uint16), with checksums of the regenerated inputs.
"""
import json
import os
import sys

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import moe as omoe  # noqa: E402


def c1_inputs():
    """Seeded inputs of the small bf16 configuration (CPU generator, so every machine sees the same bits)."""
    g = torch.Generator().manual_seed(0)
    T, d, E, k, f2 = 128, 512, 8, 2, 2048
    x = torch.randn((T, d), generator=g).to(torch.bfloat16)
    logits = torch.randn((T, E), generator=g)
    w1 = (torch.randn((E, d, f2), generator=g) * 0.02).to(torch.bfloat16)
    w2 = (torch.randn((E, f2 // 2, d), generator=g) * 0.02).to(torch.bfloat16)
    b1 = torch.zeros((E, f2), dtype=torch.bfloat16)
    b2 = torch.zeros((E, d), dtype=torch.bfloat16)
    return x, logits, k, w1, b1, w2, b2


def checksum(t: torch.Tensor) -> int:
    raw = t.contiguous().view(torch.uint8).numpy().astype(np.uint64)
    return int((raw * (np.arange(raw.size, dtype=np.uint64).reshape(raw.shape) % 251 + 1)).sum() % (1 << 61))


def bf16_bits(t: torch.Tensor) -> np.ndarray:
    return t.contiguous().view(torch.int16).numpy().view(np.uint16)


def main():
    mx = {
        "source": "python/triton_kernels/tests/test_mxfp.py:92-141",
        "round_up": {
            "input_head": [6, 0, 0.24, 0.25, 0.75, 0.99, 1.2, 1.3, -1.25],
            "tenth_element_by_dtype": {"bfloat16": 0.251953125, "float16": 0.250244140625, "float32": 0.2500000298023223877},
            "zeros_appended": 22,
            "dequantised_head": [6, 0, 0, 0.0, 1.0, 1.0, 1.0, 1.5, -1.0, 0.5],
            "scale_byte": 127,
        },
        "round_down": {
            "input_head": [33.0, 24.0, 16.0, 8.0, 4.0, 0.0, -32.0, 0.0],
            "zeros_appended": 24,
            "scale_byte": 130,
            "exact_from_index": 1,
        },
        "e2m1_values": [0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0],
        "e2m1_ties_go_to": {"0.25": 0.0, "0.75": 1.0, "1.25": 1.0, "1.75": 2.0, "2.5": 2.0, "3.5": 4.0, "5.0": 4.0},
    }
    with open(os.path.join(HERE, "mx_vectors.json"), "w") as f:
        json.dump(mx, f, indent=1)

    routing = {
        "bitmatrix": {
            "source": "python/triton_kernels/triton_kernels/tensor_details/bitmatrix.py:11-19",
            "rows": [[0, 0, 1, 0, 1, 1, 0], [0, 1, 0, 0, 0, 1, 0], [1, 1, 1, 0, 0, 0, 1], [0, 0, 1, 0, 1, 0, 0]],
            "col_sum": [1, 2, 3, 0, 2, 2, 1],
            "col_sorted_indx": [5, 3, 6, 0, 7, 9, 1, 10, 2, 4, 8],
            "row_sorted_indx": [3, 6, 8, 1, 9, 0, 2, 4, 10, 5, 7],
        },
        "ragged": {
            "source": "python/triton_kernels/triton_kernels/tensor_details/ragged_tensor.py:16-29",
            "slice_sizes": [15, 17, 0, 127],
            "block_offs": {"16": [0, 1, 3, 3, 11], "32": [0, 1, 2, 2, 6], "64": [0, 1, 2, 2, 4], "128": [0, 1, 2, 2, 3]},
        },
    }
    with open(os.path.join(HERE, "routing_examples.json"), "w") as f:
        json.dump(routing, f, indent=1)

    x, logits, k, w1, b1, w2, b2 = c1_inputs()
    out, inter = omoe.moe_layer(x, logits, k, w1, b1, w2, b2, return_intermediates=True)
    r = inter["routing"]
    np.savez_compressed(
        os.path.join(HERE, "c1_layer.npz"),
        input_checksums=np.array([checksum(t) for t in (x, logits, w1, w2)], dtype=np.uint64),
        vals=r.vals.numpy(), indx=r.indx.numpy().astype(np.int16), col_sum=r.meta.col_sum.numpy(),
        col_sorted_indx=r.meta.col_sorted_indx.numpy(), row_sorted_indx=r.meta.row_sorted_indx.numpy(),
        gather_indx=r.gather_indx.numpy(), gammas=r.gammas.numpy(), slice_offs=r.ragged.slice_offs.numpy(),
        block_offs=r.ragged.block_offs_data.numpy(), y=bf16_bits(inter["y"]), out=bf16_bits(out),
        h_row0=bf16_bits(inter["h"][0]), a_row0=bf16_bits(inter["a"][0]),
    )


if __name__ == "__main__":
    main()
