"""Writes tests/golden/dropout_vectors.npz: what Triton's own ``tl.rand`` returns, and the masks that the
reference's ``recompute_mask_kernel`` draws with it.

The dropout of flash attention keeps a probability when ``tl.rand(seed, counter, n_rounds=6)`` exceeds
``dropout_p`` (``src/flag_attn/flash.py:367-371, 454-457`` of the reference).  ``tl.rand`` belongs to
Triton (``triton/language/random.py``, installed here as 3.6.0), which runs its kernels on the CPU when
``TRITON_INTERPRET=1``; no GPU is needed.  Two parts:

  rand_*   a kernel of this file stores ``tl.rand(seed, offset + arange, n_rounds=6)``: seeds and offsets
           below and above 2^31 and 2^32, so that the 32- and the 64-bit argument forms both occur;
  mask_*   ``recompute_mask_kernel`` of ``src/flag_attn/testing/dropout.py:5-17``, loaded from the reference
           checkout by file path (that file imports torch and triton only) and launched on CPU tensors
           with the grid of its wrapper (``:19-27``, whose ``torch.cuda.device`` needs a GPU).

Run once, in a container that holds the reference at /root/reference:

    python tests/golden/make_dropout_vectors.py

The fixture is data (inputs and outputs); tests/test_oracle_dropout.py holds oracle/dropout.py against it.
"""
import importlib.util
import os

os.environ["TRITON_INTERPRET"] = "1"      # before triton is imported

import numpy as np      # noqa: E402
import torch            # noqa: E402
import triton           # noqa: E402
import triton.language as tl      # noqa: E402

HERE = os.path.dirname(os.path.abspath(__file__))
REFERENCE_DROPOUT = "/root/reference/src/flag_attn/testing/dropout.py"

RAND_CASES = [        # (seed, first counter, count)
    (0, 0, 256),
    (1234, 8, 256),
    (2 ** 31 - 1, 2 ** 31 - 300, 256),            # 32-bit arguments up to their end
    (5, 2 ** 31 - 100, 256),                       # 32-bit counters that wrap into the sign bit
    (2 ** 31 + 5, 12, 256),                        # a seed that needs 64 bits
    (2 ** 40 + 77, 2 ** 32 + 100, 256),            # counters beyond 2^32: the high word enters
    (0x7FFFFFFFFFFFFFFF, 2 ** 45 + 4, 256),
    (67280421310721, 2 ** 32 - 128, 256),          # counters that cross 2^32 (torch's default seed)
]

MASK_CASES = [        # (B, H, M, N, dropout_p, seed, offset)
    (1, 1, 3, 17, 0.5, 0, 0),
    (2, 3, 5, 70, 0.2, 1234, 8),
    (1, 2, 2, 1100, 0.1, 42, 4096),                # more than one 1024-wide step of the reference's loop
    (1, 1, 4, 64, 0.9, 2 ** 40 + 77, 2 ** 32 + 100),
]


@triton.jit
def rand_kernel(out, seed, offset, n, BLOCK: tl.constexpr):
    offs = tl.arange(0, BLOCK)
    tl.store(out + offs, tl.rand(seed, offset + offs, n_rounds=6), mask=offs < n)


def main():
    arrays = {}
    for i, (seed, first, count) in enumerate(RAND_CASES):
        out = torch.empty(count, dtype=torch.float32)
        rand_kernel[(1,)](out, seed, first, count, BLOCK=triton.next_power_of_2(count))
        arrays[f"rand_{i}_args"] = np.array([seed, first, count], dtype=np.uint64)
        arrays[f"rand_{i}_values"] = out.numpy().copy()

    spec = importlib.util.spec_from_file_location("reference_testing_dropout", REFERENCE_DROPOUT)
    reference = importlib.util.module_from_spec(spec)
    spec.loader.exec_module(reference)
    for i, (B, H, M, N, p, seed, offset) in enumerate(MASK_CASES):
        mask = torch.full((B, H, M, N), True, dtype=torch.bool)
        reference.recompute_mask_kernel[(M, B, H)](mask, B, H, M, N, p, seed, offset)
        arrays[f"mask_{i}_args"] = np.array([B, H, M, N, seed, offset], dtype=np.uint64)
        arrays[f"mask_{i}_p"] = np.array(p, dtype=np.float64)
        arrays[f"mask_{i}_bits"] = np.packbits(mask.numpy().reshape(-1))
    arrays["triton_version"] = np.array(triton.__version__)
    path = os.path.join(HERE, "dropout_vectors.npz")
    np.savez_compressed(path, **arrays)
    print(f"wrote {path}: {len(RAND_CASES)} tl.rand cases, {len(MASK_CASES)} masks, triton {triton.__version__}")


if __name__ == "__main__":
    main()
