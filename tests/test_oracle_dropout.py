"""Pins oracle/dropout.py: Philox-4x32 against the Random123 known-answer vectors, the uniform map
against its defining properties, the mask against its drop rate -- and both against what Triton's own
``tl.rand`` and the reference's ``recompute_mask_kernel`` produce (tests/golden/dropout_vectors.npz, written
by tests/golden/make_dropout_vectors.py with Triton's CPU interpreter)."""
import os

import numpy as np
import pytest

from oracle.dropout import keep_mask, philox4x32, uniform_from_bits

# Random123 kat_vectors, "philox4x32 10": counter words, key words, expected output words
KAT = [
    ((0x00000000, 0x00000000, 0x00000000, 0x00000000), (0x00000000, 0x00000000),
     (0x6627e8d5, 0xe169c58d, 0xbc57ac4c, 0x9b00dbd8)),
    ((0xffffffff, 0xffffffff, 0xffffffff, 0xffffffff), (0xffffffff, 0xffffffff),
     (0x408f276d, 0x41c83b0e, 0xa20bc7c6, 0x6d5451fd)),
    ((0x243f6a88, 0x85a308d3, 0x13198a2e, 0x03707344), (0xa4093822, 0x299f31d0),
     (0xd16cfe09, 0x94fdcceb, 0x5001e420, 0x24126ea1)),
]


@pytest.mark.parametrize("ctr,key,expected", KAT)
def test_philox_known_answers(ctr, key, expected):
    out = philox4x32(*[np.array([c], dtype=np.uint32) for c in ctr], key[0], key[1], 10)
    assert tuple(int(o[0]) for o in out) == expected


def test_philox_is_a_bijection_of_the_counter_per_round():
    # one round maps distinct counters to distinct outputs (it is a Feistel-like permutation)
    c0 = np.arange(4096, dtype=np.uint32)
    z = np.zeros_like(c0)
    out = np.stack(philox4x32(c0, z, z, z, 123, 456, 1), axis=1)
    assert len({tuple(r) for r in out.tolist()}) == 4096


def test_uniform_map():
    x = np.array([0, 1, 0x7fffffff, 0x80000000, 0xffffffff], dtype=np.uint32)
    u = uniform_from_bits(x)
    assert u[0] == 0 and u[4] == 0            # 0 and -1 (folded to 0)
    assert u[2] == u[3]                       # INT_MAX and INT_MIN fold to the same value
    assert 0.0 <= u.min() and u.max() < 1.0
    big = uniform_from_bits(np.random.default_rng(0).integers(0, 2 ** 32, 1 << 20, dtype=np.uint64).astype(np.uint32))
    assert abs(big.mean() - 0.5) < 2e-3 and big.max() < 1.0


@pytest.mark.parametrize("p", [0.1, 0.5, 0.9])
def test_mask_drop_rate_and_determinism(p):
    m1 = keep_mask(2, 3, 64, 100, p, seed=1234, offset=40)
    m2 = keep_mask(2, 3, 64, 100, p, seed=1234, offset=40)
    assert (m1 == m2).all()
    assert abs((~m1).float().mean().item() - p) < 0.02
    assert (keep_mask(2, 3, 64, 100, p, seed=1235, offset=40) != m1).any()
    # the counter is offset + linear index: shifting the offset by one row shifts the mask by one row
    shifted = keep_mask(1, 1, 8, 16, p, seed=7, offset=16)
    base = keep_mask(1, 1, 9, 16, p, seed=7, offset=0)
    assert (shifted[0, 0] == base[0, 0, 1:]).all()
    assert keep_mask(1, 1, 4, 4, 0.0, 1, 0).all()


def test_flash_oracle_with_dropout_mask():
    import torch
    from oracle import flash_attention
    torch.manual_seed(0)
    q, k, v = (torch.randn(1, 2, 5, 8, dtype=torch.float64) for _ in range(3))
    plain = flash_attention(q, k, v, True)
    ones = torch.ones(1, 2, 5, 5, dtype=torch.bool)
    assert torch.allclose(flash_attention(q, k, v, True, dropout_p=0.0, dropout_mask=ones), plain)
    # explicit loop: dropped probabilities are zeroed AFTER normalisation, kept ones scaled by 1 / (1 - p)
    mask = keep_mask(1, 2, 5, 5, 0.4, seed=3, offset=0)
    out = flash_attention(q, k, v, True, dropout_p=0.4, dropout_mask=mask)
    ref = torch.zeros_like(out)
    for h in range(2):
        for m in range(5):
            s = torch.tensor([float(q[0, h, m] @ k[0, h, n]) / 8 ** 0.5 if n <= m else float("-inf") for n in range(5)],
                             dtype=torch.float64)
            p = torch.softmax(s.float(), 0).double()
            for n in range(5):
                if mask[0, h, m, n]:
                    ref[0, h, m] += p[n] * v[0, h, n] / 0.6
    assert torch.allclose(out, ref, atol=1e-6)


GOLDEN = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "dropout_vectors.npz"))
RAND_CASES = sorted(int(k.split("_")[1]) for k in GOLDEN.files if k.startswith("rand_") and k.endswith("_args"))
MASK_CASES = sorted(int(k.split("_")[1]) for k in GOLDEN.files if k.startswith("mask_") and k.endswith("_args"))


@pytest.mark.parametrize("case", RAND_CASES)
def test_uniform_numbers_equal_tritons_rand_bit_for_bit(case):
    """tl.rand(seed, first + arange(count), n_rounds=6) of Triton 3.6.0: seeds and counters on both sides of
    2^31 and 2^32, so the 32-bit and the 64-bit argument forms are both covered."""
    seed, first, count = (int(x) for x in GOLDEN[f"rand_{case}_args"])
    counter = np.uint64(first) + np.arange(count, dtype=np.uint64)
    zeros = np.zeros(count, dtype=np.uint32)
    x, _, _, _ = philox4x32((counter & np.uint64(0xFFFFFFFF)).astype(np.uint32), (counter >> np.uint64(32)).astype(np.uint32),
                            zeros, zeros, seed & 0xFFFFFFFF, seed >> 32, 6)
    assert np.array_equal(uniform_from_bits(x).view(np.uint32), GOLDEN[f"rand_{case}_values"].view(np.uint32))


@pytest.mark.parametrize("case", MASK_CASES)
def test_mask_equals_the_references_recomputed_mask(case):
    """recompute_mask_kernel (src/flag_attn/testing/dropout.py:5-17 of the reference) on the same arguments."""
    B, H, M, N, seed, offset = (int(x) for x in GOLDEN[f"mask_{case}_args"])
    p = float(GOLDEN[f"mask_{case}_p"])
    expected = np.unpackbits(GOLDEN[f"mask_{case}_bits"])[:B * H * M * N].astype(bool).reshape(B, H, M, N)
    assert np.array_equal(keep_mask(B, H, M, N, p, seed, offset).numpy(), expected)


def test_the_fixture_covers_both_argument_widths():
    firsts = [int(GOLDEN[f"rand_{c}_args"][1]) for c in RAND_CASES]
    seeds = [int(GOLDEN[f"rand_{c}_args"][0]) for c in RAND_CASES]
    assert min(firsts) < 2 ** 31 < 2 ** 32 < max(firsts) and min(seeds) < 2 ** 31 < 2 ** 32 < max(seeds)
    assert len(MASK_CASES) >= 4 and str(GOLDEN["triton_version"]) == "3.6.0"
