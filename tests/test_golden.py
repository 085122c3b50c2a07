"""Fixed vectors (tests/golden/attention_vectors.npz, written by tests/golden/make_vectors.py from scalar
fp64 loops): the oracle, the kernels in the host lane simulator and the kernels on the GPU against the
same frozen numbers."""
import math
import os

import numpy as np
import pytest
import torch

from oracle import flash_attention as oracle_flash, piecewise_attention as oracle_pw, paged_attention as oracle_paged

VECTORS = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "attention_vectors.npz"))
FLASH = ["flash_causal_gqa", "flash_rows_without_keys", "flash_noncausal"]
PIECEWISE = ["piecewise_causal", "piecewise_noncausal_cross"]


def t(name, device="cpu"):
    return torch.from_numpy(VECTORS[name]).to(device)


def close(hyp, expected, atol):
    hyp, expected = hyp.detach().float().cpu(), expected.float()
    finite = torch.isfinite(expected)
    assert torch.equal(torch.isfinite(hyp), finite)          # -inf log-normalizers in the same places
    assert (hyp[finite] - expected[finite]).abs().max().item() <= atol


@pytest.mark.parametrize("name", FLASH)
def test_oracle_flash_matches_the_fixed_vectors(name):
    q, k, v = t(name + ".q").float(), t(name + ".k").float(), t(name + ".v").float()   # fp32 in, fp32 out
    o, L, tot, *_ = oracle_flash(q, k, v, bool(VECTORS[name + ".causal"]), upcast=True, return_log_normalizer=True,
                                 return_total_attention=True)
    close(o, t(name + ".o"), 2e-5)
    close(L, t(name + ".L"), 2e-5)
    close(tot, t(name + ".tot"), 2e-5)


@pytest.mark.parametrize("name", PIECEWISE)
def test_oracle_piecewise_matches_the_fixed_vectors(name):
    args = [t(f"{name}.{x}").float() for x in ("q1", "k1", "q2", "k2", "v")]
    o = oracle_pw(*args, int(VECTORS[name + ".w"]), bool(VECTORS[name + ".causal"]), upcast=True)
    close(o, t(name + ".o"), 2e-5)


def test_oracle_paged_matches_the_fixed_vectors():
    q = t("paged.q")
    out = oracle_paged(q.float(), t("paged.kc").float(), t("paged.vc").float(), t("paged.table"), t("paged.lens"),
                       q.shape[-1] ** -0.5)
    close(out, t("paged.out"), 2e-5)


# fp16 kernels: P and the output are rounded to fp16 (values of order 1)
KERNEL_ATOL = 4e-3


@pytest.mark.gpu
@pytest.mark.parametrize("name", FLASH)
def test_gpu_flash_matches_the_fixed_vectors(name):
    import flagattention_amd as flag_attn
    q, k, v = t(name + ".q", "cuda"), t(name + ".k", "cuda"), t(name + ".v", "cuda")
    o, L, tot, _, _ = flag_attn.flash_attention(q, k, v, bool(VECTORS[name + ".causal"]), return_log_normalizer=True,
                                                return_total_attention=True)
    close(o, t(name + ".o"), KERNEL_ATOL)
    close(L, t(name + ".L"), KERNEL_ATOL)
    close(tot, t(name + ".tot"), KERNEL_ATOL)


@pytest.mark.gpu
@pytest.mark.parametrize("name", PIECEWISE)
def test_gpu_piecewise_matches_the_fixed_vectors(name):
    import flagattention_amd as flag_attn
    args = [t(f"{name}.{x}", "cuda") for x in ("q1", "k1", "q2", "k2", "v")]
    o = flag_attn.piecewise_attention(*args, int(VECTORS[name + ".w"]), causal=bool(VECTORS[name + ".causal"]))
    close(o, t(name + ".o"), KERNEL_ATOL)


@pytest.mark.gpu
@pytest.mark.parametrize("num_splits", [0, 1, 2])
def test_gpu_paged_matches_the_fixed_vectors(num_splits):
    import flagattention_amd as flag_attn
    q = t("paged.q", "cuda")
    lens = t("paged.lens", "cuda")
    out = flag_attn.paged_attention(q, t("paged.kc", "cuda"), t("paged.vc", "cuda"), lens, t("paged.table", "cuda"),
                                    q.shape[-1] ** -0.5, int(lens.max()), num_splits=num_splits)
    close(out, t("paged.out"), 2e-3)


@pytest.mark.parametrize("name", FLASH)
def test_simulated_kernels_match_the_fixed_vectors(name):
    from tests.sim import simlib
    from flagattention_amd import _abi
    lib = simlib.get()
    q, k, v = t(name + ".q"), t(name + ".k"), t(name + ".v")
    B, H, M, D = q.shape
    o = torch.full_like(q, float("nan"))
    L = torch.full((B, H, M), float("nan"))
    causal = bool(VECTORS[name + ".causal"])
    _abi.fa_fwd(lib, q, k, v, o, L, causal, 1.0 / math.sqrt(D))
    tot = torch.full((B, H, k.shape[2]), float("nan"))
    _abi.fa_total_attn(lib, q, k, L, tot, causal, 1.0 / math.sqrt(D))
    close(o, t(name + ".o"), KERNEL_ATOL)
    close(L, t(name + ".L"), KERNEL_ATOL)
    close(tot, t(name + ".tot"), KERNEL_ATOL)
