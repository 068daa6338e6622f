"""Shared helpers of the GPU parity tests: seeded inputs rounded once to the GPU dtype (the same
values feed the HIP path and the FP32 CPU checker), tolerances, comparison."""
import numpy as np
import torch

import oracle

# rel-L2, max-abs against the FP32 checker. bf16 is the stated bar of the port; fp16 is tighter,
# in line with the reference's 1e-3 traced-vs-fused bound (tests/test_flux_blocks.cpp:288-290).
TOL = {"bf16": (5e-3, 2e-2), "fp16": (1e-3, 5e-3)}
TORCH_DT = {"bf16": torch.bfloat16, "fp16": torch.float16}


def randn(seed: int, shape, dtype: str) -> np.ndarray:
    """N(0,1) from the seeded generator, rounded to `dtype`, stored as float32."""
    n = int(np.prod(shape))
    x = oracle.torch_randn_f32(seed, max(n, 16))[:n].reshape(shape)
    return oracle.round_to(x, dtype)


def to_dev(x: np.ndarray, dtype: str) -> torch.Tensor:
    bits = oracle.to_bits(x, dtype)
    return torch.from_numpy(bits.view(np.int16)).view(TORCH_DT[dtype]).cuda()


def to_np(t: torch.Tensor) -> np.ndarray:
    return t.detach().float().cpu().numpy()


def assert_close(ref: np.ndarray, got: np.ndarray, dtype: str, what: str = ""):
    m = oracle.compare(ref, got)
    rel, mx = TOL[dtype]
    assert np.isfinite(got).all(), f"{what}: non-finite output"
    assert m["rel_l2"] <= rel and m["max_abs"] <= mx, f"{what}: {m} exceeds rel_l2 {rel} / max_abs {mx}"
    return m
