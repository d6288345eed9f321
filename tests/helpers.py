"""Synthetic inputs shared by the tests: the weight and activation recipes of the benchmark
configurations, at arbitrary shapes."""
import numpy as np
import torch


def bf16_bits(t: torch.Tensor) -> np.ndarray:
    """bf16 tensor -> numpy uint16 bit patterns."""
    return t.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


def bits_to_bf16(a: np.ndarray) -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(a).view(np.int16)).view(torch.bfloat16)


def make_weight_kn(out_features: int, in_features: int, seed: int, std: float = 0.02) -> torch.Tensor:
    """nn.Linear-oriented N(0, std) bf16 weight, returned transposed to [K=in, N=out]."""
    g = torch.Generator("cpu").manual_seed(seed)
    w = (torch.randn(out_features, in_features, generator=g, dtype=torch.float32) * std).to(torch.bfloat16)
    return w.t().contiguous()


def make_x(M: int, K: int, seed: int) -> torch.Tensor:
    g = torch.Generator("cpu").manual_seed(seed)
    return torch.randn(M, K, generator=g, dtype=torch.float32).to(torch.bfloat16)


def zipf_bytes(n: int, skew: float, seed: int) -> np.ndarray:
    rng = np.random.default_rng(seed)
    p = 1.0 / np.arange(1, 257) ** skew
    p /= p.sum()
    return rng.choice(256, size=n, p=p).astype(np.uint8)
