"""Seeded synthetic weights shared by the CPU and GPU tests."""
import numpy as np
import torch


def gaussian_weight(M, K, seed=0, std=0.02):
    g = torch.Generator().manual_seed(seed)
    return (torch.randn(M, K, generator=g) * std).bfloat16()


def student_t_weight(M, K, seed=0, std=0.02, nu=3.0):
    g = torch.Generator().manual_seed(seed)
    z = torch.randn(M, K, generator=g)
    chi2 = torch.zeros(M, K)
    for _ in range(int(nu)):
        chi2 += torch.randn(M, K, generator=g) ** 2
    t = z / torch.sqrt(chi2 / nu)
    return (t * (std / (nu / (nu - 2)) ** 0.5)).bfloat16()


def random_bits_weight(M, K, seed=0):
    g = torch.Generator().manual_seed(seed)
    return torch.randint(0, 65536, (M, K), generator=g, dtype=torch.int32).to(torch.int16).view(torch.bfloat16)


def special_values_weight(M, K, seed=0):
    """Gaussian weights salted with zeros, denormals, infinities and NaNs."""
    w = gaussian_weight(M, K, seed).view(torch.int16).clone()
    g = torch.Generator().manual_seed(seed + 1)
    idx = torch.randint(0, M * K, (M * K // 50,), generator=g)
    pats = torch.tensor([0x0000, 0x8000, 0x0001, 0x807F, 0x7F80, 0xFF80, 0x7FC0, 0xFFFF, 0x7F7F, 0x0080],
                        dtype=torch.int32).to(torch.int16)
    w.view(-1)[idx] = pats[torch.randint(0, len(pats), idx.shape, generator=g)]
    return w.view(torch.bfloat16)


def bits_of(w: torch.Tensor) -> np.ndarray:
    return w.contiguous().view(torch.int16).cpu().numpy().view(np.uint16)


def pair_counts(bits: np.ndarray) -> np.ndarray:
    e = ((bits.astype(np.int64) >> 7) & 0xFF)
    return np.bincount((e[:, 0::2] | (e[:, 1::2] << 8)).reshape(-1), minlength=65536)
