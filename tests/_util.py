"""Helpers shared by the tests: seeded inputs and torch <-> numpy bit views."""
import numpy as np
import torch


def bits(t: torch.Tensor) -> np.ndarray:
    """bf16 tensor (any device) -> uint16 bit patterns."""
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view(np.uint16)


def from_bits(b: np.ndarray, device="cpu") -> torch.Tensor:
    return torch.from_numpy(np.ascontiguousarray(b).view(np.int16)).view(torch.bfloat16).to(device)


def codes(t: torch.Tensor) -> np.ndarray:
    """float8 / uint8 tensor -> uint8 codes."""
    return t.detach().cpu().contiguous().view(torch.uint8).numpy()


def f32(t: torch.Tensor) -> np.ndarray:
    return t.detach().cpu().contiguous().to(torch.float32).numpy()


def f32_bits(a) -> np.ndarray:
    return np.ascontiguousarray(a, dtype=np.float32).view(np.uint32)


def randn_bf16(shape, seed, std=1.0, outlier_frac=0.0, outlier_mul=1.0) -> torch.Tensor:
    g = torch.Generator(device="cpu").manual_seed(seed)
    x = torch.randn(shape, generator=g, dtype=torch.float32) * std
    if outlier_frac > 0:
        n = x.numel()
        k = max(1, round(outlier_frac * n))
        idx = torch.randperm(n, generator=g)[:k]
        x.view(-1)[idx] *= outlier_mul
    return x.to(torch.bfloat16)


def laplace_bf16(shape, seed, scale=1.0) -> torch.Tensor:
    """Unit-variance Laplace via the inverse CDF of a uniform draw, times `scale`."""
    g = torch.Generator(device="cpu").manual_seed(seed)
    u = torch.rand(shape, generator=g, dtype=torch.float32) - 0.5
    b = 1.0 / np.sqrt(2.0)
    x = -b * torch.sign(u) * torch.log1p(-2.0 * u.abs().clamp(max=0.4999999))
    return (x * scale).to(torch.bfloat16)


def special_bf16_rows(cols=128) -> torch.Tensor:
    """Rows that exercise the corners of the quantizer: zeros, one tiny value, subnormal bf16,
    +-max in a group, exact ties, mixed signs of zero."""
    rows = []
    rows.append(torch.zeros(cols))
    r = torch.zeros(cols); r[3] = 1e-30; rows.append(r)
    r = torch.zeros(cols); r[5] = -1e-38; r[9] = 5e-39; rows.append(r)          # bf16 subnormals
    r = torch.linspace(-448, 448, cols); rows.append(r)
    r = torch.full((cols,), 3.0); r[0] = 448.0; r[1] = -448.0; r[2] = 17.0; r[3] = 19.0; rows.append(r)
    r = torch.arange(cols, dtype=torch.float32) - 64.0; rows.append(r)
    r = torch.zeros(cols); r[0] = -0.0; r[1] = 1.0; r[2] = -2.0 ** -10; r[3] = 2.0 ** -10; rows.append(r)
    r = torch.full((cols,), 3.3895e38); r[1] = -1.0; rows.append(r)             # near bf16 max
    r = torch.full((cols,), 1e-12); r[7] = 2e-12; rows.append(r)                 # around the eps clamp
    r = torch.full((cols,), 1e-13); rows.append(r)                               # below the eps clamp
    return torch.stack(rows).to(torch.bfloat16)


def nonfinite_bf16(rows=256, cols=512, seed=5) -> torch.Tensor:
    """Seeded normal data with NaN, +Inf and -Inf planted in known 128-wide groups (and groups left
    clean beside them): (0, 0..127) a NaN, (1, 128..255) +Inf, (2, 256..383) -Inf and a NaN,
    (130, 0..127) -Inf, (131, 384..511) a negative NaN."""
    x = randn_bf16((rows, cols), seed).clone()
    x[0, 5] = float("nan")
    x[1, 128 + 77] = float("inf")
    x[2, 256 + 1] = float("-inf")
    x[2, 256 + 100] = float("nan")
    x[130, 127] = float("-inf")
    v = x.view(torch.int16)
    v[131, 384 + 64] = -64                 # 0xFFC0: a NaN with its sign bit set
    return x


def canon_nan_codes(c: np.ndarray) -> np.ndarray:
    """E4M3 codes with the sign of NaN codes dropped (0xFF -> 0x7F): which of the two a cast writes for
    a NaN is not part of the numeric recipe."""
    c = np.asarray(c, dtype=np.uint8)
    return np.where((c & 0x7F) == 0x7F, np.uint8(0x7F), c)


def same_f32_or_nan(a, b) -> bool:
    """fp32 arrays equal bit for bit where both are numbers, and NaN in the same places."""
    a = np.asarray(a, dtype=np.float32).reshape(-1)
    b = np.asarray(b, dtype=np.float32).reshape(-1)
    na, nb = np.isnan(a), np.isnan(b)
    return a.shape == b.shape and np.array_equal(na, nb) and np.array_equal(a[~na].view(np.uint32), b[~nb].view(np.uint32))
