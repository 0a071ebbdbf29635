"""Toeplitz factors of the two-pass chunked convolution, under the names and signatures of
vortex/ops/hyena_se/utils.py (`from hyena_ops.utils import toeplitz, correction_toeplitz`).

With a filter in convolution orientation h [g, K] (for the operator's weights: `h[:, 0].flip(-1)`) and chunks
of `size` samples, chunk c of y = conv(h, x) is  T @ x_c + T_hat @ x_{c-1}:
    T[g, i, j]     = h[g, i - j]            for 0 <= i - j < K        (vortex/ops/hyena_se/utils.py:5-25)
    T_hat[g, i, j] = h[g, i + size - j]     for j >= i, i + size - j < K   (utils.py:38-51)
Built with index arithmetic instead of the reference's Python double loop."""
import torch


def _lagged(h, lag, keep, dtype, device):
    dtype = h.dtype if dtype is None else dtype
    device = h.device if device is None else device
    K = h.shape[1]
    lag, keep = lag.to(h.device), keep.to(h.device)
    vals = h[:, lag.clamp(0, K - 1)]
    out = torch.where((keep & (lag >= 0) & (lag < K))[None], vals, torch.zeros((), dtype=h.dtype, device=h.device))
    return out.to(device=device, dtype=dtype)


def toeplitz(h, size, dtype=None, device=None):
    """h [g, K] -> lower-triangular Toeplitz matrices [g, size, size]."""
    i = torch.arange(size)
    lag = i[:, None] - i[None, :]
    return _lagged(h, lag, lag >= 0, dtype, device)


def correction_toeplitz(h, size, dtype=None, device=None):
    """h [g, K] -> the factor that carries the previous chunk into the current one, [g, size, size]."""
    i = torch.arange(size)
    lag = i[:, None] - i[None, :]
    return _lagged(h, lag + size, lag <= 0, dtype, device)


def toeplitz_from_empty(T, h):
    """Fills T [g, size, size] in place with toeplitz(h, size)."""
    return T.copy_(toeplitz(h, T.shape[1], dtype=T.dtype, device=T.device))


def correction_toeplitz_from_empty(T, h):
    """Fills T [g, size, size] in place with correction_toeplitz(h, size)."""
    return T.copy_(correction_toeplitz(h, T.shape[1], dtype=T.dtype, device=T.device))
