"""Error statements shared by the GPU parity tests.

Two measures are asserted side by side:

* rel_err: max|a-b| / max|b|, the normalised figure the tolerances 2e-2 (bf16 outputs) and 1e-4 (float32
  long-convolution output, modal state) are stated on;
* a per-element forward-error bound for the gated bf16 outputs out = bf16(x2 * z), z = bf16(y [+ bias term]):

      |got - ref| <= |x2| * (eps_acc * S + ulps_z * ulp_bf16(z)) + ulp_bf16(ref)

  where S[t] = sum_k |h[k]| * |u[t-k]| (+ |bias*u|) is the magnitude the accumulation ran over, eps_acc the
  relative precision of the coefficients and the accumulation (2^-8 for taps rounded to one bf16 term on the
  matrix cores, 2^-16 for split-precision or float32 arithmetic), and the two ulp terms are the roundings the
  reference itself applies (a sum that lands on the other side of a rounding boundary moves z by one ulp).
  A sample that picked up a wrong tap, a neighbouring segment's halo or a stale ring slot is off by a term of
  order |h|*|u| ~ S / sqrt(K), hundreds of times this bound, wherever in the tensor it sits -- which the
  normalised maximum alone does not see for small samples.
"""
import torch


def rel_err(a, b):
    a, b = a.double().cpu(), b.double().cpu()
    return ((a - b).abs().max() / b.abs().max().clamp_min(1e-30)).item()


def bf16_ulp(x):
    """Spacing of bfloat16 at |x| (float64 in, float64 out; 2^-133 at zero)."""
    x = x.double().abs().clamp_min(2.0 ** -126)
    return torch.pow(2.0, torch.floor(torch.log2(x)) - 7)


def abs_scale(u, h_conv, extra=None):
    """S[b, d, t] = sum_k |h[d, k]| |u[b, d, t-k]| (+ |extra|) in float64.  h_conv: [D, K] in convolution order
    (h[:, 0] on the current sample)."""
    B, D, L = u.shape
    K = h_conv.shape[1]
    n = 1
    while n < L + K:
        n *= 2
    U = torch.fft.rfft(u.double().abs(), n=n)
    H = torch.fft.rfft(h_conv.double().abs(), n=n)
    S = torch.fft.irfft(U * H[None], n=n)[..., :L]
    S = S.clamp_min(0) + 1e-12 * S.abs().max()          # FFT noise floor
    if extra is not None:
        S = S + extra.double().abs()
    return S


def assert_gated_close(got, ref, z_ref, x2, S, eps_acc, ulps_z=1.0, gate_ulps=0.0, fft_floor=0.0, what=""):
    """The per-element bound above.  got, ref: outputs; z_ref: the reference's bf16 pre-gate value; x2: the
    output gate (None for an ungated operator); S from abs_scale.  gate_ulps: bf16 ulps by which the output gate
    itself may differ (a fused featurizer computes it; 0 when the gate is an input).  fft_floor: absolute noise of a
    reference that convolves through a float32 FFT, as a fraction of max S (its error is uniform over the row, not
    proportional to the local magnitude; 4e-6 covers lengths up to 2^20).  Returns the largest error/bound ratio."""
    got, ref, z_ref, S = (t.double().cpu() for t in (got, ref, z_ref, S))
    g = x2.double().cpu().abs() if x2 is not None else torch.ones_like(ref)
    bound = g * (eps_acc * S + ulps_z * bf16_ulp(z_ref) + fft_floor * S.max()) + bf16_ulp(ref) \
        + gate_ulps * 2.0 ** -7 * ref.abs()
    err = (got - ref).abs()
    ratio = (err / bound).max().item()
    n_bad = int((err > bound).sum())
    off2 = int((err > 2 * bf16_ulp(ref) + 2 * g * bf16_ulp(z_ref)).sum())
    assert n_bad == 0, (f"{what}: {n_bad} of {err.numel()} elements outside the per-element bound, worst ratio "
                        f"{ratio:.2f} at {tuple(int(i) for i in (err / bound).argmax().unsqueeze(0))}; "
                        f"{off2} elements differ by more than 2 bf16 ulps of the pre-gate value")
    return ratio


def log_uniform_modal(G, S, cplx, seed, pmin=0.05, pmax=0.9999):
    """Modal parameters with log-uniform |p| in [pmin, pmax]: slow poles as in the benchmark configurations and the
    fast-decaying ones a trained or randn-initialised log_poles parameter (vortex/model/model.py:202) also holds.
    Returns (log_poles [G, S, 1], residues [G, S]), complex64 or float32."""
    import math
    g = torch.Generator().manual_seed(seed)
    lm = math.log(pmin) + (math.log(pmax) - math.log(pmin)) * torch.rand(G, S, generator=g, dtype=torch.float64)
    if cplx:
        ang = math.pi * torch.rand(G, S, generator=g, dtype=torch.float64)
        lp = torch.complex(lm, ang).to(torch.complex64)[..., None]
        r = (torch.complex(torch.randn(G, S, generator=g), torch.randn(G, S, generator=g)) / 2 ** 0.5).to(torch.complex64)
        return lp, r
    return lm.to(torch.float32)[..., None], torch.randn(G, S, generator=g)
