"""GPU parity of the Hyena-LI chunked modal scan against the CPU oracle, through the C ABI.

Tolerances: 1e-4 max relative error (max|a-b| / max|b|) for the fp32 long-convolution
output, 2e-2 for the gated bf16 output, 1e-4 for the modal state."""
import pytest
import torch

import vortex_amd as va
from oracle import hyena_oracle as O

pytestmark = pytest.mark.gpu


def rel_err(a, b):
    a, b = a.double().cpu(), b.double().cpu()
    return ((a - b).abs().max() / b.abs().max().clamp_min(1e-30)).item()


@pytest.mark.parametrize("B,D,L,G,cplx", [
    (1, 32, 1024, 2, True),
    (2, 64, 2048, 4, True),
    (1, 32, 1544, 2, True),       # L not a multiple of the 512-sample step
    (1, 16, 8, 1, True),          # a single octet
    (1, 32, 4096, 1, False),      # real poles (vortex's own parametrisation), one group of 32 channels
    (1, 16, 520, 1, False),
])
def test_li_vs_oracle(B, D, L, G, cplx):
    x2, x1, v = O.make_gates(B, D, L, seed=L + D)
    lp, r = (O.make_modal_complex if cplx else O.make_modal_real)(G, 16, seed=L)
    Db = torch.randn(D, generator=torch.Generator().manual_seed(1)).bfloat16()
    ref, y32_ref, st_ref = O.li_prefill(x2, x1, v, lp, r, Db)
    out, y32, st = va.hyena_li_fwd(x1.cuda(), x2.cuda(), v.cuda(), lp.cuda(), r.cuda(), Db.cuda(),
                                   want_state=True, want_fp32=True)
    torch.cuda.synchronize()
    assert rel_err(y32, y32_ref) <= 1e-4
    assert rel_err(out, ref) <= 2e-2
    assert st.dtype == st_ref.dtype and st.shape == st_ref.shape
    assert rel_err(torch.view_as_real(st) if cplx else st, torch.view_as_real(st_ref) if cplx else st_ref) <= 1e-4


def test_li_state_feeds_decode():
    # prefill on L tokens, then decode steps from the emitted state reproduce a longer prefill
    B, D, L, G, n_dec = 2, 32, 1024, 2, 4
    x2, x1, v = O.make_gates(B, D, L + 8, seed=3)
    lp, r = O.make_modal_complex(G, 16, seed=4)
    Db = torch.randn(D, generator=torch.Generator().manual_seed(1)).bfloat16()
    full, _, _ = O.li_prefill(x2, x1, v, lp, r, Db, want_state=False)
    d = lambda t: t.cuda()
    _, _, st = va.hyena_li_fwd(d(x1[..., :L].contiguous()), d(x2[..., :L].contiguous()), d(v[..., :L].contiguous()),
                               d(lp), d(r), d(Db), want_state=True)
    poles = torch.exp(lp[..., 0]).cuda()
    for i in range(n_dec):
        y = va.iir_step(d(x1[..., L + i].contiguous()), d(x2[..., L + i].contiguous()), d(v[..., L + i].contiguous()),
                        st, poles, d(r), d(Db))
        assert rel_err(y, full[..., L + i]) <= 2e-2


def test_li_impulse_gives_filter():
    # x1 = delta, v = x2 = 1, D = 0: y32 = h exactly as the modal formula defines it
    B, D, L, G = 1, 32, 2048, 2
    lp, r = O.make_modal_complex(G, 16, seed=9)
    x1 = torch.zeros(B, D, L, dtype=torch.bfloat16)
    x1[..., 5] = 1
    one = torch.ones(B, D, L, dtype=torch.bfloat16)
    _, y32, _ = va.hyena_li_fwd(x1.cuda(), one.cuda(), one.cuda(), lp.cuda(), r.cuda(), torch.zeros(D).bfloat16().cuda(),
                                want_fp32=True)
    h = O.modal_filter(lp, r, L, dtype=torch.float64)[0].repeat_interleave(D // G, 0)
    exp = torch.zeros(B, D, L, dtype=torch.float64)
    exp[0, :, 5:] = h[:, : L - 5]
    assert rel_err(y32, exp) <= 2e-5
