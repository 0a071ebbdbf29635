"""hyena_li_fwd_static, the entry point that allocates nothing (coefficient tables in a static device array),
against hyena_li_plan + hyena_li_fwd through the C ABI: same kernels, so the outputs must be bit-identical.
Two calls in a row, the second with a smaller problem, so that what the first left in the array cannot leak."""
import ctypes

import pytest
import torch

from oracle import hyena_oracle as O
from vortex_amd import _lib, ops

pytestmark = pytest.mark.gpu


def _both(B, D, L, G, S, cplx, seed, want_state=True, want_fp32=True):
    dev = torch.device("cuda:0")
    x2, x1, v = (t.to(dev) for t in O.make_gates(B, D, L, seed=seed))
    lp, r = (O.make_modal_complex if cplx else O.make_modal_real)(G, S, seed=seed + 1)
    Db = torch.randn(D, generator=torch.Generator().manual_seed(seed)).to(dev)
    pairs = lambda t: torch.view_as_real(t.reshape(G, S).to(torch.complex64).contiguous()).contiguous().to(dev)
    lpp, rp = pairs(lp), pairs(r)
    L_ = _lib.lib()
    stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    r1, r2, rv = ops.rows_of(x1), ops.rows_of(x2), ops.rows_of(v)
    ref = ctypes.byref
    res = []
    for static in (False, True):
        out = torch.full((B, D, L), float("nan"), dtype=torch.bfloat16, device=dev)
        y32 = torch.full((B, D, L), float("nan"), dtype=torch.float32, device=dev) if want_fp32 else None
        st = torch.full((B, D, S, 2), float("nan"), dtype=torch.float32, device=dev) if want_state else None
        p = lambda t: ctypes.c_void_p(t.data_ptr()) if t is not None else None
        if static:
            rc = L_.hyena_li_fwd_static(ref(r1), ref(r2), ref(rv), p(lpp), p(rp), p(Db), 1, p(out), p(y32), p(st),
                                        B, D, L, G, S, stream)
            _lib.check(rc, "hyena_li_fwd_static")
        else:
            ws = torch.empty(L_.hyena_li_plan_bytes(G, S) // 4, dtype=torch.float32, device=dev)
            _lib.check(L_.hyena_li_plan(p(lpp), p(rp), G, S, p(ws), stream), "hyena_li_plan")
            rc = L_.hyena_li_fwd(ref(r1), ref(r2), ref(rv), p(ws), p(Db), 1, p(out), p(y32), p(st), B, D, L, G, S, stream)
            _lib.check(rc, "hyena_li_fwd")
        torch.cuda.synchronize()
        res.append((out, y32, st))
    return res


def test_static_form_matches_workspace_form_twice_in_a_row():
    for (B, D, L, G, S, cplx, seed) in [(2, 64, 2048 + 520, 16, 16, True, 1),      # first call: 16 groups
                                         (1, 16, 1000, 2, 8, False, 2)]:           # then a smaller one: 2 groups, 8 modes
        (o0, y0, s0), (o1, y1, s1) = _both(B, D, L, G, S, cplx, seed)
        assert not torch.isnan(o1.float()).any() and not torch.isnan(s1).any()
        assert torch.equal(o0, o1), (B, D, L, G)
        assert torch.equal(y0, y1)
        assert torch.equal(s0, s1)
    # and the bf16-only variant (no side outputs) on a third, again different shape
    (o0, _, _), (o1, _, _) = _both(1, 32, 4096, 32, 16, True, 3, want_state=False, want_fp32=False)
    assert torch.equal(o0, o1)


def test_static_form_rejects_more_groups_than_its_table_holds():
    L_ = _lib.lib()
    P = 4096
    r = _lib.Rows(P, 16384 * 64, 64, 16384, 16384)
    rc = L_.hyena_li_fwd_static(ctypes.byref(r), ctypes.byref(r), ctypes.byref(r), P, P, None, 1, P, None, None,
                                1, 16384, 64, 16384, 16, None)
    assert rc == -3 and b"8192" in L_.hyena_last_error_string()
    with pytest.raises(NotImplementedError):
        _lib.check(rc, "hyena_li_fwd_static")
