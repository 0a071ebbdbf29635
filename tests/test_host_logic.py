"""Host-side logic that needs no GPU: row descriptors against the reference's split / column_split
index maps, the ring-cache ordering, tap slicing, and the interleave permutation of the decode path."""
import ctypes

import pytest
import torch

from oracle import hyena_oracle as O
from vortex_amd import ops
from vortex_amd.engine import _group_taps


def gather_rows(u, r, D):
    """Reads channel d of batch b the way the kernels do: through the descriptor arithmetic."""
    B, C, L = u.shape
    flat = u.reshape(-1)
    base = (r.ptr - u.data_ptr()) // u.element_size()
    out = torch.empty(B, D, L, dtype=u.dtype)
    for b in range(B):
        for d in range(D):
            row = (d // r.ch_inner) * r.ch_outer + d % r.ch_inner
            s = base + b * r.batch_stride + row * r.row_stride
            out[b, d] = flat[s:s + L]
    return out


@pytest.mark.parametrize("cs", [False, True])
def test_row_descriptors_match_reference_split(cs):
    B, D, L, H = 2, 24, 8, 4
    u = torch.arange(B * 3 * D * L, dtype=torch.float32).reshape(B, 3 * D, L).bfloat16()
    hd = D // H
    ref = O.column_split(u, H, hd) if cs else u.split(D, dim=1)
    for i in range(3):
        r = ops.rows_of_projection(u, D, i, hd if cs else None)
        assert torch.equal(gather_rows(u, r, D), ref[i])


def test_rows_of_strided_view():
    u = torch.arange(2 * 12 * 16, dtype=torch.float32).reshape(2, 12, 16).bfloat16()
    x = u[:, 4:8]
    r = ops.rows_of(x)
    assert torch.equal(gather_rows(u, r, 4), x)
    with pytest.raises(ValueError):
        ops.rows_of(u.permute(0, 2, 1))           # samples not contiguous
    with pytest.raises(TypeError):
        ops.rows_of(u.float())


def test_size_one_dimensions_get_dense_strides():
    # torch leaves the stride of a size-one dimension arbitrary (here 1 for the time axis of a permuted [B, D, 1]
    # tensor); the descriptors handed to the C entry points carry the dense value, which passes the alignment checks
    t = torch.zeros(3, 48, 1, dtype=torch.bfloat16).permute(0, 2, 1)
    assert t.stride() == (48, 1, 1)
    assert ops._strides(t) == [48, 48, 1]
    c = ops._cl_of(t)
    assert (c.batch_stride, c.time_stride) == (48, 48)
    r = ops.rows_of(torch.zeros(1, 1, 64, dtype=torch.bfloat16))
    assert (r.batch_stride, r.row_stride) == (64, 64)
    assert ops._strides(torch.zeros(4, 6, 16)[:, :3]) == [96, 16, 1]


def test_fir_ring_reference_order_and_rotation():
    B, D, R = 2, 3, 5
    st = torch.arange(B * D * R, dtype=torch.float32).reshape(B, D, R)
    ring = ops.FirRing.from_reference(st)
    assert ring.shape == torch.Size((B, D, R))
    assert torch.equal(ring.reference_order(), st)
    # emulate two steps: the oldest slot is overwritten, then the oldest moves on
    for step in range(2):
        new = torch.full((B, D), 100.0 + step)
        ring.slots()[:, ring.pos] = new.bfloat16()        # block = D: slots() is a view of the cache
        ring.pos = (ring.pos + 1) % R
        st = torch.cat([st[..., 1:], new[..., None]], dim=-1)
        assert torch.equal(ring.reference_order(), st)


def test_group_taps_undoes_repeat_interleave():
    G, D, K = 4, 32, 7
    h = torch.randn(G, 1, K)
    assert torch.equal(_group_taps(h.repeat_interleave(D // G, 0), D, G), h[:, 0])
    assert torch.equal(_group_taps(h, D, G), h[:, 0])
    w = torch.randn(D, 1, 3)
    assert torch.equal(_group_taps(w, D, None), w[:, 0])


def test_decode_interleave_permutation_matches_reference():
    C = 24
    z = torch.arange(2 * C, dtype=torch.float32).reshape(2, C)
    j = torch.arange(C)
    perm = (j % (C // 3)) * 3 + j // (C // 3)      # the index map vortex_amd.cascade builds for decode
    assert torch.equal(z[:, perm], O.interleave(z))


def test_return_codes_map_to_exceptions():
    from vortex_amd import _lib
    assert _lib.check(0, "x") is None
    for rc, exc in ((-1, ValueError), (-2, ValueError), (-3, NotImplementedError), (700, RuntimeError)):
        with pytest.raises(exc):
            _lib.check(rc, "some call")


def test_rows_struct_layout_matches_header():
    # hyena_rows: one pointer and four int64, no padding
    assert ctypes.sizeof(ops.Rows) == 40
    assert [f[0] for f in ops.Rows._fields_] == ["ptr", "batch_stride", "row_stride", "ch_inner", "ch_outer"]


@pytest.mark.parametrize("cs,il", [(False, False), (True, False), (False, True)])
def test_gate_channel_map_matches_reference_split(cs, il):
    # the closed channel maps the fused layer kernels use == interleave / split / column_split of the reference
    D, H = 48, 4
    z = torch.arange(3 * D, dtype=torch.float32)[None]            # value = projection channel index
    ref = O.interleave(z) if il else z
    x2, x1, v = O.split_gates(ref, (D, H, D // H), cs, False)
    ci, co, gs, cst = ops.gate_channel_map(D, interleave=il, head_dim=D // H if cs else None)
    d = torch.arange(D)
    for gate, want in enumerate((x2, x1, v)):
        ch = (d // ci) * co + gate * gs + (d % ci) * cst
        assert torch.equal(ch.float(), want[0])
    assert ops.gate_channel_map(D, interleave=True, head_dim=D // H) is None


def test_proj_structs_match_header():
    from vortex_amd import _lib
    # hyena_proj_step: 7 pointer/int64 fields, 4 int64 map fields, one int (padded to 8), one pointer
    assert ctypes.sizeof(_lib.ProjStep) == 13 * 8
    assert _lib.ProjStep.flip_x1x2.offset == 11 * 8 and _lib.ProjStep.pos_dev.offset == 12 * 8
    # hyena_proj_fwd: 5 pointer/int64 fields, two ints, 4 int64 map fields
    assert ctypes.sizeof(_lib.ProjFwd) == 10 * 8
    assert _lib.ProjFwd.Ks.offset == 5 * 8 and _lib.ProjFwd.flip_x1x2.offset == 5 * 8 + 4
    assert _lib.ProjFwd.ch_inner.offset == 6 * 8
    assert ctypes.sizeof(_lib.Cl) == 3 * 8


def test_from_vortex_shares_parameters_and_config():
    # a stand-in with the attributes of vortex's HyenaCascade (vortex/model/model.py:125-210)
    import types
    from vortex_amd.cascade import HyenaCascade, use_hip_filters

    class Cfg(dict):
        __getattr__ = dict.__getitem__

    cfg = Cfg(hidden_size=64, num_attention_heads=4, state_size=16, short_filter_length=3, short_filter_bias=False,
              interleave=True, column_split_hyena=False, hyena_flip_x1x2=True)
    ref = types.SimpleNamespace(config=cfg, layer_idx=3, hyena_filter_groups=4, fir_inner_filter_length=7,
                                short_filter_weight=torch.nn.Parameter(torch.randn(192, 1, 3)), short_filter_bias=None,
                                h=torch.nn.Parameter(torch.randn(4, 1, 7)), D=None)
    m = HyenaCascade.from_vortex(ref)
    assert m.h is ref.h and m.short_filter_weight is ref.short_filter_weight and m.D is None
    assert (m.layer_idx, m.interleave, m.column_split_hyena, m.hyena_flip_x1x2) == (3, True, False, True)
    modal = types.SimpleNamespace(config=cfg, layer_idx=5, hyena_filter_groups=64, fir_inner_filter_length=None,
                                  short_filter_weight=torch.nn.Parameter(torch.randn(192, 1, 3)), short_filter_bias=None,
                                  h=None, D=torch.nn.Parameter(torch.zeros(64)),
                                  log_poles=torch.nn.Parameter(torch.randn(64, 16, 1)),
                                  residues=torch.nn.Parameter(torch.randn(64, 16)))
    blocks = [types.SimpleNamespace(filter=ref), types.SimpleNamespace(), types.SimpleNamespace(filter=modal)]
    model = types.SimpleNamespace(blocks=blocks)
    assert use_hip_filters(model) == 2 and use_hip_filters(model) == 0
    assert isinstance(blocks[2].filter, HyenaCascade) and blocks[2].filter.log_poles is modal.log_poles
    # sequence_major_projections wraps the projection of the Hyena-LI block only, keeps the layer's parameters, and
    # falls back to the layer itself wherever the one-launch path does not apply (here: tensors on the CPU)
    from vortex_amd.cascade import SequenceMajorProjection, project_sequence_major
    lin_fir, lin_modal = torch.nn.Linear(64, 192, bias=False), torch.nn.Linear(64, 192, bias=False)
    blocks[0].projections, blocks[2].projections = lin_fir, lin_modal
    assert use_hip_filters(model, sequence_major_projections=True) == 0
    assert blocks[0].projections is lin_fir
    wrapped = blocks[2].projections
    assert isinstance(wrapped, SequenceMajorProjection) and wrapped.linear is lin_modal and wrapped.weight is lin_modal.weight
    x = torch.randn(2, 16, 64)
    assert torch.equal(wrapped(x), lin_modal(x)) and wrapped(x).is_contiguous()
    z = project_sequence_major(lin_modal.weight.detach(), x)
    assert z.shape == (2, 16, 192) and z.stride(1) == 1 and z.stride(2) == 16
    assert torch.allclose(z, lin_modal(x), atol=1e-5)


def test_hyena_ops_utils_toeplitz_factors():
    # `from hyena_ops.utils import toeplitz, correction_toeplitz` (vortex/ops/hyena_se/ref_fwd.py:24): the definition
    # by brute force on the arange filter of vortex/ops/hyena_se/tests/test_toeplitz.py:33-66, the in-place forms, and the
    # two-pass identity y_c = T x_c + T_hat x_{c-1} against a direct causal convolution
    from hyena_ops.utils import correction_toeplitz, correction_toeplitz_from_empty, toeplitz, toeplitz_from_empty
    from hyena_ops.kernel_utils import BwdKernelConfig, FwdKernelConfig
    assert FwdKernelConfig() is not None and BwdKernelConfig() is not None
    for g, K, C in [(1, 4, 16), (2, 4, 32), (3, 7, 8), (2, 32, 32)]:
        h = torch.arange(1, g * K + 1).reshape(g, 1, K)
        hf = h[:, 0].flip(-1)
        T, Th = toeplitz(hf, C), correction_toeplitz(hf, C)
        assert T.shape == Th.shape == (g, C, C) and T.dtype == hf.dtype
        for gi in range(g):
            for i in range(C):
                for j in range(C):
                    assert int(T[gi, i, j]) == (int(hf[gi, i - j]) if 0 <= i - j < K else 0)
                    assert int(Th[gi, i, j]) == (int(hf[gi, i + C - j]) if (j >= i and i + C - j < K) else 0)
        assert torch.equal(toeplitz_from_empty(torch.empty(g, C, C), hf), T.float())
        assert torch.equal(correction_toeplitz_from_empty(torch.empty(g, C, C), hf), Th.float())
    gen = torch.Generator().manual_seed(3)
    g, K, C, n = 2, 5, 8, 4
    hf = torch.randn(g, K, generator=gen, dtype=torch.float64)
    x = torch.randn(g, n * C, generator=gen, dtype=torch.float64)
    T, Th = toeplitz(hf, C), correction_toeplitz(hf, C, dtype=torch.float64)
    xc = x.reshape(g, n, C)
    prev = torch.cat([torch.zeros(g, 1, C, dtype=torch.float64), xc[:, :-1]], 1)
    y = (torch.einsum("gij,gnj->gni", T, xc) + torch.einsum("gij,gnj->gni", Th, prev)).reshape(g, n * C)
    direct = torch.stack([sum(hf[gi, k] * torch.cat([torch.zeros(k, dtype=torch.float64), x[gi, :n * C - k]])
                              for k in range(K)) for gi in range(g)])
    assert torch.allclose(y, direct, atol=1e-12)


def test_operator_module_compute_filter_matches_the_closed_form():
    # HyenaCascade.compute_filter / update_time (vortex/model/model.py:377-398) on the CPU: h[g, t] = sum_s r e^(lp t)
    from vortex_amd.cascade import HyenaCascade
    cfg = dict(hidden_size=16, num_attention_heads=2, state_size=4, short_filter_length=3, short_filter_bias=False)
    mod = HyenaCascade(cfg, 0, hyena_filter_groups=2)
    with torch.no_grad():
        mod.log_poles.copy_(-torch.rand(2, 4, 1))
    h, dt, lp, r = mod.compute_filter(10, "cpu")
    assert h.shape == (1, 2, 10) and dt == torch.float32 and mod.t.shape == (1, 1, 10)
    want = torch.stack([sum(r[g, s] * torch.exp(lp[g, s, 0] * torch.arange(10)) for s in range(4)) for g in range(2)])
    assert torch.allclose(h[0], want, atol=1e-6)
    assert torch.allclose(h[0, :, 0], r.sum(1), atol=1e-6)          # h[0] = sum of the residues
    mod.update_time(6, "cpu")
    assert mod.t.shape == (1, 1, 6)


def test_per_element_bound_catches_a_single_wrong_halo_sample():
    # the error statement of tests/parity.py, exercised on the CPU: an output that read one wrong input sample at a
    # segment start fails it even where the sample is small, while one-ulp roundings of the pre-gate value pass
    import pytest
    from parity import abs_scale, assert_gated_close, rel_err
    g = torch.Generator().manual_seed(0)
    B, D, L, K = 1, 4, 512, 128
    x2, x1, v = O.make_gates(B, D, L, seed=1)
    h = torch.randn(D, K, generator=g) / K ** 0.5 * torch.exp(-0.08 * torch.arange(K))     # decaying: lag 127 is tiny
    u = x1 * v
    z32 = O.fft_causal_conv_fp32(u.float(), h)
    z_ref = z32.bfloat16()
    ref = x2 * z_ref
    S = abs_scale(u, h)
    # legitimate: sums that land on the other side of a rounding boundary
    nudged = (z32 * (1 + 2.0 ** -10)).bfloat16()
    assert_gated_close(x2 * nudged, ref, z_ref, x2, S, 2.0 ** -8, fft_floor=4e-6)
    # a slip: output t = 256 misses input t - 127 (what a halo sample lost at a segment start does)
    bad32 = z32.clone()
    bad32[..., 256] -= h[:, 127] * u[..., 256 - 127].float()
    bad = x2 * bad32.bfloat16()
    assert rel_err(bad, ref) < 2e-2                     # invisible to the normalised maximum ...
    hflat = torch.randn(D, K, generator=g) / K ** 0.5   # ... unless the oldest tap carries weight
    z32f = O.fft_causal_conv_fp32(u.float(), hflat)
    badf = z32f.clone()
    badf[..., 256] -= hflat[:, 127] * u[..., 256 - 127].float()
    with pytest.raises(AssertionError):
        assert_gated_close(x2 * badf.bfloat16(), x2 * z32f.bfloat16(), z32f.bfloat16(), x2, abs_scale(u, hflat),
                           2.0 ** -8, fft_floor=4e-6)


def test_hyena_ops_reshape_helpers_follow_the_index_definitions():
    # vortex/ops/hyena_se/interface.py:272-339: every layout is a re-indexing of channel d = g*dg + j; checked
    # element by element against that definition, and against the oracle's restatement for the bdl inner layout
    from hyena_ops.interface import (DefaultTwoPassChunkedGateConvGateBwdConfig, DefaultTwoPassChunkedGateConvGateFwdConfig,
                                     gate_gate, reshape_inputs, reshape_outputs)
    from oracle import hyena_oracle as O
    B, G, dg, Ls = 2, 3, 4, 5
    D = G * dg
    bdl = torch.arange(B * D * Ls, dtype=torch.float32).reshape(B, D, Ls)
    blgdg = torch.empty(B, Ls, G, dg)
    bgdgl = torch.empty(B, G, dg, Ls)
    for b in range(B):
        for g in range(G):
            for j in range(dg):
                for t in range(Ls):
                    blgdg[b, t, g, j] = bgdgl[b, g, j, t] = bdl[b, g * dg + j, t]
    forms = {"bdl": bdl, "blgdg": blgdg, "bgdgl": bgdgl}
    for src, dst in [("bdl", "bdl"), ("bdl", "blgdg"), ("blgdg", "bdl"), ("blgdg", "bgdgl"), ("bgdgl", "bdl"),
                     ("bgdgl", "bgdgl")]:
        for got in reshape_inputs(forms[src], forms[src], forms[src], G, src, dst):
            assert torch.equal(got, forms[dst]), (src, dst)
        if dst == "bdl":
            assert all(torch.equal(a, b_) for a, b_ in zip(reshape_inputs(forms[src], forms[src], forms[src], G, src, dst),
                                                           O.reshape_inputs(forms[src], forms[src], forms[src], G, src)))
    with pytest.raises(NotImplementedError):
        reshape_inputs(bdl, bdl, bdl, G, "bdl", "bgdgl")
    with pytest.raises(AssertionError):
        reshape_inputs(blgdg, blgdg, blgdg, G + 1, "blgdg", "bdl")
    bld = bdl.permute(0, 2, 1)
    for out_layout, want in (("bdl", bdl), ("bld", bld), ("blgdg", blgdg)):
        assert torch.equal(reshape_outputs(bdl, G, out_layout, "bdl"), want)
        assert torch.equal(reshape_outputs(bdl, G, out_layout, "bdl"), O.reshape_outputs(bdl, G, out_layout))
    assert torch.equal(reshape_outputs(blgdg, G, "bld", "blgdg"), bld)
    assert torch.equal(reshape_outputs(blgdg, G, "blgdg", "blgdg"), blgdg)
    with pytest.raises(NotImplementedError):
        reshape_outputs(blgdg, G, "bdl", "blgdg")
    assert torch.equal(gate_gate(bdl, 2 * bdl, 3 * bdl), 6 * bdl ** 3)
    f, w = DefaultTwoPassChunkedGateConvGateFwdConfig(), DefaultTwoPassChunkedGateConvGateBwdConfig()
    assert (f.autotune, f.CHUNK_SIZE, f.BLOCK_D, f.RETURN_Y2) == (True, 128, 32, True)
    assert (w.LOAD_TOEPLITZ, w.LOAD_BX_LAG, w.name) == (False, False, "bwd")


def test_projection_row_descriptors_reject_maps_outside_the_tensor():
    # the row descriptors address rows up to 3*hidden - 1 of the projection; a head size that does not divide the
    # width, or a tensor of another height, would make a kernel read outside it
    import pytest
    import torch
    from vortex_amd import ops
    p = torch.zeros(1, 3 * 64, 16, dtype=torch.bfloat16)
    with pytest.raises(ValueError):
        ops.rows_of_projection(p, 64, 2, head_dim=128)
    with pytest.raises(ValueError):
        ops.projection_rows(p, 64, head_dim=48)
    with pytest.raises(ValueError):
        ops.projection_rows(p, 32)
    with pytest.raises(ValueError):
        ops.projection_rows(p, 64, interleave=True, head_dim=16)
    rows, chan = ops.projection_rows(p, 64, head_dim=16)
    assert chan.shape == (3, 64) and int(chan.max()) == 3 * 64 - 1 and len(set(chan.flatten().tolist())) == 3 * 64
    rows, chan = ops.projection_rows(p, 64, interleave=True)
    assert chan[:, 5].tolist() == [15, 16, 17]
