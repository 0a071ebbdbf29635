"""Oracle vs the committed vectors of the reference's decode steps
(tests/golden/decode_steps.npz, written by tests/golden/make_decode_golden.py)."""
import os

import numpy as np
import pytest
import torch

from oracle import hyena_oracle as O

G = np.load(os.path.join(os.path.dirname(__file__), "golden", "decode_steps.npz"))


@pytest.mark.parametrize("name", ["se", "mr", "feat", "partial", "partial_flip"])
def test_step_fir_golden(name):
    K, cache, flip, gated, y_is_bf16, st_is_f32 = G[f"fir_{name}_meta"].tolist()
    u = torch.from_numpy(G[f"fir_{name}_u"]).bfloat16()
    st = torch.from_numpy(G[f"fir_{name}_state"]).bfloat16()
    w = torch.from_numpy(G[f"fir_{name}_w"])
    bias = torch.from_numpy(G[f"fir_{name}_bias"]) if f"fir_{name}_bias" in G else None
    y, st2 = O.step_fir(u, st, w, bias=bias, gated_bias=bool(gated), flip_filter=bool(flip))
    assert (y.dtype == torch.bfloat16) == bool(y_is_bf16) and (st2.dtype == torch.float32) == bool(st_is_f32)
    assert np.array_equal(y.float().numpy(), G[f"fir_{name}_y"])
    assert np.array_equal(st2.numpy(), G[f"fir_{name}_state_out"])


@pytest.mark.parametrize("name", ["real_bf16D", "real_f32D", "cplx_f32D"])
def test_step_iir_golden(name):
    x2, x1, v = (torch.from_numpy(G[f"iir_{name}_{k}"]).bfloat16() for k in ("x2", "x1", "v"))
    D = torch.from_numpy(G[f"iir_{name}_D"])
    if "bf16D" in name:
        D = D.bfloat16()
    lp, r, st = (torch.from_numpy(G[f"iir_{name}_{k}"]) for k in ("lp", "r", "state"))
    y, st2 = O.step_iir(x2, x1, v, D, r, lp, st)
    assert str(y.dtype) == str(G[f"iir_{name}_ydtype"])
    assert np.array_equal(y.numpy(), G[f"iir_{name}_y"])
    assert np.array_equal(st2.numpy(), G[f"iir_{name}_state_out"])
