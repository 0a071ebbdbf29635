"""Writes tests/golden/decode_steps.npz: input/output vectors of the reference's
step_fir / step_iir (vortex/model/engine.py:406-467), the two hot-path functions
that none of the reference's own tests pins.  Run once in the build container,
where the reference checkout is mounted; the fixture (data only) is committed.

    cd /tmp && python /root/repo/tests/golden/make_decode_golden.py /root/reference
"""
import os
import sys

import numpy as np
import torch

ref_root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
sys.path.insert(0, ref_root)
from vortex.model.engine import HyenaInferenceEngine  # noqa: E402

eng = HyenaInferenceEngine()
g = torch.Generator().manual_seed(2024)
out = {}


def f32(t):
    return t.detach().to(torch.float32).numpy()


B, D = 3, 8
for name, K, cache, flip, gated, with_bias in [
    ("se", 7, 6, False, False, False),
    ("mr", 128, 127, True, True, True),
    ("feat", 3, 2, False, False, True),
    ("partial", 7, 3, False, False, False),
    ("partial_flip", 128, 50, True, True, True),
]:
    u = torch.randn(B, D, generator=g).bfloat16()
    st = torch.randn(B, D, cache, generator=g).bfloat16()
    w = torch.randn(D, 1, K, generator=g)
    bias = torch.randn(D, generator=g) if with_bias else None
    y, st2 = eng.step_fir(u, st.clone(), w, bias=bias, gated_bias=gated, flip_filter=flip)
    out[f"fir_{name}_u"] = f32(u)
    out[f"fir_{name}_state"] = f32(st)
    out[f"fir_{name}_w"] = f32(w)
    if bias is not None:
        out[f"fir_{name}_bias"] = f32(bias)
    out[f"fir_{name}_y"] = f32(y)
    out[f"fir_{name}_state_out"] = f32(st2)
    out[f"fir_{name}_meta"] = np.array([K, cache, int(flip), int(gated), int(y.dtype == torch.bfloat16),
                                        int(st2.dtype == torch.float32)])

S = 16
for name, cplx, dtypeD in [("real_bf16D", False, torch.bfloat16), ("real_f32D", False, torch.float32),
                           ("cplx_f32D", True, torch.float32)]:
    x2, x1, v = (torch.randn(B, D, generator=g).bfloat16() for _ in range(3))
    Dp = torch.randn(D, generator=g).to(dtypeD)
    if cplx:
        lp = torch.complex(-0.1 * torch.rand(D, S, 1, generator=g), 3.0 * torch.rand(D, S, 1, generator=g))
        r = torch.complex(torch.randn(D, S, generator=g), torch.randn(D, S, generator=g))
        st = torch.complex(torch.randn(B, D, S, generator=g), torch.randn(B, D, S, generator=g))
    else:
        lp = -0.1 * torch.rand(D, S, 1, generator=g)
        r = torch.randn(D, S, generator=g)
        st = torch.randn(B, D, S, generator=g)
    y, st2 = eng.step_iir(x2, x1, v, Dp, r, lp, st.clone())
    for k, t in [("x2", x2), ("x1", x1), ("v", v), ("D", Dp)]:
        out[f"iir_{name}_{k}"] = f32(t)
    for k, t in [("lp", lp), ("r", r), ("state", st), ("y", y), ("state_out", st2)]:
        out[f"iir_{name}_{k}"] = t.detach().numpy()
    out[f"iir_{name}_ydtype"] = np.array(str(y.dtype))

dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "decode_steps.npz")
np.savez_compressed(dst, **out)
print("wrote", dst, len(out), "arrays")
