"""Writes tests/golden/quantizer_script.npz: input/output vectors of the reference's offline
quantizer function, `quantize_int4_per_group` of scripts/quantize_gpt2_int4.py, evaluated in
the build container (numpy 2.2.6).  Run once, by hand, where the reference checkout exists:

    python tests/golden/make_quantizer_fixture.py /root/reference

Only that one function is imported (the script's main() is not run).  The fixture pins what
reading the source leaves open: float32-vs-float64 evaluation of `w / scale` and numpy's
round-half-to-even on exact ties.
"""
import importlib.util
import os
import sys

import numpy as np

ref_root = sys.argv[1] if len(sys.argv) > 1 else "/root/reference"
spec = importlib.util.spec_from_file_location("quantize_gpt2_int4", os.path.join(ref_root, "scripts", "quantize_gpt2_int4.py"))
mod = importlib.util.module_from_spec(spec)
spec.loader.exec_module(mod)

rng = np.random.default_rng(20240607)
out = {}

# case A: random N(0, 0.02) weights, [out=8, in=64], group 32
wa = (rng.standard_normal((8, 64)) * 0.02).astype(np.float32)
pa, sa = mod.quantize_int4_per_group(wa, group_size=32)
out.update(a_weight=wa, a_packed=pa, a_scales=sa, a_group=np.int32(32))

# case B: exact .5 ties.  Column max is 7.0 so scale is exactly 1.0 and w/scale = w.
wb = np.zeros((4, 32), np.float32)
wb[:, 0] = 7.0
ties = np.array([0.5, 1.5, 2.5, 3.5, -0.5, -1.5, -2.5, -3.5, 4.5, 5.5, 6.5, -4.5, -5.5, -6.5, -7.5, 0.49999997], np.float32)
wb[0, 1:17] = ties
wb[1, 1:17] = -ties
wb[2, 1:17] = ties * 0.5
wb[3, 1:9] = np.array([-8.0, -7.49, 7.0, 6.9999995, 1e-13, 0.0, -0.0, 3.0], np.float32)
pb, sb = mod.quantize_int4_per_group(wb, group_size=32)
out.update(b_weight=wb, b_packed=pb, b_scales=sb, b_group=np.int32(32))

# case C: group 128 default, short last group (in=136 -> groups of 128 and 8), an all-zero group
wc = (rng.standard_normal((6, 136)) * 0.05).astype(np.float32)
wc[2, 128:] = 0.0
pc, sc = mod.quantize_int4_per_group(wc, group_size=128)
out.update(c_weight=wc, c_packed=pc, c_scales=sc, c_group=np.int32(128))

dst = os.path.join(os.path.dirname(os.path.abspath(__file__)), "quantizer_script.npz")
np.savez(dst, **out)
print("wrote", dst, {k: (v.shape, v.dtype) for k, v in out.items() if hasattr(v, "shape")})
