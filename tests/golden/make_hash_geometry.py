"""Re-derives tests/golden/hash_geometry.json with exact rational arithmetic.

N_l = floor(N_min * b**l) where b = exp((ln N_max - ln N_min)/(L-1)) + 1e-5 rounded to
float32 (the reference evaluates the power on a float32 tensor,
triton_helpers/layers/hash_encoding/helpers.py:37-39).  The power is evaluated here
exactly with fractions; a level whose exact value lies within 2e-6 (relative) of an
integer is reported as ambiguous, because a float32 pow could round across it
(level 0 is exact: b**0 == 1).

Run: python tests/golden/make_hash_geometry.py   (prints the JSON body; CPU only)
"""
import json
import math
from fractions import Fraction

import numpy as np


def exact_geometry(T, levels, dims, min_res, max_res):
    b64 = math.exp((math.log(max_res) - math.log(min_res)) / (levels - 1)) + 1e-5
    b = Fraction(float(np.float32(b64)))
    res, ambiguous = [], []
    for l in range(levels):
        v = b**l * min_res
        n = v.numerator // v.denominator
        frac = float(v - n)
        if l > 0 and min(frac, 1 - frac) < 2e-6 * float(v):
            ambiguous.append(l)
        res.append(int(n))
    rows = [min((n + 1) ** dims, T) for n in res]
    first = next((i for i, n in enumerate(res) if (n + 1) ** dims > T), levels + 1)
    return dict(T=T, levels=levels, dims=dims, min_res=min_res, max_res=max_res, resolutions=res, rows=rows,
                first_hash_level=first, total_rows=sum(rows), ambiguous_levels=ambiguous)


if __name__ == "__main__":
    print(json.dumps({"bench": exact_geometry(2**19, 16, 3, 16, 7006), "default": exact_geometry(2**14, 16, 3, 16, 512)}, indent=1))
