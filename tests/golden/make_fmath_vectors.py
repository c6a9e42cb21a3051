"""Writes tests/golden/fmath_exp_vectors.npz with the reference's own exponent.

Runs oracle/_ref/fmath_exp (the reference's contrib/libs/fmath/fmath.hpp built by
oracle/build_ref.sh, AVX2 path) on seeded inputs: runs of 1, 3, 4, 10 and 128 values, which is how
the result processor calls it (single values, per-document softmax, 128-document blocks), over
ordinary magnitudes, the clamps at +-708/709, infinities and NaN.

    bash oracle/build_ref.sh && python tests/golden/make_fmath_vectors.py
"""
import os
import subprocess
import tempfile

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
TOOL = os.path.join(HERE, "..", "..", "oracle", "_ref", "fmath_exp")


def main():
    rng = np.random.default_rng(20240607)
    x = np.concatenate([
        rng.normal(0.0, 3.0, 4000), rng.uniform(-40.0, 40.0, 3000), rng.uniform(-720.0, 720.0, 2000),
        -np.abs(rng.normal(0.0, 1e-3, 500)), np.array([0.0, -0.0, 1.0, -1.0, 700.0, -700.0, 709.78, 709.7827128933839,
                                                      709.79, 710.0, -708.3, -708.4, -708.39641853226408, -745.0, 1e308,
                                                      -1e308, np.inf, -np.inf, np.nan, 5e-324, 1e-300, 88.7, -87.3]),
    ])
    rng.shuffle(x)
    out = {"x": x}
    with tempfile.TemporaryDirectory() as tmp:
        src, dst = os.path.join(tmp, "in.f64"), os.path.join(tmp, "out.f64")
        x.tofile(src)
        for chunk in (1, 3, 4, 10, 128):
            subprocess.check_call([TOOL, src, dst, str(chunk)])
            out["chunk_%d" % chunk] = np.fromfile(dst)
    np.savez_compressed(os.path.join(HERE, "fmath_exp_vectors.npz"), **out)
    print("wrote %d inputs x %d run lengths" % (len(x), len(out) - 1))


if __name__ == "__main__":
    main()
