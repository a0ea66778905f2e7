"""Writes the small known-answer fixtures of tests/golden/ (inputs + expected int8 O).

The reference ships no data files and regenerates its inputs from library-defined distributions on every run
(test_fmha_i8.cpp:49-89), so there is nothing of the reference's to record here.  These vectors are regression anchors:
inputs from this repository's seeded generators, expected outputs from the CPU checker after it passed the closed-form
and cross-implementation tests in tests/test_oracle_*.py.  Run from the repository root:
    python tests/golden/make_fixtures.py
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

import fmha_cases as fc  # noqa: E402
import __graft_entry__ as g  # noqa: E402

CASES = {
    # name: make_inputs keyword arguments
    "c1_b1h2s128d64": dict(B=1, H=2, S=128, d=64),
    "prefix_b1h1s256d128": dict(B=1, H=1, S=256, d=128, valid_lengths=[160]),
    "scatter_b1h1s256d64_reference_style": dict(B=1, H=1, S=256, d=64, dist="reference", pad="scatter"),
    "student_t_b1h1s384d64": dict(B=1, H=1, S=384, d=64, dist="student_t", sigma=0.5),
}


def main():
    orc = g.load_oracle()
    for name, kw in CASES.items():
        c = fc.make_inputs(seed=fc.MASTER_SEED, **kw)
        o = orc.fmha_i8_blockwise(c["q"], c["k"], c["v"], c["mask"], c["q_amax"], c["k_amax"], c["v_amax"],
                                  c["o_amax"])
        # the same inputs through the checker's 255-step mode (P = rne(255 p); README.md:15,186 of the reference plans it)
        o_full = orc.fmha_i8_blockwise_cross(c["q"], c["k"], c["v"], c["mask"], c["q_amax"], c["k_amax"], c["v_amax"],
                                             c["o_amax"], full_range_p=True)
        np.savez_compressed(os.path.join(HERE, name + ".npz"), q=c["q"], k=c["k"], v=c["v"], mask=c["mask"],
                            amax=np.array([c["q_amax"], c["k_amax"], c["v_amax"], c["o_amax"]], np.float32), o=o,
                            o_full_range_p=o_full)
        print(name, o.shape, "saturated:", float((np.abs(o) == 127).mean()))


if __name__ == "__main__":
    main()
