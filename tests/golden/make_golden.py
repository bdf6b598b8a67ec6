"""Writes the golden fixtures of tests/golden/ from the compiled reference
translation units (oracle/_ref/libref_cpu.so; build with `make -C oracle ref`
in a container that has the reference checkout).

    python -m tests.golden.make_golden

i4_bounds.json: for seeded int4 code matrices, the k_tile the reference's
INT16-partial certificate (src/rk_npu_i4_bounds.cpp) selects when asked for the
largest safe tile (requested = 0) and whether explicit tiles certify.  The
matrices are regenerated from (seed, K, N, low, high, heavy_columns) by the
tests; only inputs' recipes and expected outputs are stored.
"""
import json
import os

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))


def i4_matrix(seed, K, N, low, high, heavy):
    rng = np.random.default_rng(seed)
    B = rng.integers(low, high + 1, (K, N)).astype(np.int8)
    for c in range(heavy):
        B[:, (c * 7) % N] = -8 if c % 2 == 0 else 7
    return B


I4_RECIPES = [
    dict(seed=1, K=2048, N=64, low=1, high=1, heavy=0),
    dict(seed=2, K=2048, N=64, low=-8, high=-8, heavy=0),
    dict(seed=3, K=4096, N=96, low=-7, high=7, heavy=0),
    dict(seed=4, K=4096, N=96, low=-7, high=7, heavy=2),
    dict(seed=5, K=1000, N=33, low=-8, high=7, heavy=1),
    dict(seed=6, K=513, N=65, low=-3, high=3, heavy=0),
    dict(seed=7, K=20003, N=17, low=-8, high=7, heavy=3),
    dict(seed=8, K=64, N=300, low=-8, high=7, heavy=0),
]


def i4_bound_cases():
    from oracle import ref_binding as ref
    cases = []
    for r in I4_RECIPES:
        B = i4_matrix(**r)
        auto = ref.bound_i4(B, 0)
        explicit = {str(t): int(ref.bound_i4(B, t) == t) for t in (512, 1024, 2048) if t <= 2048}
        cases.append(dict(recipe=r, auto_k_tile=int(auto), explicit=explicit))
    return cases


def main():
    with open(os.path.join(HERE, "i4_bounds.json"), "w") as f:
        json.dump(i4_bound_cases(), f, indent=1)
    print("wrote i4_bounds.json")


if __name__ == "__main__":
    main()
