"""Writes tests/golden/dispatch_plan.txt: what the library launches for every (entry, M, N, K) of the grid below,
as bitlinear_plan_name reports it (host only, no GPU).  Run it after a deliberate change of a dispatch threshold
or a kernel's template arguments, and read the diff: every changed row is a call that now takes another kernel or
launch shape.

    python tests/golden/make_dispatch_plan.py
"""
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)

# (N, K) of the reference's dispatch table (gpu/bitnet_kernels/bitnet_kernels.cu:4-33)
REFERENCE_SHAPES = [(3840, 2560), (2560, 2560), (13824, 2560), (2560, 6912), (4800, 3200), (3200, 3200), (20480, 3200),
                    (3200, 10240), (5120, 27648), (55296, 5120)]
TOKENS = [1, 2, 4, 5, 8, 16, 17, 128, 512, 2048]
ENTRIES = {0: "bitlinear_int8xint2", 1: "bitlinear_forward_bf16", 2: "bitlinear_norm_forward_bf16",
           3: "bitlinear_norm_forward_bf16+residual", 4: "bitlinear_norm_forward_bf16+gate+residual"}


def rows():
    from bitnet_amd import _lib

    lib = _lib.load_library()
    assert lib.bitlinear_set_tuning(0, 0, 0, 0) == 0
    for entry, name in ENTRIES.items():
        shapes = REFERENCE_SHAPES if entry <= 1 else REFERENCE_SHAPES[:4]  # the norm-folded calls: the decoder's four
        for n, k in shapes:
            for m in TOKENS:
                yield f"{name} M={m} N={n} K={k}: {_lib.plan_name(entry, m, n, k)}"


PATH = os.path.join(ROOT, "tests", "golden", "dispatch_plan.txt")

if __name__ == "__main__":
    with open(PATH, "w") as f:
        f.write("\n".join(rows()) + "\n")
    print(PATH)
