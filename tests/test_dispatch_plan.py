"""Which kernel and launch shape the library picks, pinned over a grid of shapes (no GPU needed): the ten (N, K)
of the reference's dispatch table (gpu/bitnet_kernels/bitnet_kernels.cu:4-33) x ten token counts through the
drop-in product and the forward call, and the decoder's four shapes through the norm-folded calls, against the
committed table tests/golden/dispatch_plan.txt.  A changed threshold or plan shows up as changed rows."""
import os
import sys

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "tests", "golden"))

import make_dispatch_plan as mk  # noqa: E402

from bitnet_amd import _lib  # noqa: E402


def test_dispatch_matches_the_committed_table():
    want = open(mk.PATH).read().splitlines()
    got = list(mk.rows())
    assert len(got) == len(want) == (2 * 10 + 3 * 4) * 10
    changed = [f"- {w}\n+ {g}" for w, g in zip(want, got) if w != g]
    assert not changed, f"{len(changed)} rows differ (regenerate with tests/golden/make_dispatch_plan.py if intended):\n" + "\n".join(changed[:10])


def test_plan_rows_say_what_the_design_says():
    """A few rows spelled out, so that the table cannot drift as a whole: one token goes through the kernel whose
    waves prepare their own slices, five to eight tokens (short rows) through the kernel whose lanes quantize for their
    own token, up to sixteen through a quantizer kernel plus the product without staging, more than sixteen through the MFMA GEMM, the largest matrix through the streaming kernel."""
    p = _lib.plan_name
    assert p(1, 1, 2560, 2560).startswith("bitlinear_solo_kernel<5, 5, 1, false, 0, false, 1> grid=(160,1,1) block=512")
    assert p(1, 1, 13824, 2560).startswith("bitlinear_solo_kernel<5, 5, 1, false, 0, false, 4> grid=(216,1,1)")
    assert p(2, 1, 3840, 2560).startswith("bitlinear_solo_kernel<5, 1, 1, true, 1, false, 1>")
    assert p(1, 8, 3840, 2560).startswith("bitlinear_solo_tok_kernel<5, 1> grid=(240,1,1) block=512")
    two = p(1, 16, 3840, 2560).split(" + ")
    assert len(two) == 2 and two[0].startswith("quant_absmax_rows_kernel<0, 5>") and two[1].startswith("gemv_i2_solo_kernel<5, 1, false>")
    assert "gemm_i2_prefill_kernel" in p(0, 17, 13824, 2560) and "gemm_i2_prefill_dma_kernel<2, 2, 256>" in p(0, 2048, 13824, 2560)
    # 2048 x 2560 outputs are 320 tiles of 64 x 256: one round of the machine plus a quarter -> tiles of two sizes in one
    # launch (256 + 256 workgroups); 2560 x 2560 outputs (400 tiles) leave too large a rest for that
    assert p(0, 2048, 2560, 6912).startswith("gemm_i2_prefill_mix_kernel<256> grid=(512,1,1) block=256")
    assert "gemm_i2_prefill_mix_kernel" not in p(0, 2560, 2560, 2560) and "gemm_i2_prefill_mix_kernel" not in p(0, 2048, 3840, 2560)
    assert p(0, 1, 55296, 5120).startswith("gemv_i2_stream_kernel<5, true>")
    assert p(0, 1, 20480, 3200).startswith("bitlinear_fused_kernel<")


def test_plan_name_argument_checks():
    import ctypes

    lib = _lib.load_library()
    buf = ctypes.create_string_buffer(64)
    assert lib.bitlinear_plan_name(5, 1, 2560, 2560, buf, 64) == 4 and lib.bitlinear_plan_name(0, 1, 2560, 2560, None, 64) == 2
    assert lib.bitlinear_plan_name(0, 1, 100, 2560, buf, 64) == 1 and buf.value == b""  # a shape the library refuses
    assert lib.bitlinear_plan_name(0, 1, 2560, 2560, buf, 8) == 0 and len(buf.value) == 7  # truncated, terminated
