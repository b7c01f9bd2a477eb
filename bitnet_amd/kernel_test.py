"""Known-answer check and timing of the drop-in product at the reference's shapes.

What gpu/test.py:31-86 of the reference does, for the library built here:
`python -m bitnet_amd.kernel_test` draws, per (N, K) of the reference's list, a
ternary weight matrix and one int8 activation row, packs the weights, calls
`bitlinear_int8xint2` with unit scales and compares the bf16 result with an
exact integer matmul (printed as the reference prints it: `custom == np True`);
then it times the call against torch's bf16 matmul on the same operands and
prints `Shape(N, K), W2A8: .. us, torch BF16: .. us`.  Two timings are given
per kernel: calls issued one after the other from the host (what the
reference's `benchmark.Timer` measures: launch overhead included) and the same
calls replayed from a captured graph (GPU time per call in a dependent chain).
"""
import argparse
import time
from typing import Callable, List, Sequence, Tuple

import torch

from .bitlinear import bitnet_int8xint2_linear
from .pack_weight import convert_weight_int8_to_int2

# gpu/test.py:32-41
REFERENCE_SHAPES: Tuple[Tuple[int, int], ...] = (
    (2560, 2560), (3840, 2560), (13824, 2560), (2560, 6912), (3200, 3200), (4800, 3200), (3200, 10240), (20480, 3200),
)


def _host_loop_us(fn: Callable[[], object], iters: int) -> float:
    for _ in range(5):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for _ in range(iters):
        fn()
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) * 1e6 / iters


def _graph_us(fn: Callable[[], object], calls: int, replays: int) -> float:
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        fn()  # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        for _ in range(calls):
            fn()
    graph.replay()
    torch.cuda.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(replays):
        graph.replay()
    end.record()
    torch.cuda.synchronize()
    return start.elapsed_time(end) * 1e3 / (calls * replays)


def check_and_time(shapes: Sequence[Tuple[int, int]] = REFERENCE_SHAPES, M: int = 1, iters: int = 50, seed: int = 42,
                   out=print) -> List[dict]:
    """One entry per shape: {"N", "K", "equal", "w2a8_us", "bf16_us", "w2a8_graph_us", "bf16_graph_us"}."""
    if not torch.cuda.is_available():
        raise RuntimeError("kernel_test needs a GPU: the HIP library is the only compute path")
    dev = torch.device("cuda")
    gen = torch.Generator(device=dev).manual_seed(seed)
    results = []
    for N, K in shapes:
        weight = torch.randint(-1, 2, (N, K), dtype=torch.int8, device=dev, generator=gen)
        packed = convert_weight_int8_to_int2(weight, keep_device=True)
        act = torch.randint(-128, 127, (M, K), dtype=torch.int8, device=dev, generator=gen)
        s = torch.ones(M, dtype=torch.bfloat16, device=dev)
        ws = torch.ones(6, dtype=torch.bfloat16, device=dev)
        want = (act.double() @ weight.double().T).to(torch.bfloat16)  # exact in fp64: |acc| < 2^53
        ret = torch.empty(M, N, dtype=torch.bfloat16, device=dev)
        got = bitnet_int8xint2_linear(act, packed, s, ws, out=ret)
        equal = bool(torch.all(got == want))
        out(f"custom == np {equal}")
        act_bf16, weight_bf16 = act.to(torch.bfloat16), weight.to(torch.bfloat16).T.contiguous()
        ours = lambda: bitnet_int8xint2_linear(act, packed, s, ws, out=ret)
        dense = lambda: torch.matmul(act_bf16, weight_bf16)
        r = {"N": N, "K": K, "equal": equal,
             "w2a8_us": _host_loop_us(ours, iters), "bf16_us": _host_loop_us(dense, iters),
             "w2a8_graph_us": _graph_us(ours, 20, 10), "bf16_graph_us": _graph_us(dense, 20, 10)}
        out(f"Shape{(N, K)}, W2A8: {r['w2a8_us']:.2f}us, torch BF16: {r['bf16_us']:.2f}us"
            f"   (from a graph: {r['w2a8_graph_us']:.2f}us, {r['bf16_graph_us']:.2f}us)")
        results.append(r)
    return results


def main(argv=None) -> int:
    ap = argparse.ArgumentParser(description=__doc__.split("\n\n")[0])
    ap.add_argument("--m", type=int, default=1, help="activation rows (the reference tests one)")
    ap.add_argument("--iters", type=int, default=50)
    args = ap.parse_args(argv)
    results = check_and_time(M=args.m, iters=args.iters)
    return 0 if all(r["equal"] for r in results) else 1


if __name__ == "__main__":
    raise SystemExit(main())
