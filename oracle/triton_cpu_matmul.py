"""TEST / MEASUREMENT INFRASTRUCTURE ONLY -- the reference's CPU path for the 512^3 matmul.

The reference runs on a CPU by handing the Triton kernel it generates to Triton's interpreter
(``TRITON_INTERPRET=1``).  The reference package does not travel with this repository, so this file
carries its own ``@triton.jit`` kernel with the structure of the kernel the reference generates for the
README matmul (README.md:40-62; launch and indexing rules src/ninetoothed/generation.py:629-636,
676-706, 746-817): a one-dimensional grid over output tiles, the tile id unravelled row-major, masked
loads with zero fill, ``tl.dot`` accumulating in fp32, fixed 64 x 64 x 64 blocks (so no autotuner runs),
the accumulator stored into the fp16 output.  The interpreter executes the programs of the grid one after
another in Python, with numpy doing each tile product.

Run as a program (a process of its own, so that the interpreter switch is set before Triton is imported):

    python -m oracle.triton_cpu_matmul [size]

prints one JSON object: seconds per run, TFLOP/s, threads, and the largest deviation from ``torch.matmul``.
"""

import json
import os
import sys
import time

os.environ["TRITON_INTERPRET"] = "1"


def main():
    size = int(sys.argv[1]) if len(sys.argv) > 1 else 512
    try:
        import torch
        import triton
        import triton.language as tl
    except ImportError as error:
        print(json.dumps({"error": f"triton not importable: {error}"}))
        return

    @triton.jit
    def matmul_kernel(lhs, rhs, out, m, n, k, lhs_s0, lhs_s1, rhs_s0, rhs_s1, out_s0, out_s1, BM: tl.constexpr, BN: tl.constexpr, BK: tl.constexpr):
        tile = tl.program_id(0)
        tiles_n = tl.cdiv(n, BN)
        tile_m = tile // tiles_n
        tile_n = tile % tiles_n
        rows = tile_m * BM + tl.arange(0, BM)
        cols = tile_n * BN + tl.arange(0, BN)
        acc = tl.zeros((BM, BN), dtype=tl.float32)
        for step in range(tl.cdiv(k, BK)):
            ks = step * BK + tl.arange(0, BK)
            a = tl.load(lhs + rows[:, None] * lhs_s0 + ks[None, :] * lhs_s1, mask=(rows[:, None] < m) & (ks[None, :] < k), other=0.0)
            b = tl.load(rhs + ks[:, None] * rhs_s0 + cols[None, :] * rhs_s1, mask=(ks[:, None] < k) & (cols[None, :] < n), other=0.0)
            acc += tl.dot(a, b)
        tl.store(out + rows[:, None] * out_s0 + cols[None, :] * out_s1, acc, mask=(rows[:, None] < m) & (cols[None, :] < n))

    generator = torch.Generator().manual_seed(0)
    lhs = torch.randn(size, size, generator=generator).to(torch.float16)
    rhs = torch.randn(size, size, generator=generator).to(torch.float16)
    out = torch.empty(size, size, dtype=torch.float16)
    block = 64
    grid = (triton.cdiv(size, block) * triton.cdiv(size, block),)

    def run():
        matmul_kernel[grid](lhs, rhs, out, size, size, size, lhs.stride(0), lhs.stride(1), rhs.stride(0), rhs.stride(1), out.stride(0), out.stride(1), BM=block, BN=block, BK=block)

    run()  # warm-up
    times = []
    for _ in range(3):
        start = time.perf_counter()
        run()
        times.append(time.perf_counter() - start)
    seconds = sorted(times)[1]
    expected = torch.matmul(lhs.float(), rhs.float())
    print(json.dumps({
        "seconds": seconds,
        "value": 2.0 * size**3 / seconds / 1e12,
        "unit": "TFLOP/s",
        "cores": 1,
        "threads_available": torch.get_num_threads(),
        "max_abs_error": float((out.float() - expected).abs().max()),
        "sample": f"own @triton.jit matmul under TRITON_INTERPRET=1 (triton {triton.__version__}), fp16 {size}^3, 64x64x64 blocks, "
                  f"{grid[0]} programs run one after another in Python, median of 3 runs: {seconds:.2f} s",
    }))


if __name__ == "__main__":
    main()
