"""Writes ``triton_rand_vectors.json``: outputs of ``tl.rand(seed, offsets)`` from the
installed Triton package run by its CPU interpreter (``TRITON_INTERPRET=1``).

Triton is the third-party package that the reference's ``ntl.rand`` resolves to
(src/ninetoothed/generation.py:849-855); the reference itself is not involved.
The vectors pin what ``oracle.programs.triton_rand`` adds on top of Philox: which
output word is used, where the offset's halves and the seed's halves go, the
mirroring of negative words and the scale.  Floats are stored as their bit patterns.

Usage:  python tests/golden/make_triton_rand_vectors.py
"""

import json
import os
import pathlib

os.environ["TRITON_INTERPRET"] = "1"

import torch  # noqa: E402
import triton  # noqa: E402
import triton.language as tl  # noqa: E402


@triton.jit
def rand_kernel(out, offsets, seed, N: tl.constexpr):
    lanes = tl.arange(0, N)
    tl.store(out + lanes, tl.rand(seed, tl.load(offsets + lanes)))


OFFSETS_32 = [0, 1, 2, 3, 17, 348, 65535, 65536, 1 << 20, (1 << 31) - 2, (1 << 31) - 1, 12345678, 99, 100, 101, 7]
OFFSETS_64 = [0, 1, 2, 3, (1 << 31) - 1, 1 << 31, (1 << 31) + 1, (1 << 32) - 1, 1 << 32, (1 << 32) + 5, (1 << 40) + 7, (1 << 62) + 1, 348, 17, 5, 6]
SEEDS = [0, 1, 42, 1234, (1 << 31) + 11, (1 << 32) - 1, 1 << 32, (1 << 40) + 3, (1 << 62) + 12345]


def main():
    cases = []
    for dtype, name, offsets in ((torch.int32, "int32", OFFSETS_32), (torch.int64, "int64", OFFSETS_64)):
        for seed in SEEDS:
            out = torch.empty(len(offsets), dtype=torch.float32)
            rand_kernel[(1,)](out, torch.tensor(offsets, dtype=dtype), seed, N=len(offsets))
            cases.append({"seed": seed, "offset_dtype": name, "offsets": offsets, "bits": out.view(torch.int32).tolist()})
    payload = {"source": f"triton {triton.__version__}, tl.rand under TRITON_INTERPRET=1", "cases": cases}
    path = pathlib.Path(__file__).resolve().parent / "triton_rand_vectors.json"
    path.write_text(json.dumps(payload))
    print(f"wrote {len(cases)} cases to {path}")


if __name__ == "__main__":
    main()
