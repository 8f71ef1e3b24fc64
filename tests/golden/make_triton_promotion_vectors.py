"""Writes ``triton_promotion_vectors.json``: how the installed Triton package (the third-party
package the reference's generated kernels are compiled by) types a tile times a Python literal
and a tile times a run-time scalar, run by its CPU interpreter (``TRITON_INTERPRET=1``).

* ``(q * 1.44269504089).to(q.dtype)`` -- the first line of the reference's attention
  application (tests/test_attention.py:46);
* ``q * (scale * 1.44269504089)`` with a run-time ``scale`` -- this build's scaled variant;
* ``beta * input + alpha * product.to(float16)`` with run-time ``beta`` / ``alpha`` -- the
  epilogue of the reference's addmm application (tests/test_addmm.py:36-38).

The reference itself is not involved.  Floats are stored as bit patterns.  A compiled Triton
kernel receives a Python float argument as an fp32 scalar; the interpreter would hand the
Python object through (and so type it like a literal), so the run-time scalars are read from
one-element fp32 tensors here, which gives them the compiled kernel's type.

Usage:  python tests/golden/make_triton_promotion_vectors.py
"""

import json
import os
import pathlib

os.environ["TRITON_INTERPRET"] = "1"

import torch  # noqa: E402
import triton  # noqa: E402
import triton.language as tl  # noqa: E402


@triton.jit
def literal_kernel(q, out, N: tl.constexpr):
    lanes = tl.arange(0, N)
    tile = tl.load(q + lanes)
    tl.store(out + lanes, (tile * 1.44269504089).to(tile.dtype))


@triton.jit
def scaled_kernel(q, scale_pointer, out, N: tl.constexpr):
    lanes = tl.arange(0, N)
    tile = tl.load(q + lanes)
    scale = tl.load(scale_pointer)
    tl.store(out + lanes, (tile * (scale * 1.44269504089)).to(tile.dtype))


@triton.jit
def epilogue_kernel(input, product, beta_pointer, alpha_pointer, out, N: tl.constexpr):
    lanes = tl.arange(0, N)
    beta = tl.load(beta_pointer)
    alpha = tl.load(alpha_pointer)
    rounded = tl.load(product + lanes).to(tl.float16)
    tl.store(out + lanes, beta * tl.load(input + lanes) + alpha * rounded)


def bits(tensor):
    return tensor.view(torch.int16 if tensor.element_size() == 2 else torch.int32).tolist()


def main():
    torch.manual_seed(20240607)
    n = 256
    cases = {}
    # fp16 only: the interpreter has no bf16 constants, and it narrows fp32 to bf16 by dropping
    # bits where a compiled kernel rounds to nearest, so its bf16 outputs would pin the wrong thing
    for name, dtype in (("fp16", torch.float16),):
        q = (torch.randn(n) * 3).to(dtype)
        out = torch.empty_like(q)
        literal_kernel[(1,)](q, out, N=n)
        cases[f"literal_{name}"] = {"q": bits(q), "out": bits(out)}
        out = torch.empty_like(q)
        scaled_kernel[(1,)](q, torch.tensor([128**-0.5], dtype=torch.float32), out, N=n)
        cases[f"scaled_{name}"] = {"q": bits(q), "scale": 128**-0.5, "out": bits(out)}
    input = torch.randn(n).to(torch.float16)
    product = torch.randn(n) * 40
    out = torch.empty(n, dtype=torch.float16)
    epilogue_kernel[(1,)](input, product, torch.tensor([0.3]), torch.tensor([1.7]), out, N=n)
    cases["addmm_epilogue_fp16"] = {"input": bits(input), "product": bits(product), "beta": 0.3, "alpha": 1.7, "out": bits(out)}
    payload = {"source": f"triton {triton.__version__} under TRITON_INTERPRET=1", "cases": cases}
    path = pathlib.Path(__file__).resolve().parent / "triton_promotion_vectors.json"
    path.write_text(json.dumps(payload))
    print(f"wrote {len(cases)} cases to {path}")


if __name__ == "__main__":
    main()
