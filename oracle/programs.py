"""TEST INFRASTRUCTURE ONLY -- CPU restatement (numpy) of the five programs of
the hot path, program by program and tile by tile, as the reference's
generated kernels execute them.  Nothing in the product imports this module.

Every function builds the arrangement with :mod:`oracle.arrangement` exactly
as the reference program does, then loops over the launch grid: for every
program it gathers the tiles through the offset tables (masked positions read
the tensor's ``other`` value, ``0`` when it is ``None``), applies the
application with the stated rounding points, and scatters the result.

* matmul   -- tests/test_matmul.py:14-45 (arrangement, application); README.md:40-62
* addmm    -- tests/test_addmm.py:13-38
* softmax  -- tests/test_softmax.py:10-27
* attention-- tests/test_attention.py:14-70
* conv2d   -- tests/test_conv2d.py:13-48
(all paths relative to the reference checkout)

Arithmetic conventions restated from the kernels the reference generates:
``ntl.dot`` multiplies fp16/bf16 tiles exactly and accumulates in fp32;
``.to(dtype)`` and stores into a narrower tensor round to nearest even;
a tile times a Python float keeps the tile's dtype, a tile times a run-time
fp32 scalar promotes to fp32 (Triton promotion rules:
``language/semantic.py`` of triton 3.6, binary arithmetic type checks).

Pinned (tests/test_oracle_programs.py) against the library routines the
reference's own tests compare with -- ``torch.matmul``, ``torch.addmm``,
``torch.softmax``, ``F.scaled_dot_product_attention``, ``F.conv2d`` -- and
against closed forms (identity matrices, constant rows, one-key attention,
1x1 convolution == matmul).  The typing rules above and ``triton_rand`` are
pinned by vectors the installed Triton package itself produced under its CPU
interpreter (tests/golden/make_triton_*_vectors.py).
"""

import numpy as np

from oracle.arrangement import View, gather, scatter

LOG2E = 1.44269504089  # the literal of tests/test_attention.py:46


def _round(values, dtype):
    """Round-to-nearest-even conversion, with bfloat16 emulated on top of fp32."""
    if dtype == "bf16":
        as_f32 = np.asarray(values, dtype=np.float32)
        bits = as_f32.view(np.uint32)
        rounded = ((bits + 0x7FFF + ((bits >> 16) & 1)) & 0xFFFF0000).astype(np.uint32)
        result = rounded.view(np.float32)
        return np.where(np.isnan(as_f32), as_f32, result)
    return np.asarray(values).astype({"fp16": np.float16, "fp32": np.float32}[dtype])


def arrange_matmul(lhs_view, rhs_view, out_view, bm, bn, bk):
    """tests/test_matmul.py:22-38 applied to already prepared 2-d views."""
    out = out_view.tile((bm, bn))
    grid = out.level_shape(0)
    lhs = lhs_view.tile((bm, bk)).tile((1, -1)).expand((-1, grid[1])).squeeze(0, level=1)
    rhs = rhs_view.tile((bk, bn)).tile((-1, 1)).expand((grid[0], -1)).squeeze(1, level=1)
    return lhs, rhs, out


def _matmul_programs(a_flat, b_flat, lhs, rhs, out, on_tile):
    grid = out.level_shape(0)
    for i in range(grid[0]):
        for j in range(grid[1]):
            acc = np.zeros(out.table.shape[2:], dtype=np.float32)
            for k in range(lhs.table.shape[2]):
                a = gather(a_flat, lhs.table[i, j, k], None).astype(np.float32)
                b = gather(b_flat, rhs.table[i, j, k], None).astype(np.float32)
                acc += a @ b
            on_tile(i, j, acc)


def matmul(a, b, bm=64, bn=64, bk=64, out_dtype="fp16"):
    """C = A @ B per (bm, bn) program with a loop over bk blocks."""
    m, n = a.shape[0], b.shape[1]
    lhs, rhs, out = arrange_matmul(View.of_shape(a.shape), View.of_shape(b.shape), View.of_shape((m, n)), bm, bn, bk)
    c = np.zeros(m * n, dtype=np.float32)

    def store(i, j, acc):
        scatter(c, out.table[i, j], _round(acc, out_dtype).astype(np.float32))

    _matmul_programs(a.reshape(-1), b.reshape(-1), lhs, rhs, out, store)
    return c.reshape(m, n)


def addmm(input, mat1, mat2, beta, alpha, bm=64, bn=64, bk=64, dtype="fp16"):
    """out = beta * input + alpha * round(mat1 @ mat2), the combination in fp32
    (beta, alpha are run-time fp32 scalars), rounded again on store."""
    m, n = mat1.shape[0], mat2.shape[1]
    lhs, rhs, out = arrange_matmul(View.of_shape(mat1.shape), View.of_shape(mat2.shape), View.of_shape((m, n)), bm, bn, bk)
    input_view = View.of_shape((m, n)).tile((bm, bn))
    input_flat = input.reshape(-1)
    c = np.zeros(m * n, dtype=np.float32)
    beta32, alpha32 = np.float32(beta), np.float32(alpha)

    def store(i, j, acc):
        product = _round(acc, dtype).astype(np.float32)
        tile_in = gather(input_flat, input_view.table[i, j], None).astype(np.float32)
        value = beta32 * tile_in + alpha32 * product
        scatter(c, out.table[i, j], _round(value, dtype).astype(np.float32))

    _matmul_programs(mat1.reshape(-1), mat2.reshape(-1), lhs, rhs, out, store)
    return c.reshape(m, n)


def softmax(x, block_size=None):
    """One program per (row, block): softmax over that block, fp32 arithmetic,
    out-of-bounds input reads -inf.  ``block_size`` defaults to the row length
    (rounded up to a power of two by the launch, which only adds masked lanes)."""
    rows, cols = x.shape
    block = cols if block_size is None else block_size
    padded_block = 1 << (block - 1).bit_length()
    view = View.of_shape(x.shape).tile((1, block))
    flat = x.reshape(-1).astype(np.float32)
    out = np.zeros(rows * cols, dtype=np.float32)
    for i in range(view.table.shape[0]):
        for j in range(view.table.shape[1]):
            table = view.table[i, j]
            table = np.concatenate([table, np.full((1, padded_block - block), -1, dtype=np.intp)], axis=1)
            row = gather(flat, table, float("-inf"))
            row_minus_max = row - np.max(row)
            numerator = np.exp(row_minus_max, dtype=np.float32)
            denominator = np.sum(numerator, dtype=np.float32)
            scatter(out, table, (numerator / denominator).astype(np.float32))
    return out.reshape(rows, cols)


def attention(q, k, v, is_causal=False, scale=None, bm=64, bn=32, dtype="fp16"):
    """Online-softmax attention forward, q block by q block, k/v block by k/v
    block (no block is skipped; causal and tail positions are masked to -inf).

    ``scale=None`` is the reference program as it stands (tests/test_attention.py:46):
    ``q * 1.44269504089`` multiplies a tile by a Python literal, which Triton first
    turns into a constant of the tile's type (fp16: 1.4423828125, bf16: 1.4453125) and
    then multiplies in that type -- one rounding of the exact product.  With a number,
    the program is this build's variant with a run-time ``scale`` argument,
    ``q * (scale * 1.44269504089)``: a run-time scalar is fp32, so the factor and the
    product are fp32 and ``.to(q.dtype)`` rounds once."""
    batch, heads, seq_q, dim = q.shape
    seq_k = k.shape[2]

    def arrange_q_or_o(shape):
        return View.of_shape(shape).tile((1, 1, bm, -1)).squeeze((0, 1), level=1)

    def arrange_k_or_v(shape, q_blocks):
        view = View.of_shape(shape).tile((1, 1, bn, -1)).tile((1, 1, -1, -1)).expand((-1, -1, q_blocks, -1))
        return view.squeeze((0, 1, 3), level=1).squeeze((0, 1), level=2)

    q_view = arrange_q_or_o(q.shape)
    o_view = arrange_q_or_o(q.shape)
    k_view = arrange_k_or_v(k.shape, q_view.table.shape[2])
    v_view = arrange_k_or_v(v.shape, q_view.table.shape[2])
    q_flat, k_flat, v_flat = q.reshape(-1), k.reshape(-1), v.reshape(-1)
    out = np.zeros(q.size, dtype=np.float32)
    if scale is None:
        factor = _round(np.float32(LOG2E), dtype).astype(np.float32)
    else:
        factor = np.float32(scale) * np.float32(LOG2E)

    for b in range(batch):
        for h in range(heads):
            for qb in range(q_view.table.shape[2]):
                q_tile = gather(q_flat, q_view.table[b, h, qb, 0], None)
                q_loaded = _round(q_tile.astype(np.float32) * factor, dtype).astype(np.float32)
                q_offsets = qb * bm + np.arange(bm)
                acc = np.zeros((bm, dim), dtype=np.float32)
                l_i = np.ones(bm, dtype=np.float32)
                m_i = np.full(bm, -np.inf, dtype=np.float32)
                for i in range(k_view.table.shape[4]):
                    k_tile = gather(k_flat, k_view.table[b, h, qb, 0, i], None).astype(np.float32)
                    v_tile = gather(v_flat, v_view.table[b, h, qb, 0, i], None).astype(np.float32)
                    k_offsets = i * bn + np.arange(bn)
                    qk = q_loaded @ k_tile.T
                    qk = np.where(k_offsets[None, :] < seq_k, qk, -np.inf)
                    if is_causal:
                        qk = np.where(q_offsets[:, None] >= k_offsets[None, :], qk, -np.inf)
                    m_ij = np.maximum(m_i, np.max(qk, axis=1))
                    with np.errstate(invalid="ignore"):
                        p = np.exp2(qk - m_ij[:, None]).astype(np.float32)
                        alpha = np.exp2(m_i - m_ij).astype(np.float32)
                    l_ij = np.sum(p, axis=1, dtype=np.float32)
                    acc = acc * alpha[:, None] + _round(p, dtype).astype(np.float32) @ v_tile
                    m_i = m_ij
                    l_i = l_i * alpha + l_ij
                acc = acc / l_i[:, None]
                scatter(out, o_view.table[b, h, qb, 0], _round(acc, dtype).astype(np.float32))
    return out.reshape(q.shape)


def conv2d(x, w, padding=(0, 0), bm=64, bn=64, bk=64, dtype="fp16", stride=(1, 1), dilation=(1, 1), floor_mode=True):
    """conv2d through the implicit-GEMM arrangement (reference tests/test_conv2d.py:13-48); `stride`, `dilation`
    and `floor_mode` go to the `tile` that cuts the padded input into windows (src/ninetoothed/tensor.py:199-286:
    without `floor_mode` the count of windows is rounded up, and what the last one reads beyond the padded input
    is masked, i.e. zero)."""
    n, c, h, width = x.shape
    k, _, r, s = w.shape
    pad_h, pad_w = padding

    def windows(size, pad, taps, spacing, step):
        span = size + 2 * pad - spacing * (taps - 1) - 1
        return max(span // step + 1 if floor_mode else -(-span // step) + 1, 0)

    p, q = windows(h, pad_h, r, dilation[0], stride[0]), windows(width, pad_w, s, dilation[1], stride[1])

    x_view = View.of_shape(x.shape).pad(((0, 0), (0, 0), (pad_h, pad_h), (pad_w, pad_w)))
    x_view = x_view.tile((1, c, r, s), strides=(-1, -1, *stride), dilation=(1, 1, *dilation), floor_mode=floor_mode).squeeze(1).squeeze(0, level=1)
    x_view = x_view.ravel().flatten(end_dim=3).flatten(start_dim=1)
    w_view = View.of_shape(w.shape).flatten(start_dim=1).permute((1, 0))
    y_view = View.of_shape((n, k, p, q)).permute((0, 2, 3, 1)).flatten(end_dim=3)

    lhs, rhs, out = arrange_matmul(x_view, w_view, y_view, bm, bn, bk)
    y = np.zeros(n * k * p * q, dtype=np.float32)

    def store(i, j, acc):
        scatter(y, out.table[i, j], _round(acc, dtype).astype(np.float32))

    _matmul_programs(x.reshape(-1), w.reshape(-1), lhs, rhs, out, store)
    return y.reshape(n, k, p, q)


# ---- tile maps: element-wise / reducing programs ----------------------------------------


def tile_map(application, inputs, out_flat, out_view):
    """Runs a program whose application maps tiles to a tile, the way the
    reference's generated kernel does (src/ninetoothed/generation.py:638-744):
    one program per position of the launch grid (the outermost level, equal for
    all operands); every program gathers its input tiles through the offset
    tables (masked positions read ``other``), calls ``application(*tiles)``
    and scatters the result through the output's table (masked positions are
    skipped).

    ``inputs`` is a list of ``(flat array, View, other)``; a view with a single
    level is a grid of single elements.  Programs of the reference this
    restates: tests/test_add.py:9-23, tests/test_clone.py:10-21,
    tests/test_pad.py:9-15, tests/test_pow.py:10-20, tests/test_dropout.py:12-18,
    tests/test_max_pool2d.py:13-40, tests/test_generation.py:139-151.
    """

    grid = out_view.level_shape(0)
    grid_rank = len(grid)
    for _, view, _ in inputs:
        assert tuple(view.level_shape(0)) == tuple(grid), "operands disagree on the launch grid"
    for program in np.ndindex(*grid):
        tiles = [gather(flat, view.table[program], other) for flat, view, other in inputs]
        result = application(*tiles)
        table = out_view.table[program]
        values = np.broadcast_to(np.asarray(result).astype(out_flat.dtype), table.shape)
        scatter(out_flat, np.asarray(table), values)
    assert grid_rank == len(grid)


def philox4x32(counter, key, rounds=10):
    """Philox-4x32 (Salmon et al., "Parallel random numbers: as easy as 1, 2, 3",
    SC'11): ``counter`` = four uint32 arrays, ``key`` = two.  Pinned by the known
    answers of the Random123 distribution (tests/test_oracle_programs.py)."""
    mask = np.uint64(0xFFFFFFFF)
    c = [np.asarray(word, dtype=np.uint64) & mask for word in counter]
    k0, k1 = (np.asarray(word, dtype=np.uint64) & mask for word in key)
    round_a, round_b = np.uint64(0xD2511F53), np.uint64(0xCD9E8D57)
    for _ in range(rounds):
        prev0, prev2 = c[0], c[2]
        c[0] = ((round_b * prev2) >> np.uint64(32)) ^ c[1] ^ k0
        c[2] = ((round_a * prev0) >> np.uint64(32)) ^ c[3] ^ k1
        c[1] = (round_b * prev2) & mask
        c[3] = (round_a * prev0) & mask
        k0 = (k0 + np.uint64(0x9E3779B9)) & mask
        k1 = (k1 + np.uint64(0xBB67AE85)) & mask
    return c


def triton_rand(seed, offsets):
    """``tl.rand(seed, offsets)``: Philox-4x32 with 10 rounds on the counter
    ``(offset_lo, offset_hi, 0, 0)`` keyed by the two halves of ``seed``; the
    first output word, read as int32 and mirrored when negative, times 2^-31
    (the published algorithm of Triton's ``language/random.py``, the package the
    reference's ``ntl.rand`` resolves to, src/ninetoothed/generation.py:849-855).
    Pinned bit for bit by outputs of the installed Triton's own ``tl.rand`` for 32- and
    64-bit offsets and seeds up to 2^62 (tests/golden/triton_rand_vectors.json)."""
    offsets = np.asarray(offsets, dtype=np.int64).astype(np.uint64)
    seed = np.uint64(seed)
    mask = np.uint64(0xFFFFFFFF)
    zeros = np.zeros_like(offsets)
    words = philox4x32((offsets & mask, offsets >> np.uint64(32), zeros, zeros), (seed & mask, seed >> np.uint64(32)))
    word = words[0].astype(np.uint32).view(np.int32).astype(np.int64)
    word = np.where(word < 0, -word - 1, word)
    return word.astype(np.float32) * np.float32(4.6566127342e-10)
