"""The arrange-and-apply programs this build executes with hand-written kernels.

Each program is written with the public API exactly as a user would write it
(the matmul is the README program of the reference, README.md:30-68; addmm,
softmax, attention and conv2d follow the programs of the reference's tests,
tests/test_addmm.py:13-38, tests/test_softmax.py:10-27,
tests/test_attention.py:14-70, tests/test_conv2d.py:13-48).  They have two
jobs: users can call them directly (``programs.matmul.kernel()``), and their
traced applications are the dictionary against which
:mod:`ninetoothed_amd.recognition` matches user applications.
"""

import functools

import ninetoothed_amd.language as ntl
from ninetoothed_amd.symbol import Symbol, block_size
from ninetoothed_amd.tensor import Tensor

BLOCK_SIZE_M = block_size()
BLOCK_SIZE_N = block_size()
BLOCK_SIZE_K = block_size()


class matmul:
    @staticmethod
    def arrangement(lhs, rhs, output, BLOCK_SIZE_M=BLOCK_SIZE_M, BLOCK_SIZE_N=BLOCK_SIZE_N, BLOCK_SIZE_K=BLOCK_SIZE_K):
        output_arranged = output.tile((BLOCK_SIZE_M, BLOCK_SIZE_N))

        lhs_arranged = lhs.tile((BLOCK_SIZE_M, BLOCK_SIZE_K)).tile((1, -1)).expand((-1, output_arranged.shape[1]))
        lhs_arranged.dtype = lhs_arranged.dtype.squeeze(0)

        rhs_arranged = rhs.tile((BLOCK_SIZE_K, BLOCK_SIZE_N)).tile((-1, 1)).expand((output_arranged.shape[0], -1))
        rhs_arranged.dtype = rhs_arranged.dtype.squeeze(1)

        return lhs_arranged, rhs_arranged, output_arranged

    @staticmethod
    def application(lhs, rhs, output):
        accumulator = ntl.zeros(output.shape, dtype=ntl.float32)
        for k in range(lhs.shape[0]):
            accumulator += ntl.dot(lhs[k], rhs[k])
        output = accumulator  # noqa: F841

    @staticmethod
    def application_with_cast(lhs, rhs, output):
        accumulator = ntl.zeros(output.shape, dtype=ntl.float32)
        for k in range(lhs.shape[0]):
            accumulator += ntl.dot(lhs[k], rhs[k])
        output = accumulator.to(ntl.float16)  # noqa: F841

    @staticmethod
    def application_with_bfloat16_cast(lhs, rhs, output):
        accumulator = ntl.zeros(output.shape, dtype=ntl.float32)
        for k in range(lhs.shape[0]):
            accumulator += ntl.dot(lhs[k], rhs[k])
        output = accumulator.to(ntl.bfloat16)  # noqa: F841

    tensors = staticmethod(lambda: (Tensor(2), Tensor(2), Tensor(2)))

    # The same application over a batch of products: tensors [B, M, K], [B, K, N], [B, M, N], the batch
    # dimension tiled by 1 and squeezed out of the tiles, so that `lhs[k]` / `rhs[k]` / `output` are the
    # matrices' blocks as before and the grid is (batch, blocks of M, blocks of N).
    @staticmethod
    def batched_arrangement(lhs, rhs, output, BLOCK_SIZE_M=BLOCK_SIZE_M, BLOCK_SIZE_N=BLOCK_SIZE_N, BLOCK_SIZE_K=BLOCK_SIZE_K):
        output_arranged = output.tile((1, BLOCK_SIZE_M, BLOCK_SIZE_N))
        output_arranged.dtype = output_arranged.dtype.squeeze(0)

        lhs_arranged = lhs.tile((1, BLOCK_SIZE_M, BLOCK_SIZE_K)).tile((1, 1, -1)).expand((-1, -1, output_arranged.shape[2]))
        lhs_arranged.dtype = lhs_arranged.dtype.squeeze((0, 1))
        lhs_arranged.dtype.dtype = lhs_arranged.dtype.dtype.squeeze(0)

        rhs_arranged = rhs.tile((1, BLOCK_SIZE_K, BLOCK_SIZE_N)).tile((1, -1, 1)).expand((-1, output_arranged.shape[1], -1))
        rhs_arranged.dtype = rhs_arranged.dtype.squeeze((0, 2))
        rhs_arranged.dtype.dtype = rhs_arranged.dtype.dtype.squeeze(0)

        return lhs_arranged, rhs_arranged, output_arranged

    batched_tensors = staticmethod(lambda: (Tensor(3), Tensor(3), Tensor(3)))


class addmm:
    @staticmethod
    def arrangement(input, mat1, mat2, beta, alpha, output, BLOCK_SIZE_M=BLOCK_SIZE_M, BLOCK_SIZE_N=BLOCK_SIZE_N, BLOCK_SIZE_K=BLOCK_SIZE_K):
        _, _, input_arranged = matmul.arrangement(mat1, mat2, input, BLOCK_SIZE_M, BLOCK_SIZE_N, BLOCK_SIZE_K)
        mat1_arranged, mat2_arranged, output_arranged = matmul.arrangement(mat1, mat2, output, BLOCK_SIZE_M, BLOCK_SIZE_N, BLOCK_SIZE_K)
        return input_arranged, mat1_arranged, mat2_arranged, beta, alpha, output_arranged

    @staticmethod
    def application(input, mat1, mat2, beta, alpha, output):
        matmul_output = ntl.zeros(output.shape, dtype=ntl.float32)
        matmul.application_with_cast(mat1, mat2, matmul_output)
        output = beta * input + alpha * matmul_output  # noqa: F841

    @staticmethod
    def application_bfloat16(input, mat1, mat2, beta, alpha, output):
        matmul_output = ntl.zeros(output.shape, dtype=ntl.float32)
        matmul.application_with_bfloat16_cast(mat1, mat2, matmul_output)
        output = beta * input + alpha * matmul_output  # noqa: F841

    tensors = staticmethod(lambda: (Tensor(2), Tensor(2), Tensor(2), Tensor(0), Tensor(0), Tensor(2)))


class softmax:
    BLOCK_SIZE = Symbol("BLOCK_SIZE", constexpr=True)

    @staticmethod
    def arrangement(input, output, BLOCK_SIZE=BLOCK_SIZE):
        return input.tile((1, BLOCK_SIZE)), output.tile((1, BLOCK_SIZE))

    @staticmethod
    def application(input_row, output_row):
        row_minus_max = input_row - ntl.max(input_row)
        numerator = ntl.exp(row_minus_max)
        denominator = ntl.sum(numerator)
        output_row = numerator / denominator  # noqa: F841

    tensors = staticmethod(lambda: (Tensor(2, other=float("-inf")), Tensor(2)))


class attention:
    BLOCK_SIZE_M = block_size(lower_bound=64, upper_bound=128)
    BLOCK_SIZE_N = block_size(lower_bound=32, upper_bound=64)

    @staticmethod
    def _arrange(q, k, v, o, BLOCK_SIZE_M, BLOCK_SIZE_N):
        def arrange_q_or_o(input):
            arranged = input.tile((1, 1, BLOCK_SIZE_M, -1))
            arranged.dtype = arranged.dtype.squeeze((0, 1))
            return arranged

        def arrange_k_or_v(input):
            arranged = input.tile((1, 1, BLOCK_SIZE_N, -1)).tile((1, 1, -1, -1)).expand((-1, -1, q_arranged.shape[-2], -1))
            arranged.dtype = arranged.dtype.squeeze((0, 1, 3))
            arranged.dtype.dtype = arranged.dtype.dtype.squeeze((0, 1))
            return arranged

        q_arranged = arrange_q_or_o(q)
        return q_arranged, arrange_k_or_v(k), arrange_k_or_v(v), arrange_q_or_o(o)

    @staticmethod
    def arrangement(q, k, v, is_causal, o, BLOCK_SIZE_M=BLOCK_SIZE_M, BLOCK_SIZE_N=BLOCK_SIZE_N):
        q_arranged, k_arranged, v_arranged, o_arranged = attention._arrange(q, k, v, o, BLOCK_SIZE_M, BLOCK_SIZE_N)
        return q_arranged, k_arranged, v_arranged, is_causal, o_arranged

    @staticmethod
    def arrangement_with_scale(q, k, v, is_causal, scale, o, BLOCK_SIZE_M=BLOCK_SIZE_M, BLOCK_SIZE_N=BLOCK_SIZE_N):
        q_arranged, k_arranged, v_arranged, o_arranged = attention._arrange(q, k, v, o, BLOCK_SIZE_M, BLOCK_SIZE_N)
        return q_arranged, k_arranged, v_arranged, is_causal, scale, o_arranged

    @staticmethod
    def application(q, k, v, is_causal, o):
        q_loaded = (q * 1.44269504089).to(q.dtype)

        acc = ntl.zeros((q.shape[-2], q.shape[-1]), dtype=ntl.float32)
        l_i = ntl.full((q.shape[-2],), 1, dtype=ntl.float32)
        m_i = ntl.full((q.shape[-2],), float("-inf"), dtype=ntl.float32)

        for i in range(k.shape[0]):
            qk = ntl.dot(q_loaded, ntl.trans(k[i]))
            qk = ntl.where(k[i].offsets(-2) < k.source.shape[-2], qk, float("-inf"))

            if is_causal:
                mask = q.offsets(-2)[:, None] >= k[i].offsets(-2)[None, :]
                qk = ntl.where(mask, qk, float("-inf"))

            m_ij = ntl.maximum(m_i, ntl.max(qk, 1))
            p = ntl.exp2(qk - m_ij[:, None])
            l_ij = ntl.sum(p, 1)

            alpha = ntl.exp2(m_i - m_ij)
            acc = acc * alpha[:, None] + ntl.dot(p.to(v[i].dtype), v[i])
            m_i = m_ij
            l_i = l_i * alpha + l_ij

        acc /= l_i[:, None]
        o = acc  # noqa: F841

    @staticmethod
    def application_with_scale(q, k, v, is_causal, scale, o):
        q_loaded = (q * (scale * 1.44269504089)).to(q.dtype)

        acc = ntl.zeros((q.shape[-2], q.shape[-1]), dtype=ntl.float32)
        l_i = ntl.full((q.shape[-2],), 1, dtype=ntl.float32)
        m_i = ntl.full((q.shape[-2],), float("-inf"), dtype=ntl.float32)

        for i in range(k.shape[0]):
            qk = ntl.dot(q_loaded, ntl.trans(k[i]))
            qk = ntl.where(k[i].offsets(-2) < k.source.shape[-2], qk, float("-inf"))

            if is_causal:
                mask = q.offsets(-2)[:, None] >= k[i].offsets(-2)[None, :]
                qk = ntl.where(mask, qk, float("-inf"))

            m_ij = ntl.maximum(m_i, ntl.max(qk, 1))
            p = ntl.exp2(qk - m_ij[:, None])
            l_ij = ntl.sum(p, 1)

            alpha = ntl.exp2(m_i - m_ij)
            acc = acc * alpha[:, None] + ntl.dot(p.to(v[i].dtype), v[i])
            m_i = m_ij
            l_i = l_i * alpha + l_ij

        acc /= l_i[:, None]
        o = acc  # noqa: F841

    @staticmethod
    def tensors(with_scale=False):
        options = (None, None, {"constexpr": True}, {"constexpr": True, "upper_bound": 128})
        q, k, v, o = (Tensor(4, shape_options=options) for _ in range(4))
        is_causal = Tensor(0, constexpr=True)
        if with_scale:
            return q, k, v, is_causal, Tensor(0), o
        return q, k, v, is_causal, o


class conv2d:
    @staticmethod
    def arrangement(input, filter, output, enable_padding=True, BLOCK_SIZE_M=BLOCK_SIZE_M, BLOCK_SIZE_N=BLOCK_SIZE_N, BLOCK_SIZE_K=BLOCK_SIZE_K,
                    stride=(1, 1), dilation=(1, 1), floor_mode=False):
        """`stride`, `dilation`: steps of the window over the (padded) input and between its taps -- one more
        argument to `tile` (src/ninetoothed/tensor.py:199-286).  With a stride, `floor_mode=True` gives the output
        size of the usual convolution; `tile` otherwise adds a window that hangs over the edge."""
        if enable_padding:
            padding_h = Symbol("padding_h", constexpr=True)
            padding_w = Symbol("padding_w", constexpr=True)
            input = input.pad(((0, 0), (0, 0), (padding_h, padding_h), (padding_w, padding_w)))

        input_tiled = input.tile((1, *filter.shape[1:]), strides=(-1, -1, *stride), dilation=(1, 1, *dilation), floor_mode=floor_mode)
        input_squeezed = input_tiled.squeeze(1)
        input_squeezed.dtype = input_squeezed.dtype.squeeze(0)
        input_flattened = input_squeezed.ravel().flatten(end_dim=3).flatten(start_dim=1)

        filter_permuted = filter.flatten(start_dim=1).permute((1, 0))

        output_flattened = output.permute((0, 2, 3, 1)).flatten(end_dim=3)

        return functools.partial(matmul.arrangement, BLOCK_SIZE_M=BLOCK_SIZE_M, BLOCK_SIZE_N=BLOCK_SIZE_N, BLOCK_SIZE_K=BLOCK_SIZE_K)(
            input_flattened, filter_permuted, output_flattened
        )

    application = matmul.application_with_cast

    tensors = staticmethod(lambda: (Tensor(4), Tensor(4, shape_options={"constexpr": True}), Tensor(4)))

    @staticmethod
    def premake(n=None, c=None, h=None, w=None, k=None, r=None, s=None, dtype=None, block_size_m=64, block_size_n=64, block_size_k=64):
        """The unpadded convolution with sizes fixed or left open, for ``build`` (after the
        reference's tests/test_conv2d.py:51-87)."""
        arrangement = functools.partial(
            conv2d.arrangement, enable_padding=False, BLOCK_SIZE_M=block_size_m, BLOCK_SIZE_N=block_size_n, BLOCK_SIZE_K=block_size_k
        )
        p = h - r + 1 if h is not None and r is not None else None
        q = w - s + 1 if w is not None and s is not None else None
        tensors = (Tensor(shape=(n, c, h, w), dtype=dtype), Tensor(shape=(k, c, r, s), dtype=dtype), Tensor(shape=(n, k, p, q), dtype=dtype))
        return arrangement, matmul.application, tensors
