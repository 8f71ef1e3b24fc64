// Shape- and stride-agnostic tiled GEMM main loop for gfx950.  The problem
// description (how A, B elements are fetched and how C elements are stored) is
// a policy type, so the same MFMA loop serves arbitrarily strided matmul /
// addmm operands and the implicit-GEMM view of conv2d.
//
// 128x128x32 tile, 4 waves in a 2x2 grid, each wave 64x64 of C as 2x2 MFMA
// 32x32x16 tiles.  Operands pass through registers on their way to LDS (the
// policy may gather them), rows of 32 k-values are padded to 40 elements so
// the 16-byte fragment reads are bank-conflict free.
#pragma once

#include "nt_common.h"

namespace nt {

constexpr int kGenBM = 128;
constexpr int kGenBN = 128;
constexpr int kGenBK = 32;
constexpr int kGenPitch = 40;  // elements per LDS row
constexpr int kGenThreads = 256;

// Policy concept:
//   typedef ... elem;                       // half_t, bf16_t or float
//   int m, n, k;                            // GEMM extents
//   void load_a16(int row, int k0, elem out[16]) const;  // A[row][k0..k0+15], zero outside
//   void load_b16(int col, int k0, elem out[16]) const;  // B[k0..k0+15][col], zero outside
//   void store_c(int row, int col, float v) const;        // row < m, col < n guaranteed
//   void select_batch(int index);                         // the grid's y coordinate: which of several independent products
template <typename Problem>
__global__ __launch_bounds__(kGenThreads) void gemm_generic_kernel(Problem prob) {
    typedef typename Problem::elem T;
    typedef Elem<T> E;
    typedef typename E::vec8 vec8;

    __shared__ __attribute__((aligned(32))) T lds_a[kGenBM * kGenPitch];
    __shared__ __attribute__((aligned(32))) T lds_b[kGenBN * kGenPitch];

    prob.select_batch((int)blockIdx.y);  // independent products of one launch: the operands move by the batch strides
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = tid >> 6;
    const int wave_m = wave >> 1;
    const int wave_n = wave & 1;
    const int g = lane >> 5;
    const int l32 = lane & 31;

    const int tiles_n = ceil_div(prob.n, kGenBN);
    const int tile_m = blockIdx.x / tiles_n;
    const int tile_n = blockIdx.x % tiles_n;
    const int m0 = tile_m * kGenBM;
    const int n0 = tile_n * kGenBN;

    // staging assignment: thread -> one tile row (of A and of B^T), one k half
    const int stage_row = tid & 127;
    const int stage_k = (tid >> 7) * 16;

    float16_t acc[2][2];
#pragma unroll
    for (int ti = 0; ti < 2; ++ti)
#pragma unroll
        for (int tj = 0; tj < 2; ++tj)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[ti][tj][r] = 0.0f;

    T ra[16], rb[16];
    const int num_k = ceil_div(prob.k, kGenBK);
    if (num_k > 0) {
        prob.load_a16(m0 + stage_row, stage_k, ra);
        prob.load_b16(n0 + stage_row, stage_k, rb);
    }

    for (int kt = 0; kt < num_k; ++kt) {
        __syncthreads();  // previous tile fully consumed
        {
            vec8 *da = (vec8 *)&lds_a[stage_row * kGenPitch + stage_k];
            vec8 *db = (vec8 *)&lds_b[stage_row * kGenPitch + stage_k];
            vec8 v0, v1, w0, w1;
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                v0[i] = ra[i];
                v1[i] = ra[8 + i];
                w0[i] = rb[i];
                w1[i] = rb[8 + i];
            }
            da[0] = v0;
            da[1] = v1;
            db[0] = w0;
            db[1] = w1;
        }
        __syncthreads();
        if (kt + 1 < num_k) {  // prefetch the next tile while this one is multiplied
            prob.load_a16(m0 + stage_row, (kt + 1) * kGenBK + stage_k, ra);
            prob.load_b16(n0 + stage_row, (kt + 1) * kGenBK + stage_k, rb);
        }
#pragma unroll
        for (int ks = 0; ks < kGenBK / 16; ++ks) {
            vec8 af[2], bf[2];
#pragma unroll
            for (int ti = 0; ti < 2; ++ti)
                af[ti] = *(const vec8 *)&lds_a[(wave_m * 64 + ti * 32 + l32) * kGenPitch + ks * 16 + 8 * g];
#pragma unroll
            for (int tj = 0; tj < 2; ++tj)
                bf[tj] = *(const vec8 *)&lds_b[(wave_n * 64 + tj * 32 + l32) * kGenPitch + ks * 16 + 8 * g];
#pragma unroll
            for (int ti = 0; ti < 2; ++ti)
#pragma unroll
                for (int tj = 0; tj < 2; ++tj) acc[ti][tj] = E::mfma32(af[ti], bf[tj], acc[ti][tj]);
        }
    }

#pragma unroll
    for (int ti = 0; ti < 2; ++ti) {
#pragma unroll
        for (int tj = 0; tj < 2; ++tj) {
            const int col = n0 + wave_n * 64 + tj * 32 + l32;
#pragma unroll
            for (int r = 0; r < 16; ++r) {
                const int row = m0 + wave_m * 64 + ti * 32 + 8 * (r >> 2) + 4 * g + (r & 3);
                if (row < prob.m && col < prob.n) prob.store_c(row, col, acc[ti][tj][r]);
            }
        }
    }
}

// ---- policy: plain strided matrices (matmul / addmm with any strides) ----
template <typename T, typename TOut>
struct StridedProblem {
    typedef T elem;
    int m, n, k;
    const T *a;
    const T *b;
    TOut *c;
    const T *bias;
    int64_t sam, sak, sbk, sbn, scm, scn, sbm_, sbn_;  // sbm_/sbn_: bias strides
    float alpha, beta;
    int64_t a_batch, b_batch, c_batch, bias_batch;  // element strides between the products of a batched launch
    int k_chunk;  // > 0: the grid's y coordinate is a part of the k range of one product, this many positions long

    NT_DEVICE void select_batch(int index) {
        if (k_chunk > 0) {
            a += (int64_t)index * k_chunk * sak;
            b += (int64_t)index * k_chunk * sbk;
            c += index * c_batch;
            k = min(k_chunk, k - index * k_chunk);
            return;
        }
        a += index * a_batch;
        b += index * b_batch;
        c += index * c_batch;
        if (bias != nullptr) bias += index * bias_batch;
    }

    NT_DEVICE void load_a16(int row, int k0, T out[16]) const {
        const T *src = a + (int64_t)row * sam + (int64_t)k0 * sak;
        if (row < m && k0 + 16 <= k && sak == 1 && (((uintptr_t)src) & 15) == 0) {
            typedef typename Elem<T>::vec8 vec8;
            vec8 v0 = ((const vec8 *)src)[0];
            vec8 v1 = ((const vec8 *)src)[1];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                out[i] = v0[i];
                out[8 + i] = v1[i];
            }
            return;
        }
#pragma unroll
        for (int i = 0; i < 16; ++i) out[i] = (row < m && k0 + i < k) ? src[(int64_t)i * sak] : (T)0.0f;
    }

    NT_DEVICE void load_b16(int col, int k0, T out[16]) const {
        const T *src = b + (int64_t)k0 * sbk + (int64_t)col * sbn;
        if (col < n && k0 + 16 <= k && sbk == 1 && (((uintptr_t)src) & 15) == 0) {
            typedef typename Elem<T>::vec8 vec8;
            vec8 v0 = ((const vec8 *)src)[0];
            vec8 v1 = ((const vec8 *)src)[1];
#pragma unroll
            for (int i = 0; i < 8; ++i) {
                out[i] = v0[i];
                out[8 + i] = v1[i];
            }
            return;
        }
#pragma unroll
        for (int i = 0; i < 16; ++i) out[i] = (col < n && k0 + i < k) ? src[(int64_t)i * sbk] : (T)0.0f;
    }

    NT_DEVICE void store_c(int row, int col, float v) const {
        if (bias != nullptr) {
            const float mm = Elem<T>::to_float(Elem<T>::from_float(v));
            const float in = Elem<T>::to_float(bias[(int64_t)row * sbm_ + (int64_t)col * sbn_]);
            v = beta * in + alpha * mm;
        }
        c[(int64_t)row * scm + (int64_t)col * scn] = from_float<TOut>(v);
    }
};

// ---- policy: fp8 (e5m2) operands, any strides ----
// An e5m2 value is the upper byte of the fp16 value with the same sign and
// exponent, so widening is a shift and the fp16 MFMA multiplies exactly.
template <typename TOut>
struct Fp8E5m2Problem {
    typedef half_t elem;
    int m, n, k;
    const uint8_t *a;
    const uint8_t *b;
    TOut *c;
    const uint8_t *bias;  // addmm input (fp8 as well), or null
    int64_t sam, sak, sbk, sbn, scm, scn, sbm_, sbn_;
    float alpha, beta;

    NT_DEVICE void select_batch(int) {}

    static NT_DEVICE half_t widen(uint8_t byte) {
        const unsigned short bits = (unsigned short)((unsigned short)byte << 8);
        return __builtin_bit_cast(half_t, bits);
    }

    NT_DEVICE void load_a16(int row, int k0, half_t out[16]) const {
        const uint8_t *src = a + (int64_t)row * sam + (int64_t)k0 * sak;
#pragma unroll
        for (int i = 0; i < 16; ++i) out[i] = (row < m && k0 + i < k) ? widen(src[(int64_t)i * sak]) : (half_t)0.0f;
    }

    NT_DEVICE void load_b16(int col, int k0, half_t out[16]) const {
        const uint8_t *src = b + (int64_t)k0 * sbk + (int64_t)col * sbn;
#pragma unroll
        for (int i = 0; i < 16; ++i) out[i] = (col < n && k0 + i < k) ? widen(src[(int64_t)i * sbk]) : (half_t)0.0f;
    }

    NT_DEVICE void store_c(int row, int col, float v) const {
        if (bias != nullptr) {  // the product is rounded to fp16 first, the combination happens in fp32
            const float mm = (float)(half_t)v;
            const float in = (float)widen(bias[(int64_t)row * sbm_ + (int64_t)col * sbn_]);
            v = beta * in + alpha * mm;
        }
        c[(int64_t)row * scm + (int64_t)col * scn] = from_float<TOut>(v);
    }
};

// ---- policy: conv2d as implicit GEMM (any window stride and dilation, zero padding) ----
// GEMM row  = (image, out_y, out_x), GEMM k = (channel, filter_y, filter_x),
// GEMM col  = output channel.
template <typename T>
struct Conv2dProblem {
    typedef T elem;
    int m, n, k;  // m = N*P*Q, n = K, k = C*R*S
    const T *x;
    const T *w;
    T *y;
    int C, H, W, R, S, P, Q, pad_h, pad_w;
    int stride_h, stride_w, dil_h, dil_w;  // steps of the window over the input and between its taps
    int64_t xs[4], ws[4], ys[4];

    NT_DEVICE void select_batch(int) {}

    NT_DEVICE void load_a16(int row, int k0, T out[16]) const {
        if (row >= m) {
#pragma unroll
            for (int i = 0; i < 16; ++i) out[i] = (T)0.0f;
            return;
        }
        const int img = row / (P * Q);
        const int pq = row - img * (P * Q);
        const int oy = pq / Q;
        const int ox = pq - oy * Q;
        const T *base = x + (int64_t)img * xs[0];
        int c = k0 / (R * S);
        int rs = k0 - c * (R * S);
        int fy = rs / S;
        int fx = rs - fy * S;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            const int iy = oy * stride_h + fy * dil_h - pad_h;
            const int ix = ox * stride_w + fx * dil_w - pad_w;
            const bool ok = (k0 + i < k) && iy >= 0 && iy < H && ix >= 0 && ix < W;
            out[i] = ok ? base[(int64_t)c * xs[1] + (int64_t)iy * xs[2] + (int64_t)ix * xs[3]] : (T)0.0f;
            if (++fx == S) {
                fx = 0;
                if (++fy == R) {
                    fy = 0;
                    ++c;
                }
            }
        }
    }

    NT_DEVICE void load_b16(int col, int k0, T out[16]) const {
        if (col >= n) {
#pragma unroll
            for (int i = 0; i < 16; ++i) out[i] = (T)0.0f;
            return;
        }
        const T *base = w + (int64_t)col * ws[0];
        int c = k0 / (R * S);
        int rs = k0 - c * (R * S);
        int fy = rs / S;
        int fx = rs - fy * S;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            out[i] = (k0 + i < k) ? base[(int64_t)c * ws[1] + (int64_t)fy * ws[2] + (int64_t)fx * ws[3]] : (T)0.0f;
            if (++fx == S) {
                fx = 0;
                if (++fy == R) {
                    fy = 0;
                    ++c;
                }
            }
        }
    }

    NT_DEVICE void store_c(int row, int col, float v) const {
        const int img = row / (P * Q);
        const int pq = row - img * (P * Q);
        const int oy = pq / Q;
        const int ox = pq - oy * Q;
        y[(int64_t)img * ys[0] + (int64_t)col * ys[1] + (int64_t)oy * ys[2] + (int64_t)ox * ys[3]] = Elem<T>::from_float(v);
    }
};

}  // namespace nt
