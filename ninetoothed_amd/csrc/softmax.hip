// Row softmax for gfx950.  Bandwidth-bound: every element is read once and
// written once; a row (or row segment) lives in registers between the two.
//
// A "segment" is what one program of the arrange-and-apply softmax handles:
// columns [s * block, min((s + 1) * block, N)) of one row.  With block >= N
// (the usual call) a segment is a whole row.
#include "nt_common.h"
#include "tune.h"
#include "workspace.h"

#include <algorithm>
#include <cstdlib>

namespace nt {
namespace {

struct SoftmaxParams {
    const void *in;
    void *out;
    int64_t rows, cols;
    int64_t in_row_stride, in_col_stride, out_row_stride, out_col_stride;
    int64_t block;      // segment length
    int64_t segments;   // per row
};

constexpr float kLog2e = 1.4426950408889634f;

// reductions over aligned groups of kLanes lanes of a wave
template <int kLanes = 64>
NT_DEVICE float wave_max(float v) {
#pragma unroll
    for (int off = kLanes / 2; off > 0; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}

template <int kLanes = 64>
NT_DEVICE float wave_sum(float v) {
#pragma unroll
    for (int off = kLanes / 2; off > 0; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

// Reduction over the kRowThreads threads that share a segment.  Up to 64 it is a
// pure wave reduction; for more, partial results cross waves through LDS.
template <int kRowThreads, bool kIsMax>
NT_DEVICE float group_reduce(float v, float *scratch) {
    constexpr int kLanes = kRowThreads < 64 ? kRowThreads : 64;
    v = kIsMax ? wave_max<kLanes>(v) : wave_sum<kLanes>(v);
    if constexpr (kRowThreads > 64) {
        constexpr int kWaves = kRowThreads / 64;
        const int wave = threadIdx.x >> 6;
        __syncthreads();  // scratch may still be read from a previous reduction
        if ((threadIdx.x & 63) == 0) scratch[wave] = v;
        __syncthreads();
        v = scratch[0];
#pragma unroll
        for (int w = 1; w < kWaves; ++w) v = kIsMax ? fmaxf(v, scratch[w]) : v + scratch[w];
    }
    return v;
}

template <typename T>
struct Vec16 {  // 16 bytes of T
    static constexpr int kWidth = 16 / sizeof(T);
    typedef T type __attribute__((ext_vector_type(16 / sizeof(T))));
};

// Vector path: unit column strides, 16-byte aligned segments whose length is a
// multiple of the vector width.  Thread t of a segment's group owns vectors
// t, t + kRowThreads, ...  (coalesced 16-byte accesses).
template <typename T, int kRowThreads, int kVecs>
__global__ __launch_bounds__(kRowThreads > 256 ? kRowThreads : 256) void softmax_vec_kernel(SoftmaxParams p) {
    typedef typename Vec16<T>::type vec_t;
    constexpr int W = Vec16<T>::kWidth;
    constexpr int kGroups = kRowThreads > 256 ? 1 : 256 / kRowThreads;  // segments per workgroup
    __shared__ float scratch[16];

    const int group = threadIdx.x / kRowThreads;
    const int t = threadIdx.x % kRowThreads;
    const int64_t seg = (int64_t)blockIdx.x * kGroups + group;
    const int64_t total = p.rows * p.segments;
    // whole groups leave together, so the barriers below stay uniform (kGroups == 1 when they exist)
    const bool active = seg < total;
    const int64_t row = active ? seg / p.segments : 0;
    const int64_t start = active ? (seg % p.segments) * p.block : 0;
    const int len = active ? (int)min(p.block, p.cols - start) : 0;
    const int nvec = len / W;

    const T *src = (const T *)p.in + row * p.in_row_stride + start;
    T *dst = (T *)p.out + row * p.out_row_stride + start;

    float x[kVecs][W];
    float m = -INFINITY;
#pragma unroll
    for (int j = 0; j < kVecs; ++j) {
        const int v = j * kRowThreads + t;
        if (v < nvec) {
            vec_t raw = *((const vec_t *)src + v);  // (a non-temporal load here costs 7-20 % of the rate; the non-temporal store below gains)
#pragma unroll
            for (int e = 0; e < W; ++e) {
                x[j][e] = (float)raw[e];
                m = fmaxf(m, x[j][e]);
            }
        } else {
#pragma unroll
            for (int e = 0; e < W; ++e) x[j][e] = -INFINITY;
        }
    }
    m = group_reduce<kRowThreads, true>(m, scratch);
    const float shift = m * kLog2e;
    float s = 0.0f;
#pragma unroll
    for (int j = 0; j < kVecs; ++j)
#pragma unroll
        for (int e = 0; e < W; ++e) {
            // exp(x - m) as exp2(x * log2e - m * log2e); padding (-inf) gives 0
            x[j][e] = __builtin_amdgcn_exp2f(fmaf(x[j][e], kLog2e, -shift));
            s += x[j][e];
        }
    s = group_reduce<kRowThreads, false>(s, scratch);
    const float inv = 1.0f / s;
#pragma unroll
    for (int j = 0; j < kVecs; ++j) {
        const int v = j * kRowThreads + t;
        if (v < nvec) {
            vec_t o;
#pragma unroll
            for (int e = 0; e < W; ++e) o[e] = (T)(x[j][e] * inv);
            __builtin_nontemporal_store(o, (vec_t *)dst + v);
        }
    }
}

// Rows of up to 64 bytes (a softmax over 4 or 8 classes, for millions of rows): one THREAD per row.  A group of
// 8 lanes per row, the smallest the vector path has, leaves most lanes without a vector on such rows.  A thread
// fetches its row in pieces of kBytes (the largest power of two that divides the row's bytes and its pitch),
// consecutive threads consecutive rows.
template <typename T, int kBytes>
__global__ __launch_bounds__(256) void softmax_thread_per_row_kernel(SoftmaxParams p, int pieces) {
    constexpr int kWidth = kBytes / (int)sizeof(T);  // elements per piece
    constexpr int kMaxPieces = 64 / kBytes;
    typedef T piece_t __attribute__((ext_vector_type(kWidth)));
    const int64_t row = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (row >= p.rows) return;
    const piece_t *src = (const piece_t *)((const T *)p.in + row * p.in_row_stride);
    piece_t *dst = (piece_t *)((T *)p.out + row * p.out_row_stride);
    float x[kMaxPieces][kWidth];
    float m = -INFINITY;
#pragma unroll
    for (int j = 0; j < kMaxPieces; ++j) {
        if (j < pieces) {
            const piece_t raw = src[j];
#pragma unroll
            for (int e = 0; e < kWidth; ++e) {
                x[j][e] = (float)raw[e];
                m = fmaxf(m, x[j][e]);
            }
        } else {
#pragma unroll
            for (int e = 0; e < kWidth; ++e) x[j][e] = -INFINITY;
        }
    }
    const float shift = m * kLog2e;
    float s = 0.0f;
#pragma unroll
    for (int j = 0; j < kMaxPieces; ++j)
#pragma unroll
        for (int e = 0; e < kWidth; ++e) {
            x[j][e] = __builtin_amdgcn_exp2f(fmaf(x[j][e], kLog2e, -shift));  // (as in softmax_vec_kernel)
            s += x[j][e];
        }
    const float inv = 1.0f / s;
#pragma unroll
    for (int j = 0; j < kMaxPieces; ++j) {
        if (j < pieces) {
            piece_t o;
#pragma unroll
            for (int e = 0; e < kWidth; ++e) o[e] = (T)(x[j][e] * inv);
            dst[j] = o;
        }
    }
}

template <typename T, int kBytes>
hipError_t launch_thread_per_row(const SoftmaxParams &p, hipStream_t stream) {
    note_launch(kLaunchSoftmax, 1, "softmax_thread_per_row_kernel, rows of up to 64 bytes");
    softmax_thread_per_row_kernel<T, kBytes><<<dim3((unsigned)((p.rows + 255) / 256)), dim3(256), 0, stream>>>(p, (int)(p.cols * (int64_t)sizeof(T) / kBytes));
    return hipGetLastError();
}

// Element path: any strides / alignment / length up to kRowThreads * kElems.
template <typename T, int kRowThreads, int kElems>
__global__ __launch_bounds__(kRowThreads > 256 ? kRowThreads : 256) void softmax_elem_kernel(SoftmaxParams p) {
    constexpr int kGroups = kRowThreads > 256 ? 1 : 256 / kRowThreads;
    __shared__ float scratch[16];

    const int group = threadIdx.x / kRowThreads;
    const int t = threadIdx.x % kRowThreads;
    const int64_t seg = (int64_t)blockIdx.x * kGroups + group;
    const int64_t total = p.rows * p.segments;
    const bool active = seg < total;
    const int64_t row = active ? seg / p.segments : 0;
    const int64_t start = active ? (seg % p.segments) * p.block : 0;
    const int len = active ? (int)min(p.block, p.cols - start) : 0;

    const T *src = (const T *)p.in + row * p.in_row_stride + start * p.in_col_stride;
    T *dst = (T *)p.out + row * p.out_row_stride + start * p.out_col_stride;

    float x[kElems];
    float m = -INFINITY;
#pragma unroll
    for (int j = 0; j < kElems; ++j) {
        const int c = j * kRowThreads + t;
        x[j] = c < len ? (float)src[(int64_t)c * p.in_col_stride] : -INFINITY;
        m = fmaxf(m, x[j]);
    }
    m = group_reduce<kRowThreads, true>(m, scratch);
    const float shift = m * kLog2e;
    float s = 0.0f;
#pragma unroll
    for (int j = 0; j < kElems; ++j) {
        x[j] = __builtin_amdgcn_exp2f(fmaf(x[j], kLog2e, -shift));
        s += x[j];
    }
    s = group_reduce<kRowThreads, false>(s, scratch);
    const float inv = 1.0f / s;
#pragma unroll
    for (int j = 0; j < kElems; ++j) {
        const int c = j * kRowThreads + t;
        if (c < len) dst[(int64_t)c * p.out_col_stride] = (T)(x[j] * inv);
    }
}

// One access of the kernels for long segments: 16 bytes of a segment whose columns are one element apart (global
// accesses need the element's alignment only), else one element.
template <typename T, bool kVec>
struct WideAccess {
    static constexpr int kWidth = kVec ? Vec16<T>::kWidth : 1;
    typedef typename Vec16<T>::type aligned_type;
    typedef aligned_type type __attribute__((aligned(sizeof(T))));
};

template <typename T, bool kVec>
NT_DEVICE void wide_load(const T *src, int64_t col_stride, int64_t index, int64_t count, float (&x)[WideAccess<T, kVec>::kWidth]) {
    constexpr int W = WideAccess<T, kVec>::kWidth;
    if constexpr (kVec) {
        if ((index + 1) * W <= count) {
            const typename WideAccess<T, kVec>::type v = *(const typename WideAccess<T, kVec>::type *)(src + index * W);
#pragma unroll
            for (int e = 0; e < W; ++e) x[e] = (float)v[e];
        } else {
#pragma unroll
            for (int e = 0; e < W; ++e) x[e] = index * W + e < count ? (float)src[index * W + e] : -INFINITY;
        }
    } else {
        x[0] = index < count ? (float)src[index * col_stride] : -INFINITY;
    }
}

// exp(x - maximum) / sum of one access, stored
template <typename T, bool kVec>
NT_DEVICE void wide_store(T *dst, int64_t col_stride, int64_t index, int64_t count, const float (&x)[WideAccess<T, kVec>::kWidth], float shift, float inv) {
    constexpr int W = WideAccess<T, kVec>::kWidth;
    if constexpr (kVec) {
        if ((index + 1) * W <= count) {
            typename WideAccess<T, kVec>::type v;
#pragma unroll
            for (int e = 0; e < W; ++e) v[e] = (T)(__builtin_amdgcn_exp2f(fmaf(x[e], kLog2e, -shift)) * inv);
            *(typename WideAccess<T, kVec>::type *)(dst + index * W) = v;
        } else {
#pragma unroll
            for (int e = 0; e < W; ++e)
                if (index * W + e < count) dst[index * W + e] = (T)(__builtin_amdgcn_exp2f(fmaf(x[e], kLog2e, -shift)) * inv);
        }
    } else {
        if (index < count) dst[index * col_stride] = (T)(__builtin_amdgcn_exp2f(fmaf(x[0], kLog2e, -shift)) * inv);
    }
}

// Long segments: one workgroup of 1024 threads per segment, two sweeps over memory: running
// maximum and sum together (a thread rescales its sum once per round of independent loads),
// then the write; the second sweep hits L2 for segments that fit there.
constexpr int kLoopThreads = 1024;

template <typename T, bool kVec>
__global__ __launch_bounds__(kLoopThreads) void softmax_loop_kernel(SoftmaxParams p) {
    constexpr int W = WideAccess<T, kVec>::kWidth;
    constexpr int kLoopUnroll = kVec ? 2 : 8;
    __shared__ float scratch[kLoopThreads / 64];
    const int64_t seg = blockIdx.x;
    const int64_t row = seg / p.segments;
    const int64_t start = (seg % p.segments) * p.block;
    const int64_t len = min(p.block, p.cols - start);
    const T *src = (const T *)p.in + row * p.in_row_stride + start * p.in_col_stride;
    T *dst = (T *)p.out + row * p.out_row_stride + start * p.out_col_stride;
    const int64_t pieces = (len + W - 1) / W;

    float m = -INFINITY, s = 0.0f;
    for (int64_t base = threadIdx.x; base < pieces; base += kLoopThreads * kLoopUnroll) {
        float x[kLoopUnroll][W];
        float round_max = -INFINITY;
#pragma unroll
        for (int u = 0; u < kLoopUnroll; ++u) {
            wide_load<T, kVec>(src, p.in_col_stride, base + u * kLoopThreads, len, x[u]);
#pragma unroll
            for (int e = 0; e < W; ++e) round_max = fmaxf(round_max, x[u][e]);
        }
        if (round_max > m) {  // (a first round of -inf only leaves m at -inf and s at 0)
            s *= __builtin_amdgcn_exp2f((m - round_max) * kLog2e);
            m = round_max;
        }
        if (m > -INFINITY) {
            const float shift = m * kLog2e;
#pragma unroll
            for (int u = 0; u < kLoopUnroll; ++u)
#pragma unroll
                for (int e = 0; e < W; ++e) s += __builtin_amdgcn_exp2f(fmaf(x[u][e], kLog2e, -shift));
        }
    }
    const float total_max = group_reduce<kLoopThreads, true>(m, scratch);
    // every thread's sum is relative to its own maximum
    s = m > -INFINITY ? s * __builtin_amdgcn_exp2f((m - total_max) * kLog2e) : 0.0f;
    s = group_reduce<kLoopThreads, false>(s, scratch);
    const float inv = 1.0f / s;
    const float shift = total_max * kLog2e;
    for (int64_t base = threadIdx.x; base < pieces; base += kLoopThreads * kLoopUnroll) {
        float x[kLoopUnroll][W];
#pragma unroll
        for (int u = 0; u < kLoopUnroll; ++u) wide_load<T, kVec>(src, p.in_col_stride, base + u * kLoopThreads, len, x[u]);
#pragma unroll
        for (int u = 0; u < kLoopUnroll; ++u) wide_store<T, kVec>(dst, p.out_col_stride, base + u * kLoopThreads, len, x[u], shift, inv);
    }
}

// Few long segments: each is cut into parts, a workgroup of 256 threads per part, two launches.  The first leaves
// every part's maximum and its sum of exponentials relative to that maximum in `partials`; the second combines
// the parts of its segment and writes its own part (its input is the first launch's and comes from the caches).
// kVec: unit column strides, 16 bytes per access (global accesses need the element's alignment only).
constexpr int kSplitThreads = 256;
constexpr int kSplitUnroll = 4;

struct SplitPartial {
    float max, sum;
};

template <typename T, bool kVec>
__global__ __launch_bounds__(kSplitThreads) void softmax_split_partial_kernel(SoftmaxParams p, int64_t part_len, SplitPartial *partials) {
    constexpr int W = WideAccess<T, kVec>::kWidth;
    __shared__ float scratch[kSplitThreads / 64];
    const int64_t seg = blockIdx.y;
    const int64_t row = seg / p.segments;
    const int64_t start = (seg % p.segments) * p.block + (int64_t)blockIdx.x * part_len;
    const int64_t seg_end = min((seg % p.segments + 1) * p.block, p.cols);
    const int64_t count = max((int64_t)0, min(part_len, seg_end - start));
    const T *src = (const T *)p.in + row * p.in_row_stride + start * p.in_col_stride;
    const int64_t pieces = (count + W - 1) / W;
    float m = -INFINITY, s = 0.0f;
    for (int64_t base = threadIdx.x; base < pieces; base += kSplitThreads * kSplitUnroll) {
        float x[kSplitUnroll][W];
        float round_max = -INFINITY;
#pragma unroll
        for (int u = 0; u < kSplitUnroll; ++u) {
            wide_load<T, kVec>(src, p.in_col_stride, base + u * kSplitThreads, count, x[u]);
#pragma unroll
            for (int e = 0; e < W; ++e) round_max = fmaxf(round_max, x[u][e]);
        }
        if (round_max > m) {
            s *= __builtin_amdgcn_exp2f((m - round_max) * kLog2e);
            m = round_max;
        }
        if (m > -INFINITY) {
            const float shift = m * kLog2e;
#pragma unroll
            for (int u = 0; u < kSplitUnroll; ++u)
#pragma unroll
                for (int e = 0; e < W; ++e) s += __builtin_amdgcn_exp2f(fmaf(x[u][e], kLog2e, -shift));
        }
    }
    const float part_max = group_reduce<kSplitThreads, true>(m, scratch);
    s = m > -INFINITY ? s * __builtin_amdgcn_exp2f((m - part_max) * kLog2e) : 0.0f;
    s = group_reduce<kSplitThreads, false>(s, scratch);
    if (threadIdx.x == 0) {
        SplitPartial r;
        r.max = part_max;
        r.sum = s;
        partials[seg * gridDim.x + blockIdx.x] = r;
    }
}

template <typename T, bool kVec>
__global__ __launch_bounds__(kSplitThreads) void softmax_split_finish_kernel(SoftmaxParams p, int64_t part_len, const SplitPartial *partials) {
    constexpr int W = WideAccess<T, kVec>::kWidth;
    __shared__ float scratch[kSplitThreads / 64];
    const int64_t seg = blockIdx.y;
    const int64_t row = seg / p.segments;
    const int64_t start = (seg % p.segments) * p.block + (int64_t)blockIdx.x * part_len;
    const int64_t seg_end = min((seg % p.segments + 1) * p.block, p.cols);
    const int64_t count = max((int64_t)0, min(part_len, seg_end - start));
    // the parts of this segment (at most one per thread)
    SplitPartial mine;
    mine.max = -INFINITY;
    mine.sum = 0.0f;
    if (threadIdx.x < gridDim.x) mine = partials[seg * gridDim.x + threadIdx.x];
    const float total_max = group_reduce<kSplitThreads, true>(mine.max, scratch);
    const float scaled = mine.max > -INFINITY ? mine.sum * __builtin_amdgcn_exp2f((mine.max - total_max) * kLog2e) : 0.0f;
    const float inv = 1.0f / group_reduce<kSplitThreads, false>(scaled, scratch);
    const float shift = total_max * kLog2e;
    const T *src = (const T *)p.in + row * p.in_row_stride + start * p.in_col_stride;
    T *dst = (T *)p.out + row * p.out_row_stride + start * p.out_col_stride;
    const int64_t pieces = (count + W - 1) / W;
    for (int64_t base = threadIdx.x; base < pieces; base += kSplitThreads * kSplitUnroll) {
        float x[kSplitUnroll][W];
#pragma unroll
        for (int u = 0; u < kSplitUnroll; ++u) wide_load<T, kVec>(src, p.in_col_stride, base + u * kSplitThreads, count, x[u]);
#pragma unroll
        for (int u = 0; u < kSplitUnroll; ++u) wide_store<T, kVec>(dst, p.out_col_stride, base + u * kSplitThreads, count, x[u], shift, inv);
    }
}

// true when the segments were served by the two launches over parts.  `in_registers`: the segments are short
// enough for the kernels that read them once (those win unless too few workgroups are left to fetch: measured
// fp32 [128, 65536] 13 us against 18 us in parts, [16, 65536] 9.1 against 8.1, [16, 262144] fp16 77 against 12).
template <typename T>
bool run_split(const SoftmaxParams &p, int64_t len, bool in_registers, hipStream_t stream, hipError_t *status) {
    const int64_t total = p.rows * p.segments;
    const int64_t bytes = len * (int64_t)sizeof(T);
    if (total > 128) return false;
    if (in_registers ? (bytes < (1 << 18) || total > 16) : bytes < (1 << 16)) return false;
    const int64_t wanted = std::min<int64_t>(kSplitThreads, std::max<int64_t>(2, 1024 / total));  // (the finishing launch reads one part per thread)
    int64_t part_len = std::max<int64_t>(4096, (((len + wanted - 1) / wanted + 2047) / 2048) * 2048);
    const int64_t parts = (len + part_len - 1) / part_len;
    if (parts < 2 || parts > kSplitThreads) return false;
    WorkspaceLease lease(stream);
    SplitPartial *partials = (SplitPartial *)lease.get(kWorkspaceSoftmaxParts, (size_t)(total * parts) * sizeof(SplitPartial));
    if (partials == nullptr) return false;  // no scratch: one workgroup per segment
    const dim3 grid((unsigned)parts, (unsigned)total), block(kSplitThreads);
    note_launch(kLaunchSoftmax, kSplitThreads, "softmax_split_partial_kernel + softmax_split_finish_kernel, long segments cut into parts");
    if (p.in_col_stride == 1 && p.out_col_stride == 1) {
        softmax_split_partial_kernel<T, true><<<grid, block, 0, stream>>>(p, part_len, partials);
        softmax_split_finish_kernel<T, true><<<grid, block, 0, stream>>>(p, part_len, partials);
    } else {
        softmax_split_partial_kernel<T, false><<<grid, block, 0, stream>>>(p, part_len, partials);
        softmax_split_finish_kernel<T, false><<<grid, block, 0, stream>>>(p, part_len, partials);
    }
    *status = hipGetLastError();
    return true;
}

template <typename T, int kRowThreads>
hipError_t launch_vec(const SoftmaxParams &p, int vecs_needed, hipStream_t stream) {
    const int64_t total = p.rows * p.segments;
    constexpr int kGroups = kRowThreads > 256 ? 1 : 256 / kRowThreads;
    const dim3 grid((unsigned)((total + kGroups - 1) / kGroups)), block(kRowThreads > 256 ? kRowThreads : 256);
    note_launch(kLaunchSoftmax, kRowThreads, "softmax_vec_kernel, 16-byte vectors, this many threads per row segment");
    if (vecs_needed <= 1)
        softmax_vec_kernel<T, kRowThreads, 1><<<grid, block, 0, stream>>>(p);
    else if (vecs_needed <= 2)
        softmax_vec_kernel<T, kRowThreads, 2><<<grid, block, 0, stream>>>(p);
    else if (vecs_needed <= 4)
        softmax_vec_kernel<T, kRowThreads, 4><<<grid, block, 0, stream>>>(p);
    else if (vecs_needed <= 8)
        softmax_vec_kernel<T, kRowThreads, 8><<<grid, block, 0, stream>>>(p);
    else
        softmax_vec_kernel<T, kRowThreads, 16><<<grid, block, 0, stream>>>(p);
    return hipGetLastError();
}

template <typename T, int kRowThreads, int kElems>
hipError_t launch_elem(const SoftmaxParams &p, hipStream_t stream) {
    const int64_t total = p.rows * p.segments;
    constexpr int kGroups = kRowThreads > 256 ? 1 : 256 / kRowThreads;
    const dim3 grid((unsigned)((total + kGroups - 1) / kGroups)), block(kRowThreads > 256 ? kRowThreads : 256);
    note_launch(kLaunchSoftmax, kRowThreads, "softmax_elem_kernel, element by element, this many threads per row segment");
    softmax_elem_kernel<T, kRowThreads, kElems><<<grid, block, 0, stream>>>(p);
    return hipGetLastError();
}

// `variant`: 0 = library's choice, 1 = one wave per segment, 2 = one workgroup per segment
template <typename T>
int run_softmax(const SoftmaxParams &p, int variant, hipStream_t stream) {
    constexpr int W = Vec16<T>::kWidth;
    const int64_t total = p.rows * p.segments;
    if (total == 0 || p.cols == 0) return 0;
    if (total > 0x7fffffffll) return NINETOOTHED_NO_KERNEL;
    const int64_t len = p.block < p.cols ? p.block : p.cols;
    const bool vector_ok = p.in_col_stride == 1 && p.out_col_stride == 1 && p.cols % W == 0 &&
                           (p.segments == 1 || p.block % W == 0) && p.in_row_stride % W == 0 &&
                           p.out_row_stride % W == 0 && ((uintptr_t)p.in & 15) == 0 && ((uintptr_t)p.out & 15) == 0;
    // rows of up to 64 bytes, many of them: a thread per row
    if (variant == 0 && p.segments == 1 && p.in_col_stride == 1 && p.out_col_stride == 1 && p.cols * (int64_t)sizeof(T) <= 64 && p.rows >= 4096 &&
        (p.rows + 255) / 256 <= 0x7fffffffll) {
        const uint64_t bits = (uint64_t)(p.cols * sizeof(T)) | (uint64_t)(p.in_row_stride * (int64_t)sizeof(T)) | (uint64_t)(p.out_row_stride * (int64_t)sizeof(T)) |
                              (uint64_t)(uintptr_t)p.in | (uint64_t)(uintptr_t)p.out;  // what every piece's address and size is a multiple of
        if (bits % 16 == 0) return (int)launch_thread_per_row<T, 16>(p, stream);
        if (bits % 8 == 0) return (int)launch_thread_per_row<T, 8>(p, stream);
        if (bits % 4 == 0) return (int)launch_thread_per_row<T, 4>(p, stream);
        if constexpr (sizeof(T) == 2) {
            if (p.cols <= 8) return (int)launch_thread_per_row<T, 2>(p, stream);  // (up to 32 pieces of one element would not stay in registers)
        }
    }
    // (a row of 16 vectors of 2-byte elements per thread -- 128 floats -- does not stay in the registers of 1024 threads)
    const bool in_registers = vector_ok && len <= (int64_t)1024 * 64;
    if (variant == 0) {
        hipError_t status = hipSuccess;
        if (run_split<T>(p, len, in_registers, stream, &status)) return (int)status;
    }
    if (in_registers || (vector_ok && variant != 0 && len <= (int64_t)1024 * 16 * W)) {
        const bool wave_fits = len <= (int64_t)64 * 16 * W;
        bool use_wave = wave_fits && len <= (int64_t)64 * 8 * W;  // default: keep <= 8 vectors per lane
        // few segments: a workgroup each, so that more of the chip has something to fetch
        if (use_wave && len > (int64_t)64 * W && total < 4096) use_wave = false;
        if (variant == 1 && wave_fits) use_wave = true;
        if (variant == 2) use_wave = false;
        const int64_t nvec = len / W;
        if (variant == 0 && p.segments == 1) {  // short rows: 8, 16 or 32 lanes each, one vector per lane
            if (nvec <= 8) return (int)launch_vec<T, 8>(p, 1, stream);
            if (nvec <= 16) return (int)launch_vec<T, 16>(p, 1, stream);
            if (nvec <= 32) return (int)launch_vec<T, 32>(p, 1, stream);
        }
        if (use_wave) return (int)launch_vec<T, 64>(p, (int)((nvec + 63) / 64), stream);
        // more than 8 vectors per thread of a 256-thread workgroup: 1024 threads (registers per thread, not LDS, hold the row)
        if (nvec > 256 * 8 && variant != 2) return (int)launch_vec<T, 1024>(p, (int)((nvec + 1023) / 1024), stream);
        if (nvec > 256 * 16) return (int)launch_vec<T, 1024>(p, (int)((nvec + 1023) / 1024), stream);
        return (int)launch_vec<T, 256>(p, (int)((nvec + 255) / 256), stream);
    }
    // element by element (any strides / alignment): as many threads per segment as keep every thread at
    // 4 .. 16 elements, from 8 lanes of a wave to a workgroup of 1024
    if (len <= 8 * 4) return (int)launch_elem<T, 8, 4>(p, stream);
    if (len <= 16 * 4) return (int)launch_elem<T, 16, 4>(p, stream);
    if (len <= 32 * 4) return (int)launch_elem<T, 32, 4>(p, stream);
    if (len <= 64 * 4) return (int)launch_elem<T, 64, 4>(p, stream);
    if (len <= 64 * 16) return (int)launch_elem<T, 64, 16>(p, stream);
    if (len <= 256 * 16) return (int)launch_elem<T, 256, 16>(p, stream);
    // (measured: 8192 x 4099 fp32 3.0 TB/s with 256 threads, 2.5 with 1024; 4096 x 12289 fp16 1.3 against 1.9;
    // 2048 x 30001 fp32 2.1 in registers of 1024 threads, 3.9 with the loop kernel)
    if (len <= 256 * 32) return (int)launch_elem<T, 256, 64>(p, stream);
    if (len <= 1024 * 16) return (int)launch_elem<T, 1024, 16>(p, stream);
    note_launch(kLaunchSoftmax, kLoopThreads, "softmax_loop_kernel, two sweeps over a long row segment");
    if (p.in_col_stride == 1 && p.out_col_stride == 1)
        softmax_loop_kernel<T, true><<<dim3((unsigned)total), dim3(kLoopThreads), 0, stream>>>(p);
    else
        softmax_loop_kernel<T, false><<<dim3((unsigned)total), dim3(kLoopThreads), 0, stream>>>(p);
    return (int)hipGetLastError();
}

int softmax_entry(NineToothedStream stream, const NineToothedTensor &input, const NineToothedTensor &output, int dtype,
                  int block_size, int variant) {
    if (!input.shape || !output.shape || !input.strides || !output.strides) return hipErrorInvalidValue;
    if (input.shape[0] != output.shape[0] || input.shape[1] != output.shape[1]) return hipErrorInvalidValue;
    SoftmaxParams p;
    p.in = input.data;
    p.out = output.data;
    p.rows = (int64_t)input.shape[0];
    p.cols = (int64_t)input.shape[1];
    p.in_row_stride = input.strides[0];
    p.in_col_stride = input.strides[1];
    p.out_row_stride = output.strides[0];
    p.out_col_stride = output.strides[1];
    p.block = block_size > 0 ? block_size : (p.cols > 0 ? p.cols : 1);
    p.segments = p.cols > 0 ? (p.cols + p.block - 1) / p.block : 0;
    switch (dtype) {
        case NINETOOTHED_FLOAT32:
            return run_softmax<float>(p, variant, (hipStream_t)stream);
        case NINETOOTHED_FLOAT16:
            return run_softmax<half_t>(p, variant, (hipStream_t)stream);
        case NINETOOTHED_BFLOAT16:
            return run_softmax<bf16_t>(p, variant, (hipStream_t)stream);
        default:
            return NINETOOTHED_NO_KERNEL;
    }
}

}  // namespace
}  // namespace nt

extern "C" {

NineToothedResult launch_nt_softmax(NineToothedStream stream, NineToothedTensor input, NineToothedTensor output,
                                    int dtype, int block_size) {
    return nt::softmax_entry(stream, input, output, dtype, block_size, 0);
}

NineToothedResult launch_nt_softmax_config(NineToothedStream stream, int config, NineToothedTensor input,
                                           NineToothedTensor output, int dtype, int block_size) {
    if (config < 0 || config > 2) return NINETOOTHED_NO_KERNEL;
    return nt::softmax_entry(stream, input, output, dtype, block_size, config);
}

}  // extern "C"
