// C ABI for the GEMM family: launch_nt_matmul, launch_nt_addmm,
// launch_nt_conv2d and the tile-selection entry points.
#include <algorithm>
#include <memory>
#include <mutex>
#include <type_traits>
#include <shared_mutex>
#include <unordered_map>
#include <vector>
#include <cstdio>
#include <cstdlib>
#include <cstring>

#include "conv2d.h"
#include "gemm_fast.h"
#include "gemm_generic.h"
#include "tune.h"
#include "workspace.h"

namespace nt {
namespace {

struct GemmProblem {
    int dtype, out_dtype;
    int m, n, k;
    const void *a, *b, *bias;
    void *c;
    int64_t sam, sak, sbk, sbn, scm, scn, sim, sin;
    float alpha, beta;
    int batch = 1;  // independent products that share the shapes; operands move by these element strides
    int64_t a_batch = 0, b_batch = 0, c_batch = 0, bias_batch = 0;
    // set by the entry point that allocates nothing: split-K parts go here instead of the stream's workspace
    float *fixed_scratch = nullptr;
    size_t fixed_scratch_bytes = 0;
    bool hinted = false;  // the caller gave block sizes: the call stays on kernels without scratch memory
    bool addmm() const { return bias != nullptr; }
};

int g_tile_order = 0;  // see GemmParams::order; changed only by measurement builds

typedef hipError_t (*LaunchFn)(const GemmProblem &, hipStream_t);
typedef bool (*AcceptFn)(const GemmProblem &);

struct GemmInstance {
    const char *name;
    int bm, bn, bk;
    AcceptFn accepts;
    LaunchFn launch;
};

// the fast instances take B row-major ([K, N], unit column stride) or transposed ([N, K] storage, unit k stride)
bool b_is_transposed(const GemmProblem &q) { return q.sbn != 1 && q.sbk == 1; }

template <int BM, int BN, int BK, int kStages, bool kTail = false>
bool fast_accepts(const GemmProblem &q) {
    if (q.dtype != NINETOOTHED_FLOAT16 && q.dtype != NINETOOTHED_BFLOAT16) return false;
    // the element type, or fp32 for a plain product (the accumulators as they are)
    if (q.out_dtype != q.dtype && !(q.out_dtype == NINETOOTHED_FLOAT32 && !q.addmm())) return false;
    if (q.m <= 0 || q.n <= 0 || q.k <= 0) return false;
    // any number of rows: rows past M read as zeros and are not stored; N and K must fit the tile,
    // or, for the instances with tails, be multiples of 8 (whole 16-byte chunks)
    // (K: whole 16-byte chunks of the k-contiguous rows; N: only where rows of B run along it.  With a
    // transposed B any N goes: C is then stored element by element when its rows are not 16-byte aligned)
    if (kTail ? (q.k % 8 || (q.n % 8 && !b_is_transposed(q))) : (q.n % BN || q.k % BK)) return false;
    if (q.sak != 1 || q.scn != 1) return false;
    if (q.sam % 8 || q.sam < q.k || q.scm < q.n) return false;
    if (((uintptr_t)q.a & 15) || ((uintptr_t)q.b & 15)) return false;
    if (!kTail && (((uintptr_t)q.c & 15) || q.scm % 8)) return false;
    // (a batch: the operands of every product on 16-byte boundaries; the outputs too, unless the instance stores element by element)
    if (q.batch > 1 && ((q.a_batch | q.b_batch) % 8 || (!kTail && q.c_batch % 8) || (int64_t)((q.m + BM - 1) / BM) * ((q.n + BN - 1) / BN) * q.batch > 0x7fffffffll)) return false;
    // per-lane 32-bit byte offsets inside one tile panel
    if ((int64_t)BM * q.sam * 2 >= (int64_t(1) << 31)) return false;
    if (b_is_transposed(q)) {  // B as [N, K] with K contiguous (`x @ w.T`)
        if (q.sbn % 8 || q.sbn < q.k) return false;
        if ((int64_t)BN * q.sbn * 2 >= (int64_t(1) << 31)) return false;
    } else {
        if (q.sbn != 1 || q.sbk % 8 || q.sbk < q.n) return false;
        if ((int64_t)q.k * q.sbk * 2 >= (int64_t(1) << 31)) return false;
    }
    return true;
}

void fill_params(GemmParams &p, const GemmProblem &q, int bm, int bn) {
    p.a = q.a;
    p.b = q.b;
    p.c = q.c;
    p.bias = q.bias;
    p.m = q.m;
    p.n = q.n;
    p.k = q.k;
    p.lda = q.sam;
    p.ldb = b_is_transposed(q) ? q.sbn : q.sbk;
    p.ldc = q.scm;
    p.bias_stride_m = q.sim;
    p.bias_stride_n = q.sin;
    p.alpha = q.alpha;
    p.beta = q.beta;
    p.tiles_m = (q.m + bm - 1) / bm;
    p.tiles_n = (q.n + bn - 1) / bn;
    p.order = g_tile_order;
    p.bias_vector = q.bias != nullptr && q.sin == 1 && q.sim % 8 == 0 && ((uintptr_t)q.bias & 15) == 0 && q.n % 8 == 0 && (q.batch == 1 || q.bias_batch % 8 == 0);
    p.c_vector = ((uintptr_t)q.c & 15) == 0 && q.scm % 8 == 0 && q.n % 8 == 0 && (q.batch == 1 || q.c_batch % 8 == 0);
    p.kt_per_split = 0;
    p.batch = q.batch;
    p.a_batch = q.a_batch;
    p.b_batch = q.b_batch;
    p.c_batch = q.c_batch;
    p.bias_batch = q.bias_batch;
}

template <typename T, int BM, int BN, int BK, int WM, int WN, int kStages, int kOcc, int kAblate, int kLoad, int kAux, bool kTail>
hipError_t fast_launch_typed(const GemmProblem &q, hipStream_t stream) {
    GemmParams p;
    fill_params(p, q, BM, BN);
    const dim3 grid(p.tiles_m * p.tiles_n * q.batch), block(WM * WN * 64);
    const bool f32 = q.out_dtype == NINETOOTHED_FLOAT32, addmm = q.addmm();
    if (b_is_transposed(q)) {
        if (f32) gemm_nn_fast_kernel<T, BM, BN, BK, WM, WN, kStages, kOcc, false, kAblate, kLoad, kAux, true, true, kTail><<<grid, block, 0, stream>>>(p);
        else if (addmm) gemm_nn_fast_kernel<T, BM, BN, BK, WM, WN, kStages, kOcc, true, kAblate, kLoad, kAux, false, true, kTail><<<grid, block, 0, stream>>>(p);
        else gemm_nn_fast_kernel<T, BM, BN, BK, WM, WN, kStages, kOcc, false, kAblate, kLoad, kAux, false, true, kTail><<<grid, block, 0, stream>>>(p);
    } else {
        if (f32) gemm_nn_fast_kernel<T, BM, BN, BK, WM, WN, kStages, kOcc, false, kAblate, kLoad, kAux, true, false, kTail><<<grid, block, 0, stream>>>(p);
        else if (addmm) gemm_nn_fast_kernel<T, BM, BN, BK, WM, WN, kStages, kOcc, true, kAblate, kLoad, kAux, false, false, kTail><<<grid, block, 0, stream>>>(p);
        else gemm_nn_fast_kernel<T, BM, BN, BK, WM, WN, kStages, kOcc, false, kAblate, kLoad, kAux, false, false, kTail><<<grid, block, 0, stream>>>(p);
    }
    return hipGetLastError();
}

template <int BM, int BN, int BK, int WM, int WN, int kStages, int kOcc, int kAblate = 0, int kLoad = 1, int kAux = 0, bool kTail = false>
hipError_t fast_launch(const GemmProblem &q, hipStream_t stream) {
    if (q.dtype == NINETOOTHED_FLOAT16) return fast_launch_typed<half_t, BM, BN, BK, WM, WN, kStages, kOcc, kAblate, kLoad, kAux, kTail>(q, stream);
    return fast_launch_typed<bf16_t, BM, BN, BK, WM, WN, kStages, kOcc, kAblate, kLoad, kAux, kTail>(q, stream);
}

// ---- split-K: problems with too few output tiles for 256 CUs (a few rows, or small M x N with a long K) ----
// The k range is cut into parts, each (tile, part) is a workgroup that writes an fp32 tile to scratch
// memory of the stream, and a second kernel sums the parts and applies the epilogue.

// number of parts for tiles of bm x bn x bk, 1 = do not split
// (`scratch_limit`: bytes the partial products may take)
int split_parts(const GemmProblem &q, int bm, int bn, int bk, int *kt_per_part, int64_t scratch_limit = int64_t(64) << 20) {
    const int64_t tiles = (int64_t)((q.m + bm - 1) / bm) * ((q.n + bn - 1) / bn);
    const int num_kt = (q.k + bk - 1) / bk;
    if (tiles >= 320) return 1;  // (the untuned choice only splits below 192 tiles; between, the tuner decides)
    // about two workgroups per CU; of 256 x 256 tiles a CU holds one, so there all of them should run at once
    int64_t parts = bm * bn >= 256 * 256 ? 256 / tiles : (512 + tiles - 1) / tiles;
    parts = std::min<int64_t>(parts, num_kt / 2);                  // at least two k tiles each
    parts = std::min<int64_t>(parts, 256);
    while (parts >= 2 && parts * q.m * ((q.n + 7) / 8 * 8) * 4 > scratch_limit) --parts;  // scratch of at most 64 MiB, or what the caller's fixed array holds
    if (parts < 2) return 1;
    const int per_part = (int)((num_kt + parts - 1) / parts);
    if (kt_per_part) *kt_per_part = per_part;
    return (num_kt + per_part - 1) / per_part;                      // every part has at least one k tile
}

template <int BM, int BN, int BK, int kStages>
bool split_accepts(const GemmProblem &q) {
    // the operands, outputs and epilogues of the one-pass instances with tails (the second kernel writes four
    // consecutive elements of C at a time where N, the row pitch and the address of C allow it, else one)
    if (q.batch != 1) return false;
    return fast_accepts<BM, BN, BK, kStages, true>(q) && split_parts(q, BM, BN, BK, nullptr) >= 2;
}

// out[m][n] = epilogue(sum over parts): four consecutive columns per thread.  The parts are [m][pitch] tiles, pitch = N
// rounded up to 8; kVector: N is a multiple of 4 and the rows of C start on 16-byte (fp32) / 8-byte boundaries -- else
// the four values are stored one by one, those inside N
template <typename T, typename TOut, bool kAddmm, bool kVector = true>
__global__ __launch_bounds__(256) void gemm_split_reduce_kernel(const float *parts, int num_parts, int m, int n, TOut *c, int64_t ldc, const T *bias,
                                                               int64_t bias_stride_m, int64_t bias_stride_n, float alpha, float beta) {
    typedef float float4_t __attribute__((ext_vector_type(4)));
    typedef TOut out4_t __attribute__((ext_vector_type(4)));
    const int pitch = (n + 7) / 8 * 8;
    const int groups = pitch / 4;
    const int64_t total = (int64_t)m * groups;
    for (int64_t index = (int64_t)blockIdx.x * 256 + threadIdx.x; index < total; index += (int64_t)gridDim.x * 256) {
        const int row = (int)(index / groups);
        const int col = (int)(index - (int64_t)row * groups) * 4;
        if (col >= n) continue;
        const float *src = parts + (int64_t)row * pitch + col;
        float4_t sum = *(const float4_t *)src;
        for (int part = 1; part < num_parts; ++part) sum += *(const float4_t *)(src + (int64_t)part * m * pitch);
        out4_t out;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            if constexpr (kAddmm) {
                // as in the one-pass kernels: the product is rounded to the element type, then combined in fp32
                const float product = Elem<T>::to_float(Elem<T>::from_float(sum[e]));
                const float input = kVector || col + e < n ? Elem<T>::to_float(bias[(int64_t)row * bias_stride_m + (int64_t)(col + e) * bias_stride_n]) : 0.0f;
                out[e] = Elem<T>::from_float(beta * input + alpha * product);
            } else if constexpr (std::is_same<TOut, float>::value) {
                out[e] = sum[e];
            } else {
                out[e] = Elem<T>::from_float(sum[e]);
            }
        }
        if constexpr (kVector) {
            __builtin_nontemporal_store(out, (out4_t *)(c + (int64_t)row * ldc + col));
        } else {
#pragma unroll
            for (int e = 0; e < 4; ++e)
                if (col + e < n) c[(int64_t)row * ldc + col + e] = out[e];
        }
    }
}

template <typename T, int BM, int BN, int BK, int WM, int WN, int kStages, int kOcc>
hipError_t split_launch_typed(const GemmProblem &q, hipStream_t stream) {
    int kt_per_part = 0;
    // with a fixed array the part count shrinks until the partial products fit; the call is refused when not even two parts do
    const int parts = q.fixed_scratch != nullptr ? split_parts(q, BM, BN, BK, &kt_per_part, (int64_t)q.fixed_scratch_bytes) : split_parts(q, BM, BN, BK, &kt_per_part);
    if (parts < 2) return (hipError_t)(q.fixed_scratch != nullptr && split_parts(q, BM, BN, BK, nullptr) >= 2 ? NINETOOTHED_SCRATCH_LIMIT : NINETOOTHED_NO_KERNEL);
    const int pitch = (q.n + 7) / 8 * 8;  // of the partial tiles: whole 16-byte chunks, whatever N is
    const size_t scratch_bytes = (size_t)parts * q.m * pitch * sizeof(float);
    // the lock of the workspace registry also serialises host threads that enqueue onto the fixed array
    WorkspaceLease lease(stream);
    float *scratch;
    if (q.fixed_scratch != nullptr) {
        if (scratch_bytes > q.fixed_scratch_bytes) return (hipError_t)NINETOOTHED_SCRATCH_LIMIT;
        scratch = q.fixed_scratch;
    } else {
        scratch = (float *)lease.get(kWorkspaceGemmParts, scratch_bytes);
        if (scratch == nullptr) return (hipError_t)NINETOOTHED_NO_KERNEL;  // no scratch (graph capture, out of memory): the caller takes a one-pass instance
    }
    GemmParams p;
    fill_params(p, q, BM, BN);
    p.c = scratch;
    p.ldc = pitch;
    p.c_vector = 1;  // (the scratch tensor is aligned and its rows hold whole chunks: a chunk that begins inside N is stored whole)
    p.bias = nullptr;
    p.kt_per_split = kt_per_part;
    const dim3 grid(p.tiles_m * p.tiles_n * parts), block(WM * WN * 64);
    if (b_is_transposed(q)) gemm_nn_fast_kernel<T, BM, BN, BK, WM, WN, kStages, kOcc, false, 0, 1, 0, true, true, true, true><<<grid, block, 0, stream>>>(p);
    else gemm_nn_fast_kernel<T, BM, BN, BK, WM, WN, kStages, kOcc, false, 0, 1, 0, true, false, true, true><<<grid, block, 0, stream>>>(p);
    hipError_t err = hipGetLastError();
    if (err != hipSuccess) return err;
    const int64_t groups = (int64_t)q.m * (pitch / 4);
    const dim3 reduce_grid((unsigned)std::min<int64_t>((groups + 255) / 256, 256 * 8));
    const int64_t out_size = q.out_dtype == NINETOOTHED_FLOAT32 ? 4 : 2;
    const bool vector = q.n % 4 == 0 && (q.scm * out_size) % (4 * out_size) == 0 && ((uintptr_t)q.c & (4 * out_size - 1)) == 0;
    const auto reduce = [&](auto vector_tag) {
        constexpr bool kVector = decltype(vector_tag)::value;
        if (q.addmm())
            gemm_split_reduce_kernel<T, T, true, kVector><<<reduce_grid, dim3(256), 0, stream>>>(scratch, parts, q.m, q.n, (T *)q.c, q.scm, (const T *)q.bias, q.sim, q.sin, q.alpha, q.beta);
        else if (q.out_dtype == NINETOOTHED_FLOAT32)
            gemm_split_reduce_kernel<T, float, false, kVector><<<reduce_grid, dim3(256), 0, stream>>>(scratch, parts, q.m, q.n, (float *)q.c, q.scm, nullptr, 0, 0, 1.0f, 0.0f);
        else
            gemm_split_reduce_kernel<T, T, false, kVector><<<reduce_grid, dim3(256), 0, stream>>>(scratch, parts, q.m, q.n, (T *)q.c, q.scm, nullptr, 0, 0, 1.0f, 0.0f);
    };
    if (vector) reduce(std::true_type());
    else reduce(std::false_type());
    return hipGetLastError();
}

template <int BM, int BN, int BK, int WM, int WN, int kStages, int kOcc>
hipError_t split_launch(const GemmProblem &q, hipStream_t stream) {
    if (q.dtype == NINETOOTHED_FLOAT16) return split_launch_typed<half_t, BM, BN, BK, WM, WN, kStages, kOcc>(q, stream);
    return split_launch_typed<bf16_t, BM, BN, BK, WM, WN, kStages, kOcc>(q, stream);
}

bool generic_accepts(const GemmProblem &q) {
    if (q.batch < 1 || q.batch > 65535) return false;  // (the batch is the grid's y extent)
    if (q.dtype == NINETOOTHED_FLOAT8_E5M2 && q.batch != 1) return false;
    if (q.dtype == NINETOOTHED_FLOAT8_E5M2)  // widened to fp16; addmm rounds its product to fp16, so it writes fp16
        return (q.out_dtype == NINETOOTHED_FLOAT16 || (q.out_dtype == NINETOOTHED_FLOAT32 && !q.addmm())) && q.m >= 0 && q.n >= 0 && q.k >= 0;
    if (q.dtype != NINETOOTHED_FLOAT16 && q.dtype != NINETOOTHED_BFLOAT16 && q.dtype != NINETOOTHED_FLOAT32) return false;
    if (q.out_dtype != q.dtype && q.out_dtype != NINETOOTHED_FLOAT32) return false;
    return q.m >= 0 && q.n >= 0 && q.k >= 0;
}

// out = epilogue(sum over the parts of the k range), any output strides; fp32 throughout (an fp32 addmm does not round its product)
__global__ __launch_bounds__(256) void gemm_generic_reduce_kernel(const float *parts, int num_parts, int m, int n, float *c, int64_t scm, int64_t scn, const float *bias,
                                                                 int64_t bias_stride_m, int64_t bias_stride_n, float alpha, float beta) {
    const int64_t total = (int64_t)m * n;
    for (int64_t index = (int64_t)blockIdx.x * 256 + threadIdx.x; index < total; index += (int64_t)gridDim.x * 256) {
        float sum = parts[index];
        for (int part = 1; part < num_parts; ++part) sum += parts[index + (int64_t)part * total];
        const int row = (int)(index / n), col = (int)(index - (int64_t)row * n);
        if (bias != nullptr) sum = beta * bias[(int64_t)row * bias_stride_m + (int64_t)col * bias_stride_n] + alpha * sum;
        c[(int64_t)row * scm + (int64_t)col * scn] = sum;
    }
}

// fp32 products with too few 128 x 128 tiles for the chip: parts of the k range as the grid's y extent, each writing an
// fp32 tile to scratch memory of the stream, then the sum (512^3 50 -> 23 us, 1024^3 96 -> 41, [128, 4096] x [4096, 128]
// 347 -> 28, [64, 8192] x [8192, 64] 776 -> 38).  NINETOOTHED_NO_KERNEL: not worth it, or no scratch -- the caller runs the product in one pass.
hipError_t generic_launch_in_parts(const GemmProblem &q, hipStream_t stream) {
    const int64_t tiles = (int64_t)ceil_div(q.m, kGenBM) * ceil_div(q.n, kGenBN);
    const int num_kt = ceil_div(q.k, kGenBK);
    if (q.batch != 1 || q.hinted || q.fixed_scratch != nullptr || tiles == 0 || tiles >= 192) return (hipError_t)NINETOOTHED_NO_KERNEL;
    int64_t parts = std::min<int64_t>({(512 + tiles - 1) / tiles, num_kt / 4, 256});
    while (parts >= 2 && parts * q.m * q.n * 4 > (int64_t(64) << 20)) --parts;
    if (parts < 2) return (hipError_t)NINETOOTHED_NO_KERNEL;
    const int kt_per_part = (int)((num_kt + parts - 1) / parts);
    parts = (num_kt + kt_per_part - 1) / kt_per_part;  // every part has at least one k tile
    WorkspaceLease lease(stream);
    float *scratch = (float *)lease.get(kWorkspaceGemmParts, (size_t)parts * q.m * q.n * sizeof(float));
    if (scratch == nullptr) return (hipError_t)NINETOOTHED_NO_KERNEL;
    StridedProblem<float, float> prob;
    prob.m = q.m;
    prob.n = q.n;
    prob.k = q.k;
    prob.a = (const float *)q.a;
    prob.b = (const float *)q.b;
    prob.c = scratch;
    prob.bias = nullptr;
    prob.sam = q.sam;
    prob.sak = q.sak;
    prob.sbk = q.sbk;
    prob.sbn = q.sbn;
    prob.scm = q.n;
    prob.scn = 1;
    prob.sbm_ = prob.sbn_ = 0;
    prob.alpha = 1.0f;
    prob.beta = 0.0f;
    prob.a_batch = prob.b_batch = prob.bias_batch = 0;
    prob.c_batch = (int64_t)q.m * q.n;
    prob.k_chunk = kt_per_part * kGenBK;
    note_launch(kLaunchGemm, 0, "128x128x32 waves 2x2 any-stride, k range in parts, then gemm_generic_reduce_kernel");
    gemm_generic_kernel<StridedProblem<float, float>><<<dim3((unsigned)tiles, (unsigned)parts), dim3(kGenThreads), 0, stream>>>(prob);
    hipError_t err = hipGetLastError();
    if (err != hipSuccess) return err;
    const int64_t total = (int64_t)q.m * q.n;
    gemm_generic_reduce_kernel<<<dim3((unsigned)std::min<int64_t>((total + 255) / 256, 256 * 8)), dim3(256), 0, stream>>>(
        scratch, (int)parts, q.m, q.n, (float *)q.c, q.scm, q.scn, (const float *)q.bias, q.sim, q.sin, q.alpha, q.beta);
    return hipGetLastError();
}

template <typename T, typename TOut>
hipError_t generic_launch_typed(const GemmProblem &q, hipStream_t stream) {
    if constexpr (std::is_same<T, float>::value) {
        const hipError_t in_parts = generic_launch_in_parts(q, stream);
        if ((int)in_parts != NINETOOTHED_NO_KERNEL) return in_parts;
    }
    StridedProblem<T, TOut> prob;
    prob.k_chunk = 0;
    prob.m = q.m;
    prob.n = q.n;
    prob.k = q.k;
    prob.a = (const T *)q.a;
    prob.b = (const T *)q.b;
    prob.c = (TOut *)q.c;
    prob.bias = (const T *)q.bias;
    prob.sam = q.sam;
    prob.sak = q.sak;
    prob.sbk = q.sbk;
    prob.sbn = q.sbn;
    prob.scm = q.scm;
    prob.scn = q.scn;
    prob.sbm_ = q.sim;
    prob.sbn_ = q.sin;
    prob.alpha = q.alpha;
    prob.beta = q.beta;
    prob.a_batch = q.a_batch;
    prob.b_batch = q.b_batch;
    prob.c_batch = q.c_batch;
    prob.bias_batch = q.bias_batch;
    const int64_t tiles = (int64_t)ceil_div(q.m, kGenBM) * ceil_div(q.n, kGenBN);
    if (tiles == 0) return hipSuccess;  // empty launch is legal
    gemm_generic_kernel<StridedProblem<T, TOut>><<<dim3((unsigned)tiles, (unsigned)q.batch), dim3(kGenThreads), 0, stream>>>(prob);
    return hipGetLastError();
}

template <typename TOut>
hipError_t fp8_launch_typed(const GemmProblem &q, hipStream_t stream) {
    Fp8E5m2Problem<TOut> prob;
    prob.m = q.m;
    prob.n = q.n;
    prob.k = q.k;
    prob.a = (const uint8_t *)q.a;
    prob.b = (const uint8_t *)q.b;
    prob.c = (TOut *)q.c;
    prob.sam = q.sam;
    prob.sak = q.sak;
    prob.sbk = q.sbk;
    prob.sbn = q.sbn;
    prob.scm = q.scm;
    prob.scn = q.scn;
    prob.bias = (const uint8_t *)q.bias;
    prob.sbm_ = q.sim;
    prob.sbn_ = q.sin;
    prob.alpha = q.alpha;
    prob.beta = q.beta;
    const int64_t tiles = (int64_t)ceil_div(q.m, kGenBM) * ceil_div(q.n, kGenBN);
    if (tiles == 0) return hipSuccess;
    gemm_generic_kernel<Fp8E5m2Problem<TOut>><<<dim3((unsigned)tiles), dim3(kGenThreads), 0, stream>>>(prob);
    return hipGetLastError();
}

hipError_t generic_launch(const GemmProblem &q, hipStream_t stream) {
    const bool f32out = q.out_dtype == NINETOOTHED_FLOAT32;
    if (q.dtype == NINETOOTHED_FLOAT8_E5M2) return f32out ? fp8_launch_typed<float>(q, stream) : fp8_launch_typed<half_t>(q, stream);
    if (q.dtype == NINETOOTHED_FLOAT32) return generic_launch_typed<float, float>(q, stream);
    if (q.dtype == NINETOOTHED_FLOAT16)
        return f32out ? generic_launch_typed<half_t, float>(q, stream) : generic_launch_typed<half_t, half_t>(q, stream);
    return f32out ? generic_launch_typed<bf16_t, float>(q, stream) : generic_launch_typed<bf16_t, bf16_t>(q, stream);
}

// BM, BN, BK, wave grid WM x WN, LDS stages, waves per SIMD the register budget allows
#define NT_FAST_INSTANCE(BM, BN, BK, WM, WN, ST, OCC) \
    {#BM "x" #BN "x" #BK " waves " #WM "x" #WN " stages " #ST " lds-direct", BM, BN, BK, fast_accepts<BM, BN, BK, ST>, fast_launch<BM, BN, BK, WM, WN, ST, OCC>}

// the same kernels with partial last tiles along N and K (both multiples of 8)
#define NT_TAIL_INSTANCE(BM, BN, BK, WM, WN, ST, OCC) \
    {#BM "x" #BN "x" #BK " waves " #WM "x" #WN " stages " #ST " lds-direct tails", BM, BN, BK, fast_accepts<BM, BN, BK, ST, true>, fast_launch<BM, BN, BK, WM, WN, ST, OCC, 0, 1, 0, true>}

#define NT_SPLIT_INSTANCE(BM, BN, BK, WM, WN, ST, OCC) \
    {#BM "x" #BN "x" #BK " waves " #WM "x" #WN " stages " #ST " lds-direct tails split-k", BM, BN, BK, split_accepts<BM, BN, BK, ST>, split_launch<BM, BN, BK, WM, WN, ST, OCC>}

// positions in kInstances (the tuning cache and the heuristics refer to instances by position)
enum InstanceIndex {
    kAnyStride, k256x256x32, k256x256x64, k128x128x64, k64x64x64, k128x256x32,
    kTail256x256x32, kTail128x256x32, kTail128x128x64, kTail64x64x64, kSplit64x64x64, kSplit128x128x64,
    kSplit128x256x32, kSplit256x256x32,
};

const GemmInstance kInstances[] = {
    {"128x128x32 waves 2x2 any-stride", kGenBM, kGenBN, kGenBK, generic_accepts, generic_launch},
    NT_FAST_INSTANCE(256, 256, 32, 2, 4, 5, 2),  // 5 x 32 KiB: the whole LDS of a CU
    NT_FAST_INSTANCE(256, 256, 64, 2, 4, 2, 2),
    NT_FAST_INSTANCE(128, 128, 64, 2, 2, 2, 2),
    NT_FAST_INSTANCE(64, 64, 64, 2, 2, 4, 2),  // small problems: more, smaller tiles to occupy the CUs
    NT_FAST_INSTANCE(128, 256, 32, 1, 4, 3, 2),  // two workgroups per CU: mid-size problems
    NT_TAIL_INSTANCE(256, 256, 32, 2, 4, 5, 2),
    NT_TAIL_INSTANCE(128, 256, 32, 1, 4, 3, 2),
    NT_TAIL_INSTANCE(128, 128, 64, 2, 2, 2, 2),
    NT_TAIL_INSTANCE(64, 64, 64, 2, 2, 4, 2),
    NT_SPLIT_INSTANCE(64, 64, 64, 2, 2, 4, 2),
    NT_SPLIT_INSTANCE(128, 128, 64, 2, 2, 2, 2),
    NT_SPLIT_INSTANCE(128, 256, 32, 1, 4, 3, 2),  // a few hundred rows against a wide rhs: 64 to 160 large tiles
    NT_SPLIT_INSTANCE(256, 256, 32, 2, 4, 5, 2),
#ifdef NT_GEMM_ABLATION
#define NT_LOAD_INSTANCE(BM, BN, BK, WM, WN, ST, OCC, LD, AUX) \
    {#BM "x" #BN "x" #BK " waves " #WM "x" #WN " stages " #ST " load " #LD " aux " #AUX, BM, BN, BK, fast_accepts<BM, BN, BK, ST>, fast_launch<BM, BN, BK, WM, WN, ST, OCC, 0, LD, AUX>}
#define NT_ABLATED_INSTANCE(BM, BN, BK, WM, WN, ST, OCC, AB) \
    {#BM "x" #BN "x" #BK " waves " #WM "x" #WN " stages " #ST " ABLATED " #AB " (wrong results)", BM, BN, BK, fast_accepts<BM, BN, BK, ST>, fast_launch<BM, BN, BK, WM, WN, ST, OCC, AB>}
    NT_LOAD_INSTANCE(256, 256, 32, 2, 4, 4, 2, 1, 0),
    NT_LOAD_INSTANCE(256, 256, 32, 2, 2, 4, 1, 1, 0),
    NT_LOAD_INSTANCE(256, 256, 32, 2, 2, 5, 1, 1, 0),
    NT_LOAD_INSTANCE(256, 256, 64, 2, 2, 2, 1, 1, 0),
    NT_LOAD_INSTANCE(128, 256, 32, 1, 4, 3, 2, 1, 0),
    NT_ABLATED_INSTANCE(256, 256, 32, 2, 4, 4, 2, 1),
    NT_ABLATED_INSTANCE(256, 256, 32, 2, 4, 4, 2, 2),
    NT_ABLATED_INSTANCE(256, 256, 32, 2, 4, 4, 2, 3),
#endif
};
constexpr int kNumInstances = sizeof(kInstances) / sizeof(kInstances[0]);
static_assert(kNumInstances > kSplit256x256x32, "InstanceIndex names the first instances of the table");

inline bool is_split(int instance) { return instance >= kSplit64x64x64 && instance <= kSplit256x256x32; }

// choices read from a tuning file: an instance index counts only together with the block sizes saved next to it
bool gemm_choice_known(int index, const int *extra, int extras) {
    return index >= 0 && index < kNumInstances && extras == 3 && extra[0] == kInstances[index].bm && extra[1] == kInstances[index].bn &&
           extra[2] == kInstances[index].bk;
}
const bool g_gemm_check_registered = tune_register_check(kTuneGemm, gemm_choice_known);

// ---- tuned choices: (dtype, output dtype, M, N, K, addmm, rhs layout) -> instance ----
void tune_values(const GemmProblem &q, int (&values)[7]) {
    int layout = b_is_transposed(q) ? 1 : (q.sbn == 1 ? 0 : 2);  // rhs row-major, transposed, other strides
    // + 4: operands that the direct-to-LDS instances cannot read in place (they run on dense copies, whose own
    // problem -- same sizes when K is a multiple of 8 -- must not share this one's entry)
    const bool in_place = q.sak == 1 && q.sam % 8 == 0 && q.k % 8 == 0 && (((uintptr_t)q.a | (uintptr_t)q.b) & 15) == 0 &&
                          (b_is_transposed(q) ? q.sbn % 8 == 0 : (q.sbn == 1 && q.sbk % 8 == 0 && q.n % 8 == 0));
    if (!in_place && (q.dtype == NINETOOTHED_FLOAT16 || q.dtype == NINETOOTHED_BFLOAT16)) layout += 4;
    const int v[7] = {q.dtype, q.out_dtype, q.m, q.n, q.k, q.addmm() ? 1 : 0, layout};
    for (int i = 0; i < 7; ++i) values[i] = v[i];
}

int lookup_tuned(const GemmProblem &q) {
    int values[7];
    tune_values(q, values);
    const int choice = tune_lookup(kTuneGemm, values, 7);
    return choice >= 0 && choice < kNumInstances ? choice : -1;
}

// Untuned choice: the largest direct-to-LDS tile that still gives every CU a
// tile (256 CUs), falling back to smaller tiles, then to the any-stride kernel.
int heuristic_choice(const GemmProblem &q, int bm, int bn, int bk) {
    if (bm > 0 && bn > 0) {  // caller fixed the blocks: nearest accepting instance
        int best = -1;
        long best_d = 0;
        for (int i = 0; i < kNumInstances; ++i) {
            if (!kInstances[i].accepts(q)) continue;
            long d = labs(kInstances[i].bm - bm) + labs(kInstances[i].bn - bn) + (bk > 0 ? labs(kInstances[i].bk - bk) : 0);
            if (best < 0 || d < best_d) {
                best = i;
                best_d = d;
            }
        }
        return best;
    }
    // untuned preference (measured on square problems): 256x256 tiles from 256 tiles up,
    // 128x256 from 128 tiles up, 128x128 from 256 tiles up, else the smallest tile that divides
    struct Rule { int instance; int64_t min_tiles; };
    // too few tiles for the chip: split K (64-row tiles for up to 64 rows, else 128 x 128)
    // (64 x 64 tiles of the product: where they fill the chip, a skinny product runs on them in one pass -- 256 x 4096 x 4096
    // 19 us against 27 with K in parts of 128 x 128 tiles, 128 x 4096 x 14336 33 against 42 -- and tiles that the product
    // fills to less than half along M or N are passed over: 64 x 4096 x 128256 259 us on 256 x 256 tiles, 220 on 64 x 64)
    const int64_t tiles_64 = (int64_t)((q.m + 63) / 64) * ((q.n + 63) / 64);
    const bool small_tiles_fill_the_chip = q.batch == 1 && tiles_64 >= 256 && kInstances[kTail64x64x64].accepts(q);
    const auto few_tiles = [&](int instance) {
        const GemmInstance &inst = kInstances[instance];
        // (with a short K the second kernel costs more than the idle CUs: 512^3 8 us split, 5 in one pass)
        return q.batch == 1 && !small_tiles_fill_the_chip && q.k >= 2048 && (int64_t)((q.m + inst.bm - 1) / inst.bm) * ((q.n + inst.bn - 1) / inst.bn) < 192 &&
               inst.accepts(q);
    };
    if (q.m <= 64 && few_tiles(kSplit64x64x64)) return kSplit64x64x64;
    if (few_tiles(kSplit128x128x64)) return kSplit128x128x64;
    if (few_tiles(kSplit64x64x64)) return kSplit64x64x64;
    // (an instance with tails accepts what its plain form accepts, so it comes right after it: a partial
    // last tile costs less than a smaller tile everywhere)
    const Rule rules[] = {{k256x256x32, 256}, {k256x256x64, 256}, {kTail256x256x32, 256}, {k128x256x32, 128}, {kTail128x256x32, 128},
                          {k128x128x64, 256}, {kTail128x128x64, 256}, {k64x64x64, 1}, {kTail64x64x64, 1}, {k128x128x64, 1}, {kTail128x128x64, 1},
                          {k128x256x32, 1}, {kTail128x256x32, 1}, {k256x256x64, 1}, {k256x256x32, 1}, {kTail256x256x32, 1}};
    for (const Rule &rule : rules) {
        const GemmInstance &inst = kInstances[rule.instance];
        if (!inst.accepts(q)) continue;
        const int64_t per_matrix = (int64_t)((q.m + inst.bm - 1) / inst.bm) * ((q.n + inst.bn - 1) / inst.bn);
        // (a batch of small matrices reaches any number of tiles: a tile that such a matrix fills to less than
        // 60 % is left to the rules of the second pass, which start from the small tiles -- unless 64 x 64 tiles
        // would be as empty: 197 x 197 fills 59 % of one 256 x 256 tile and 59 % of sixteen 64 x 64 ones)
        if (small_tiles_fill_the_chip && (inst.bm > 64 || inst.bn > 64) &&
            ((int64_t)q.m * 2 < (int64_t)((q.m + inst.bm - 1) / inst.bm) * inst.bm || (int64_t)q.n * 2 < (int64_t)((q.n + inst.bn - 1) / inst.bn) * inst.bn))
            continue;
        const int64_t small_tiles = tiles_64 * 64 * 64;
        if (q.batch > 1 && rule.min_tiles > 1 && (int64_t)q.m * q.n * 5 < per_matrix * inst.bm * inst.bn * 3 && per_matrix * inst.bm * inst.bn * 9 > small_tiles * 10) continue;
        if (per_matrix * q.batch >= rule.min_tiles) return rule.instance;
    }
    return kInstances[kAnyStride].accepts(q) ? kAnyStride : -1;
}

bool read_matrix(const NineToothedTensor &t, uint64_t &d0, uint64_t &d1, int64_t &s0, int64_t &s1) {
    if (t.shape == nullptr || t.strides == nullptr) return false;
    d0 = t.shape[0];
    d1 = t.shape[1];
    s0 = t.strides[0];
    s1 = t.strides[1];
    return true;
}

int build_problem(GemmProblem &q, const NineToothedTensor *input, const NineToothedTensor &a, const NineToothedTensor &b,
                  const NineToothedTensor *beta, const NineToothedTensor *alpha, const NineToothedTensor &c, int dtype,
                  int out_dtype) {
    uint64_t am, ak, bk, bn, cm, cn;
    if (!read_matrix(a, am, ak, q.sam, q.sak) || !read_matrix(b, bk, bn, q.sbk, q.sbn) || !read_matrix(c, cm, cn, q.scm, q.scn))
        return hipErrorInvalidValue;
    if (ak != bk || am != cm || bn != cn) return hipErrorInvalidValue;
    if (am > 0x7fffffffull || bn > 0x7fffffffull || ak > 0x7fffffffull) return NINETOOTHED_NO_KERNEL;
    q.dtype = dtype;
    q.out_dtype = out_dtype;
    q.m = (int)am;
    q.n = (int)bn;
    q.k = (int)ak;
    q.a = a.data;
    q.b = b.data;
    q.c = c.data;
    q.bias = nullptr;
    q.sim = q.sin = 0;
    q.alpha = 1.0f;
    q.beta = 0.0f;
    if (input != nullptr && input->data != nullptr) {
        uint64_t im, in_;
        if (!read_matrix(*input, im, in_, q.sim, q.sin)) return hipErrorInvalidValue;
        if (im != cm || in_ != cn) return hipErrorInvalidValue;
        if (beta == nullptr || alpha == nullptr || beta->data == nullptr || alpha->data == nullptr) return hipErrorInvalidValue;
        q.bias = input->data;
        q.beta = (float)Scalar0d::as_double(*beta);
        q.alpha = (float)Scalar0d::as_double(*alpha);
    }
    if ((q.m > 0 && q.n > 0) && (q.a == nullptr && q.k > 0)) return hipErrorInvalidValue;
    return 0;
}

// ---- fp8 (e5m2) operands of large products: widened copies, then the fp16 instances ----
// An e5m2 value is the upper byte of the fp16 value it equals, so widening is exact and the fp16 kernels compute
// what the widening any-stride kernel computes (every product exact, fp32 sums).  One pass per operand writes a dense
// fp16 copy in the operand's own orientation -- rows contiguous or columns contiguous -- into the stream's scratch
// buffers; the direct-to-LDS instances then run the product several times faster than the any-stride kernel.
__global__ __launch_bounds__(256) void widen_e5m2_kernel(const uint8_t *src, int64_t outer, int64_t inner, int64_t outer_stride,
                                                         int64_t inner_stride, int64_t pitch, uint16_t *dst, int vectors) {
    typedef unsigned uint4_t __attribute__((ext_vector_type(4)));
    const int64_t per_row = vectors ? inner / 16 : inner;
    const int64_t total = outer * per_row;
    for (int64_t index = (int64_t)blockIdx.x * 256 + threadIdx.x; index < total; index += (int64_t)gridDim.x * 256) {
        const int64_t row = index / per_row, piece = index - row * per_row;
        if (vectors) {  // 16 bytes in, 32 out: byte b of a dword becomes the upper byte of half b
            const uint4_t in = *(const uint4_t *)(src + row * outer_stride + piece * 16);
            uint4_t lo, hi;
            lo[0] = __builtin_amdgcn_perm(0u, in[0], 0x010c000cu);
            lo[1] = __builtin_amdgcn_perm(0u, in[0], 0x030c020cu);
            lo[2] = __builtin_amdgcn_perm(0u, in[1], 0x010c000cu);
            lo[3] = __builtin_amdgcn_perm(0u, in[1], 0x030c020cu);
            hi[0] = __builtin_amdgcn_perm(0u, in[2], 0x010c000cu);
            hi[1] = __builtin_amdgcn_perm(0u, in[2], 0x030c020cu);
            hi[2] = __builtin_amdgcn_perm(0u, in[3], 0x010c000cu);
            hi[3] = __builtin_amdgcn_perm(0u, in[3], 0x030c020cu);
            uint4_t *out = (uint4_t *)(dst + row * pitch + piece * 16);
            __builtin_nontemporal_store(lo, out);
            __builtin_nontemporal_store(hi, out + 1);
        } else {
            dst[row * pitch + piece] = (uint16_t)((unsigned)src[row * outer_stride + piece * inner_stride] << 8);
        }
    }
}

// writes the widened copy of a [d0, d1] matrix with element strides (s0, s1) and returns the copy's strides
hipError_t widen_e5m2(hipStream_t stream, const void *src, int64_t d0, int64_t d1, int64_t s0, int64_t s1, uint16_t *dst, int64_t &t0, int64_t &t1) {
    const bool by_columns = s0 == 1 && s1 != 1;  // columns contiguous: the copy keeps that orientation
    const int64_t outer = by_columns ? d1 : d0, inner = by_columns ? d0 : d1;
    const int64_t outer_stride = by_columns ? s1 : s0, inner_stride = by_columns ? s0 : s1;
    const int64_t pitch = (inner + 7) / 8 * 8;  // rows of the copy start on 16-byte boundaries
    t0 = by_columns ? 1 : pitch;
    t1 = by_columns ? pitch : 1;
    if (outer == 0 || inner == 0) return hipSuccess;
    const int vectors = inner_stride == 1 && inner % 16 == 0 && outer_stride % 16 == 0 && ((uintptr_t)src & 15) == 0;
    const int64_t work = outer * (vectors ? inner / 16 : inner);
    const unsigned blocks = (unsigned)std::min<int64_t>((work + 255) / 256, 256 * 32);
    widen_e5m2_kernel<<<dim3(blocks), dim3(256), 0, stream>>>((const uint8_t *)src, outer, inner, outer_stride, inner_stride, pitch, dst, vectors);
    return hipGetLastError();
}

int run_gemm(hipStream_t stream, const GemmProblem &q, int bm, int bn, int bk, bool may_copy = true);

// ---- fp16 / bf16 operands that the direct-to-LDS instances cannot read in place ----
// A K that is no multiple of 8, rows that do not start on 16-byte boundaries, an lhs stored by columns, operands with
// other strides: the any-stride kernel gathers such operands two bytes at a time and reaches a fifth of the fast
// instances' rate.  For products that are large enough, one pass per operand writes a dense copy with k contiguous --
// the lhs as [M][K8], the rhs as [N][K8], K8 = K rounded up to 8 with zeros in between, which add nothing to the sums --
// and the product runs on the instances with tails, which take a k-contiguous rhs with any N.
// dst[i][j] = j < d1 ? src[i * s0 + j * s1] : 0 for j < pitch; 64 x 64 tiles through LDS, so that the reads run along
// whichever dimension has the smaller stride and the writes along j, 16 bytes per lane on both sides where the
// source is contiguous along that dimension
__global__ __launch_bounds__(256) void repack_operand_kernel(const uint16_t *src, int64_t d0, int64_t d1, int64_t s0, int64_t s1, uint16_t *dst, int64_t pitch,
                                                            int64_t src_batch) {
    src += (int64_t)blockIdx.y * src_batch;  // a batch of matrices: the copies lie one after another
    dst += (int64_t)blockIdx.y * d0 * pitch;
    typedef uint16_t ushort8_t __attribute__((ext_vector_type(8)));
    typedef ushort8_t unaligned_ushort8_t __attribute__((aligned(2)));  // (global accesses need the element's alignment only)
    constexpr int kPitch = 72;  // rows of the tile start on 16-byte boundaries
    __shared__ __attribute__((aligned(16))) uint16_t tile[64 * kPitch];
    const int64_t tiles_j = (pitch + 63) / 64;
    const int64_t i0 = (int64_t)(blockIdx.x / tiles_j) * 64, j0 = (int64_t)(blockIdx.x % tiles_j) * 64;
    const int t = threadIdx.x;
    const bool along_i = s0 < s1;  // consecutive threads read consecutive i
    const int64_t fast_stride = along_i ? s0 : s1;
    if (fast_stride != 1) {  // (uniform) no dimension is contiguous: consecutive threads fetch consecutive elements
#pragma unroll 4
        for (int e = t; e < 64 * 64; e += 256) {
            const int fast = e & 63, slow = e >> 6;
            const int i = along_i ? fast : slow, j = along_i ? slow : fast;
            uint16_t value = 0;
            if (i0 + i < d0 && j0 + j < d1) value = src[(i0 + i) * s0 + (j0 + j) * s1];
            tile[i * kPitch + j] = value;
        }
    } else
    // eight consecutive elements of the source's contiguous dimension per thread, in one load
#pragma unroll
    for (int e = t; e < 64 * 8; e += 256) {
        const int fast = (e & 7) * 8, slow = e >> 3;
        const int i = along_i ? fast : slow, j = along_i ? slow : fast;
        const int64_t limit = along_i ? d0 - (i0 + i) : d1 - (j0 + j);  // elements left along the faster dimension
        const bool slow_inside = along_i ? j0 + j < d1 : i0 + i < d0;
        ushort8_t values = {0, 0, 0, 0, 0, 0, 0, 0};
        if (slow_inside && limit > 0) {
            const uint16_t *from = src + (i0 + i) * s0 + (j0 + j) * s1;
            if (fast_stride == 1 && limit >= 8) {
                values = *(const unaligned_ushort8_t *)from;
            } else {
#pragma unroll
                for (int c = 0; c < 8; ++c)
                    if (c < limit) values[c] = from[c * fast_stride];
            }
        }
        if (along_i) {
#pragma unroll
            for (int c = 0; c < 8; ++c) tile[(i + c) * kPitch + j] = values[c];
        } else {
            *(ushort8_t *)&tile[i * kPitch + j] = values;
        }
    }
    __syncthreads();
#pragma unroll
    for (int e = t; e < 64 * 8; e += 256) {
        const int j = (e & 7) * 8, i = e >> 3;
        if (i0 + i >= d0 || j0 + j >= pitch) continue;  // (pitch is a multiple of 8: whole vectors)
        *(ushort8_t *)(dst + (i0 + i) * pitch + j0 + j) = *(const ushort8_t *)&tile[i * kPitch + j];
    }
}

hipError_t repack_operand(hipStream_t stream, const void *src, int64_t d0, int64_t d1, int64_t s0, int64_t s1, uint16_t *dst, int64_t pitch, int batch = 1,
                          int64_t src_batch = 0) {
    const int64_t tiles = ((d0 + 63) / 64) * ((pitch + 63) / 64);
    if (tiles == 0 || batch == 0) return hipSuccess;
    if (tiles > 0x7fffffffll || batch > 65535) return hipErrorInvalidValue;
    repack_operand_kernel<<<dim3((unsigned)tiles, (unsigned)batch), dim3(256), 0, stream>>>((const uint16_t *)src, d0, d1, s0, s1, dst, pitch, src_batch);
    return hipGetLastError();
}

int heuristic_choice(const GemmProblem &q, int bm, int bn, int bk);

// Writes the dense copies of q's operands into the stream's buffers (`lease` must stay alive until everything that
// reads them is enqueued) and describes the product on them in `dense`.  0, an error, or NINETOOTHED_NO_KERNEL when
// this way does not apply.
int make_dense_copies(hipStream_t stream, const GemmProblem &q, int bm, int bn, int bk, WorkspaceLease &lease, GemmProblem &dense) {
    if ((q.dtype != NINETOOTHED_FLOAT16 && q.dtype != NINETOOTHED_BFLOAT16) || q.batch < 1 || q.batch > 65535) return NINETOOTHED_NO_KERNEL;
#ifndef NT_GEMM_COPY_LOG2
#define NT_GEMM_COPY_LOG2 21
#endif
    // (the any-stride kernel is slower from small sizes on: 512^3 36-45 us in place against 11-13 us on copies,
    // 256^3 22-25 against 12; below 128^3 everything is one launch's time)
    if ((int64_t)q.m * q.n * q.k * q.batch < ((int64_t)1 << NT_GEMM_COPY_LOG2) || q.fixed_scratch != nullptr) return NINETOOTHED_NO_KERNEL;
    const int64_t k8 = ((int64_t)q.k + 7) / 8 * 8;
    dense = q;
    dense.k = (int)k8;
    dense.sam = k8;
    dense.sak = 1;
    dense.sbk = 1;
    dense.sbn = k8;
    dense.a_batch = (int64_t)q.m * k8;  // (a batch: one copy per product, also of an operand that the products share)
    dense.b_batch = (int64_t)q.n * k8;
    // (alignment of the copies is a fact, not a property of these placeholder addresses)
    dense.a = dense.b = (const void *)(uintptr_t)256;
    const int choice = heuristic_choice(dense, bm, bn, bk);
    if (choice < 0 || choice == kAnyStride) return NINETOOTHED_NO_KERNEL;  // (the output's layout rules the fast instances out)
    // (buffers of their own: the sources may be the widened copies of fp8 operands)
    if (((int64_t)q.m + q.n) * k8 * 2 * q.batch > (int64_t(1) << 32)) return NINETOOTHED_NO_KERNEL;  // (a batch whose copies would take more than 4 GiB)
    uint16_t *a = (uint16_t *)lease.get(kWorkspaceGemmLhsDense, (size_t)q.m * k8 * 2 * q.batch);
    uint16_t *b = a != nullptr ? (uint16_t *)lease.get(kWorkspaceGemmRhsDense, (size_t)q.n * k8 * 2 * q.batch) : nullptr;
    if (a == nullptr || b == nullptr) return NINETOOTHED_NO_KERNEL;
    dense.a = a;
    dense.b = b;
    if (hipError_t err = repack_operand(stream, q.a, q.m, q.k, q.sam, q.sak, a, k8, q.batch, q.a_batch)) return (int)err;
    if (hipError_t err = repack_operand(stream, q.b, q.n, q.k, q.sbn, q.sbk, b, k8, q.batch, q.b_batch)) return (int)err;
    return 0;
}

// 0 / an error when the product ran on copies, NINETOOTHED_NO_KERNEL when this way does not apply
int run_gemm_on_repacked_copies(hipStream_t stream, const GemmProblem &q, int bm, int bn, int bk) {
    WorkspaceLease lease(stream);  // held until the product is enqueued: it reads the copies
    GemmProblem dense;
    if (const int status = make_dense_copies(stream, q, bm, bn, bk, lease, dense)) return status;
    return run_gemm(stream, dense, bm, bn, bk, false);
}

// 0 / an error when the product ran on widened copies, NINETOOTHED_NO_KERNEL when this way does not apply (tiny
// products; negative strides; no scratch memory, as under graph capture before a call of the same size outside one):
// the widening any-stride kernel, which reads its operands byte by byte, then serves the call (512^3: 70 us against
// 12 us this way, 8192^3: 16.8 ms against 0.83 ms)
int run_gemm_on_widened_copies(hipStream_t stream, const GemmProblem &q, int bm, int bn, int bk) {
    if (q.dtype != NINETOOTHED_FLOAT8_E5M2 || q.batch != 1) return NINETOOTHED_NO_KERNEL;
    if (q.fixed_scratch != nullptr) return NINETOOTHED_NO_KERNEL;  // (the entry point that allocates nothing: no buffers for copies)
    if (q.out_dtype != NINETOOTHED_FLOAT16 && (q.out_dtype != NINETOOTHED_FLOAT32 || q.addmm())) return NINETOOTHED_NO_KERNEL;
    if ((int64_t)q.m * q.n * q.k < ((int64_t)1 << 18)) return NINETOOTHED_NO_KERNEL;
    if (q.sam < 0 || q.sak < 0 || q.sbk < 0 || q.sbn < 0 || (q.addmm() && (q.sim < 0 || q.sin < 0))) return NINETOOTHED_NO_KERNEL;
    WorkspaceLease lease(stream);  // held until the product is enqueued: it reads the copies
    const auto bytes = [](int64_t d0, int64_t d1) { return (size_t)(std::max(d0, d1) + 8) * (size_t)(std::min(d0, d1) + 8) * 2; };  // (either orientation, padded rows)
    uint16_t *a = (uint16_t *)lease.get(kWorkspaceGemmLhsWidened, bytes(q.m, q.k));
    uint16_t *b = a != nullptr ? (uint16_t *)lease.get(kWorkspaceGemmRhsWidened, bytes(q.k, q.n)) : nullptr;
    uint16_t *bias = b != nullptr && q.addmm() ? (uint16_t *)lease.get(kWorkspaceGemmBiasWidened, bytes(q.m, q.n)) : nullptr;
    if (a == nullptr || b == nullptr || (q.addmm() && bias == nullptr)) return NINETOOTHED_NO_KERNEL;
    GemmProblem wide = q;
    wide.dtype = NINETOOTHED_FLOAT16;
    wide.a = a;
    wide.b = b;
    if (hipError_t err = widen_e5m2(stream, q.a, q.m, q.k, q.sam, q.sak, a, wide.sam, wide.sak)) return (int)err;
    if (hipError_t err = widen_e5m2(stream, q.b, q.k, q.n, q.sbk, q.sbn, b, wide.sbk, wide.sbn)) return (int)err;
    if (q.addmm()) {
        wide.bias = bias;
        if (hipError_t err = widen_e5m2(stream, q.bias, q.m, q.n, q.sim, q.sin, bias, wide.sim, wide.sin)) return (int)err;
    }
    return run_gemm(stream, wide, bm, bn, bk);
}

// an output stored by columns (`out.T`): C^T = B^T A^T is the same product with a row-major output, which the
// direct-to-LDS instances write (the any-stride kernel would store it two bytes at a time)
bool output_by_columns(const GemmProblem &q) { return q.scn != 1 && q.scm == 1 && q.n > 1; }

GemmProblem transposed_problem(const GemmProblem &q) {
    GemmProblem t = q;
    t.m = q.n;
    t.n = q.m;
    t.a = q.b;
    t.b = q.a;
    t.sam = q.sbn;
    t.sak = q.sbk;
    t.sbk = q.sak;
    t.sbn = q.sam;
    t.scm = q.scn;
    t.scn = q.scm;
    t.sim = q.sin;
    t.sin = q.sim;
    t.a_batch = q.b_batch;
    t.b_batch = q.a_batch;
    return t;
}

// A product whose 256 x 256 tiles are a few more than whole rounds of the chip's 256 CUs (17 x 17 = 289 of them for
// 4352^2) pays a whole round for the few: the tile rows that fill whole rounds run in one pass, the rows left over
// -- at most 51 tiles -- as a product of their own with the k range in parts, so that they occupy the chip once for
// a fraction of a round.  NINETOOTHED_NO_KERNEL when the shape is not of that kind or scratch memory is not to be had.
int run_gemm_last_rows_in_parts(hipStream_t stream, const GemmProblem &q) {
    if ((q.dtype != NINETOOTHED_FLOAT16 && q.dtype != NINETOOTHED_BFLOAT16) || q.batch != 1 || q.fixed_scratch != nullptr) return NINETOOTHED_NO_KERNEL;
    static const bool enabled = getenv("NT_GEMM_NO_ROW_SPLIT") == nullptr;  // (set for A/B measurements: every product in one pass)
    if (!enabled) return NINETOOTHED_NO_KERNEL;
    const int64_t tiles_m = ceil_div(q.m, 256), tiles_n = ceil_div(q.n, 256), tiles = tiles_m * tiles_n;
    // (measured, one pass -> this way: 4352 x 4096 x 4352 160 -> 143 us, 4096 x 4096 x 4352 158 -> 135, 5120 x 4096 x 3584
    // 159 -> 139, 4104^3 172 -> 143; not for more than three rounds -- 8192 x 4096 x 8448 436 -> 447 --, for more than 51
    // tiles left over -- 4608^2 x 4096, 72 of them: 162 -> 173 -- or a short k range -- 4352 x 1024 x 4352 49 -> 63)
    if (tiles <= 256 || tiles > 768 || tiles % 256 == 0 || q.k < 2048) return NINETOOTHED_NO_KERNEL;
    const int64_t top_rows = tiles / 256 * 256 / tiles_n;
    const int64_t bottom_tiles = (tiles_m - top_rows) * tiles_n;
    if (top_rows < 1 || top_rows >= tiles_m || bottom_tiles * 5 > 256) return NINETOOTHED_NO_KERNEL;
    if (ceil_div(top_rows * tiles_n, (int64_t)256) >= ceil_div(tiles, (int64_t)256)) return NINETOOTHED_NO_KERNEL;  // (no round saved)
    const int64_t size = q.dtype == NINETOOTHED_FLOAT16 || q.dtype == NINETOOTHED_BFLOAT16 ? 2 : 4;
    const int64_t out_size = q.out_dtype == NINETOOTHED_FLOAT32 ? 4 : size;
    GemmProblem top = q, bottom = q;
    top.m = (int)(top_rows * 256);
    bottom.m = q.m - top.m;
    bottom.a = (const char *)q.a + (int64_t)top.m * q.sam * size;
    bottom.c = (char *)q.c + (int64_t)top.m * q.scm * out_size;
    if (q.bias != nullptr) bottom.bias = (const char *)q.bias + (int64_t)top.m * q.sim * size;
    const int whole = kInstances[k256x256x32].accepts(top) ? (int)k256x256x32 : (int)kTail256x256x32;
    if (!kInstances[whole].accepts(top) || !kInstances[kSplit256x256x32].accepts(bottom)) return NINETOOTHED_NO_KERNEL;
    int result = (int)kInstances[kSplit256x256x32].launch(bottom, stream);  // (first: it is the one that may find no scratch memory)
    if (result != 0) return result;
    note_launch(kLaunchGemm, whole, "256x256x32 tiles: the tile rows that fill whole rounds in one pass, the last rows with the k range in parts");
    return (int)kInstances[whole].launch(top, stream);
}

int run_gemm(hipStream_t stream, const GemmProblem &q, int bm, int bn, int bk, bool may_copy) {
    if (q.m == 0 || q.n == 0) return 0;
    if (output_by_columns(q)) return run_gemm(stream, transposed_problem(q), bn, bm, bk, may_copy);
    if (bm <= 0 && bn <= 0 && bk <= 0) {
        const int rows_split = run_gemm_last_rows_in_parts(stream, q);
        if (rows_split != NINETOOTHED_NO_KERNEL) return rows_split;
    }
    if (q.dtype == NINETOOTHED_FLOAT8_E5M2) {
        const int widened = run_gemm_on_widened_copies(stream, q, bm, bn, bk);
        if (widened != NINETOOTHED_NO_KERNEL) return widened;
    }
    int choice = -1;
    if ((bm <= 0 || bn <= 0) && q.batch == 1) choice = lookup_tuned(q);  // (tuned choices are recorded for single products)
    if (choice < 0 || !kInstances[choice].accepts(q)) choice = heuristic_choice(q, bm, bn, bk);
    if (choice < 0) return NINETOOTHED_NO_KERNEL;
    if (choice == kAnyStride && may_copy) {
        const int copied = run_gemm_on_repacked_copies(stream, q, bm, bn, bk);
        if (copied != NINETOOTHED_NO_KERNEL) return copied;
    }
    note_launch(kLaunchGemm, choice, kInstances[choice].name);
    int result;
    if (bm > 0 || bn > 0 || bk > 0) {
        GemmProblem hinted = q;
        hinted.hinted = true;
        result = (int)kInstances[choice].launch(hinted, stream);
    } else {
        result = (int)kInstances[choice].launch(q, stream);
    }
    if (result == NINETOOTHED_NO_KERNEL && is_split(choice)) {  // a split-K instance without scratch memory
        for (int fallback : {(int)kTail64x64x64, (int)kTail128x128x64, (int)kTail256x256x32, (int)kAnyStride})
            if (kInstances[fallback].accepts(q)) {
                note_launch(kLaunchGemm, fallback, kInstances[fallback].name);
                return (int)kInstances[fallback].launch(q, stream);
            }
    }
    return result;
}

}  // namespace
}  // namespace nt

using namespace nt;

extern "C" {

NineToothedResult launch_nt_matmul(NineToothedStream stream, NineToothedTensor lhs, NineToothedTensor rhs,
                                   NineToothedTensor output, int dtype, int output_dtype, int block_size_m,
                                   int block_size_n, int block_size_k) {
    GemmProblem q;
    if (int err = build_problem(q, nullptr, lhs, rhs, nullptr, nullptr, output, dtype, output_dtype)) return err;
    return run_gemm((hipStream_t)stream, q, block_size_m, block_size_n, block_size_k);
}

NineToothedResult launch_nt_batched_matmul(NineToothedStream stream, NineToothedTensor lhs, NineToothedTensor rhs,
                                           NineToothedTensor output, int dtype, int output_dtype, int block_size_m,
                                           int block_size_n, int block_size_k) {
    if (!lhs.shape || !rhs.shape || !output.shape || !lhs.strides || !rhs.strides || !output.strides) return hipErrorInvalidValue;
    const uint64_t batch = output.shape[0];
    // an operand with a single matrix is shared by all products
    if ((lhs.shape[0] != batch && lhs.shape[0] != 1) || (rhs.shape[0] != batch && rhs.shape[0] != 1)) return hipErrorInvalidValue;
    if (batch > 0x7fffffffull) return NINETOOTHED_NO_KERNEL;
    const NineToothedTensor a = {lhs.data, lhs.shape + 1, lhs.strides + 1}, b = {rhs.data, rhs.shape + 1, rhs.strides + 1},
                            c = {output.data, output.shape + 1, output.strides + 1};
    GemmProblem q;
    if (int err = build_problem(q, nullptr, a, b, nullptr, nullptr, c, dtype, output_dtype)) return err;
    if (batch == 0) return 0;
    q.batch = (int)batch;
    q.a_batch = lhs.shape[0] == 1 ? 0 : lhs.strides[0];
    q.b_batch = rhs.shape[0] == 1 ? 0 : rhs.strides[0];
    q.c_batch = output.strides[0];
    return run_gemm((hipStream_t)stream, q, block_size_m, block_size_n, block_size_k);
}

NineToothedResult launch_nt_addmm(NineToothedStream stream, NineToothedTensor input, NineToothedTensor mat1,
                                  NineToothedTensor mat2, NineToothedTensor beta, NineToothedTensor alpha,
                                  NineToothedTensor output, int dtype, int block_size_m, int block_size_n,
                                  int block_size_k) {
    if (input.data == nullptr) return hipErrorInvalidValue;
    GemmProblem q;
    const int output_dtype = dtype == NINETOOTHED_FLOAT8_E5M2 ? NINETOOTHED_FLOAT16 : dtype;  // fp8 operands: the rounded product is fp16
    if (int err = build_problem(q, &input, mat1, mat2, &beta, &alpha, output, dtype, output_dtype)) return err;
    return run_gemm((hipStream_t)stream, q, block_size_m, block_size_n, block_size_k);
}

}  // extern "C"

namespace nt {
namespace {

// Scratch memory of launch_nt_matmul_static_scratch: part of the library's code object, so every GPU the
// library runs on holds its own copy from the first use until the process ends.  Host code never uses the
// array's name as an address (on the host it is a stand-in, not device memory): the device address is
// asked for once per device and only that pointer is handed to kernels.
constexpr size_t kStaticScratchBytes = size_t(NINETOOTHED_STATIC_SCRATCH_BYTES);
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kMaxDevices = 64;
std::mutex g_static_scratch_mutex;
void *g_static_scratch_address[kMaxDevices] = {};

// the array's address on the current device
int static_scratch_address(void **address) {
    int device = 0;
    hipError_t err = hipGetDevice(&device);
    if (err != hipSuccess) return (int)err;
    if (device < 0 || device >= kMaxDevices) return (int)hipErrorInvalidDevice;
    std::lock_guard<std::mutex> lock(g_static_scratch_mutex);
    if (g_static_scratch_address[device] == nullptr) {
        void *found = nullptr;
        err = hipGetSymbolAddress(&found, HIP_SYMBOL(scratch));
        if (err != hipSuccess) return (int)err;
        if (found == nullptr) return (int)hipErrorInvalidSymbol;
        g_static_scratch_address[device] = found;
    }
    *address = g_static_scratch_address[device];
    return 0;
}

}  // namespace
}  // namespace nt

extern "C" {

NineToothedResult launch_nt_matmul_static_scratch(NineToothedStream stream, NineToothedTensor lhs, NineToothedTensor rhs,
                                                  NineToothedTensor output, int dtype, int output_dtype, int block_size_m,
                                                  int block_size_n, int block_size_k) {
    GemmProblem q;
    if (int err = build_problem(q, nullptr, lhs, rhs, nullptr, nullptr, output, dtype, output_dtype)) return err;
    void *address = nullptr;
    if (int err = static_scratch_address(&address)) return err;
    q.fixed_scratch = (float *)address;
    q.fixed_scratch_bytes = kStaticScratchBytes;
    return run_gemm((hipStream_t)stream, q, block_size_m, block_size_n, block_size_k);
}

int nt_gemm_num_configs(void) { return kNumInstances; }

NineToothedResult nt_gemm_config_name(int config, char *buffer, int size) {
    if (config < 0 || config >= kNumInstances || buffer == nullptr || size <= 0) return NINETOOTHED_NO_KERNEL;
    snprintf(buffer, (size_t)size, "%s", kInstances[config].name);
    return 0;
}

NineToothedResult launch_nt_gemm_config(NineToothedStream stream, int config, NineToothedTensor input,
                                        NineToothedTensor mat1, NineToothedTensor mat2, NineToothedTensor beta,
                                        NineToothedTensor alpha, NineToothedTensor output, int dtype,
                                        int output_dtype) {
    if (config < 0 || config >= kNumInstances) return NINETOOTHED_NO_KERNEL;
    GemmProblem q;
    if (int err = build_problem(q, &input, mat1, mat2, &beta, &alpha, output, dtype, output_dtype)) return err;
    if (q.m == 0 || q.n == 0) return 0;
    if (!kInstances[config].accepts(q)) return NINETOOTHED_NO_KERNEL;
    return (int)kInstances[config].launch(q, (hipStream_t)stream);
}

NineToothedResult nt_tune_gemm(NineToothedStream stream_, NineToothedTensor input, NineToothedTensor mat1,
                               NineToothedTensor mat2, NineToothedTensor beta, NineToothedTensor alpha,
                               NineToothedTensor output, int dtype, int output_dtype, int iters, int *best_config,
                               float *best_ms) {
    hipStream_t stream = (hipStream_t)stream_;
    GemmProblem given;
    if (int err = build_problem(given, &input, mat1, mat2, &beta, &alpha, output, dtype, output_dtype)) return err;
    // (what the launch functions do first: an output stored by columns is the transposed product)
    GemmProblem q = output_by_columns(given) ? transposed_problem(given) : given;
    int best = -1;
    float best_time = 0.0f;
    // A problem that a single instance accepts has nothing to time.  Operands that only the any-stride kernel reads
    // in place run on dense copies (launch_nt_matmul / launch_nt_addmm): then the product on the copies is what
    // gets timed and recorded, under its own key, where the launch functions look it up.
    int accepting = 0;
    for (int i = 0; i < kNumInstances; ++i) accepting += kInstances[i].accepts(q) ? 1 : 0;
    std::unique_ptr<WorkspaceLease> lease;  // (keeps the copies in place while they are timed)
    if (accepting <= 1) {
        GemmProblem dense;
        lease.reset(new WorkspaceLease(stream));
        const int copied = stream_is_capturing(stream) ? NINETOOTHED_NO_KERNEL : make_dense_copies(stream, q, 0, 0, 0, *lease, dense);
        if (copied != 0) {
            if (best_config) *best_config = accepting == 1 ? -2 : -1;
            if (best_ms) *best_ms = 0.0f;
            if (copied != NINETOOTHED_NO_KERNEL) return copied;
            return accepting == 1 ? 0 : NINETOOTHED_NO_KERNEL;
        }
        q = dense;
        const int known = lookup_tuned(q);
        if (known >= 0 && kInstances[known].accepts(q)) {  // (an earlier process has timed it: the file was loaded)
            if (best_config) *best_config = known;
            if (best_ms) *best_ms = 0.0f;
            return 0;
        }
    }
    // (inside a graph capture nothing is timed: the problem stays on the fixed preference order and nothing is recorded)
    // the untuned rule's instance is timed first and stays unless another one is more than 2 % faster: timings of a
    // few launches scatter by about that much, and the choice should not differ from process to process for nothing
    const int preferred = heuristic_choice(q, 0, 0, 0);
    auto instance_of = [&](int i) { return preferred < 0 ? i : (i == 0 ? preferred : (i - 1 < preferred ? i - 1 : i)); };
    const int result = tune_time(stream, kNumInstances, iters, [&](int i) -> int {
        const int instance = instance_of(i);
        if (!kInstances[instance].accepts(q)) return NINETOOTHED_NO_KERNEL;
        return (int)kInstances[instance].launch(q, stream);
    }, &best, &best_time, 0.02f);
    if (best >= 0) best = instance_of(best);
    if (best_config) *best_config = best;
    if (best_ms) *best_ms = best_time;
    if (result != 0) return result;
    if (best < 0) return stream_is_capturing(stream) ? 0 : NINETOOTHED_NO_KERNEL;
    int values[7];
    tune_values(q, values);
    const int blocks[3] = {kInstances[best].bm, kInstances[best].bn, kInstances[best].bk};
    tune_record(kTuneGemm, values, 7, best, blocks, 3);
    return 0;
}

// The cached instance for a problem given by its sizes (row-major rhs), or -1.
int nt_tune_cache_lookup(int dtype, int output_dtype, int m, int n, int k, int addmm) {
    const int values[7] = {dtype, output_dtype, m, n, k, addmm ? 1 : 0, 0};
    const int choice = tune_lookup(kTuneGemm, values, 7);
    return choice >= 0 && choice < kNumInstances ? choice : -1;
}

}  // extern "C"

namespace nt {
namespace {

// the ways to run a convolution; kConvAuto tries them from the top (a 1 x 1 filter without padding first runs
// as a batch of plain products when it can)
enum ConvPath { kConvAuto = 0, kConvGather = 1, kConvRepack = 2, kConvDirect = 3, kConvPointwise = 4 };
bool conv2d_choice_known(int index, const int *, int) { return index >= kConvGather && index <= kConvPointwise; }
const bool g_conv2d_check_registered = tune_register_check(kTuneConv2d, conv2d_choice_known);

// validates the call and fills the request; returns 0, an error, or -1 when there is nothing to compute
int conv2d_request(Conv2dRequest &request, const NineToothedTensor &input, const NineToothedTensor &filter, const NineToothedTensor &output,
                   int dtype, int padding_h, int padding_w, int stride_h = 1, int stride_w = 1, int dilation_h = 1, int dilation_w = 1) {
    if (dtype != NINETOOTHED_FLOAT16 && dtype != NINETOOTHED_BFLOAT16 && dtype != NINETOOTHED_FLOAT32) return NINETOOTHED_NO_KERNEL;
    if (!input.shape || !filter.shape || !output.shape || !input.strides || !filter.strides || !output.strides)
        return hipErrorInvalidValue;
    if (padding_h < 0 || padding_w < 0 || stride_h < 1 || stride_w < 1 || dilation_h < 1 || dilation_w < 1) return hipErrorInvalidValue;
    const int64_t N = (int64_t)input.shape[0], C = (int64_t)input.shape[1], H = (int64_t)input.shape[2], W = (int64_t)input.shape[3];
    const int64_t K = (int64_t)filter.shape[0], R = (int64_t)filter.shape[2], S = (int64_t)filter.shape[3];
    if ((int64_t)filter.shape[1] != C) return hipErrorInvalidValue;
    // Windows start every `stride` positions of the padded input, as many as the output has rows / columns: either the
    // number that fit (floor, the usual convolution) or one more that hangs over the edge (the reference's
    // `Tensor.tile` without `floor_mode`, src/ninetoothed/tensor.py:237-248; what hangs over reads as padding).
    const int64_t span_h = H + 2 * padding_h - dilation_h * (R - 1) - 1, span_w = W + 2 * padding_w - dilation_w * (S - 1) - 1;
    const int64_t P = (int64_t)output.shape[2], Q = (int64_t)output.shape[3];
    if ((int64_t)output.shape[0] != N || (int64_t)output.shape[1] != K) return hipErrorInvalidValue;
    if (span_h < 0 || span_w < 0) {
        if (P > 0 && Q > 0) return hipErrorInvalidValue;  // the filter does not fit the padded input: no output positions
    } else {
        const int64_t fit_h = span_h / stride_h + 1, fit_w = span_w / stride_w + 1;
        const int64_t over_h = (span_h + stride_h - 1) / stride_h + 1, over_w = (span_w + stride_w - 1) / stride_w + 1;
        if ((P != fit_h && P != over_h) || (Q != fit_w && Q != over_w)) return hipErrorInvalidValue;
    }
    if (P <= 0 || Q <= 0 || N == 0 || K == 0) return -1;  // nothing to write
    if (N * P * Q > 0x7fffffffll || C * R * S > 0x7fffffffll || K > 0x7fffffffll || N > 0x7fffffffll) return NINETOOTHED_NO_KERNEL;
    request.dtype = dtype;
    request.x = input.data;
    request.w = filter.data;
    request.y = output.data;
    request.N = (int)N; request.C = (int)C; request.H = (int)H; request.W = (int)W;
    request.K = (int)K; request.R = (int)R; request.S = (int)S; request.P = (int)P; request.Q = (int)Q;
    request.pad_h = padding_h; request.pad_w = padding_w;
    request.stride_h = stride_h; request.stride_w = stride_w; request.dil_h = dilation_h; request.dil_w = dilation_w;
    for (int d = 0; d < 4; ++d) {
        request.xs[d] = input.strides[d];
        request.ws[d] = filter.strides[d];
        request.ys[d] = output.strides[d];
    }
    return 0;
}

template <typename T>
hipError_t conv2d_gather(const Conv2dRequest &r, hipStream_t stream) {
    Conv2dProblem<T> prob;
    prob.m = r.N * r.P * r.Q;
    prob.n = r.K;
    prob.k = r.C * r.R * r.S;
    prob.x = (const T *)r.x;
    prob.w = (const T *)r.w;
    prob.y = (T *)r.y;
    prob.C = r.C; prob.H = r.H; prob.W = r.W; prob.R = r.R; prob.S = r.S; prob.P = r.P; prob.Q = r.Q;
    prob.pad_h = r.pad_h;
    prob.pad_w = r.pad_w;
    prob.stride_h = r.stride_h; prob.stride_w = r.stride_w; prob.dil_h = r.dil_h; prob.dil_w = r.dil_w;
    for (int d = 0; d < 4; ++d) {
        prob.xs[d] = r.xs[d];
        prob.ws[d] = r.ws[d];
        prob.ys[d] = r.ys[d];
    }
    const int64_t tiles = (int64_t)ceil_div(prob.m, kGenBM) * ceil_div(prob.n, kGenBN);
    gemm_generic_kernel<Conv2dProblem<T>><<<dim3((unsigned)tiles), dim3(kGenThreads), 0, stream>>>(prob);
    return hipGetLastError();
}

// 1 x 1 filters without padding: per image Y[K, P*Q] = W[K, C] . X[C, P*Q], a batch of row-major products on
// the tensors as they lie (no repacking, no scratch memory).  NINETOOTHED_NO_KERNEL when the call is not that
// or no one-pass GEMM instance of the fast kind takes it.
int conv2d_pointwise(const Conv2dRequest &r, hipStream_t stream) {
    if (!(r.R == 1 && r.S == 1 && r.pad_h == 0 && r.pad_w == 0 && r.stride_h == 1 && r.stride_w == 1 && r.P == r.H && r.Q == r.W && r.xs[3] == 1 && r.xs[2] == r.W && r.ys[3] == 1 && r.ys[2] == r.Q && r.ws[1] == 1))
        return NINETOOTHED_NO_KERNEL;
    GemmProblem q;
    q.dtype = q.out_dtype = r.dtype;
    q.m = r.K;
    q.n = r.P * r.Q;
    q.k = r.C;
    q.a = r.w;
    q.b = r.x;
    q.c = r.y;
    q.bias = nullptr;
    q.sam = r.ws[0]; q.sak = 1;
    q.sbk = r.xs[1]; q.sbn = 1;
    q.scm = r.ys[1]; q.scn = 1;
    q.sim = q.sin = 0;
    q.alpha = 1.0f; q.beta = 0.0f;
    q.batch = r.N;
    q.a_batch = 0;
    q.b_batch = r.xs[0];
    q.c_batch = r.ys[0];
    const int choice = heuristic_choice(q, 0, 0, 0);
    if (choice <= kAnyStride || is_split(choice)) return NINETOOTHED_NO_KERNEL;
    note_launch(kLaunchConv2d, kConvPointwise, kInstances[choice].name);
    return (int)kInstances[choice].launch(q, stream);
}

int conv2d_run(const Conv2dRequest &r, int path, hipStream_t stream) {
    // fp32 tensors: the gathering kernel on fp32 MFMAs (the other paths move 16-bit elements)
    if (r.dtype == NINETOOTHED_FLOAT32) {
        if (path != kConvAuto && path != kConvGather) return NINETOOTHED_NO_KERNEL;
        note_launch(kLaunchConv2d, kConvGather, "gemm_generic_kernel with an im2col gather, fp32 MFMA");
        return (int)conv2d_gather<float>(r, stream);
    }
    if (path == kConvAuto || path == kConvPointwise) {
        const int pointwise = conv2d_pointwise(r, stream);
        if (pointwise != NINETOOTHED_NO_KERNEL || path == kConvPointwise) return pointwise;
    }
    if (path == kConvAuto || path == kConvDirect) {
        note_launch(kLaunchConv2d, kConvDirect, "conv2d_direct_kernel, one launch on the tensors as they lie");
        const int direct = conv2d_direct(r, stream);
        if (direct != NINETOOTHED_NO_KERNEL || path == kConvDirect) return direct;
    }
    if (path == kConvAuto || path == kConvRepack) {
        note_launch(kLaunchConv2d, kConvRepack, "conv2d_repack_kernel, then conv2d_nhwc_kernel on channels-last copies");
        const int fast = conv2d_fast(r, stream);
        if (fast != NINETOOTHED_NO_KERNEL || path == kConvRepack) return fast;
    }
    note_launch(kLaunchConv2d, kConvGather, "gemm_generic_kernel with an im2col gather");
    return r.dtype == NINETOOTHED_FLOAT16 ? (int)conv2d_gather<half_t>(r, stream) : (int)conv2d_gather<bf16_t>(r, stream);
}

void conv2d_tune_values(const Conv2dRequest &r, int (&values)[11]) {
    const int dense_x = r.xs[3] == 1 && r.xs[2] == r.W && r.xs[1] == (int64_t)r.H * r.W && r.xs[0] == (int64_t)r.C * r.H * r.W;
    const int v[11] = {r.dtype, r.N, r.C, r.H, r.W, r.K, r.R, r.S, r.pad_h, r.pad_w, dense_x};
    for (int i = 0; i < 11; ++i) values[i] = v[i];
}

}  // namespace
}  // namespace nt

extern "C" {

NineToothedResult launch_nt_conv2d(NineToothedStream stream, NineToothedTensor input, NineToothedTensor filter,
                                   NineToothedTensor output, int dtype, int padding_h, int padding_w, int block_size_m,
                                   int block_size_n, int block_size_k) {
    (void)block_size_n;
    (void)block_size_k;
    Conv2dRequest request;
    const int status = conv2d_request(request, input, filter, output, dtype, padding_h, padding_w);
    if (status != 0) return status < 0 ? 0 : status;
    // block_size_m: 1 = the gather kernel, 2 = the repacking path, 3 = the one-launch path, 4 = a 1 x 1 filter as a
    // batch of plain products; otherwise the tuned choice for this problem, else the library's order
    int path = block_size_m >= kConvGather && block_size_m <= kConvPointwise ? block_size_m : kConvAuto;
    if (block_size_m == 0) {
        int values[11];
        conv2d_tune_values(request, values);
        const int tuned = tune_lookup(kTuneConv2d, values, 11);
        if (tuned >= kConvGather && tuned <= kConvPointwise) path = tuned;
    }
    int result = conv2d_run(request, path, (hipStream_t)stream);
    // (a tuned path that needs scratch memory it cannot get, e.g. under graph capture: the library's order)
    if (result == NINETOOTHED_NO_KERNEL && path != kConvAuto && block_size_m == 0) result = conv2d_run(request, kConvAuto, (hipStream_t)stream);
    return result;
}

NineToothedResult launch_nt_conv2d_strided(NineToothedStream stream, NineToothedTensor input, NineToothedTensor filter,
                                           NineToothedTensor output, int dtype, int padding_h, int padding_w, int stride_h,
                                           int stride_w, int dilation_h, int dilation_w, int block_size_m, int block_size_n,
                                           int block_size_k) {
    if (stride_h == 1 && stride_w == 1 && dilation_h == 1 && dilation_w == 1) {
        Conv2dRequest plain;  // (an output with one more window than fits is not launch_nt_conv2d's problem)
        const int status = conv2d_request(plain, input, filter, output, dtype, padding_h, padding_w);
        if (status != 0) return status < 0 ? 0 : status;
        if (plain.P == plain.H + 2 * padding_h - plain.R + 1 && plain.Q == plain.W + 2 * padding_w - plain.S + 1)
            return launch_nt_conv2d(stream, input, filter, output, dtype, padding_h, padding_w, block_size_m, block_size_n, block_size_k);
    }
    (void)block_size_n;
    (void)block_size_k;
    Conv2dRequest request;
    const int status = conv2d_request(request, input, filter, output, dtype, padding_h, padding_w, stride_h, stride_w, dilation_h, dilation_w);
    if (status != 0) return status < 0 ? 0 : status;
    // the ways that take windows with steps: 2 = repacking pass plus GEMM loop, 1 = gather kernel (nothing is tuned here)
    const int path = block_size_m == kConvGather || block_size_m == kConvRepack ? block_size_m : kConvAuto;
    int result = conv2d_run(request, path, (hipStream_t)stream);
    if (result == NINETOOTHED_NO_KERNEL && path == kConvRepack) result = conv2d_run(request, kConvGather, (hipStream_t)stream);
    return result;
}

NineToothedResult nt_tune_conv2d(NineToothedStream stream, NineToothedTensor input, NineToothedTensor filter, NineToothedTensor output,
                                 int dtype, int padding_h, int padding_w, int iters, int *best_path, float *best_ms) {
    if (best_path) *best_path = -1;
    if (best_ms) *best_ms = 0.0f;
    Conv2dRequest request;
    const int status = conv2d_request(request, input, filter, output, dtype, padding_h, padding_w);
    if (status != 0) return status < 0 ? 0 : status;
    int values[11];
    conv2d_tune_values(request, values);
    const int paths[4] = {kConvPointwise, kConvDirect, kConvRepack, kConvGather};
    int best = -1;
    float best_time = 0.0f;
    // an earlier way stays unless a later one is more than 3 % faster: the first two need no scratch memory and one launch
    const int result = tune_time((hipStream_t)stream, 4, iters, [&](int i) -> int { return conv2d_run(request, paths[i], (hipStream_t)stream); }, &best, &best_time, 0.03f);
    if (result != 0) return result;
    if (best < 0) return 0;  // (a stream under graph capture: nothing was timed)
    tune_record(kTuneConv2d, values, 11, paths[best]);
    if (best_path) *best_path = paths[best];
    if (best_ms) *best_ms = best_time;
    return 0;
}

#ifdef NT_GEMM_ABLATION
void nt_debug_set_tile_order(int order) { g_tile_order = order; }
#endif

const char *nt_version(void) { return "nt_hip 0.1 gfx950"; }

}  // extern "C"
