// conv2d (stride 1, dilation 1, zero padding) as implicit GEMM on the direct-to-LDS
// MFMA main loop of gemm_fast.h.
//
//   GEMM row  m = (image, out_y, out_x)      M = N*P*Q
//   GEMM col  j = output channel             K_out
//   GEMM k    = (filter_y, filter_x, c)      R*S*C, channel fastest
//
// The MFMA operands need 8 consecutive k-values per lane, i.e. consecutive
// CHANNELS of one input position, while NCHW keeps channels H*W elements apart.
// A pre-pass on the launch stream therefore repacks both operands into scratch
// buffers the library keeps per stream between calls (workspace.h; the call stays
// asynchronous, and allocates only when a call needs more than any before it):
//   x[N,C,H,W]  -> xt[N,H,W,C]              (tiled transpose through LDS, 16-byte accesses)
//   w[K,C,R,S]  -> wt[(r*S+s)*C + c, K]     (row-major K x N operand of the GEMM)
// The main kernel then is the direct-to-LDS GEMM loop (256x256x32 tiles for wide layers,
// 256x128 and 128x64 for layers with fewer output channels): a K step is 32 channels of
// one filter tap (r, s); the A rows of a step are 64-byte runs of xt whose
// addresses differ from step to step by a uniform offset; taps that fall into
// the padding are fetched with an out-of-range buffer offset, which the
// hardware returns as zeros.  GEMM rows run over all images (a tile may span
// several small ones).  The epilogue writes NCHW: per output channel the
// GEMM rows of an image are contiguous, so the accumulators go through an LDS slab
// laid out [channel][row] and leave as 16-byte stores when P*Q is a multiple of 8
// (8 consecutive rows then lie in one image, aligned), element by element otherwise.
//
// Requirements of this path (anything else uses the any-stride gather kernel):
// fp16/bf16, K_out % 8 == 0, contiguous output.  The repacked operands hold C rounded up to a
// multiple of 32 channels, the extra ones zero (a 3-channel stem layer multiplies ten times the
// useful work and is still twice as fast as the gather kernel).
#include <algorithm>

#include "conv2d.h"
#include "gemm_fast.h"
#include "workspace.h"

namespace nt {
namespace {

struct ConvParams {
    const void *xt;
    const void *wt;
    void *y;
    int N, C, H, W, K, R, S, P, Q, pad_h, pad_w;
    int M, tiles_m, tiles_n;  // M = N*P*Q rows
    unsigned xt_bytes, wt_bytes;
};

// ---- pre-pass: one launch, two jobs ----
// grid layers z <  f.layers: w[K,C,R,S] (any strides) -> wt[(r*S+s)*C + c][K], grid-stride over these layers' threads
//                     (first, so that its scattered reads overlap the streaming layers behind it; as many
//                     layers as give the filter a few hundred workgroups, whatever the image size)
// grid layers z >= f.layers: x[z - f.layers] NCHW (any strides) -> xt NHWC contiguous (64 x 64 tiles through LDS)
struct FilterRepack {
    const void *w;
    void *wt;
    int K, C, R, S;
    int64_t s_k, s_c, s_r, s_s;
    int layers;
    int Cp;  // channels of the repacked operands: C rounded up to the k step, the extra ones zero
};

template <typename T>
__global__ __launch_bounds__(256) void conv2d_repack_kernel(const T *x, T *xt, int C, int HW, int W, int64_t s_n, int64_t s_c, int64_t s_h,
                                                           int64_t s_w, int vector_ok, FilterRepack f) {
    typedef typename Elem<T>::vec8 vec8;
    constexpr int kPitch = 64 + 8;  // halfs; keeps 16-byte alignment of rows
    __shared__ __attribute__((aligned(16))) T tile[64 * kPitch];
    const int t = threadIdx.x;
    if ((int)blockIdx.z < f.layers) {
        const T *w = (const T *)f.w;
        T *wt = (T *)f.wt;
        const int64_t total = (int64_t)f.K * f.Cp * f.R * f.S;
        const int64_t layer_threads = (int64_t)gridDim.x * gridDim.y * 256 * f.layers;
        for (int64_t index = (((int64_t)blockIdx.z * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x) * 256 + t; index < total; index += layer_threads) {
            const int k = (int)(index % f.K);
            const int64_t row = index / f.K;
            const int c = (int)(row % f.Cp);
            const int rs = (int)(row / f.Cp);
            wt[index] = c < f.C ? w[(int64_t)k * f.s_k + (int64_t)c * f.s_c + (int64_t)(rs / f.S) * f.s_r + (int64_t)(rs % f.S) * f.s_s] : (T)0.0f;
        }
        return;
    }
    const int hw0 = blockIdx.x * 64, c0 = blockIdx.y * 64, n = blockIdx.z - f.layers;
    const T *src = x + (int64_t)n * s_n;
    // load: rows = channels, 8 consecutive positions per thread
#pragma unroll
    for (int pass = 0; pass < 2; ++pass) {
        const int c = pass * 32 + (t >> 3);
        const int hw = hw0 + (t & 7) * 8;
        vec8 v;
        if (vector_ok && c0 + c < C && hw + 8 <= HW) {
            v = *(const vec8 *)(src + (int64_t)(c0 + c) * s_c + hw);
        } else {
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const int pos = hw + e;
                v[e] = (c0 + c < C && pos < HW) ? src[(int64_t)(c0 + c) * s_c + (int64_t)(pos / W) * s_h + (int64_t)(pos % W) * s_w] : (T)0.0f;
            }
        }
        *(vec8 *)&tile[c * kPitch + (t & 7) * 8] = v;
    }
    __syncthreads();
    // store: rows = positions, 8 consecutive channels per thread
#pragma unroll
    for (int pass = 0; pass < 2; ++pass) {
        const int hw = pass * 32 + (t >> 3);
        const int c = (t & 7) * 8;
        if (hw0 + hw < HW && c0 + c < f.Cp) {  // Cp % 8 == 0; channels from C on were loaded as zeros
            vec8 v;
#pragma unroll
            for (int e = 0; e < 8; ++e) v[e] = tile[(c + e) * kPitch + hw];
            *(vec8 *)(xt + ((int64_t)n * HW + hw0 + hw) * f.Cp + c0 + c) = v;
        }
    }
}

// ---- main kernel ----
template <typename T, int BM, int BN, int WM, int WN, int kStages, int kOcc>
__global__ __launch_bounds__(WM *WN * 64, kOcc) void conv2d_nhwc_kernel(ConvParams p) {
#if defined(__HIP_DEVICE_COMPILE__)
    typedef Elem<T> E;
    typedef typename E::vec8 vec8;
    constexpr int BK = 32;
    constexpr int kWaves = WM * WN;
    constexpr int kWaveM = BM / WM, kWaveN = BN / WN;
    constexpr int TM = kWaveM / 32, TN = kWaveN / 32;
    constexpr int kStageA = BM * BK * 2, kStageB = BK * BN * 2;
    constexpr int kAChunksPerRow = BK / 8, kARowsPerInstr = 64 / kAChunksPerRow;
    constexpr int kAInstr = kStageA / (kWaves * 1024);
    constexpr int kBChunksPerRow = BN / 8, kBRowsPerInstr = 64 / kBChunksPerRow;
    constexpr int kBInstr = kStageB / (kWaves * 1024);
    constexpr int kLoadsPerTile = kAInstr + kBInstr;
    static_assert(kStageA % (kWaves * 1024) == 0 && kStageB % (kWaves * 1024) == 0, "every wave issues whole load instructions");
    static_assert(kWaveM % 32 == 0 && kWaveN % 32 == 0, "wave tile");
    static_assert(kStages >= 3 && kStages <= 4 && kStages >= WN, "stages (the epilogue slabs of all waves live in the A stages)");

    __shared__ __attribute__((aligned(1024))) unsigned char lds_a0[kStageA];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_a1[kStageA];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_a2[kStageA];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_a3[kStages > 3 ? kStageA : 16];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_b0[kStageB];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_b1[kStageB];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_b2[kStageB];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_b3[kStages > 3 ? kStageB : 16];
    auto stage_a = [&](auto tag) -> NT_LDS unsigned char * {
        constexpr int i = decltype(tag)::value;
        if constexpr (i == 0) return (NT_LDS unsigned char *)lds_a0;
        else if constexpr (i == 1) return (NT_LDS unsigned char *)lds_a1;
        else if constexpr (i == 2) return (NT_LDS unsigned char *)lds_a2;
        else return (NT_LDS unsigned char *)lds_a3;
    };
    auto stage_b = [&](auto tag) -> NT_LDS unsigned char * {
        constexpr int i = decltype(tag)::value;
        if constexpr (i == 0) return (NT_LDS unsigned char *)lds_b0;
        else if constexpr (i == 1) return (NT_LDS unsigned char *)lds_b1;
        else if constexpr (i == 2) return (NT_LDS unsigned char *)lds_b2;
        else return (NT_LDS unsigned char *)lds_b3;
    };

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wave_m = wave / WN, wave_n = wave % WN;

    int tile_m, tile_n;
    map_tile(p.tiles_m, p.tiles_n, 0, tile_m, tile_n);
    const int m0 = tile_m * BM;
    const int n0 = tile_n * BN;
    const int PQ = p.P * p.Q;

    // ---- A: rows of the tile are output positions; per lane one 16-byte chunk of 8 channels ----
    __amdgpu_buffer_rsrc_t a_rsrc = __builtin_amdgcn_make_buffer_rsrc((void *)p.xt, 0, p.xt_bytes, 0x00020000);
    // the filter descriptor ends with the matrix: a partial last tile of output channels reads the next
    // row's values (they only feed channels that are not stored) and, in the last row, zeros
    __amdgpu_buffer_rsrc_t b_rsrc = __builtin_amdgcn_make_buffer_rsrc((void *)((const T *)p.wt + n0), 0, p.wt_bytes - (unsigned)n0 * 2u, 0x00020000);
    int a_base[kAInstr], a_y[kAInstr], a_x[kAInstr];
#pragma unroll
    for (int j = 0; j < kAInstr; ++j) {
        const int row = (j * kWaves + wave) * kARowsPerInstr + lane / kAChunksPerRow;
        const int chunk = a_phys_chunk<BK>(row, lane % kAChunksPerRow);
        const int m = m0 + row;
        const int image = m / PQ, pq = m - image * PQ;
        const int oy = pq / p.Q, ox = pq - oy * p.Q;
        a_y[j] = m < p.M ? oy - p.pad_h : -(1 << 20);  // rows past the last image never pass the bounds test
        a_x[j] = ox - p.pad_w;
        a_base[j] = m < p.M ? (((image * p.H + a_y[j]) * p.W + a_x[j]) * p.C + chunk * 8) * 2 : 0;
    }
    unsigned b_src[kBInstr];
#pragma unroll
    for (int j = 0; j < kBInstr; ++j) {
        const int krow = (j * kWaves + wave) * kBRowsPerInstr + lane / kBChunksPerRow;
        const int chunk = b_phys_chunk<BN>(krow, lane % kBChunksPerRow);
        b_src[j] = (unsigned)(krow * p.K + chunk * 8) * 2u;
    }
    auto issue_loads = [&](auto stage_tag, int kt) {
        NT_LDS unsigned char *sa = stage_a(stage_tag);
        NT_LDS unsigned char *sb = stage_b(stage_tag);
        // k order: channel block outer, filter taps inner -- the R*S taps of a block of 32 channels read the
        // same pixels shifted by a row or a column, so they hit in L2 while the lines are still there
        const int taps = p.R * p.S;
        const int cb = kt / taps;
        const int tap = kt - cb * taps;
        const int c0 = cb * BK;
        const int fy = tap / p.S, fx = tap - fy * p.S;
        const int delta = ((fy * p.W + fx) * p.C + c0) * 2;
#pragma unroll
        for (int j = 0; j < kAInstr; ++j) {
            const bool inside = (unsigned)(a_y[j] + fy) < (unsigned)p.H && (unsigned)(a_x[j] + fx) < (unsigned)p.W;
            const unsigned offset = inside ? (unsigned)(a_base[j] + delta) : 0x80000000u;  // beyond num_records: reads zeros
            __builtin_amdgcn_raw_ptr_buffer_load_lds(a_rsrc, sa + (j * kWaves + wave) * 1024, 16, offset, 0, 0, 0);
        }
        const int b_k = (tap * p.C + c0) * p.K * 2;
#pragma unroll
        for (int j = 0; j < kBInstr; ++j)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(b_rsrc, sb + (j * kWaves + wave) * 1024, 16, b_src[j], b_k, 0, 0);
    };

    // ---- LDS -> registers (as in gemm_fast.h) ----
    const int g = lane >> 5, l32 = lane & 31;
    int a_row_off[TM], a_row_sw[TM];
#pragma unroll
    for (int ti = 0; ti < TM; ++ti) {
        const int row = wave_m * kWaveM + ti * 32 + l32;
        a_row_off[ti] = row * (BK * 2);
        a_row_sw[ti] = a_phys_chunk<BK>(row, 0);
    }
    const int i16 = lane & 15, nhalf = (lane >> 4) & 1;
    const int b_krow = 8 * g + (i16 >> 2);
    int b_col_chunk[TN], b_col_in[TN];
#pragma unroll
    for (int tj = 0; tj < TN; ++tj) {
        const int ncol = wave_n * kWaveN + tj * 32 + nhalf * 16 + 4 * (i16 & 3);
        b_col_chunk[tj] = ncol >> 3;
        b_col_in[tj] = (ncol & 7) * 2;
    }

    float16_t acc[TM][TN];
#pragma unroll
    for (int ti = 0; ti < TM; ++ti)
#pragma unroll
        for (int tj = 0; tj < TN; ++tj)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[ti][tj][r] = 0.0f;

    auto multiply_stage = [&](auto stage_tag) {
        const NT_LDS unsigned char *sa = stage_a(stage_tag);
        const NT_LDS unsigned char *sb = stage_b(stage_tag);
#pragma unroll
        for (int ks = 0; ks < BK / 16; ++ks) {
            vec8 af[TM], bf[TN];
#pragma unroll
            for (int ti = 0; ti < TM; ++ti) {
                const int chunk = (ks * 2 + g) ^ a_row_sw[ti];
                af[ti] = *(const NT_LDS vec8 *)(sa + a_row_off[ti] + chunk * 16);
            }
#pragma unroll
            for (int tj = 0; tj < TN; ++tj) {
                const int k_lo = ks * 16 + b_krow, k_hi = k_lo + 4;
                const int c_lo = b_phys_chunk<BN>(k_lo, b_col_chunk[tj]);
                const int c_hi = b_phys_chunk<BN>(k_hi, b_col_chunk[tj]);
                short4_t lo = lds_read_tr16_b64(sb + k_lo * (BN * 2) + c_lo * 16 + b_col_in[tj]);
                short4_t hi = lds_read_tr16_b64(sb + k_hi * (BN * 2) + c_hi * 16 + b_col_in[tj]);
                short8_t both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                bf[tj] = __builtin_bit_cast(vec8, both);
            }
#pragma unroll
            for (int ti = 0; ti < TM; ++ti)
#pragma unroll
                for (int tj = 0; tj < TN; ++tj) acc[ti][tj] = E::mfma32(af[ti], bf[tj], acc[ti][tj]);
        }
    };

    const int num_k = p.R * p.S * (p.C / BK);
    const int last_k = num_k - 1;
    const int main_k = num_k - num_k % kStages;
    static_for<0, kStages - 1>([&](auto s) { issue_loads(s, min((int)decltype(s)::value, last_k)); });
    auto step = [&](auto s, int kt) {
        constexpr int kS = decltype(s)::value;
        wait_vmcnt<(kStages - 2) * kLoadsPerTile>();
        lds_barrier();
        issue_loads(std::integral_constant<int, (kS + kStages - 1) % kStages>(), min(kt + kS + kStages - 1, last_k));
        multiply_stage(s);
    };
    for (int kt = 0; kt < main_k; kt += kStages) static_for<0, kStages>([&](auto s) { step(s, kt); });
    static_for<0, kStages - 1>([&](auto s) {
        if (main_k + (int)decltype(s)::value < num_k) step(s, main_k);
    });
    wait_vmcnt<0>();
    lds_barrier();

    // ---- epilogue: lane holds, per 32x32 tile, output channel l32 and rows 8*(r/4) + 4*g + r%4 ----
    // slab layout [32 channels][kWaveM rows], 16-byte chunks swizzled by channel; an A stage holds WM slabs
    constexpr int kRowBytes = kWaveM * 2;
    constexpr int kSlabBytes = 32 * kRowBytes;
    constexpr int kChunks = kWaveM / 8;
    static_assert(kStageA == WM * kSlabBytes, "slabs per A stage");
    NT_LDS unsigned char *slab;
    {
        const int which = wave / WM;
        slab = which == 0 ? (NT_LDS unsigned char *)lds_a0
               : which == 1 ? (NT_LDS unsigned char *)lds_a1
               : which == 2 ? (NT_LDS unsigned char *)lds_a2
                            : (NT_LDS unsigned char *)lds_a3;
        slab += (wave % WM) * kSlabBytes;
    }
    T *Y = (T *)p.y;
    const bool whole_chunks = PQ % 8 == 0;
#pragma unroll
    for (int tj = 0; tj < TN; ++tj) {
#pragma unroll
        for (int ti = 0; ti < TM; ++ti)
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                typedef T vec4 __attribute__((ext_vector_type(4)));
                vec4 v;
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = E::from_float(acc[ti][tj][4 * r4 + e]);
                const int chunk = (ti * 4 + r4) ^ (l32 & (kChunks - 1));
                *(NT_LDS vec4 *)(slab + l32 * kRowBytes + chunk * 16 + 8 * g) = v;
            }
#pragma unroll
        for (int it = 0; it < (32 * kChunks) / 64; ++it) {
            const int idx = it * 64 + lane;
            const int channel = idx / kChunks;
            const int phys = idx % kChunks;
            const int chunk = phys ^ (channel & (kChunks - 1));
            vec8 v = *(const NT_LDS vec8 *)(slab + channel * kRowBytes + phys * 16);
            const int m = m0 + wave_m * kWaveM + chunk * 8;
            if (m >= p.M) continue;
            const int out_channel = n0 + wave_n * kWaveN + tj * 32 + channel;
            if (out_channel >= p.K) continue;  // a partial last tile of output channels
            int image = m / PQ, pq = m - image * PQ;
            if (whole_chunks) {  // the 8 rows lie in one image and start at a multiple of 8
                __builtin_nontemporal_store(v, (vec8 *)(Y + ((int64_t)image * p.K + out_channel) * PQ + pq));  // +2 % over a plain store
            } else {
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    if (m + e < p.M) Y[((int64_t)image * p.K + out_channel) * PQ + pq] = v[e];
                    if (++pq == PQ) {
                        pq = 0;
                        ++image;
                    }
                }
            }
        }
    }
#endif
}

template <typename T>
int run_fast(const Conv2dRequest &q, hipStream_t stream) {
    const int Cp = ceil_div(q.C, 32) * 32;
    const int64_t xt_bytes = (int64_t)q.N * q.H * q.W * Cp * 2;
    const int64_t wt_bytes = (int64_t)q.K * Cp * q.R * q.S * 2;
    WorkspaceLease lease(stream);
    void *xt = lease.get(kWorkspaceConvInput, (size_t)xt_bytes);
    void *wt = lease.get(kWorkspaceConvFilter, (size_t)wt_bytes);
    if (xt == nullptr || wt == nullptr) return NINETOOTHED_NO_KERNEL;  // no scratch: the caller falls back to the gather kernel
    const int HW = q.H * q.W;
    const int vector_ok = q.xs[3] == 1 && q.xs[2] == q.W && HW % 8 == 0 && q.xs[1] % 8 == 0 && q.xs[0] % 8 == 0 && ((uintptr_t)q.x & 15) == 0;
    FilterRepack f;
    f.w = q.w;
    f.wt = wt;
    f.K = q.K; f.C = q.C; f.R = q.R; f.S = q.S; f.Cp = Cp;
    f.s_k = q.ws[0]; f.s_c = q.ws[1]; f.s_r = q.ws[2]; f.s_s = q.ws[3];
    // about 512 workgroups for the filter, or one thread per element if that is less
    const int64_t per_layer = (int64_t)ceil_div(HW, 64) * ceil_div(Cp, 64);
    const int64_t wanted = std::min<int64_t>(512, ((int64_t)q.K * Cp * q.R * q.S + 255) / 256);
    f.layers = (int)std::max<int64_t>(1, std::min<int64_t>(ceil_div(wanted, per_layer), 512));
    conv2d_repack_kernel<T><<<dim3(ceil_div(HW, 64), ceil_div(Cp, 64), q.N + f.layers), dim3(256), 0, stream>>>(
        (const T *)q.x, (T *)xt, q.C, HW, q.W, q.xs[0], q.xs[1], q.xs[2], q.xs[3], vector_ok, f);
    ConvParams p;
    p.xt = xt;
    p.wt = wt;
    p.y = q.y;
    p.N = q.N; p.C = Cp; p.H = q.H; p.W = q.W; p.K = q.K; p.R = q.R; p.S = q.S; p.P = q.P; p.Q = q.Q;
    p.pad_h = q.pad_h; p.pad_w = q.pad_w;
    p.M = q.N * q.P * q.Q;
    p.xt_bytes = (unsigned)xt_bytes;
    p.wt_bytes = (unsigned)wt_bytes;
    // tile by the number of output channels: 256 wide when they fill it and there are enough tiles for the
    // chip, else 128 (two workgroups per CU), else 128 x 64 tiles of four waves
    const auto launch = [&](auto kernel, int bm, int bn, int threads) {
        p.tiles_m = ceil_div(p.M, bm);
        p.tiles_n = ceil_div(q.K, bn);
        kernel<<<dim3(p.tiles_m * p.tiles_n), dim3(threads), 0, stream>>>(p);
    };
    // the widest tile that is at least 4/5 full of output channels and leaves enough tiles for the chip
    const auto fits = [&](int bm, int bn) {
        const int64_t tiles = (int64_t)ceil_div(p.M, bm) * ceil_div(q.K, bn);
        return q.K * 5 >= ceil_div(q.K, bn) * bn * 4 && tiles >= 192;
    };
    if (fits(256, 256)) launch(conv2d_nhwc_kernel<T, 256, 256, 2, 4, 4, 2>, 256, 256, 512);
    else if (fits(256, 128)) launch(conv2d_nhwc_kernel<T, 256, 128, 4, 2, 3, 4>, 256, 128, 512);
    else launch(conv2d_nhwc_kernel<T, 128, 64, 2, 2, 4, 3>, 128, 64, 256);
    return (int)hipGetLastError();
}

}  // namespace

int conv2d_fast(const Conv2dRequest &q, hipStream_t stream) {
    if (q.dtype != NINETOOTHED_FLOAT16 && q.dtype != NINETOOTHED_BFLOAT16) return NINETOOTHED_NO_KERNEL;
    // channels are padded to the k step of 32 with zeros; below a sixteenth of useful work the gather kernel is as good
    if (q.K % 8 || q.C < 2) return NINETOOTHED_NO_KERNEL;  // (rows of the repacked filter are read in 16-byte pieces)
    if (q.ys[3] != 1 || q.ys[2] != q.Q || q.ys[1] != (int64_t)q.P * q.Q || q.ys[0] != (int64_t)q.K * q.P * q.Q) return NINETOOTHED_NO_KERNEL;
    if (((uintptr_t)q.y & 15) != 0) return NINETOOTHED_NO_KERNEL;
    const int64_t xt_bytes = (int64_t)q.N * q.H * q.W * ceil_div(q.C, 32) * 32 * 2;
    const int64_t wt_bytes = (int64_t)q.K * ceil_div(q.C, 32) * 32 * q.R * q.S * 2;
    if (xt_bytes >= (int64_t(1) << 31) || wt_bytes >= (int64_t(1) << 31)) return NINETOOTHED_NO_KERNEL;  // 32-bit buffer offsets
    if ((int64_t)q.N * q.P * q.Q > 0x7fffffffll || (int64_t)ceil_div(q.N * q.P * q.Q, 128) * ceil_div(q.K, 64) > 0x7fffffffll) return NINETOOTHED_NO_KERNEL;
    if (q.N >= 65535 - 512 || ceil_div(q.C, 64) > 65535) return NINETOOTHED_NO_KERNEL;  // grid of the repacking pass: (positions, channels, filter layers + images)
    // enough work to amortise the repacking pass
    if ((int64_t)q.N * q.P * q.Q < 1024) return NINETOOTHED_NO_KERNEL;
    return q.dtype == NINETOOTHED_FLOAT16 ? run_fast<half_t>(q, stream) : run_fast<bf16_t>(q, stream);
}

}  // namespace nt
