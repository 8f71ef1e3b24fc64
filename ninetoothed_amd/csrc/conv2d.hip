// conv2d (stride 1, dilation 1, zero padding) as implicit GEMM on the MFMA main loop of gemm_fast.h.  Two paths:
//
// (1) conv2d_direct: one launch on the tensors as they lie, no scratch memory (described with its kernel
//     below); needs an output width that is a multiple of 8, padding_w <= 1, C*R*S a multiple of 32, a contiguous
//     filter and output, and output channels that fill 256-wide tiles.
//
// (2) conv2d_fast: a repacking pre-pass plus the GEMM loop, for the shapes (1) does not take.
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
// Requirements of path (2) (anything else uses the any-stride gather kernel):
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
    int Kp;                   // row pitch of the repacked filter: K rounded up to 8 (its rows are read in 16-byte pieces)
    int dense_out;            // 1: the output is a contiguous NCHW tensor on a 16-byte boundary; 2: its channels are its
                              // innermost dimension (channels last); 0: any strides, stored element by element
    int64_t ys[4];            // element strides of the output
    int M, tiles_m, tiles_n;  // M = N*P*Q rows
    unsigned xt_bytes, wt_bytes;
    int stride_h, stride_w, dil_h, dil_w;  // steps of the window over the input and between its taps
};

// ---- pre-pass: one launch, two jobs ----
// grid layers z <  f.layers: w[K,C,R,S] (any strides) -> wt[(r*S+s)*C + c][K], grid-stride over these layers' threads
//                     (first, so that its scattered reads overlap the streaming layers behind it; as many
//                     layers as give the filter a few hundred workgroups, whatever the image size)
// grid layers z >= f.layers: x[z - f.layers] NCHW (any strides) -> xt NHWC contiguous (64 x 64 tiles through LDS;
//                     vector_ok 1: 16-byte loads along the positions; 2 and 3: the channels are innermost in x
//                     already and rows of them are copied, 3 with 16-byte loads)
struct FilterRepack {
    const void *w;
    void *wt;
    int K, C, R, S;
    int64_t s_k, s_c, s_r, s_s;
    int layers;
    int Cp;  // channels of the repacked operands: C rounded up to the k step, the extra ones zero
    int Kp;  // row pitch of the repacked filter: K rounded up to 8, the extra columns zero
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
        const int64_t total = (int64_t)f.Kp * f.Cp * f.R * f.S;
        const int64_t layer_threads = (int64_t)gridDim.x * gridDim.y * 256 * f.layers;
        for (int64_t index = (((int64_t)blockIdx.z * gridDim.y + blockIdx.y) * gridDim.x + blockIdx.x) * 256 + t; index < total; index += layer_threads) {
            const int k = (int)(index % f.Kp);
            const int64_t row = index / f.Kp;
            const int c = (int)(row % f.Cp);
            const int rs = (int)(row / f.Cp);
            wt[index] = c < f.C && k < f.K ? w[(int64_t)k * f.s_k + (int64_t)c * f.s_c + (int64_t)(rs / f.S) * f.s_r + (int64_t)(rs % f.S) * f.s_s] : (T)0.0f;
        }
        return;
    }
    const int hw0 = blockIdx.x * 64, c0 = blockIdx.y * 64, n = blockIdx.z - f.layers;
    const T *src = x + (int64_t)n * s_n;
    if (vector_ok >= 2) {
        // the channels are the innermost dimension already (a channels-last tensor): rows of 8 channels are
        // copied as they lie, padded to Cp with zeros
#pragma unroll
        for (int pass = 0; pass < 2; ++pass) {
            const int hw = hw0 + pass * 32 + (t >> 3);
            const int c = c0 + (t & 7) * 8;
            if (hw < HW && c < f.Cp) {
                const T *from = src + (int64_t)(hw / W) * s_h + (int64_t)(hw % W) * s_w + c;
                vec8 v;
                if (vector_ok == 3 && c + 8 <= C) {
                    v = *(const vec8 *)from;
                } else {
#pragma unroll
                    for (int e = 0; e < 8; ++e) v[e] = c + e < C ? from[e] : (T)0.0f;
                }
                *(vec8 *)(xt + ((int64_t)n * HW + hw) * f.Cp + c) = v;
            }
        }
        return;
    }
    // load: rows = channels, 8 consecutive positions per thread
#pragma unroll
    for (int pass = 0; pass < 2; ++pass) {
        const int c = pass * 32 + (t >> 3);
        const int hw = hw0 + (t & 7) * 8;
        vec8 v;
        if (vector_ok && c0 + c < C && hw + 8 <= HW) {
            // (the positions of a channel are contiguous; where they start does not matter: global accesses need the element's alignment only)
            typedef vec8 unaligned_vec8 __attribute__((aligned(2)));
            v = *(const unaligned_vec8 *)(src + (int64_t)(c0 + c) * s_c + hw);
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
    // Few input channels (p.C = 8 or 16 after padding): a k step of 32 contraction positions then holds 4 or 2
    // filter taps, and which tap a lane fetches follows from its chunk of the step.
    const bool narrow = p.C < BK;
    const int chunks_per_tap = narrow ? p.C / 8 : kAChunksPerRow;
    int a_base[kAInstr], a_y[kAInstr], a_x[kAInstr], a_tap[kAInstr];
#pragma unroll
    for (int j = 0; j < kAInstr; ++j) {
        const int row = (j * kWaves + wave) * kARowsPerInstr + lane / kAChunksPerRow;
        const int chunk = a_phys_chunk<BK>(row, lane % kAChunksPerRow);
        const int m = m0 + row;
        const int image = m / PQ, pq = m - image * PQ;
        const int oy = pq / p.Q, ox = pq - oy * p.Q;
        a_y[j] = m < p.M ? oy * p.stride_h - p.pad_h : -(1 << 20);  // rows past the last image never pass the bounds test
        a_x[j] = ox * p.stride_w - p.pad_w;
        a_tap[j] = chunk / chunks_per_tap;  // (narrow) the lane's tap within a k step
        a_base[j] = m < p.M ? (((image * p.H + a_y[j]) * p.W + a_x[j]) * p.C + (chunk % chunks_per_tap) * 8) * 2 : 0;
    }
    unsigned b_src[kBInstr];
#pragma unroll
    for (int j = 0; j < kBInstr; ++j) {
        const int krow = (j * kWaves + wave) * kBRowsPerInstr + lane / kBChunksPerRow;
        const int chunk = b_phys_chunk<BN>(krow, lane % kBChunksPerRow);
        b_src[j] = (unsigned)(krow * p.Kp + chunk * 8) * 2u;
    }
    auto issue_loads = [&](auto stage_tag, int kt) {
        NT_LDS unsigned char *sa = stage_a(stage_tag);
        NT_LDS unsigned char *sb = stage_b(stage_tag);
        // k order: channel block outer, filter taps inner -- the R*S taps of a block of 32 channels read the
        // same pixels shifted by a row or a column, so they hit in L2 while the lines are still there
        const int taps = p.R * p.S;
        if (narrow) {  // (uniform) rows of the repacked filter are (tap, channel) pairs in this order: k step kt is rows 32 kt ...
            const int taps_per_step = BK / p.C;
#pragma unroll
            for (int j = 0; j < kAInstr; ++j) {
                const int tap = kt * taps_per_step + a_tap[j];
                const int fy = (tap / p.S) * p.dil_h, fx = (tap % p.S) * p.dil_w;
                const bool inside = tap < taps && (unsigned)(a_y[j] + fy) < (unsigned)p.H && (unsigned)(a_x[j] + fx) < (unsigned)p.W;
                const unsigned offset = inside ? (unsigned)(a_base[j] + (fy * p.W + fx) * p.C * 2) : 0x80000000u;
                __builtin_amdgcn_raw_ptr_buffer_load_lds(a_rsrc, sa + (j * kWaves + wave) * 1024, 16, offset, 0, 0, 0);
            }
            const int b_k = kt * BK * p.Kp * 2;  // (rows past the last tap lie behind the descriptor: zeros)
#pragma unroll
            for (int j = 0; j < kBInstr; ++j)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(b_rsrc, sb + (j * kWaves + wave) * 1024, 16, b_src[j], b_k, 0, 0);
            return;
        }
        const int cb = kt / taps;
        const int tap = kt - cb * taps;
        const int c0 = cb * BK;
        const int fy = (tap / p.S) * p.dil_h, fx = (tap % p.S) * p.dil_w;  // the tap's distance from the window's corner
        const int delta = ((fy * p.W + fx) * p.C + c0) * 2;
#pragma unroll
        for (int j = 0; j < kAInstr; ++j) {
            const bool inside = (unsigned)(a_y[j] + fy) < (unsigned)p.H && (unsigned)(a_x[j] + fx) < (unsigned)p.W;
            const unsigned offset = inside ? (unsigned)(a_base[j] + delta) : 0x80000000u;  // beyond num_records: reads zeros
            __builtin_amdgcn_raw_ptr_buffer_load_lds(a_rsrc, sa + (j * kWaves + wave) * 1024, 16, offset, 0, 0, 0);
        }
        const int b_k = (tap * p.C + c0) * p.Kp * 2;
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

    const int num_k = (p.R * p.S * p.C + BK - 1) / BK;
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
    const bool whole_chunks = PQ % 8 == 0 && p.dense_out == 1;
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
        if (p.dense_out == 2) {
            // channels-last output: a lane gathers 8 channels of one row from the slab and stores them with one
            // instruction (the 32 channels of the slab are 64 consecutive bytes of the tensor)
#pragma unroll
            for (int it = 0; it < (32 * kChunks) / 64; ++it) {
                const int idx = it * 64 + lane;
                const int row = idx >> 2, first = (idx & 3) * 8;
                vec8 v;
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    const int channel = first + e;
                    v[e] = *(const NT_LDS T *)(slab + channel * kRowBytes + (((row >> 3) ^ (channel & (kChunks - 1))) * 16) + (row & 7) * 2);
                }
                const int m = m0 + wave_m * kWaveM + row;
                const int out_channel = n0 + wave_n * kWaveN + tj * 32 + first;
                if (m >= p.M || out_channel >= p.K) continue;
                const int image = m / PQ, pq = m - image * PQ;
                const int oy = pq / p.Q, ox = pq - oy * p.Q;
                T *to = Y + (int64_t)image * p.ys[0] + (int64_t)oy * p.ys[2] + (int64_t)ox * p.ys[3] + out_channel;
                if (out_channel + 8 <= p.K) {
                    typedef vec8 unaligned_vec8 __attribute__((aligned(2)));
                    *(unaligned_vec8 *)to = v;
                } else {
#pragma unroll
                    for (int e = 0; e < 8; ++e)
                        if (out_channel + e < p.K) to[e] = v[e];
                }
            }
            continue;
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
            } else if (p.dense_out == 1 && pq + 8 <= PQ && m + 8 <= p.M) {
                // the 8 rows lie in one image, only not on a 16-byte boundary (a 7 x 7 map): one store all the same
                // (global accesses need the element's alignment only)
                typedef vec8 unaligned_vec8 __attribute__((aligned(2)));
                *(unaligned_vec8 *)(Y + ((int64_t)image * p.K + out_channel) * PQ + pq) = v;
            } else {
                // (any output strides: a channels-last tensor, a slice of a wider one)
                int oy = pq / p.Q, ox = pq - oy * p.Q;
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    if (m + e < p.M) Y[(int64_t)image * p.ys[0] + (int64_t)out_channel * p.ys[1] + (int64_t)oy * p.ys[2] + (int64_t)ox * p.ys[3]] = v[e];
                    if (++ox == p.Q) {
                        ox = 0;
                        if (++oy == p.P) {
                            oy = 0;
                            ++image;
                        }
                    }
                }
            }
        }
    }
#endif
}

// ---- one launch, no scratch: the convolution on the tensors as they lie ----
//
// For NCHW the natural orientation of the product is  Y[k_out, pixel] = W[k_out, (c, r, s)] . X_col[(c, r, s), pixel]
// per image: the filter tensor IS the row-major left operand (its rows are contiguous in (c, r, s)), the output
// tensor IS the row-major result per image (pixels contiguous per output channel), and the right operand has
// pixels contiguous, which is how NCHW stores them.  The filter tiles take the direct-to-LDS route of the GEMM
// (rows of 32 contraction values, read back with ds_read_b128); a row of the right operand's tile is one
// (channel, filter tap): 256 pixels of one channel shifted by the tap, fetched in 16-byte pieces of 8 pixels
// -- through registers, because a tap that moves by one pixel leaves the pieces 2-byte aligned, which loads
// into registers accept and loads into LDS do not -- and written to a [32][256] LDS tile that the transposing
// ds_read_b64_tr_b16 turns into MFMA operands.  Pieces whose image row lies in the padding are fetched from
// behind the buffer (zeros); pixels of a piece that fall into the left / right padding are cleared in registers.
// Needs Q % 8 == 0 (a piece stays inside one image row), C*R*S % 32 == 0, contiguous filter and output, and a
// filter whose taps repeat within 25 tiles of the contraction (R*S / gcd(32, R*S) <= 25: 1x1 ... 5x5).
//
// Tiles are 256 output channels x 256 pixels.  (Measured and dropped: cutting the pixels that are left after the
// last full round of workgroups -- 392 tiles on 256 CUs -- into one round of narrower tiles, with the two waves
// of a SIMD sharing a tile's pixels so that the round takes the fraction of a full one that its MFMAs are.  A
// step of a narrow tile lasts as long as a full one: what the ring of loads has in flight does not cover the
// memory latency once the MFMAs between two barriers shrink.)
struct ConvDirectParams {
    const void *x, *w;
    void *y;
    int C, H, W, K, R, S, P, Q, pad_h, pad_w;
    int64_t xs0, xs1, xs2;  // element strides of the input's image, channel and row (pixels of a row are contiguous)
    int M;                  // pixels of all images
    int CRS;                // contraction length
    int tiles_ch;           // tiles along the output channels
    unsigned x_bytes, w_bytes;
    int period;             // tiles after which the filter taps of a tile's 32 rows repeat: R*S / gcd(32, R*S)
    int period_bytes;       // ... and by how many bytes the rows' channels have moved on by then
#ifdef NT_CONV_STAMPS
    unsigned long long *stamps;  // measurement builds: per wave {loop, waiting for loads, waiting for own LDS traffic, waiting at the barrier}
#endif
};

#ifdef NT_CONV_STAMPS
unsigned long long *g_conv_stamps = nullptr;
#endif

// rows of the table of filter taps kept in LDS: at most this many tiles per period (5 x 5 filters: 25)
constexpr int kConvDirectMaxPeriod = 25;

// Measurement builds only (wrong results): bit 0 = no pixel loads inside the loop, bit 1 = no pixel stores into
// LDS, bit 2 = no filter fills, bit 3 = no MFMAs, bit 4 = no fragment reads.  0 in the library.
#ifndef NT_CONV_ABLATE
#define NT_CONV_ABLATE 0
#endif

// kM16: the tile is computed with 16x16x32 MFMAs (per FLOP half as many accumulator values pass through the
// register file as with 32x32x16 ones, which is what the part's power limit charges for): per wave 4 blocks of
// 16 channels, whose fragments stay in registers for a k tile (two sets taking turns), times 8 blocks of 16
// pixels, whose fragments stream through four slots, each read two blocks ahead of its MFMAs.
template <typename T, bool kM16>
__global__ __launch_bounds__(512, 2) void conv2d_direct_kernel(ConvDirectParams p) {
#if defined(__HIP_DEVICE_COMPILE__)
    typedef Elem<T> E;
    typedef typename E::vec8 vec8;
    constexpr int BM = 256, BN = 256, BK = 32, kStages = 4;  // BM: output channels, BN: pixels
    constexpr int WM = 4, WN = 2, kWaves = 8;
    constexpr int kWaveM = BM / WM, kWaveN = BN / WN;          // 64 channels x 128 pixels per wave
    constexpr int TM = kWaveM / 32, TN = kWaveN / 32;
    // pixel tile [32 rows][256 pixels]: rows 64 bytes longer than their pixels, so that the 8 rows a transposing
    // read touches start in different banks and every address is affine in (row, pixel): fragments and k steps
    // are immediate offsets of one address register
    constexpr int kPitchB = BN * 2 + 64;
    constexpr int kStageA = BM * BK * 2, kStageB = BK * kPitchB;
    constexpr int kAChunksPerRow = BK / 8, kARowsPerInstr = 64 / kAChunksPerRow;
    constexpr int kAInstr = kStageA / (kWaves * 1024);
    constexpr int KS = BK / 16;
    static_assert(kAInstr == 2, "thread assignment below");

    __shared__ __attribute__((aligned(1024))) unsigned char lds_a0[kStageA];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_a1[kStageA];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_a2[kStageA];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_a3[kStageA];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_b0[kStageB];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_b1[kStageB];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_b2[kStageB];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_b3[kStageB];
    // what the 32 rows of a pixel tile are, for every tile of a period: {byte offset of the row's (channel, tap)
    // relative to the period's first channel, 31 - filter row, border mask, unused}
    typedef unsigned uint4_t __attribute__((ext_vector_type(4)));
    __shared__ __attribute__((aligned(16))) uint4_t lds_taps[kConvDirectMaxPeriod * BK];
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

#ifdef NT_CONV_STAMPS
    const unsigned long long real_entry = __builtin_amdgcn_s_memrealtime();
#endif
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wave_m = wave % WM, wave_n = wave / WM;

    // ---- which tile ----
    // The first and the last tile of pixels run the careful form of the loop, which is slower: both are dealt out first
    // (workgroup ids 0 and 1 per tile of channels), so that a launch does not end with one of them.
    const int tile_ch = blockIdx.x % p.tiles_ch;
    const int pixel_tiles = (p.M + BN - 1) / BN;
    int pixel_tile = blockIdx.x / p.tiles_ch;
    if (pixel_tiles >= 3 && pixel_tile >= 1) pixel_tile = pixel_tile == 1 ? pixel_tiles - 1 : pixel_tile - 1;
    const int n0 = pixel_tile * BN;
    const int tile_pixels = min(BN, p.M - n0);  // > 0 by construction of the grid
    const int m0 = tile_ch * BM;
    const int PQ = p.P * p.Q;
    const int RS = p.R * p.S;

    // ---- filter tile: rows of 32 contraction values, direct to LDS ----
    const int64_t w_rows = min((int64_t)BM, (int64_t)p.K - m0);
    const unsigned char *w_base = (const unsigned char *)((const T *)p.w + (int64_t)m0 * p.CRS);
    __amdgpu_buffer_rsrc_t w_rsrc = __builtin_amdgcn_make_buffer_rsrc((void *)w_base, 0, (unsigned)(w_rows * p.CRS * 2), 0x00020000);
    unsigned a_src[kAInstr];
#pragma unroll
    for (int j = 0; j < kAInstr; ++j) {
        const int row = (j * kWaves + wave) * kARowsPerInstr + lane / kAChunksPerRow;
        const int chunk = kM16 ? a_phys_chunk16<BK>(row, lane % kAChunksPerRow) : a_phys_chunk<BK>(row, lane % kAChunksPerRow);
        a_src[j] = (unsigned)(row * p.CRS + chunk * 8) * 2u;
    }
    auto issue_filter = [&](auto stage_tag, int kt) {
        NT_LDS unsigned char *sa = stage_a(stage_tag);
#pragma unroll
        for (int j = 0; j < kAInstr; ++j)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(w_rsrc, sa + (j * kWaves + wave) * 1024, 16, a_src[j], kt * BK * 2, 0, 0);
    };

    // ---- pixel tile: a thread fetches one 16-byte piece (8 pixels) of two rows, 16 contraction positions apart ----
    // A row is one (channel, filter tap).  A tap that moves the pixels by one column leaves the load 2-byte
    // aligned, which loads into registers accept; the pixel that the first / last piece of an image row then
    // takes from the neighbouring image row is cleared before the piece is stored.  A tap that moves the pixels
    // above or below the image gets an offset with the top bit set: such loads return zeros.
    constexpr int kGather = 2;
    __amdgpu_buffer_rsrc_t x_rsrc = __builtin_amdgcn_make_buffer_rsrc((void *)p.x, 0, p.x_bytes, 0x00020000);
    const int piece = tid % (BN / 8);
    const int krow0 = tid / (BN / 8);  // 0..15; the second row is krow0 + 16
    int lane_off;            // byte offset of the piece for channel 0 and the filter's first tap
    unsigned rows_outside;   // bit r: filter row r moves the pixels out of the image (or the piece lies past the tile's end)
    bool at_left, at_right;  // the piece is the first / last of an image row
    {
        const int n = n0 + piece * 8;
        const bool live = piece * 8 < tile_pixels;
        const int image = n / PQ, pq = n - image * PQ;
        const int oy = pq / p.Q, ox = pq - oy * p.Q;
        lane_off = (int)(image * p.xs0 + (int64_t)(oy - p.pad_h) * p.xs2 + ox - p.pad_w) * 2;
        rows_outside = 0xffffffffu;
        for (int r = 0; r < p.R; ++r)
            if (live && (unsigned)(oy - p.pad_h + r) < (unsigned)p.H) rows_outside &= ~(1u << r);
        at_left = ox == 0;
        at_right = ox == p.Q - 8;
    }
    // Loads that would reach below the tensor's first or beyond its last byte would lose their whole piece to the
    // range check: the first image row of the whole tensor with a tap that moves it left, the last with one that
    // moves it right.  Tiles that contain such a row run the careful form of the loop, which tests every load for
    // this and, where it happens, loads the piece one pixel further in and moves the pixels back in registers.
    const int last_live = min(BN / 8 - 1, (tile_pixels - 1) / 8);  // the lane with this piece in wave 0 has the largest offset
    const int off_first = __builtin_amdgcn_readfirstlane(lane_off);
    const int off_last = __builtin_amdgcn_readlane(lane_off, last_live);
    const int64_t reach = ((int64_t)(p.C - 1) * p.xs1 + (int64_t)(p.R - 1) * p.xs2 + p.S - 1) * 2;  // largest row offset
    const bool careful_tile = off_first < 0 || (int64_t)off_last + reach + 16 > (int64_t)p.x_bytes;
    // masks that clear the pixel left / right of the image in a piece at an image border
    const unsigned keep_left = at_left ? 0xffff0000u : 0xffffffffu;    // first dword of the piece
    const unsigned keep_right = at_right ? 0x0000ffffu : 0xffffffffu;  // last dword
    // The rows of a tile are 32 consecutive (channel, tap) pairs; which taps they are repeats every `period`
    // tiles, `period_bytes` of channels further on.  A table in LDS holds, for every tile of a period and each of
    // its rows, the row's byte offset (c * xs1 + r * xs2 + s) * 2 relative to the period's first channel, the
    // shift that brings the bit of its filter row in rows_outside to the top, and a mask over a piece's first and
    // last pixel that is zero where the tap moves the pixels across the left (low half) / right (high half)
    // image border.  A lane then derives a load's offset with three instructions and keeps no per-row state.
    for (int idx = tid; idx < p.period * BK; idx += 512) {
        const int k = idx;  // tile idx / 32 of the period, row idx % 32
        const int c = k / RS, rs = k - c * RS;
        const int r = rs / p.S, sx = rs - r * p.S;
        uint4_t entry;
        entry[0] = (unsigned)((c * (int)p.xs1 + r * (int)p.xs2 + sx) * 2);
        if ((NT_CONV_ABLATE & 32) && sx != p.pad_w) entry[0] |= 0x80000000u;  // measurement: only the aligned taps fetch
        entry[1] = (unsigned)(31 - r);
        entry[2] = (sx < p.pad_w ? 0u : 0x0000ffffu) | (sx > p.S - 1 - p.pad_w ? 0u : 0xffff0000u);
        entry[3] = 0u;
        lds_taps[idx] = entry;
    }
    __syncthreads();
    const NT_LDS uint4_t *my_taps = (const NT_LDS uint4_t *)lds_taps + krow0;  // + 16 for the second row, + 32 per tile of the period
    int tap_tile = 0;        // position of the tile fetched next in its period (uniform)
    int period_base = 0;     // byte offset of that period's first channel (uniform)
    // (kM16: the four 16-lane groups of a transposing read fetch k rows 8 apart, so rows with bit 3 of k set lie another
    // 32 bytes to the right -- inside the 64 spare bytes of a row -- and two groups served together do not meet in a bank)
    const unsigned b_dst = (unsigned)(krow0 * kPitchB + (kM16 ? ((krow0 >> 3) & 1) * 32 : 0) + piece * 16);  // the first piece in a stage; the second: 16 rows on
    // fetches this thread's pieces of the next tile and moves on to the tile after it; `cols` keeps the rows' border masks
    auto gather = [&](auto careful_tag, uint4_t (&regs)[kGather], unsigned (&cols)[kGather], int (&nudges)[kGather]) {
#pragma unroll
        for (int j = 0; j < kGather; ++j) {
            const uint4_t entry = my_taps[tap_tile * BK + 16 * j];
            cols[j] = entry[2];
            // a row outside the image (or a piece past the tile's end) gets the top bit: one and the same kind of
            // offset behind the buffer for every load that has to return zeros
            const unsigned outside = (rows_outside << entry[1]) & 0x80000000u;
            int offset = (int)((unsigned)(lane_off + period_base + (int)entry[0]) | outside);

            if constexpr (decltype(careful_tag)::value) {
                // A load that would start below the tensor or end beyond it (and is no load of zeros anyway) is moved one
                // pixel further in; its pixels are moved back by one place when the piece is stored.  Every load of a
                // careful tile goes this way, without a branch: the lanes that need no move shift by zero places.
                const bool edge = !outside && (offset < 0 || (unsigned)(offset + 16) > p.x_bytes);
                const int nudge = !edge ? 0 : (offset < 0 ? 1 : -1);
                offset += 2 * nudge;
                nudges[j] = nudge;
            }
            regs[j] = __builtin_bit_cast(uint4_t, __builtin_amdgcn_raw_buffer_load_b128(x_rsrc, offset, 0, 0));
        }
        if (++tap_tile == p.period) {
            tap_tile = 0;
            period_base += p.period_bytes;
        }
    };
    // stores the pieces, the pixel that a shifted piece at an image border took from the neighbouring image row cleared
    // (keep_left always keeps the upper pixel of a dword, keep_right the lower one: the other half of a row's mask is inert)
    auto scatter = [&](auto careful_tag, auto stage_tag, const uint4_t (&regs)[kGather], const unsigned (&cols)[kGather], const int (&nudges)[kGather]) {
        NT_LDS unsigned char *sb = stage_b(stage_tag) + b_dst;
#pragma unroll
        for (int j = 0; j < kGather; ++j) {
            uint4_t v = regs[j];
            // (the masking belongs here, two steps after the load: placed right behind the load it would wait for it)
            asm volatile("" : "+v"(v));
            if constexpr (decltype(careful_tag)::value) {
                // pixels of a piece that was loaded one pixel further in move back (byte selectors of v_perm_b32 over
                // {high operand: bytes 4..7, low operand: bytes 0..3}); what falls off is a border pixel, cleared below
                const unsigned up = nudges[j] > 0 ? 0x05040302u : 0x07060504u;    // one place up: (v[i], v[i-1])
                const unsigned down = nudges[j] < 0 ? 0x05040302u : 0x03020100u;  // one place down: (v[i+1], v[i])
                uint4_t w;
                w[0] = __builtin_amdgcn_perm(v[0], 0u, up);
                w[1] = __builtin_amdgcn_perm(v[1], v[0], up);
                w[2] = __builtin_amdgcn_perm(v[2], v[1], up);
                w[3] = __builtin_amdgcn_perm(v[3], v[2], up);
                v[0] = __builtin_amdgcn_perm(w[1], w[0], down);
                v[1] = __builtin_amdgcn_perm(w[2], w[1], down);
                v[2] = __builtin_amdgcn_perm(w[3], w[2], down);
                v[3] = __builtin_amdgcn_perm(0u, w[3], down);
            }
            v[0] &= keep_left | cols[j];
            v[3] &= keep_right | cols[j];
            *(NT_LDS uint4_t *)(sb + j * (16 * kPitchB)) = v;
        }
    };

    // ---- LDS -> registers ----
    const int g = lane >> 5, l32 = lane & 31;
    const int a_row = wave_m * kWaveM + l32;                 // + 32 * ti
    const int a_sw = a_phys_chunk<BK>(a_row, 0);             // the swizzle repeats every 16 rows
    const int a_off = a_row * (BK * 2);
    const int i16 = lane & 15, nhalf = (lane >> 4) & 1;
    // transposing read: lane i of a 16-lane group addresses row i / 4 (+ 8 g, + 4 for the upper half, + 16 ks),
    // pixels 4 * (i % 4) .. + 3 of the group's 16 (+ 32 tj)
    const int b_off = (8 * g + (i16 >> 2)) * kPitchB + (wave_n * kWaveN + nhalf * 16 + 4 * (i16 & 3)) * 2;
    auto read_frags = [&](auto stage_tag, int ks, vec8 (&af)[TM], vec8 (&bf)[TN]) {
        const NT_LDS unsigned char *sa = stage_a(stage_tag);
        const NT_LDS unsigned char *sb = stage_b(stage_tag);
#pragma unroll
        for (int ti = 0; ti < TM; ++ti) {
            const int chunk = (ks * 2 + g) ^ a_sw;
            af[ti] = *(const NT_LDS vec8 *)(sa + a_off + ti * (32 * BK * 2) + chunk * 16);
        }
#pragma unroll
        for (int tj = 0; tj < TN; ++tj) {
            short4_t lo = lds_read_tr16_b64(sb + b_off + (ks * 16) * kPitchB + tj * 64);
            short4_t hi = lds_read_tr16_b64(sb + b_off + (ks * 16 + 4) * kPitchB + tj * 64);
            short8_t both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            bf[tj] = __builtin_bit_cast(vec8, both);
        }
    };

    float16_t acc[TM][TN];
#pragma unroll
    for (int ti = 0; ti < TM; ++ti)
#pragma unroll
        for (int tj = 0; tj < TN; ++tj)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[ti][tj][r] = 0.0f;

    // 16x16x32 form: channel block ti (16 channels) is one 16-byte read per lane (row i16, 16-byte chunk kg of the k
    // tile); pixel block tj (16 pixels) is two transposing reads (16-lane group kg fetches k rows 8 kg .. + 7)
    const int kg = lane >> 4;
    constexpr int TM16 = kWaveM / 16, TN16 = kWaveN / 16;
    const int a16_off = (wave_m * kWaveM + i16) * (BK * 2) + a_phys_chunk16<BK>(wave_m * kWaveM + i16, kg) * 16;  // + ti * 16 rows (the swizzle repeats)
    const int b16_lo = (8 * kg + (i16 >> 2)) * kPitchB + (kg & 1) * 32 + (wave_n * kWaveN + 4 * (i16 & 3)) * 2;    // + tj * 32 bytes; + 4 rows for the upper half
    auto read_a16 = [&](auto stage_tag, int ti) -> vec8 { return *(const NT_LDS vec8 *)(stage_a(stage_tag) + a16_off + ti * (16 * BK * 2)); };
    auto read_b16 = [&](auto stage_tag, int tj) -> vec8 {
        const NT_LDS unsigned char *sb = stage_b(stage_tag);
        short4_t lo = lds_read_tr16_b64(sb + b16_lo + tj * 32);
        short4_t hi = lds_read_tr16_b64(sb + b16_lo + 4 * kPitchB + tj * 32);
        short8_t both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        return __builtin_bit_cast(vec8, both);
    };
    float4_t acc16[kM16 ? TM16 : 1][kM16 ? TN16 : 1];  // (cleared after the prologue, whose loads borrow the registers)

    // ---- main loop ----
    // Tile t occupies stage t % 4.  The barrier that opens step t tells that tile t + 1 is complete in LDS (so
    // that the fragments of its first k step can be fetched during step t) and that every wave is done with
    // tile t - 1.  In step t a wave stores its pieces of the pixel part of tile t + 2, fetched two steps
    // earlier, into that tile's stage, fetches its pieces of tile t + 4 into the registers that have become
    // free, and requests the filter part of tile t + 3 into the stage of tile t - 1.
    const int num_k = p.CRS / BK;
    const int last_k = num_k - 1;
#ifdef NT_CONV_STAMPS
    unsigned long long stamp_loads = 0, stamp_lds = 0, stamp_sync = 0;
    const unsigned long long stamp_begin = __builtin_amdgcn_s_memtime();
    const unsigned long long real_begin = __builtin_amdgcn_s_memrealtime();
#endif
    uint4_t held[2][kGather];  // pieces in flight, by tile parity
    unsigned held_cols[2][kGather];  // their rows' border masks
    int held_nudges[2][kGather];     // (careful tiles) by how many pixels a piece was loaded further in
    auto run = [&](auto careful_tag) {
        constexpr int kFrags = TN;
        // prologue: tiles 0 and 1 complete, the pieces of tiles 2 and 3 and the filter part of tile 2 in flight
        // every load of the prologue is requested before the first one is waited for: the pieces of tiles 0 and 1 pass
        // through registers that the accumulators take over afterwards
        {
            uint4_t first[2][kGather];
            unsigned first_cols[2][kGather];
            int first_nudges[2][kGather];
            issue_filter(std::integral_constant<int, 0>(), 0);
            gather(careful_tag, first[0], first_cols[0], first_nudges[0]);
            issue_filter(std::integral_constant<int, 1>(), min(1, last_k));
            gather(careful_tag, first[1], first_cols[1], first_nudges[1]);
            gather(careful_tag, held[0], held_cols[0], held_nudges[0]);
            issue_filter(std::integral_constant<int, 2>(), min(2, last_k));
            gather(careful_tag, held[1], held_cols[1], held_nudges[1]);
            wait_vmcnt<kAInstr + 2 * kGather>();  // (in flight: the pieces of tiles 2 and 3 and the filter part of tile 2)
            scatter(careful_tag, std::integral_constant<int, 0>(), first[0], first_cols[0], first_nudges[0]);
            scatter(careful_tag, std::integral_constant<int, 1>(), first[1], first_cols[1], first_nudges[1]);
        }
#pragma unroll
        for (int ti = 0; ti < (kM16 ? TM16 : 1); ++ti)
#pragma unroll
            for (int tj = 0; tj < (kM16 ? TN16 : 1); ++tj) acc16[ti][tj] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
        vec8 af[2][TM];
        vec8 bf[2][TN];
        vec8 ch[2][kM16 ? TM16 : 1];  // kM16: the channel fragments of a k tile, two sets taking turns
        vec8 px[4];                   // ... and the slots the pixel fragments stream through
        lds_barrier();
        if constexpr (kM16) {
#pragma unroll
            for (int ti = 0; ti < TM16; ++ti) ch[0][ti] = read_a16(std::integral_constant<int, 0>(), ti);
            px[0] = read_b16(std::integral_constant<int, 0>(), 0);
            px[1] = read_b16(std::integral_constant<int, 0>(), 1);
        } else {
            read_frags(std::integral_constant<int, 0>(), 0, af[0], bf[0]);
        }
        auto step16 = [&](auto s, auto parity_tag, int t) {
            constexpr int kS = decltype(s)::value;
            constexpr int kParity = decltype(parity_tag)::value;  // of t, t + 2 and t + 4; also the set of channel fragments in use
            typedef std::integral_constant<int, (kS + 1) % kStages> NextStage;
            constexpr int cur = kParity, nxt = cur ^ 1;
            wait_vmcnt<kAInstr + kGather>();
            lds_barrier();
            if constexpr (!(NT_CONV_ABLATE & 2)) scatter(careful_tag, std::integral_constant<int, (kS + 2) % kStages>(), held[kParity], held_cols[kParity], held_nudges[kParity]);
            if constexpr (!(NT_CONV_ABLATE & 1)) gather(careful_tag, held[kParity], held_cols[kParity], held_nudges[kParity]);
            if constexpr (!(NT_CONV_ABLATE & 4)) issue_filter(std::integral_constant<int, (kS + 3) % kStages>(), min(t + 3, last_k));
            static_for<0, TN16>([&](auto q_tag) {
                constexpr int q = decltype(q_tag)::value;
                // the pixel fragment two blocks ahead (of the next tile for the last two blocks) ...
                if constexpr (q + 2 < TN16) px[(q + 2) % 4] = read_b16(s, q + 2);
                else px[(q + 2) % 4] = read_b16(NextStage(), q + 2 - TN16);
                // ... and, under the last blocks, the channel fragments of the next tile
                constexpr bool kReadsChannels = q >= TN16 - TM16;
                if constexpr (kReadsChannels) ch[nxt][q - (TN16 - TM16)] = read_a16(NextStage(), q - (TN16 - TM16));
#pragma unroll
                for (int ti = 0; ti < TM16; ++ti) acc16[ti][q] = E::mfma16(px[q % 4], ch[cur][ti], acc16[ti][q]);
                constexpr int kReads = 2 + (kReadsChannels ? 1 : 0);
                static_for<0, TM16>([&](auto j_tag) {
                    constexpr int j = decltype(j_tag)::value;
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    if constexpr (j < kReads) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                });
            });
        };
        auto step = [&](auto s, auto parity_tag, int t) {
            constexpr int kS = decltype(s)::value;
            constexpr int kParity = decltype(parity_tag)::value;  // of t, t + 2 and t + 4
            typedef std::integral_constant<int, (kS + 1) % kStages> NextStage;
            // Loads are issued as: pieces of tile t + 4, then the filter part of tile t + 3, in every step.  All but
            // the last step's have arrived here: the pieces of tile t + 2, stored below, and the filter part of
            // tile t + 1, which with that tile's pieces, stored one step ago (the barrier waits for this wave's LDS
            // traffic), completes tile t + 1.
#if defined(NT_CONV_STAMPS) && NT_CONV_STAMPS == 1
            {
                unsigned long long t0, t1, t2, t3;
                asm volatile("s_memtime %0\n\ts_waitcnt vmcnt(4)\n\ts_memtime %1\n\ts_waitcnt lgkmcnt(0)\n\ts_memtime %2\n\ts_barrier\n\ts_memtime %3\n\ts_waitcnt lgkmcnt(0)"
                             : "=&s"(t0), "=&s"(t1), "=&s"(t2), "=&s"(t3)::"memory");
                stamp_loads += t1 - t0;
                stamp_lds += t2 - t1;
                stamp_sync += t3 - t2;
            }
#else
            wait_vmcnt<kAInstr + kGather>();
            lds_barrier();
#endif
            if constexpr (!(NT_CONV_ABLATE & 2)) scatter(careful_tag, std::integral_constant<int, (kS + 2) % kStages>(), held[kParity], held_cols[kParity], held_nudges[kParity]);
            if constexpr (!(NT_CONV_ABLATE & 1)) gather(careful_tag, held[kParity], held_cols[kParity], held_nudges[kParity]);
            if constexpr (!(NT_CONV_ABLATE & 4)) issue_filter(std::integral_constant<int, (kS + 3) % kStages>(), min(t + 3, last_k));
            static_for<0, KS>([&](auto ks_tag) {
                constexpr int ks = decltype(ks_tag)::value;
                constexpr int cur = ks & 1, nxt = cur ^ 1;
                if constexpr (NT_CONV_ABLATE & 16) {
                } else if constexpr (ks + 1 < KS) read_frags(s, ks + 1, af[nxt], bf[nxt]);
                else read_frags(NextStage(), 0, af[nxt], bf[nxt]);
                if constexpr (!(NT_CONV_ABLATE & 8))
#pragma unroll
                for (int ti = 0; ti < TM; ++ti)
#pragma unroll
                    for (int tj = 0; tj < kFrags; ++tj) acc[ti][tj] = E::mfma32(bf[cur][tj], af[cur][ti], acc[ti][tj]);
                // issue order: the fragment reads of the next k step spread under this k step's MFMAs
                constexpr int kMfma = TM * kFrags;
                constexpr int kReads = TM + 2 * kFrags;
                constexpr int kPer = kMfma > 0 ? (kReads + kMfma - 1) / kMfma : 1;
                static_for<0, kMfma>([&](auto i_tag) {
                    constexpr int i = decltype(i_tag)::value;
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    if constexpr (i * kPer < kReads) __builtin_amdgcn_sched_group_barrier(0x100, kPer, 0);
                });
            });
        };
        // stages and parities repeat every 4 tiles
        int t = 0;
        for (; t + 4 <= num_k; t += 4) {
            static_for<0, 4>([&](auto i_tag) {
                constexpr int i = decltype(i_tag)::value;
                if constexpr (kM16) step16(std::integral_constant<int, i>(), std::integral_constant<int, i & 1>(), t + i);
                else step(std::integral_constant<int, i>(), std::integral_constant<int, i & 1>(), t + i);
            });
        }
        static_for<0, 3>([&](auto i_tag) {
            constexpr int i = decltype(i_tag)::value;
            if (t + i < num_k) {
                if constexpr (kM16) step16(std::integral_constant<int, i>(), std::integral_constant<int, i & 1>(), t + i);
                else step(std::integral_constant<int, i>(), std::integral_constant<int, i & 1>(), t + i);
            }
        });
    };
    if (careful_tile) run(std::true_type());  // (the first and the last tile of a launch)
    else run(std::false_type());
#ifdef NT_CONV_STAMPS
    const unsigned long long stamp_loop_ticks = __builtin_amdgcn_s_memtime() - stamp_begin;
    const unsigned long long real_loop_end = __builtin_amdgcn_s_memrealtime();
#endif

    // ---- epilogue ----
    // lane (l32, g) holds, per 32 x 32 tile, output channel l32 and in registers 4 * r4 .. + 3 the pixels
    // 8 * r4 + 4 * g .. + 3.  Each wave passes 32 channels x 128 pixels at a time through its own LDS slab
    // (in the filter stages, idle by now: two slabs each), so that a lane stores 16 bytes of one channel's pixels.
    constexpr int kRowBytes = kWaveN * 2;
    constexpr int kCChunks = kRowBytes / 16;
    constexpr int kSlabBytes = 32 * kRowBytes;
    static_assert(2 * kSlabBytes == kStageA && kWaves == 2 * kStages, "slabs in the filter stages");
    wait_vmcnt<0>();
    lds_barrier();
    NT_LDS unsigned char *slab = (wave < 2   ? (NT_LDS unsigned char *)lds_a0
                                  : wave < 4 ? (NT_LDS unsigned char *)lds_a1
                                  : wave < 6 ? (NT_LDS unsigned char *)lds_a2
                                             : (NT_LDS unsigned char *)lds_a3) +
                                 (wave & 1) * kSlabBytes;
    T *Y = (T *)p.y;
    const int slab_sw = l32 & (kCChunks - 1);
#pragma unroll
    for (int ti = 0; ti < TM; ++ti) {
        if constexpr (kM16) {
            // 16 x 16 blocks: lane (i16, kg) holds, of channel i16, the pixels 4 kg .. + 3; two blocks of channels fill a slab
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                const int row = half * 16 + i16;
#pragma unroll
                for (int tj = 0; tj < TN16; ++tj) {
                    typedef T vec4 __attribute__((ext_vector_type(4)));
                    const float4_t a4 = acc16[kM16 ? 2 * ti + half : 0][kM16 ? tj : 0];
                    vec4 v;
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] = E::from_float(a4[e]);
                    const int chunk = (tj * 2 + (kg >> 1)) ^ (row & (kCChunks - 1));
                    *(NT_LDS vec4 *)(slab + row * kRowBytes + chunk * 16 + 8 * (kg & 1)) = v;
                }
            }
        } else
#pragma unroll
        for (int tj = 0; tj < TN; ++tj)
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                typedef T vec4 __attribute__((ext_vector_type(4)));
                vec4 v;
#pragma unroll
                for (int e = 0; e < 4; ++e) v[e] = E::from_float(acc[ti][tj][4 * r4 + e]);
                const int chunk = (tj * 4 + r4) ^ slab_sw;
                *(NT_LDS vec4 *)(slab + l32 * kRowBytes + chunk * 16 + 8 * g) = v;
            }
#pragma unroll
        for (int it = 0; it < (32 * kCChunks) / 64; ++it) {
            const int idx = it * 64 + lane;
            const int row = idx / kCChunks;
            const int phys = idx % kCChunks;
            const int chunk = phys ^ (row & (kCChunks - 1));
            vec8 v = *(const NT_LDS vec8 *)(slab + row * kRowBytes + phys * 16);
            const int channel = m0 + wave_m * kWaveM + ti * 32 + row;
            const int in_tile = wave_n * kWaveN + chunk * 8;
            if (channel >= p.K || in_tile >= tile_pixels) continue;  // (tiles are multiples of 8 pixels wide)
            const int n = n0 + in_tile;
            const int image = n / PQ, pq = n - image * PQ;
            __builtin_nontemporal_store(v, (vec8 *)(Y + ((int64_t)image * p.K + channel) * PQ + pq));
        }
    }
#ifdef NT_CONV_STAMPS
    if (p.stamps && lane == 0) {  // (100 MHz counter: loop, entry to loop, loop end to the last store issued)
        unsigned long long *dst = p.stamps + ((size_t)blockIdx.x * kWaves + wave) * 4;
        dst[0] = stamp_loop_ticks;
        dst[1] = NT_CONV_STAMPS == 2 ? real_loop_end - real_begin : stamp_loads;
        dst[2] = NT_CONV_STAMPS == 2 ? real_begin - real_entry : stamp_lds;
        dst[3] = NT_CONV_STAMPS == 2 ? __builtin_amdgcn_s_memrealtime() - real_loop_end : stamp_sync;
    }
#endif
#endif
}

// the one-launch path on the tensors as they lie; NINETOOTHED_NO_KERNEL when the request does not fit it
template <typename T>
int run_direct(const Conv2dRequest &q, hipStream_t stream) {
    const int CRS = q.C * q.R * q.S;
    if (!q.unit_steps()) return NINETOOTHED_NO_KERNEL;  // pixels of a row must be consecutive, taps one pixel apart
    if (q.P != q.H + 2 * q.pad_h - q.R + 1 || q.Q != q.W + 2 * q.pad_w - q.S + 1) return NINETOOTHED_NO_KERNEL;
    if (q.Q % 8 || q.W < 8 || q.pad_w > 1 || CRS % 32 || q.R > 16 || q.S > 16) return NINETOOTHED_NO_KERNEL;
    if (q.xs[3] != 1 || q.xs[0] < 0 || q.xs[1] < 0 || q.xs[2] < 0) return NINETOOTHED_NO_KERNEL;
    // Offsets must grow with (image, channel, row): the kernel decides from the first and the last piece of a tile
    // whether any of its loads could start before the tensor or end behind it, which an input whose images, channels
    // or rows overlap in memory (a stride of 0 from `expand`, say) would defeat.
    const int64_t row_span = q.W, channel_span = (int64_t)(q.H - 1) * q.xs[2] + row_span, image_span = (int64_t)(q.C - 1) * q.xs[1] + channel_span;
    if ((q.H > 1 && q.xs[2] < row_span) || (q.C > 1 && q.xs[1] < channel_span) || (q.N > 1 && q.xs[0] < image_span)) return NINETOOTHED_NO_KERNEL;
    if (q.ws[3] != 1 || q.ws[2] != q.S || q.ws[1] != (int64_t)q.R * q.S || q.ws[0] != CRS || ((uintptr_t)q.w & 15)) return NINETOOTHED_NO_KERNEL;
    // at least four fifths of the 256 output channels of a tile in use
    if ((int64_t)q.K * 5 < (int64_t)ceil_div(q.K, 256) * 256 * 4) return NINETOOTHED_NO_KERNEL;
    const int64_t x_extent = ((int64_t)(q.N - 1) * q.xs[0] + (int64_t)(q.C - 1) * q.xs[1] + (int64_t)(q.H - 1) * q.xs[2] + q.W) * 2;
    const int64_t w_bytes = (int64_t)q.K * CRS * 2;
    if (x_extent >= (int64_t(1) << 31) || w_bytes >= (int64_t(1) << 31)) return NINETOOTHED_NO_KERNEL;  // 32-bit buffer offsets
    ConvDirectParams p;
    p.x = q.x; p.w = q.w; p.y = q.y;
    p.C = q.C; p.H = q.H; p.W = q.W; p.K = q.K; p.R = q.R; p.S = q.S; p.P = q.P; p.Q = q.Q;
    p.pad_h = q.pad_h; p.pad_w = q.pad_w;
    p.xs0 = q.xs[0]; p.xs1 = q.xs[1]; p.xs2 = q.xs[2];
    p.M = q.N * q.P * q.Q;
    p.CRS = CRS;
    p.x_bytes = (unsigned)x_extent;
    p.w_bytes = (unsigned)w_bytes;
    int divisor = q.R * q.S;  // gcd(32, R * S)
    for (int rest = 32 % divisor; rest != 0;) {
        const int next = divisor % rest;
        divisor = rest;
        rest = next;
    }
    p.period = q.R * q.S / divisor;
    if (p.period > kConvDirectMaxPeriod) return NINETOOTHED_NO_KERNEL;
    p.period_bytes = (int)((32 / divisor) * q.xs[1] * 2);  // (the extent check above covers this product)
    p.tiles_ch = ceil_div(q.K, 256);
    const int64_t grid = (int64_t)ceil_div(p.M, 256) * p.tiles_ch;
    if (grid <= 0 || grid > 0x7fffffffll) return NINETOOTHED_NO_KERNEL;
#ifdef NT_CONV_STAMPS
    p.stamps = g_conv_stamps;
#endif
    // 16x16x32 MFMAs draw less power per FLOP and finish a tile sooner (at [32, 256, 56, 56] * [256, 256, 3, 3]: 55 against
    // 59 us per tile), but the careful form of that loop -- the first and the last tile of pixels -- runs out of registers
    // and is slower than the 32x32x16 one (92 against 80 us): with more tiles than compute units those two are dealt out
    // first and the others hide them; a launch of a single round would wait for them.
    int units = compute_units();
#ifdef NT_CONV_M32
    units = 0;
#endif
    if (units > 0 && grid > units) conv2d_direct_kernel<T, true><<<dim3((unsigned)grid), dim3(512), 0, stream>>>(p);
    else conv2d_direct_kernel<T, false><<<dim3((unsigned)grid), dim3(512), 0, stream>>>(p);
    return (int)hipGetLastError();
}

// channels of the repacked operands: the k step of 32 holds whole blocks of channels -- or, for up to 16 channels
// (the first layer of an image network), 4 or 2 filter taps of 8 or 16 channels each; the extra channels are zeros
inline int conv2d_padded_channels(int channels) { return channels <= 16 ? ceil_div(channels, 8) * 8 : ceil_div(channels, 32) * 32; }

template <typename T>
int run_fast(const Conv2dRequest &q, hipStream_t stream) {
    const int Cp = conv2d_padded_channels(q.C);
    const int64_t xt_bytes = (int64_t)q.N * q.H * q.W * Cp * 2;
    const int Kp = ceil_div(q.K, 8) * 8;
    const int64_t wt_bytes = (int64_t)Kp * Cp * q.R * q.S * 2;
    WorkspaceLease lease(stream);
    const int HW = q.H * q.W;
    // an input that lies as the kernel reads it -- channels last, contiguous, whole k steps of channels -- is read where it is
    const bool in_place = q.xs[1] == 1 && q.C == Cp && q.xs[3] == Cp && q.xs[2] == (int64_t)q.W * Cp && q.xs[0] == (int64_t)HW * Cp && ((uintptr_t)q.x & 15) == 0;
    void *xt = in_place ? const_cast<void *>(q.x) : lease.get(kWorkspaceConvInput, (size_t)xt_bytes);
    void *wt = lease.get(kWorkspaceConvFilter, (size_t)wt_bytes);
    if (xt == nullptr || wt == nullptr) return NINETOOTHED_NO_KERNEL;  // no scratch: the caller falls back to the gather kernel
    const bool aligned = ((uintptr_t)q.x & 15) == 0;
    int vector_ok = q.xs[3] == 1 && q.xs[2] == q.W;  // 16-byte loads along the positions of a channel
    if (q.xs[1] == 1 && q.C > 1) vector_ok = q.C % 8 == 0 && q.xs[3] % 8 == 0 && q.xs[2] % 8 == 0 && q.xs[0] % 8 == 0 && aligned ? 3 : 2;
    FilterRepack f;
    f.w = q.w;
    f.wt = wt;
    f.K = q.K; f.C = q.C; f.R = q.R; f.S = q.S; f.Cp = Cp; f.Kp = Kp;
    f.s_k = q.ws[0]; f.s_c = q.ws[1]; f.s_r = q.ws[2]; f.s_s = q.ws[3];
    // about 512 workgroups for the filter, or one thread per element if that is less
    const int64_t per_layer = (int64_t)ceil_div(HW, 64) * ceil_div(Cp, 64);
    const int64_t wanted = std::min<int64_t>(512, ((int64_t)Kp * Cp * q.R * q.S + 255) / 256);
    f.layers = (int)std::max<int64_t>(1, std::min<int64_t>(ceil_div(wanted, per_layer), 512));
    conv2d_repack_kernel<T><<<dim3(ceil_div(HW, 64), ceil_div(Cp, 64), (in_place ? 0 : q.N) + f.layers), dim3(256), 0, stream>>>(
        (const T *)q.x, (T *)xt, q.C, HW, q.W, q.xs[0], q.xs[1], q.xs[2], q.xs[3], vector_ok, f);
    ConvParams p;
    p.xt = xt;
    p.wt = wt;
    p.y = q.y;
    p.N = q.N; p.C = Cp; p.H = q.H; p.W = q.W; p.K = q.K; p.R = q.R; p.S = q.S; p.P = q.P; p.Q = q.Q;
    p.Kp = Kp;
    p.dense_out = q.ys[3] == 1 && q.ys[2] == q.Q && q.ys[1] == (int64_t)q.P * q.Q && q.ys[0] == (int64_t)q.K * q.P * q.Q && ((uintptr_t)q.y & 15) == 0;
    if (!p.dense_out && q.ys[1] == 1 && q.K > 1) p.dense_out = 2;
    for (int d = 0; d < 4; ++d) p.ys[d] = q.ys[d];
    p.stride_h = q.stride_h; p.stride_w = q.stride_w; p.dil_h = q.dil_h; p.dil_w = q.dil_w;
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
    if (q.C < 1) return NINETOOTHED_NO_KERNEL;
    // (an output that is no contiguous NCHW tensor -- channels last, a slice -- is stored element by element)
    const int64_t xt_bytes = (int64_t)q.N * q.H * q.W * conv2d_padded_channels(q.C) * 2;
    const int64_t wt_bytes = (int64_t)ceil_div(q.K, 8) * 8 * conv2d_padded_channels(q.C) * q.R * q.S * 2;
    if (xt_bytes >= (int64_t(1) << 31) || wt_bytes >= (int64_t(1) << 31)) return NINETOOTHED_NO_KERNEL;  // 32-bit buffer offsets
    if ((int64_t)q.N * q.P * q.Q > 0x7fffffffll || (int64_t)ceil_div(q.N * q.P * q.Q, 128) * ceil_div(q.K, 64) > 0x7fffffffll) return NINETOOTHED_NO_KERNEL;
    if (q.N >= 65535 - 512 || ceil_div(q.C, 64) > 65535) return NINETOOTHED_NO_KERNEL;  // grid of the repacking pass: (positions, channels, filter layers + images)
    // (even a few output positions are served sooner by two short launches than by the gather kernel, whose lanes
    // fetch their 16 values of a k step one after another: [2, 32, 9, 9] * [16, 32, 3, 3] 48 against 13 us)
    if ((int64_t)q.N * q.P * q.Q < 1) return NINETOOTHED_NO_KERNEL;
    return q.dtype == NINETOOTHED_FLOAT16 ? run_fast<half_t>(q, stream) : run_fast<bf16_t>(q, stream);
}

int conv2d_direct(const Conv2dRequest &q, hipStream_t stream) {
    if (q.dtype != NINETOOTHED_FLOAT16 && q.dtype != NINETOOTHED_BFLOAT16) return NINETOOTHED_NO_KERNEL;
    if (q.ys[3] != 1 || q.ys[2] != q.Q || q.ys[1] != (int64_t)q.P * q.Q || q.ys[0] != (int64_t)q.K * q.P * q.Q) return NINETOOTHED_NO_KERNEL;
    if (((uintptr_t)q.y & 15) != 0 || q.K % 8) return NINETOOTHED_NO_KERNEL;
    if ((int64_t)q.N * q.P * q.Q > 0x7fffffffll - 512) return NINETOOTHED_NO_KERNEL;
    return q.dtype == NINETOOTHED_FLOAT16 ? run_direct<half_t>(q, stream) : run_direct<bf16_t>(q, stream);
}

}  // namespace nt

#ifdef NT_CONV_STAMPS
extern "C" void nt_debug_conv_stamps(void *buffer) { nt::g_conv_stamps = (unsigned long long *)buffer; }
#endif
