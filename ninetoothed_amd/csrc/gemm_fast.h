// Tiled GEMM for gfx950: C[M,N] = A[M,K] @ B[K,N] (+ addmm epilogue), fp16/bf16
// inputs, fp32 accumulation on 16x16x32 MFMAs (32x32x16 in the measurement instances).
//
// Fast path requirements (checked on the host before launch):
//   A row-major with unit K stride, B row-major with unit N stride, C with unit
//   N stride and the element type of A/B; any M (rows of the last tile past M
//   read as zeros through the A buffer descriptor and are not stored),
//   N % BN == 0, K % BK == 0; row pitches and base addresses multiples of 16 bytes.
//
// Data movement per workgroup and K step:
//   HBM/L2 --buffer_load ... lds (16 B per lane, no registers)--> LDS stage
//   LDS --ds_read_b128 (A) / ds_read_b64_tr_b16 (B)--> MFMA operand registers
// LDS tiles are XOR-swizzled at 16-byte granularity so both the row-wise A
// reads and the transposing B reads spread over all 64 banks.
#pragma once

#include <type_traits>

#include "nt_common.h"

namespace nt {

struct GemmParams {
    const void *a;
    const void *b;
    void *c;
    const void *bias;  // addmm `input`; nullptr for plain matmul
    int m, n, k;
    int64_t lda, ldb, ldc;            // row pitches in elements
    int64_t bias_stride_m, bias_stride_n;
    float alpha, beta;
    int tiles_m, tiles_n;
    int bias_vector;  // addmm input readable with aligned 16-byte loads along N
    int order;  // tile order: 0 = XCD-aware strips of 8 tile rows; other values are measurement aids
    int kt_per_split;  // split-K instances: k tiles per part (the grid holds tiles * parts workgroups)
    int c_vector;      // rows of C take aligned 16-byte stores (else, in the instances with tails: element stores)
    // batch > 1: the grid holds tiles * batch workgroups; product b uses the operands moved by these element strides
    int batch;
    int64_t a_batch, b_batch, c_batch, bias_batch;
};

// A tile [BM][BK]: rows of BK * 2 bytes, split into 16-byte chunks.  Rows that
// share a 256-byte bank window get different chunk permutations.
template <int BK>
NT_HOST_DEVICE constexpr int a_phys_chunk(int row, int chunk) {
    constexpr int kChunksPerRow = BK / 8;
    constexpr int kRowsPerWindow = (256 / (BK * 2)) > 0 ? (256 / (BK * 2)) : 1;
    return chunk ^ ((row / kRowsPerWindow) % kChunksPerRow);
}

// B tile [BK][BN]: a transposing read touches 4 consecutive k rows x 64 bytes;
// shifting each row by a different multiple of 64 bytes separates them.
template <int BN>
NT_HOST_DEVICE constexpr int b_phys_chunk(int krow, int chunk) {
    constexpr int kChunksPerRow = BN / 8;
    constexpr int kMask = (kChunksPerRow / 4 - 1) < 7 ? (kChunksPerRow / 4 - 1) : 7;
    return chunk ^ ((krow & kMask) << 2);
}

// The A tile for the 16x16x32 MFMA form, whose 16-byte reads address row lane % 16, chunk lane / 16: the LDS
// serves such a read in four passes of 16 lanes -- {0-3, 12-15, 20-27}, {4-11, 16-19, 28-31} and the same
// + 32 (measured with two active lanes at a time) -- and with rows of 64 bytes the plain XOR of the row
// group puts two row groups of a pass on the same banks; XOR with the negated row group does not.  Rows of
// 128 bytes and more are conflict-free as they are.
template <int BK>
NT_HOST_DEVICE constexpr int a_phys_chunk16(int row, int chunk) {
    if (BK == 32) return chunk ^ ((4 - (row / 4) % 4) % 4);
    return a_phys_chunk<BK>(row, chunk);
}

// The same for the 16x16x32 MFMA's transposing reads, where the four 16-lane groups of a wave read k rows
// 8 apart (k % 8 equal): rows with bit 3 of k set move by another 32 bytes, so that two groups served
// together do not meet in a bank.
template <int BN>
NT_HOST_DEVICE constexpr int b_phys_chunk16(int krow, int chunk) {
    return b_phys_chunk<BN>(krow, chunk) ^ (((krow >> 3) & 1) << 1);
}

// Maps the hardware workgroup id to an output tile.  Workgroup ids are dealt
// round-robin to the 8 XCDs, so ids congruent mod 8 share an L2: give each
// XCD a contiguous range of tile ids, ordered in column strips of kGroupM
// tile-rows so that concurrently running tiles reuse A and B panels in L2.
NT_DEVICE void map_tile(int tiles_m, int tiles_n, int order, int &tile_m, int &tile_n, int bid = blockIdx.x, int nblocks = gridDim.x) {
    // order: low 8 bits = tile rows per strip (0 -> 8), bit 8 = skip the XCD remap
    const int group_m = (order & 0xff) ? (order & 0xff) : 8;
    if ((nblocks & 7) == 0 && !(order & 0x100)) {
        const int per_xcd = nblocks >> 3;
        bid = (bid & 7) * per_xcd + (bid >> 3);
    }
    const int group_size = group_m * tiles_n;
    const int group = bid / group_size;
    const int first_m = group * group_m;
    const int rows = min(tiles_m - first_m, group_m);
    const int in_group = bid - group * group_size;
    tile_m = first_m + in_group % rows;
    tile_n = in_group / rows;
}

template <int I, int N, typename F>
NT_DEVICE void static_for(F &&f) {
    if constexpr (I < N) {
        f(std::integral_constant<int, I>());
        static_for<I + 1, N>(f);
    }
}

// Workgroup barrier for the LDS ring.  Written as an opaque statement with a
// memory clobber: the compiler moves no LDS access across it, and -- unlike a
// workgroup fence -- it does not make the wave wait for its outstanding
// global -> LDS fills of later stages (they are waited for explicitly with
// wait_vmcnt<N>()).  The stage that is refilled right after the barrier was
// read just before it, and an LDS read that is merely issued can still sit in
// the queue behind other waves' reads when the refill (an L2 hit) lands: the
// MFMAs that consume it are not memory operations and may be scheduled below
// the barrier, taking their wait with them.  So a wave first waits for its own
// LDS reads and only then arrives at the barrier.
NT_DEVICE void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// The same without the wait, for loops whose LDS reads still in flight at the barrier are known to target
// a stage that is not refilled after it.  No instruction is scheduled across it, so every MFMA of the
// code before it -- and with it the wait for its operand reads -- is issued before the wave arrives.
NT_DEVICE void lds_barrier_reads_in_flight() {
    __builtin_amdgcn_sched_barrier(0);
    asm volatile("s_barrier" ::: "memory");
    __builtin_amdgcn_sched_barrier(0);
}

#ifndef NT_GEMM_SCHEDULE
#define NT_GEMM_SCHEDULE 1
#endif
#ifndef NT_GEMM_M16
#define NT_GEMM_M16 1
#endif
#ifndef NT_GEMM_PAIR_A
#define NT_GEMM_PAIR_A 1
#endif

// kAblate is a measurement aid (bit 0: no global loads inside the K loop,
// bit 1: operand fragments read from LDS only once); 0 in every shipped instance.
template <typename T, int BM, int BN, int BK, int WM, int WN, int kStages, int kWavesPerSimd, bool kAddmm, int kAblate = 0, int kLoad = 0, int kAux = 0,
          bool kFloatOut = false, bool kBT = false, bool kTail = false, bool kSplit = false>
__global__ __launch_bounds__(WM *WN * 64, kWavesPerSimd) void gemm_nn_fast_kernel(GemmParams p) {
#if defined(__HIP_DEVICE_COMPILE__)  // the body uses device-only builtins; the host pass only needs the stub
    typedef Elem<T> E;
    typedef typename E::vec8 vec8;
    constexpr int kWaves = WM * WN;
    constexpr int kWaveM = BM / WM;   // rows of C per wave
    constexpr int kWaveN = BN / WN;   // cols of C per wave
    constexpr int TM = kWaveM / 32;   // 32x32 MFMA tiles per wave along M
    constexpr int TN = kWaveN / 32;
    constexpr int kStageA = BM * BK * 2;  // bytes
    constexpr int kStageB = BK * BN * 2;
    constexpr int kAChunksPerRow = BK / 8;
    constexpr int kARowsPerInstr = 64 / kAChunksPerRow;
    constexpr int kAInstr = kStageA / (kWaves * 1024);
    constexpr int kBChunksPerRow = BN / 8;
    constexpr int kBRowsPerInstr = 64 / kBChunksPerRow > 0 ? 64 / kBChunksPerRow : 1;
    constexpr int kBInstr = kStageB / (kWaves * 1024);
    constexpr int kLoadsPerTile = kAInstr + kBInstr;
    // the tiles are laid out for the reads of the 16x16x32 MFMA form (see kM16 below)
    constexpr bool kTile16 = NT_GEMM_M16 && kAblate == 0 && BK % 32 == 0 && sizeof(T) == 2;
    // kPairA (the 5 x 32 KiB ring of the large tile): A is staged two k tiles at a time, in three stages of rows of
    // 128 bytes, B one k tile at a time in four stages.  A fill instruction then asks for whole cache lines of A
    // (16 half lines otherwise: a k tile of A is 64 bytes per row), which is worth 3 % at 8192^3.  The compute
    // steps stay one k tile long; a tile of B and half a pair of A stay in flight across a barrier (the pair whose
    // stage becomes free in an even step is requested half in that step and half in the next).
    constexpr bool kPairA = NT_GEMM_PAIR_A && kTile16 && BK == 32 && kStages == 5 && kLoad == 1 && !kSplit &&
                            (BM / WM / 16) % 4 == 0 && BM / WM >= BN / WN;
    constexpr int kBytesA = kPairA ? 2 * kStageA : kStageA;
    // kTail: N and K need not fit the tile (multiples of 8 elements, so that 16-byte chunks stay whole).
    // Columns of B past N feed only columns of C that are not stored; the k positions past K of the last
    // tile must read as zeros in both operands (a stray Inf times a zero would be a NaN): rows of a
    // row-major B past K lie behind the end of its descriptor, and lanes whose chunk of a k-contiguous
    // row (A, transposed B) starts past K get an offset behind the end of theirs.
    static_assert(!kTail || kLoad == 1, "tails rely on the range check of buffer loads");
    // kSplit: the grid holds tiles x parts workgroups; part s multiplies k tiles [s * kt_per_split, ...) and
    // writes its fp32 accumulators to slice s of a [parts][M][N] scratch tensor (p.c, pitch p.ldc), which a
    // second kernel sums -- for problems with too few output tiles to occupy the chip
    static_assert(!kSplit || (kFloatOut && kTail && !kAddmm), "split-K parts are fp32 tiles with tails");
    static_assert(kStageA % (kWaves * 1024) == 0 && kStageB % (kWaves * 1024) == 0, "tile/wave mismatch");
    static_assert(kBChunksPerRow <= 64, "BN too large for one-instruction rows");
    static_assert(kWaveM % 32 == 0 && kWaveN % 32 == 0 && BK % 16 == 0, "wave tile");
    static_assert(kStages >= 2 && kStages <= 5, "2..5 stages");
    static_assert((kStages - 2) * kLoadsPerTile < 64, "vmcnt range");

    // One array per stage and operand: distinct LDS objects let the compiler prove
    // that the asynchronous fill of one stage does not alias reads of another,
    // so it does not wait for the fill before the MFMA operand reads.
    // (kPairA uses a0 .. a2 and b0 .. b3; arrays that nothing refers to take no LDS)
    __shared__ __attribute__((aligned(1024))) unsigned char lds_a0[kBytesA];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_a1[kBytesA];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_a2[kStages > 2 ? kBytesA : 16];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_a3[kStages > 3 ? kStageA : 16];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_a4[kStages > 4 ? kStageA : 16];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_b0[kStageB];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_b1[kStageB];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_b2[kStages > 2 ? kStageB : 16];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_b3[kStages > 3 ? kStageB : 16];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_b4[kStages > 4 ? kStageB : 16];
    auto stage_a = [&](auto tag) -> NT_LDS unsigned char * {
        constexpr int i = decltype(tag)::value;
        if constexpr (i == 0) return (NT_LDS unsigned char *)lds_a0;
        else if constexpr (i == 1) return (NT_LDS unsigned char *)lds_a1;
        else if constexpr (i == 2) return (NT_LDS unsigned char *)lds_a2;
        else if constexpr (i == 3) return (NT_LDS unsigned char *)lds_a3;
        else return (NT_LDS unsigned char *)lds_a4;
    };
    auto stage_b = [&](auto tag) -> NT_LDS unsigned char * {
        constexpr int i = decltype(tag)::value;
        if constexpr (i == 0) return (NT_LDS unsigned char *)lds_b0;
        else if constexpr (i == 1) return (NT_LDS unsigned char *)lds_b1;
        else if constexpr (i == 2) return (NT_LDS unsigned char *)lds_b2;
        else if constexpr (i == 3) return (NT_LDS unsigned char *)lds_b3;
        else return (NT_LDS unsigned char *)lds_b4;
    };

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wave_m = wave / WN;
    const int wave_n = wave % WN;

    int tile_m, tile_n;
    const int tiles = p.tiles_m * p.tiles_n;
    const int part = kSplit ? blockIdx.x / tiles : 0;
    const int batch = !kSplit && p.batch > 1 ? blockIdx.x / tiles : 0;
    if (kSplit || p.batch > 1) map_tile(p.tiles_m, p.tiles_n, p.order, tile_m, tile_n, blockIdx.x - (part + batch) * tiles, tiles);
    else map_tile(p.tiles_m, p.tiles_n, p.order, tile_m, tile_n);
    const int m0 = tile_m * BM;
    const int n0 = tile_n * BN;

    const T *A = (const T *)p.a + batch * p.a_batch;
    const T *B = (const T *)p.b + batch * p.b_batch;

    // ---- global -> LDS assignments (per lane, fixed over the K loop) ----
    // Byte offsets relative to the tile's first A row / B column stay below
    // 2^31 (checked on the host), so addresses are a uniform base + 32-bit lane offset.
    // A: instruction j of this wave fills rows [(j*kWaves+wave)*kARowsPerInstr, +kARowsPerInstr)
    const unsigned char *a_base = (const unsigned char *)(A + (int64_t)m0 * p.lda);
    // kBT: B is given as [N, K] with K contiguous (`x @ w.T`): its tile is staged and read exactly
    // like A's (rows = columns of C, 16-byte chunks of 8 consecutive k), no transposing read
    const unsigned char *b_base = (const unsigned char *)(kBT ? B + (int64_t)n0 * p.ldb : B + n0);
    unsigned a_src[kAInstr];
#pragma unroll
    for (int j = 0; j < kAInstr; ++j) {
        const int row = (j * kWaves + wave) * kARowsPerInstr + lane / kAChunksPerRow;
        const int phys = lane % kAChunksPerRow;
        const int chunk = kTile16 ? a_phys_chunk16<BK>(row, phys) : a_phys_chunk<BK>(row, phys);  // XOR is an involution
        a_src[j] = (unsigned)(row * (int)p.lda + chunk * 8) * 2u;
    }
    unsigned b_src[kBInstr];
#pragma unroll
    for (int j = 0; j < kBInstr; ++j) {
        if constexpr (kBT) {
            const int row = (j * kWaves + wave) * kARowsPerInstr + lane / kAChunksPerRow;
            const int chunk = kTile16 ? a_phys_chunk16<BK>(row, lane % kAChunksPerRow) : a_phys_chunk<BK>(row, lane % kAChunksPerRow);
            b_src[j] = (unsigned)(row * (int)p.ldb + chunk * 8) * 2u;
        } else {
            const int krow = (j * kWaves + wave) * kBRowsPerInstr + lane / kBChunksPerRow;
            const int phys = lane % kBChunksPerRow;
            const int chunk = kTile16 ? b_phys_chunk16<BN>(krow, phys) : b_phys_chunk<BN>(krow, phys);
            b_src[j] = (unsigned)(krow * (int)p.ldb + chunk * 8) * 2u;
        }
    }

    // kPairA: instruction j of a wave fills rows [(j * kWaves + wave) * 8, + 8) of a pair stage, 128 bytes each
    constexpr int kPairInstr = 2 * kAInstr;
    unsigned a_pair_src[kPairA ? kPairInstr : 1];
    if constexpr (kPairA) {
#pragma unroll
        for (int j = 0; j < kPairInstr; ++j) {
            const int row = (j * kWaves + wave) * 8 + lane / 8;
            const int chunk = a_phys_chunk16<64>(row, lane % 8);
            a_pair_src[j] = (unsigned)(row * (int)p.lda + chunk * 8) * 2u;
        }
    }

    // kLoad 0: global_load_lds (64-bit base + lane offset); 1: buffer_load ... lds
    // (buffer resource on the tile panel, 32-bit lane offset, scalar K offset)
    __amdgpu_buffer_rsrc_t a_rsrc, b_rsrc;
    if constexpr (kLoad == 1) {
        // the A descriptor ends with the last row of the matrix: rows of the tile past M read as zeros
        const int64_t a_rows = min((int64_t)BM, (int64_t)p.m - m0);
        const unsigned a_bytes = (unsigned)(((a_rows - 1) * p.lda + p.k) * 2);
        a_rsrc = __builtin_amdgcn_make_buffer_rsrc((void *)a_base, 0, a_bytes, 0x00020000);
        unsigned b_bytes = 0xffffffff;
        if constexpr (kTail) {
            const int64_t b_cols = (int64_t)p.n - n0;  // > 0
            b_bytes = kBT ? (unsigned)(((min((int64_t)BN, b_cols) - 1) * p.ldb + p.k) * 2) : (unsigned)((((int64_t)p.k - 1) * p.ldb + b_cols) * 2);
        }
        b_rsrc = __builtin_amdgcn_make_buffer_rsrc((void *)b_base, 0, b_bytes, 0x00020000);
    }
    const int all_k = kTail ? (p.k + BK - 1) / BK : p.k / BK;  // k tiles of the problem
    const int k_first = kSplit ? part * p.kt_per_split : 0;     // this workgroup's first
    const int num_k = kSplit ? min(p.kt_per_split, all_k - k_first) : all_k;
    const int last_k = num_k - 1;
    // 16-byte chunks of the problem's last k tile that lie inside K (all of them without a tail)
    const int tail_chunks = kTail ? (p.k - (all_k - 1) * BK) / 8 : kAChunksPerRow;
    auto issue_loads = [&](auto stage_tag, int kt) {
        NT_LDS unsigned char *sa = stage_a(stage_tag);
        NT_LDS unsigned char *sb = stage_b(stage_tag);
        kt += k_first;
        if constexpr (kLoad == 1) {
            const int a_k = kt * BK * 2;
            const int b_k = kBT ? a_k : kt * BK * (int)p.ldb * 2;
            if constexpr (kTail) {
                // the partial last k tile, without a branch: a lane whose 16-byte chunk lies beyond K reads from behind
                // the descriptor, zeros (the chunk a lane fills is the same for every instruction: their rows are a
                // multiple of the swizzle's period of 16 apart)
                constexpr unsigned kBehind = 0x7fffffffu;  // behind every descriptor (their sizes stay below 2^31)
                static_assert(kWaves * kARowsPerInstr % 16 == 0, "the swizzle of a row repeats every 16 rows");
                const int chunks = kt == all_k - 1 ? tail_chunks : kAChunksPerRow;
                const int row = wave * kARowsPerInstr + lane / kAChunksPerRow;
                const bool inside = (kTile16 ? a_phys_chunk16<BK>(row, lane % kAChunksPerRow) : a_phys_chunk<BK>(row, lane % kAChunksPerRow)) < chunks;
#pragma unroll
                for (int j = 0; j < kAInstr; ++j)
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(a_rsrc, sa + (j * kWaves + wave) * 1024, 16, inside ? a_src[j] : kBehind, a_k, 0, kAux);
#pragma unroll
                for (int j = 0; j < kBInstr; ++j)
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(b_rsrc, sb + (j * kWaves + wave) * 1024, 16, kBT && !inside ? kBehind : b_src[j], b_k, 0, kAux);
                return;
            }
#pragma unroll
            for (int j = 0; j < kAInstr; ++j)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(a_rsrc, sa + (j * kWaves + wave) * 1024, 16, a_src[j], a_k, 0, kAux);
#pragma unroll
            for (int j = 0; j < kBInstr; ++j)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(b_rsrc, sb + (j * kWaves + wave) * 1024, 16, b_src[j], b_k, 0, kAux);
        } else {
            const unsigned char *a_tile = a_base + (int64_t)kt * BK * 2;
            const unsigned char *b_tile = b_base + (kBT ? (int64_t)kt * BK * 2 : (int64_t)kt * BK * p.ldb * 2);
#pragma unroll
            for (int j = 0; j < kAInstr; ++j)
                __builtin_amdgcn_global_load_lds((const NT_GLOBAL void *)(a_tile + a_src[j]), sa + (j * kWaves + wave) * 1024, 16, 0, kAux);
#pragma unroll
            for (int j = 0; j < kBInstr; ++j)
                __builtin_amdgcn_global_load_lds((const NT_GLOBAL void *)(b_tile + b_src[j]), sb + (j * kWaves + wave) * 1024, 16, 0, kAux);
        }
    };

    // ---- LDS -> register read offsets (bytes, within a stage) ----
    const int g = lane >> 5;        // k half of the MFMA operand this lane holds
    const int l32 = lane & 31;
    int a_row_off[TM];              // byte offset of this lane's A row
    int a_row_sw[TM];               // swizzle term of that row
#pragma unroll
    for (int ti = 0; ti < TM; ++ti) {
        const int row = wave_m * kWaveM + ti * 32 + l32;
        a_row_off[ti] = row * (BK * 2);
        a_row_sw[ti] = a_phys_chunk<BK>(row, 0);
    }
    // B (transposing read): lane i of a 16-lane group addresses row i/4,
    // columns 4*(i%4).. of the group's 4(k) x 16(n) block.
    const int i16 = lane & 15;
    const int nhalf = (lane >> 4) & 1;
    const int b_krow = 8 * g + (i16 >> 2);  // + 16*ks (+4 for the upper half)
    int b_col_chunk[TN];                    // 16-byte chunk index of the column
    int b_col_in[TN];                       // byte offset inside the chunk
#pragma unroll
    for (int tj = 0; tj < TN; ++tj) {
        const int ncol = wave_n * kWaveN + tj * 32 + nhalf * 16 + 4 * (i16 & 3);
        b_col_chunk[tj] = ncol >> 3;
        b_col_in[tj] = (ncol & 7) * 2;
    }

    int bt_row_off[TN], bt_row_sw[TN];  // kBT: this lane's B row (a column of C), as for A
#pragma unroll
    for (int tj = 0; tj < TN; ++tj) {
        const int row = wave_n * kWaveN + tj * 32 + l32;
        bt_row_off[tj] = row * (BK * 2);
        bt_row_sw[tj] = a_phys_chunk<BK>(row, 0);
    }

    float16_t acc[TM][TN];
#pragma unroll
    for (int ti = 0; ti < TM; ++ti)
#pragma unroll
        for (int tj = 0; tj < TN; ++tj)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[ti][tj][r] = 0.0f;

    auto read_frags = [&](auto stage_tag, int ks, vec8 (&af)[TM], vec8 (&bf)[TN]) {
        const NT_LDS unsigned char *sa = stage_a(stage_tag);
        const NT_LDS unsigned char *sb = stage_b(stage_tag);
#pragma unroll
        for (int ti = 0; ti < TM; ++ti) {
            const int chunk = (ks * 2 + g) ^ a_row_sw[ti];
            af[ti] = *(const NT_LDS vec8 *)(sa + a_row_off[ti] + chunk * 16);
        }
#pragma unroll
        for (int tj = 0; tj < TN; ++tj) {
            if constexpr (kBT) {
                const int chunk = (ks * 2 + g) ^ bt_row_sw[tj];
                bf[tj] = *(const NT_LDS vec8 *)(sb + bt_row_off[tj] + chunk * 16);
            } else {
                const int k_lo = ks * 16 + b_krow;
                const int k_hi = k_lo + 4;
                const int c_lo = b_phys_chunk<BN>(k_lo, b_col_chunk[tj]);
                const int c_hi = b_phys_chunk<BN>(k_hi, b_col_chunk[tj]);
                short4_t lo = lds_read_tr16_b64(sb + k_lo * (BN * 2) + c_lo * 16 + b_col_in[tj]);
                short4_t hi = lds_read_tr16_b64(sb + k_hi * (BN * 2) + c_hi * 16 + b_col_in[tj]);
                short8_t both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                bf[tj] = __builtin_bit_cast(vec8, both);
            }
        }
    };

    vec8 af_once[TM];
    vec8 bf_once[TN];

    auto multiply_stage = [&](auto stage_tag) {
#pragma unroll
        for (int ks = 0; ks < BK / 16; ++ks) {
            vec8 af[TM];
            vec8 bf[TN];
            if constexpr (kAblate & 2) {
#pragma unroll
                for (int ti = 0; ti < TM; ++ti) af[ti] = af_once[ti];
#pragma unroll
                for (int tj = 0; tj < TN; ++tj) bf[tj] = bf_once[tj];
            } else {
                read_frags(stage_tag, ks, af, bf);
            }
#pragma unroll
            for (int ti = 0; ti < TM; ++ti)
#pragma unroll
                for (int tj = 0; tj < TN; ++tj) acc[ti][tj] = E::mfma32(bf[tj], af[ti], acc[ti][tj]);  // transposed tile
        }
    };

    // K loop, unrolled over the stages so every LDS array is named statically.
    // Past the end the last tile is fetched again into a stage nobody needs, which keeps the
    // outstanding-load count the same in every step.
    const int main_k = num_k - num_k % kStages;
    constexpr int KS = BK / 16;
    // kCross (rings of three or more stages): the barrier that opens the step for tile t tells that every
    // wave's fills of tile t+1 have landed (one tile EARLIER than needed for t itself) and that every wave
    // is done with tile t-1, whose stage is refilled right after it.  A wave can then fetch the operand
    // fragments of the first k step of tile t+1 during the last k step of tile t: the first MFMAs after a
    // barrier have their operands in registers, and no wave starts a step by waiting for LDS.
    constexpr bool kCross = kStages >= 3 && kAblate == 0 && KS % 2 == 0;

    // kM16: the wave's tile is computed with 16x16x32 MFMAs instead of 32x32x16 ones.  Per FLOP they move
    // half as many accumulator values through the register file, and on operands with random bits that
    // is what the power limit of the part charges for (8192^3 addmm, N(0,1) fp16: +8 %).
    constexpr bool kM16 = NT_GEMM_M16 && kAblate == 0 && BK % 32 == 0 && sizeof(T) == 2;
    constexpr int TM16 = kWaveM / 16, TN16 = kWaveN / 16, KS16 = BK / 32;
    // ... with the fragment reads of the next k step under the MFMAs of this one, across the barrier
    constexpr bool kCross16 = kM16 && kStages >= 3 && (KS16 * TM16) % 4 == 0 && TM16 >= TN16;
    float4_t acc16[kM16 ? TM16 : 1][kM16 ? TN16 : 1];
#pragma unroll
    for (int ti = 0; ti < (kM16 ? TM16 : 1); ++ti)
#pragma unroll
        for (int tj = 0; tj < (kM16 ? TN16 : 1); ++tj) acc16[ti][tj] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
    // Operand fragments of the 16x16x32 MFMA: A block ti (16 rows) is one 16-byte read per lane (row i16,
    // k chunk kg of the k step); B block tj (16 columns) is two transposing reads (16-lane group kg reads
    // k rows 8 kg .. + 7 of the k step), or, for a k-contiguous B, one read like A's.
    const int kg = lane >> 4;
    int a16_off[KS16], bt16_off[KS16];
    {
        const int a_row = wave_m * kWaveM + i16;  // + 16 * ti, which leaves the swizzle term as it is
        const int bt_row = wave_n * kWaveN + i16;
#pragma unroll
        for (int ks = 0; ks < KS16; ++ks) {
            a16_off[ks] = a_row * (BK * 2) + (a_phys_chunk16<BK>(a_row, ks * 4 + kg) * 16);
            bt16_off[ks] = bt_row * (BK * 2) + (a_phys_chunk16<BK>(bt_row, ks * 4 + kg) * 16);
        }
    }
    int b16_lo[kM16 && !kBT ? TN16 : 1], b16_hi[kM16 && !kBT ? TN16 : 1];
    if constexpr (kM16 && !kBT) {
#pragma unroll
        for (int tj = 0; tj < TN16; ++tj) {
            const int k_lo = 8 * kg + (i16 >> 2), k_hi = k_lo + 4;  // + 32 * ks: the swizzle only looks at k % 16
            const int ncol = wave_n * kWaveN + tj * 16 + 4 * (i16 & 3);
            b16_lo[tj] = k_lo * (BN * 2) + b_phys_chunk16<BN>(k_lo, ncol >> 3) * 16 + (ncol & 7) * 2;
            b16_hi[tj] = k_hi * (BN * 2) + b_phys_chunk16<BN>(k_hi, ncol >> 3) * 16 + (ncol & 7) * 2;
        }
    }
    auto read_a16 = [&](auto stage_tag, int ks, int ti) -> vec8 {
        return *(const NT_LDS vec8 *)(stage_a(stage_tag) + a16_off[ks] + ti * 16 * (BK * 2));
    };
    auto read_b16 = [&](auto stage_tag, int ks, int tj) -> vec8 {
        const NT_LDS unsigned char *sb = stage_b(stage_tag);
        if constexpr (kBT) {
            return *(const NT_LDS vec8 *)(sb + bt16_off[ks] + tj * 16 * (BK * 2));
        } else {
            short4_t lo = lds_read_tr16_b64(sb + b16_lo[kBT ? 0 : tj] + ks * 32 * (BN * 2));
            short4_t hi = lds_read_tr16_b64(sb + b16_hi[kBT ? 0 : tj] + ks * 32 * (BN * 2));
            short8_t both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
            return __builtin_bit_cast(vec8, both);
        }
    };

    if constexpr (kPairA) {
        // Tile t uses B stage t % 4 and half t % 2 of A pair stage (t / 2) % 3.  The barrier that opens step t tells that
        // tile t + 1 is complete in LDS and that every wave is done with tile t - 1; after it B of tile t + 3 is
        // requested into the stage of tile t - 1 and A of tiles t + 4, t + 5 (t even; half of it in step t, half in
        // step t + 1) into the stage of tiles t - 2, t - 1.  Stage, half, B set and A slot are compile-time constants over a body of 12 steps.
        const int last_pair = last_k >> 1;
        int a16p_off[2];
        {
            const int a_row = wave_m * kWaveM + i16;  // + 16 * ti, which leaves the swizzle term as it is
#pragma unroll
            for (int h = 0; h < 2; ++h) a16p_off[h] = a_row * 128 + a_phys_chunk16<64>(a_row, 4 * h + kg) * 16;
        }
        auto read_a_pair = [&](auto stage_tag, int half, int ti) -> vec8 {
            return *(const NT_LDS vec8 *)(stage_a(stage_tag) + a16p_off[half] + ti * 16 * 128);
        };
        // (kTail: 16-byte chunks of the last pair that lie inside K; the others must read as zeros, see kTail above)
        const int pair_chunks = kTail ? min(8, (p.k - last_pair * 64) / 8) : 8;
        auto issue_a_pair = [&](auto stage_tag, int pair, auto first_tag, auto last_tag) {
            constexpr int kFirst = decltype(first_tag)::value, kLast = decltype(last_tag)::value;  // instructions [kFirst, kLast) of the pair
            NT_LDS unsigned char *sa = stage_a(stage_tag);
            if constexpr (kTail) {
                // no branch: a lane whose chunk lies beyond K in the last pair reads from behind the descriptor
                // (the chunk a lane fills is the same for every instruction: their rows are 8 * kWaves apart)
                constexpr unsigned kBehind = 0x7fffffffu;  // behind every descriptor (their sizes stay below 2^31)
                const int chunks = pair == last_pair ? pair_chunks : 8;
                const bool inside = a_phys_chunk16<64>(wave * 8 + lane / 8, lane % 8) < chunks;
                static_assert(kWaves * 8 % 16 == 0, "the swizzle of a row repeats every 16 rows");
#pragma unroll
                for (int j = kFirst; j < kLast; ++j)
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(a_rsrc, sa + (j * kWaves + wave) * 1024, 16, inside ? a_pair_src[j] : kBehind, pair * 128, 0, kAux);
                return;
            }
#pragma unroll
            for (int j = kFirst; j < kLast; ++j)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(a_rsrc, sa + (j * kWaves + wave) * 1024, 16, a_pair_src[j], pair * 128, 0, kAux);
        };
        typedef std::integral_constant<int, 0> I0;
        typedef std::integral_constant<int, kPairInstr / 2> IHalf;
        typedef std::integral_constant<int, kPairInstr> IAll;
        auto issue_b = [&](auto stage_tag, int kt) {
            NT_LDS unsigned char *sb = stage_b(stage_tag);
            const int b_k = kBT ? kt * BK * 2 : kt * BK * (int)p.ldb * 2;
            if constexpr (kTail && kBT) {  // the partial last k tile of a k-contiguous rhs, without a branch (see issue_a_pair)
                constexpr unsigned kBehind = 0x7fffffffu;
                static_assert(kWaves * kARowsPerInstr % 16 == 0, "the swizzle of a row repeats every 16 rows");
                const int chunks = kt == last_k ? tail_chunks : kAChunksPerRow;
                const bool inside = a_phys_chunk16<BK>(wave * kARowsPerInstr + lane / kAChunksPerRow, lane % kAChunksPerRow) < chunks;
#pragma unroll
                for (int j = 0; j < kBInstr; ++j)
                    __builtin_amdgcn_raw_ptr_buffer_load_lds(b_rsrc, sb + (j * kWaves + wave) * 1024, 16, inside ? b_src[j] : kBehind, b_k, 0, kAux);
                return;
            }
#pragma unroll
            for (int j = 0; j < kBInstr; ++j)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(b_rsrc, sb + (j * kWaves + wave) * 1024, 16, b_src[j], b_k, 0, kAux);
        };
        typedef std::integral_constant<int, 0> S0;
        typedef std::integral_constant<int, 1> S1;
        typedef std::integral_constant<int, 2> S2;
        // (in the order of the steps: the last requests before step 0 are half a pair and a tile of B, as after any step)
        issue_a_pair(S0(), 0, I0(), IAll());
        issue_a_pair(S1(), min(1, last_pair), I0(), IHalf());
        issue_b(S0(), 0);
        issue_b(S1(), min(1, last_k));
        issue_a_pair(S1(), min(1, last_pair), IHalf(), IAll());
        issue_b(S2(), min(2, last_k));
        vec8 as[4];
        vec8 bs[2][TN16];
        wait_vmcnt<2 * kBInstr + kPairInstr / 2>();
        lds_barrier();
#pragma unroll
        for (int tj = 0; tj < TN16; ++tj) bs[0][tj] = read_b16(S0(), 0, tj);
        as[0] = read_a_pair(S0(), 0, 0);
        as[1] = read_a_pair(S0(), 0, 1);
        auto step = [&](auto i_tag, int kt) {
            constexpr int kI = decltype(i_tag)::value;  // position in the body of 12 steps
            typedef std::integral_constant<int, (kI / 2) % 3> PairStage;
            typedef std::integral_constant<int, ((kI + 1) / 2) % 3> NextPairStage;
            typedef std::integral_constant<int, (kI + 1) % 4> NextStageB;
            constexpr int half = kI & 1, next_half = half ^ 1;
            constexpr int cur = kI & 1, nxt = cur ^ 1;
            // the pair that becomes free in an even step is requested half in that step, half in the next one
            constexpr int kFillsOfStep = kPairInstr / 2 + kBInstr;
            wait_vmcnt<kPairInstr / 2 + kBInstr>();  // in flight across the barrier: what the step before requested
            lds_barrier_reads_in_flight();
            if constexpr (half == 0) issue_a_pair(std::integral_constant<int, (kI / 2 + 2) % 3>(), min((kt + kI) / 2 + 2, last_pair), I0(), IHalf());
            else issue_a_pair(std::integral_constant<int, (kI / 2 + 2) % 3>(), min((kt + kI) / 2 + 2, last_pair), IHalf(), IAll());
            issue_b(std::integral_constant<int, (kI + 3) % 4>(), min(kt + kI + 3, last_k));
            static_for<0, TM16>([&](auto q_tag) {
                constexpr int q = decltype(q_tag)::value;
                constexpr bool kReadsB = q >= TM16 - TN16;
                if constexpr (q + 2 < TM16) as[(q + 2) % 4] = read_a_pair(PairStage(), half, q + 2);
                else as[(q + 2) % 4] = read_a_pair(NextPairStage(), next_half, q + 2 - TM16);
                if constexpr (kReadsB) bs[nxt][q - (TM16 - TN16)] = read_b16(NextStageB(), 0, q - (TM16 - TN16));
#pragma unroll
                for (int tj = 0; tj < TN16; ++tj) acc16[q][tj] = E::mfma16(bs[cur][tj], as[q % 4], acc16[q][tj]);  // transposed block
#if NT_GEMM_SCHEDULE
                constexpr int kReads = 1 + (kReadsB ? (kBT ? 1 : 2) : 0);
                static_for<0, TN16>([&](auto j_tag) {
                    constexpr int j = decltype(j_tag)::value;
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    if constexpr (j < kReads) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                    if constexpr (j == 1 && q < kFillsOfStep) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
                });
#endif
            });
        };
        constexpr int kBody = 12;
        const int body_k = num_k - num_k % kBody;
        for (int kt = 0; kt < body_k; kt += kBody) {
            static_for<0, kBody>([&](auto i) { step(i, kt); });
        }
        static_for<0, kBody - 1>([&](auto i) {
            if (body_k + (int)decltype(i)::value < num_k) step(i, body_k);
        });
    }
    if constexpr (!kPairA) static_for<0, kStages - 1>([&](auto s) { issue_loads(s, min((int)decltype(s)::value, last_k)); });
    if constexpr (kPairA) {
        // (done above)
    } else if constexpr (kCross16) {
        // All TN16 B fragments of a k step stay in registers (two sets, taking turns k step by k step); the
        // A fragments stream through four slots, each read two blocks ahead of its MFMAs.
        constexpr int Q = KS16 * TM16;  // A fragments of a k tile, in the order they are used
        vec8 as[4];
        vec8 bs[2][TN16];
        wait_vmcnt<(kStages - 2) * kLoadsPerTile>();
        lds_barrier();
#pragma unroll
        for (int tj = 0; tj < TN16; ++tj) bs[0][tj] = read_b16(std::integral_constant<int, 0>(), 0, tj);
        as[0] = read_a16(std::integral_constant<int, 0>(), 0, 0);
        as[1] = read_a16(std::integral_constant<int, 0>(), 1 / TM16, 1 % TM16);
        auto step = [&](auto i_tag, int kt) {
            constexpr int kI = decltype(i_tag)::value;  // position in the unrolled loop body: stage and B set follow from it
            constexpr int kS = kI % kStages;
            typedef std::integral_constant<int, kS> Stage;
            typedef std::integral_constant<int, (kS + 1) % kStages> NextStage;
            wait_vmcnt<(kStages - 3) * kLoadsPerTile>();
            lds_barrier_reads_in_flight();
            issue_loads(std::integral_constant<int, (kS + kStages - 1) % kStages>(), min(kt + kI + kStages - 1, last_k));
            static_for<0, Q>([&](auto q_tag) {
                constexpr int q = decltype(q_tag)::value;
                constexpr int ks = q / TM16, ti = q % TM16;
                constexpr int cur = (kI * KS16 + ks) & 1, nxt = cur ^ 1;
                constexpr int kBReadsPerBlock = kBT ? 1 : 2;
                constexpr bool kReadsB = ti >= TM16 - TN16;
                if constexpr (q + 2 < Q) as[(q + 2) % 4] = read_a16(Stage(), (q + 2) / TM16, (q + 2) % TM16);
                else as[(q + 2) % 4] = read_a16(NextStage(), (q + 2 - Q) / TM16, (q + 2 - Q) % TM16);
                if constexpr (kReadsB) {
                    constexpr int tj = ti - (TM16 - TN16);
                    if constexpr (ks + 1 < KS16) bs[nxt][tj] = read_b16(Stage(), ks + 1, tj);
                    else bs[nxt][tj] = read_b16(NextStage(), 0, tj);
                }
#pragma unroll
                for (int tj = 0; tj < TN16; ++tj) acc16[ti][tj] = E::mfma16(bs[cur][tj], as[q % 4], acc16[ti][tj]);  // transposed block
#if NT_GEMM_SCHEDULE
                // issue order: reads and ring refills spread under the MFMAs
                constexpr int kReads = 1 + (kReadsB ? kBReadsPerBlock : 0);
                constexpr int kFillsPer = (kLoadsPerTile + Q - 1) / Q;
                constexpr int kFills = q * kFillsPer < kLoadsPerTile ? (kLoadsPerTile - q * kFillsPer < kFillsPer ? kLoadsPerTile - q * kFillsPer : kFillsPer) : 0;
                static_for<0, TN16>([&](auto j_tag) {
                    constexpr int j = decltype(j_tag)::value;
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    if constexpr (TN16 >= kReads) {
                        if constexpr (j < kReads) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
                    } else if constexpr (j == 0) {
                        __builtin_amdgcn_sched_group_barrier(0x100, kReads, 0);
                    }
                    if constexpr (j == (TN16 > 1 ? 1 : 0) && kFills > 0) __builtin_amdgcn_sched_group_barrier(0x020, kFills, 0);
                });
#endif
            });
        };
        // (with an odd number of k steps per tile the B sets are back in place after an even number of tiles)
        constexpr int kBody = (KS16 & 1) ? 2 * kStages : kStages;
        const int body_k = num_k - num_k % kBody;
        for (int kt = 0; kt < body_k; kt += kBody) {
            static_for<0, kBody>([&](auto i) { step(i, kt); });
        }
        static_for<0, kBody - 1>([&](auto i) {
            if (body_k + (int)decltype(i)::value < num_k) step(i, body_k);
        });
    } else if constexpr (kM16) {
        auto step = [&](auto s, int kt) {
            constexpr int kS = decltype(s)::value;
            wait_vmcnt<(kStages - 2) * kLoadsPerTile>();
            lds_barrier();
            issue_loads(std::integral_constant<int, (kS + kStages - 1) % kStages>(), min(kt + kS + kStages - 1, last_k));
#pragma unroll
            for (int ks = 0; ks < KS16; ++ks) {
                vec8 bfr[TN16];
#pragma unroll
                for (int tj = 0; tj < TN16; ++tj) bfr[tj] = read_b16(s, ks, tj);
#pragma unroll
                for (int ti = 0; ti < TM16; ++ti) {
                    const vec8 afr = read_a16(s, ks, ti);
#pragma unroll
                    for (int tj = 0; tj < TN16; ++tj) acc16[ti][tj] = E::mfma16(bfr[tj], afr, acc16[ti][tj]);  // transposed block
                }
            }
        };
        for (int kt = 0; kt < main_k; kt += kStages) {
            static_for<0, kStages>([&](auto s) { step(s, kt); });
        }
        static_for<0, kStages - 1>([&](auto s) {
            if (main_k + (int)decltype(s)::value < num_k) step(s, main_k);
        });
    }
    if constexpr (kAblate & 2) {
        wait_vmcnt<0>();
        lds_barrier();
        read_frags(std::integral_constant<int, 0>(), 0, af_once, bf_once);
    }
    if constexpr (kM16) {
        // (done above)
    } else if constexpr (kCross) {
        vec8 af[2][TM];
        vec8 bf[2][TN];
        wait_vmcnt<(kStages - 2) * kLoadsPerTile>();
        lds_barrier();
        read_frags(std::integral_constant<int, 0>(), 0, af[0], bf[0]);
        auto step = [&](auto s, int kt) {
            constexpr int kS = decltype(s)::value;
            typedef std::integral_constant<int, (kS + 1) % kStages> NextStage;
            // (the reads in flight here fetch the first k step of this step's own tile; the stage refilled
            // below belongs to the tile before it, whose reads fed MFMAs that have been issued)
            wait_vmcnt<(kStages - 3) * kLoadsPerTile>();
            lds_barrier_reads_in_flight();
            issue_loads(std::integral_constant<int, (kS + kStages - 1) % kStages>(), min(kt + kS + kStages - 1, last_k));
            static_for<0, KS>([&](auto ks_tag) {
                constexpr int ks = decltype(ks_tag)::value;
                constexpr int cur = ks & 1, nxt = cur ^ 1;
                if constexpr (ks + 1 < KS) read_frags(s, ks + 1, af[nxt], bf[nxt]);
                else read_frags(NextStage(), 0, af[nxt], bf[nxt]);
#pragma unroll
                for (int ti = 0; ti < TM; ++ti)
#pragma unroll
                    for (int tj = 0; tj < TN; ++tj) acc[ti][tj] = E::mfma32(bf[cur][tj], af[cur][ti], acc[ti][tj]);  // transposed tile
#if NT_GEMM_SCHEDULE
                // issue order: the fragment reads of the next k step (and, in a step's first k step, the
                // refills of the ring) spread under this k step's MFMAs
                constexpr int kReads = TM + (kBT ? TN : 2 * TN);
                constexpr int kFills = ks == 0 ? kLoadsPerTile : 0;
                static_for<0, TM * TN>([&](auto i_tag) {
                    constexpr int i = decltype(i_tag)::value;
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    constexpr int kPer = (kReads + TM * TN - 1) / (TM * TN);
                    if constexpr (i * kPer < kReads) __builtin_amdgcn_sched_group_barrier(0x100, kPer, 0);
                    if constexpr (i < kFills) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);
                });
#endif
            });
        };
        for (int kt = 0; kt < main_k; kt += kStages) {
            static_for<0, kStages>([&](auto s) { step(s, kt); });
        }
        static_for<0, kStages - 1>([&](auto s) {
            if (main_k + (int)decltype(s)::value < num_k) step(s, main_k);
        });
    } else {
        // Step for tile t: wait until tile t has landed, barrier (which also tells
        // that all waves finished tile t-1), refill the stage tile t-1 used with
        // tile t+kStages-1, multiply tile t.
        auto step = [&](auto s, int kt) {
            constexpr int kS = decltype(s)::value;
            wait_vmcnt<(kAblate & 1) ? 0 : (kStages - 2) * kLoadsPerTile>();
            lds_barrier();
            if constexpr (!(kAblate & 1))
                issue_loads(std::integral_constant<int, (kS + kStages - 1) % kStages>(), min(kt + kS + kStages - 1, last_k));
            multiply_stage(s);
        };
        for (int kt = 0; kt < main_k; kt += kStages) {
            static_for<0, kStages>([&](auto s) { step(s, kt); });
        }
        // remaining num_k % kStages tiles continue the stage rotation
        static_for<0, kStages - 1>([&](auto s) {
            if (main_k + (int)decltype(s)::value < num_k) step(s, main_k);
        });
    }

    // ---- epilogue ----
    // The accumulators hold C transposed per 32x32 tile: lane (l32, g) has, in
    // registers 4*r4 .. 4*r4+3, the columns 8*r4 + 4*g .. +3 of row l32.  Each
    // wave passes its tile through its own LDS slab 32 rows at a time, so that
    // global stores (and addmm input loads) are 16 bytes per lane and cover
    // whole 128-byte lines.  (All fills have landed and all waves are done with
    // the stages before the slabs overwrite them.)
    // (fp32 output, matmul and split-K parts only, takes the same route with rows twice as long.)
    static_assert(!(kFloatOut && kAddmm), "the fp32 output path has no addmm epilogue");
    using TOut = std::conditional_t<kFloatOut, float, T>;
    constexpr int kChunkElems = 16 / (int)sizeof(TOut);
    constexpr int kRowBytes = kWaveN * (int)sizeof(TOut);
    constexpr int kCChunks = kRowBytes / 16;  // 16-byte chunks per slab row
    constexpr int kCShift = kRowBytes >= 256 ? 0 : (kRowBytes == 128 ? 1 : 2);
    // the slabs live in the (now idle) stage memory: A0, B0, A1, B1 in this order
    constexpr int kSlabBytes = 32 * kRowBytes;
    constexpr int kSlabsA = kStageA / kSlabBytes;
    constexpr int kSlabsB = kStageB / kSlabBytes;
    static_assert(kWaves <= 2 * (kSlabsA + kSlabsB), "epilogue slabs do not fit two stages");
    wait_vmcnt<0>();
    lds_barrier();
    NT_LDS unsigned char *slab;
    {
        int w = wave;
        if (w < kSlabsA) {
            slab = (NT_LDS unsigned char *)lds_a0;
        } else if ((w -= kSlabsA) < kSlabsB) {
            slab = (NT_LDS unsigned char *)lds_b0;
        } else if ((w -= kSlabsB) < kSlabsA) {
            slab = (NT_LDS unsigned char *)lds_a1;
        } else {
            w -= kSlabsA;
            slab = (NT_LDS unsigned char *)lds_b1;
        }
        slab += w * kSlabBytes;
    }
    TOut *C = (TOut *)p.c + (kSplit ? (int64_t)part * p.m * p.ldc : batch * p.c_batch);
    const T *bias = (const T *)p.bias + batch * p.bias_batch;
    typedef TOut vec_out __attribute__((ext_vector_type(kChunkElems)));
    const int slab_sw = (l32 >> kCShift) & (kCChunks - 1);
#pragma unroll
    for (int ti = 0; ti < TM; ++ti) {
        if constexpr (kM16) {
            // 16x16 blocks: lane (i16, kg) holds columns 4 kg .. + 3 of row i16; two blocks of rows fill a slab
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                const int row = half * 16 + i16;
                const int sw = (row >> kCShift) & (kCChunks - 1);
#pragma unroll
                for (int tj = 0; tj < TN16; ++tj) {
                    typedef TOut vec4 __attribute__((ext_vector_type(4)));
                    const float4_t a4 = acc16[kM16 ? 2 * ti + half : 0][kM16 ? tj : 0];
                    vec4 v;
                    if constexpr (kFloatOut) {
#pragma unroll
                        for (int e = 0; e < 4; ++e) v[e] = a4[e];
                        *(NT_LDS vec4 *)(slab + row * kRowBytes + ((tj * 4 + kg) ^ sw) * 16) = v;
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e) v[e] = E::from_float(a4[e]);
                        *(NT_LDS vec4 *)(slab + row * kRowBytes + ((tj * 2 + (kg >> 1)) ^ sw) * 16 + 8 * (kg & 1)) = v;
                    }
                }
            }
        } else
#pragma unroll
        for (int tj = 0; tj < TN; ++tj) {
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                typedef TOut vec4 __attribute__((ext_vector_type(4)));
                vec4 v;
                if constexpr (kFloatOut) {  // four columns are one chunk
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] = acc[ti][tj][4 * r4 + e];
                    const int chunk = (2 * (tj * 4 + r4) + g) ^ slab_sw;
                    *(NT_LDS vec4 *)(slab + l32 * kRowBytes + chunk * 16) = v;
                } else {  // ... half a chunk
#pragma unroll
                    for (int e = 0; e < 4; ++e) v[e] = E::from_float(acc[ti][tj][4 * r4 + e]);
                    const int chunk = (tj * 4 + r4) ^ slab_sw;
                    *(NT_LDS vec4 *)(slab + l32 * kRowBytes + chunk * 16 + 8 * g) = v;
                }
            }
        }
#pragma unroll
        for (int it = 0; it < kCChunks / 2; ++it) {
            const int idx = it * 64 + lane;
            const int row = idx / kCChunks;
            const int phys = idx % kCChunks;
            const int chunk = phys ^ ((row >> kCShift) & (kCChunks - 1));
            vec_out v = *(const NT_LDS vec_out *)(slab + row * kRowBytes + phys * 16);
            const int grow = m0 + wave_m * kWaveM + ti * 32 + row;
            const int gcol = n0 + wave_n * kWaveN + chunk * kChunkElems;
            if (grow >= p.m) continue;  // a partial last tile of rows
            if (kTail && gcol >= p.n) continue;  // ... of columns (with vector stores N is a multiple of 8: whole chunks)
            if constexpr (kAddmm) {
                // the matmul result was rounded to the element type; beta, alpha
                // are fp32 scalars, so the combination happens in fp32
                const T *src = bias + (int64_t)grow * p.bias_stride_m + (int64_t)gcol * p.bias_stride_n;
                vec8 in;
                if (p.bias_vector) {
                    in = *(const vec8 *)src;
                } else if (p.bias_stride_n == 1 && (!kTail || gcol + 8 <= p.n)) {
                    // a whole chunk of a row that does not start on a 16-byte boundary: one load all the same
                    // (global accesses need no more than the element's alignment)
                    typedef vec8 unaligned_vec8 __attribute__((aligned(2)));
                    in = *(const unaligned_vec8 *)src;
                } else {
#pragma unroll
                    for (int e = 0; e < 8; ++e) in[e] = (!kTail || gcol + e < p.n) ? src[(int64_t)e * p.bias_stride_n] : E::from_float(0.0f);
                }
#pragma unroll
                for (int e = 0; e < 8; ++e) v[e] = E::from_float(p.beta * E::to_float(in[e]) + p.alpha * E::to_float(v[e]));
            }
            if (kTail && !p.c_vector) {  // N or the row pitch of C no multiple of 8
                if (gcol + kChunkElems <= p.n) {  // a whole chunk, only not on a 16-byte boundary
                    typedef vec_out unaligned_vec_out __attribute__((aligned(sizeof(TOut))));
                    *(unaligned_vec_out *)(C + (int64_t)grow * p.ldc + gcol) = v;
                    continue;
                }
#pragma unroll
                for (int e = 0; e < kChunkElems; ++e)  // the row's last, partial chunk: element by element
                    if (gcol + e < p.n) C[(int64_t)grow * p.ldc + gcol + e] = v[e];
                continue;
            }
            // non-temporal: C is not read again, and its lines then do not displace A / B panels in L2
            // (4096^3 addmm +3 %, 8192^3 +0.3 %)
            __builtin_nontemporal_store(v, (vec_out *)(C + (int64_t)grow * p.ldc + gcol));
        }
    }
#endif
}

}  // namespace nt
