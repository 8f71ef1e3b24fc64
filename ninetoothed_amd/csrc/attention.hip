// Fused scaled-dot-product attention forward for gfx950 (flash-attention style
// online softmax, fp16/bf16 operands, fp32 accumulation on 32x32x16 MFMA).
//
// One workgroup = 4 waves handles kQTiles * 128 query rows of one (batch, head);
// each wave owns kQTiles * 32 query rows and walks all key/value blocks of 64
// rows.  Everything is computed TRANSPOSED so that a lane owns one query row:
//   S^T[kv, q] = K[kv, :] . Q'[q, :]          (A operand = K from LDS, B = Q' in registers)
//   O^T[d, q] += V^T[d, kv] . P^T[kv, q]      (A operand = V via transposing LDS reads,
//                                              B = P^T straight from the S^T accumulators)
// With this orientation the row max / row sum of the online softmax are
// reductions over a lane's own registers plus one exchange with lane ^ 32, and
// the MFMA accumulator layout of S^T is already the operand layout of P^T
// (the 8 contraction slots of a lane map to kv rows {4g..4g+3, 8+4g..8+4g+3};
// V^T is read with the same slot order, which a sum does not care about).
//
// Q' = round_to_elem(Q * scale * log2(e)); probabilities are exp2 of the
// difference to the running row maximum.
#include <type_traits>

#include <algorithm>

#include "gemm_fast.h"  // swizzle helpers, static_for, lds_barrier
#include "tune.h"
#include "workspace.h"

namespace nt {
namespace {

struct AttentionParams {
    const void *q, *k, *v;
    void *o;
    int batch, heads, seq_q, seq_k;
    int64_t q_strides[3], k_strides[3], v_strides[3], o_strides[3];  // batch, head, seq (head_dim stride is 1)
    float q_scale;  // scale * log2(e)
    int causal;
    int q_blocks;
    int head_dim;  // elements per row in memory (a multiple of 8; the kernel's D when it is not padded)
    // split key range: the grid holds `parts` workgroups per (batch, head, query block); part s takes key
    // blocks [s * blocks_per_part, ...) and writes a normalised fp32 partial output and the base-2
    // logarithm of its softmax denominator (times 2^max) to scratch memory, which a second kernel merges
    int parts, blocks_per_part;
    float *part_o;    // [parts][batch * heads][seq_q][D]
    float *part_lse;  // [parts][batch * heads][seq_q]
#ifdef NT_ATTN_STAMPS
    unsigned long long *stamps;  // measurement builds: per wave {entry to loop, loop, epilogue} in 10 ns units and the loop in clocks
#endif
};

#ifdef NT_ATTN_STAMPS
unsigned long long *g_attn_stamps = nullptr;
#endif

constexpr int kAttnWaves = 4;

// BN: key/value rows per block; kOcc: waves per SIMD the register budget is held to;
// kPipelined: overlap the softmax of a block with the MFMAs of its neighbours
// TIO: element type of Q and O in memory -- T, or float for fp32 tensors (their K and V
// are converted to T beforehand; Q is converted while it is scaled, O is stored unrounded)
// kPadded: the head dimension in memory (p.head_dim, a multiple of 8) is smaller than D: the missing
// columns of Q, K and V read as zeros (scores and the stored columns are unchanged by them)
template <typename T, int D, int kQTiles, int BN, int kOcc, bool kPipelined, typename TIO = T, int kWaves = kAttnWaves, bool kPadded = false, bool kSplitKV = false, bool kFold = true>
__global__ __launch_bounds__(kWaves * 64, kOcc) void attention_fwd_kernel(AttentionParams p) {
    static_assert(!kSplitKV || !kPipelined, "the key range is split in the plain loop only");
#if defined(__HIP_DEVICE_COMPILE__)
    typedef Elem<T> E;
    typedef typename E::vec8 vec8;
    constexpr int BM = kWaves * 32 * kQTiles;
    constexpr int KT = BN / 32;          // kv tiles of S^T per block
    constexpr int DT = D / 32;           // d tiles of O^T
    constexpr int KS = D / 16;           // contraction steps of S^T
    constexpr int PS = BN / 16;          // contraction steps of O^T
    constexpr int kTileBytes = BN * D * 2;
    constexpr int kChunksPerRow = D / 8;
    constexpr int kRowsPerInstr = 64 / kChunksPerRow;
    constexpr int kInstr = kTileBytes / (kWaves * 1024);
    static_assert(D % 32 == 0 && D >= 32 && D <= 256, "head dim");
    static_assert(kTileBytes % (kWaves * 1024) == 0, "tile/wave mismatch");

    __shared__ __attribute__((aligned(1024))) unsigned char lds_k0[kTileBytes];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_v0[kTileBytes];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_k1[kTileBytes];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_v1[kTileBytes];
    auto stage_k = [&](auto tag) __attribute__((always_inline)) -> NT_LDS unsigned char * {
        if constexpr (decltype(tag)::value == 0) return (NT_LDS unsigned char *)lds_k0;
        else return (NT_LDS unsigned char *)lds_k1;
    };
    auto stage_v = [&](auto tag) __attribute__((always_inline)) -> NT_LDS unsigned char * {
        if constexpr (decltype(tag)::value == 0) return (NT_LDS unsigned char *)lds_v0;
        else return (NT_LDS unsigned char *)lds_v1;
    };

#ifdef NT_ATTN_STAMPS
    const unsigned long long real_entry = __builtin_amdgcn_s_memrealtime();
#endif
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int g = lane >> 5;
    const int l32 = lane & 31;

    // workgroup -> (batch, head, query block).  Hardware workgroup ids are dealt
    // round-robin to the 8 XCDs, each with its own L2, so ids are first renumbered to
    // give every XCD a contiguous range.
    // Non-causal: consecutive ids are the query blocks of one (batch, head): they run
    // on one XCD and its K/V are fetched from HBM once, not once per XCD.
    // Causal: the work of a query block grows with its index, so inside an XCD's range
    // ids walk groups of kCausalGroup (batch, head) pairs, and inside a group the query
    // blocks from last (longest) to first, pair by pair: a CU gets a mix of long and
    // short blocks while only the K/V of one group (plus the next one's beginning)
    // is live in the XCD's L2.  Pair counts that are no multiple of 8 walk pair by pair.
    constexpr int kCausalGroup = 4;
    const int total = kSplitKV ? gridDim.x / p.parts : gridDim.x;
    const int part = kSplitKV ? blockIdx.x / total : 0;
    int wg = kSplitKV ? blockIdx.x - part * total : blockIdx.x;
    const bool renumber = total % 8 == 0;
    if (renumber) wg = (wg & 7) * (total >> 3) + (wg >> 3);
    int qb, bh;
    if (p.causal) {
        const int pairs = p.batch * p.heads;
        if (renumber && pairs % 8 == 0) {
            // (fewer pairs per XCD than a group: groups of two, or single pairs -- eight heads of a long sequence then
            // run one per XCD, whose CUs stream that head's K / V together instead of eight heads' at once)
            const int per_xcd = pairs >> 3;
            const int in_a_group = per_xcd % kCausalGroup == 0 ? kCausalGroup : (per_xcd % 2 == 0 ? 2 : 1);
            const int per_group = in_a_group * p.q_blocks;
            const int group = wg / per_group;
            const int in_group = wg % per_group;
            qb = p.q_blocks - 1 - in_group / in_a_group;
            bh = group * in_a_group + in_group % in_a_group;
        } else {
            // pair by pair, each from its longest block down: ids that run at one time belong to one or two pairs
            qb = p.q_blocks - 1 - wg % p.q_blocks;
            bh = wg / p.q_blocks;
        }
    } else {
        qb = wg % p.q_blocks;
        bh = wg / p.q_blocks;
    }
    const int head = bh % p.heads;
    const int batch = bh / p.heads;
    const int q0 = qb * BM;

    const TIO *Q = (const TIO *)p.q + batch * p.q_strides[0] + head * p.q_strides[1];
    const T *K = (const T *)p.k + batch * p.k_strides[0] + head * p.k_strides[1];
    const T *V = (const T *)p.v + batch * p.v_strides[0] + head * p.v_strides[1];
    TIO *O = (TIO *)p.o + batch * p.o_strides[0] + head * p.o_strides[1];

    // ---- Q' fragments (B operand of S^T): lane holds row l32 of its q tile, 8 d's per step ----
    vec8 qf[kQTiles][KS];
    int q_row[kQTiles];
#pragma unroll
    for (int qt = 0; qt < kQTiles; ++qt) {
        q_row[qt] = q0 + (wave * kQTiles + qt) * 32 + l32;
        const int row = min(q_row[qt], p.seq_q - 1);
        const TIO *src = Q + (int64_t)row * p.q_strides[2];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            vec8 raw;
            if (kPadded && ks * 16 + 8 * g >= p.head_dim) {
#pragma unroll
                for (int e = 0; e < 8; ++e) raw[e] = E::from_float(0.0f);
            } else if constexpr (std::is_same<TIO, float>::value) {
                const float4_t lo = *(const float4_t *)(src + ks * 16 + 8 * g);
                const float4_t hi = *(const float4_t *)(src + ks * 16 + 8 * g + 4);
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    raw[e] = E::from_float(lo[e] * p.q_scale);
                    raw[4 + e] = E::from_float(hi[e] * p.q_scale);
                }
            } else {
                raw = *(const vec8 *)(src + ks * 16 + 8 * g);  // (scaled below, once the first K blocks have been requested)
            }
            qf[qt][ks] = raw;
        }
    }
    // Q' = round(Q * scale * log2 e).  Called after the first K / V blocks have been requested, so that the queries and
    // those blocks are on their way at the same time (the multiplication is the first thing that waits for the queries).
    auto scale_queries = [&]() __attribute__((always_inline)) {
        if constexpr (!std::is_same<TIO, float>::value) {
#pragma unroll
            for (int qt = 0; qt < kQTiles; ++qt)
#pragma unroll
                for (int ks = 0; ks < KS; ++ks) {
                    if (kPadded && ks * 16 + 8 * g >= p.head_dim) continue;  // (zeros stay zeros)
#pragma unroll
                    for (int e = 0; e < 8; ++e) qf[qt][ks][e] = E::from_float(E::to_float(qf[qt][ks][e]) * p.q_scale);
                }
        }
    };

    // ---- number of kv blocks this query block needs ----
    int kv_end = p.seq_k;
    if (p.causal) kv_end = min(kv_end, q0 + BM);  // keys beyond the last query row are masked for all rows
    int num_blocks = ceil_div(kv_end, BN);  // one past the last key block of this workgroup
    int first_block = 0;
    if constexpr (kSplitKV) {
        first_block = part * p.blocks_per_part;
        num_blocks = min(num_blocks, first_block + p.blocks_per_part);  // may leave nothing (causal: parts past the diagonal)
    }
    const int last_block = num_blocks - 1;

    // ---- global -> LDS assignment ----
    // K and V of this (batch, head) are addressed through buffer descriptors that
    // end with the last key row: the per-lane byte offset is fixed for the whole
    // kernel, the block offset travels in a scalar register, and rows past the end
    // of the sequence read as zeros (the range check covers the scalar offset too).
    const int row_elements = kPadded ? p.head_dim : D;
    const unsigned k_bytes = (unsigned)((p.seq_k - 1) * p.k_strides[2] + row_elements) * 2u;
    const unsigned v_bytes = (unsigned)((p.seq_k - 1) * p.v_strides[2] + row_elements) * 2u;
    __amdgpu_buffer_rsrc_t k_rsrc = __builtin_amdgcn_make_buffer_rsrc((void *)K, 0, k_bytes, 0x00020000);
    __amdgpu_buffer_rsrc_t v_rsrc = __builtin_amdgcn_make_buffer_rsrc((void *)V, 0, v_bytes, 0x00020000);
    const unsigned k_block_bytes = (unsigned)(BN * p.k_strides[2]) * 2u;
    const unsigned v_block_bytes = (unsigned)(BN * p.v_strides[2]) * 2u;
    // load instruction j of a wave covers the rows kLoadRowStep * j further down; where the
    // swizzle repeats with that period, one lane offset serves every j and the
    // row step goes into the scalar offset as well (K rows of 256 elements: one offset per j).
    // Padded rows: a lane whose 16-byte chunk starts past the row's end gets an offset behind the
    // descriptor (these stay below 2^31 bytes, checked on the host) and so fetches zeros.
    constexpr int kLoadRowStep = kWaves * kRowsPerInstr;
    constexpr bool kPeriodicK = a_phys_chunk<D>(kLoadRowStep, 0) == 0;
    constexpr int kOffsetsK = kPeriodicK ? 1 : kInstr;
    static_assert(b_phys_chunk<D>(kLoadRowStep, 0) == 0, "swizzle period");
    const unsigned k_step_bytes = (unsigned)(kLoadRowStep * p.k_strides[2]) * 2u;
    const unsigned v_step_bytes = (unsigned)(kLoadRowStep * p.v_strides[2]) * 2u;
    constexpr unsigned kBehind = 0x80000000u;
    unsigned ld_k_off[kOffsetsK], ld_v_off;
    {
        const int phys = lane % kChunksPerRow;
#pragma unroll
        for (int j = 0; j < kOffsetsK; ++j) {
            const int row = (j * kWaves + wave) * kRowsPerInstr + lane / kChunksPerRow;
            const int chunk = a_phys_chunk<D>(row, phys);
            ld_k_off[j] = ((unsigned)row * (unsigned)p.k_strides[2] + chunk * 8) * 2u;
            if (kPadded && chunk * 8 >= p.head_dim) ld_k_off[j] = kBehind;
        }
        const int row = wave * kRowsPerInstr + lane / kChunksPerRow;
        const int chunk = b_phys_chunk<D>(row, phys);
        ld_v_off = ((unsigned)row * (unsigned)p.v_strides[2] + chunk * 8) * 2u;
        if (kPadded && chunk * 8 >= p.head_dim) ld_v_off = kBehind;
    }
    auto issue_k = [&](auto stage_tag, int blk) __attribute__((always_inline)) {
        NT_LDS unsigned char *sk = stage_k(stage_tag);
        const unsigned block_off = (unsigned)blk * k_block_bytes;
#pragma unroll
        for (int j = 0; j < kInstr; ++j) {
            if constexpr (kPeriodicK)
                __builtin_amdgcn_raw_ptr_buffer_load_lds(k_rsrc, sk + (j * kWaves + wave) * 1024, 16, ld_k_off[0], block_off + j * k_step_bytes, 0, 0);
            else
                __builtin_amdgcn_raw_ptr_buffer_load_lds(k_rsrc, sk + (j * kWaves + wave) * 1024, 16, ld_k_off[j], block_off, 0, 0);
        }
    };
    auto issue_v = [&](auto stage_tag, int blk) __attribute__((always_inline)) {
        NT_LDS unsigned char *sv = stage_v(stage_tag);
        const unsigned block_off = (unsigned)blk * v_block_bytes;
#pragma unroll
        for (int j = 0; j < kInstr; ++j)
            __builtin_amdgcn_raw_ptr_buffer_load_lds(v_rsrc, sv + (j * kWaves + wave) * 1024, 16, ld_v_off, block_off + j * v_step_bytes, 0, 0);
    };

    // ---- LDS read offsets ----
    // K: lane reads row kt * 32 + l32, 16-byte chunk 2 * ks + g.  The swizzle of a
    // row repeats every 16 rows, so one offset per contraction step serves all kt
    // (the tile offset is an immediate).
    static_assert(a_phys_chunk<D>(32, 0) == 0, "K swizzle period");
    int k_off[KS];
#pragma unroll
    for (int ks = 0; ks < KS; ++ks) k_off[ks] = l32 * (D * 2) + a_phys_chunk<D>(l32, ks * 2 + g) * 16;
    // V (transposing read): lane i of a 16-lane group addresses row 4g + i/4 (+ 16 per
    // contraction step, + 8 for the upper slots), columns 4 * (i % 4) of the group's 16.
    // The swizzle only looks at the row modulo 8 or less, so one offset per d tile.
    static_assert(b_phys_chunk<D>(8, 0) == 0, "V swizzle period");
    const int i16 = lane & 15;
    int v_off[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
        const int row = 4 * g + (i16 >> 2);
        const int col = dt * 32 + 16 * ((lane >> 4) & 1) + 4 * (i16 & 3);
        v_off[dt] = row * (D * 2) + b_phys_chunk<D>(row, col >> 3) * 16 + (col & 7) * 2;
    }

    float16_t o_acc[DT][kQTiles];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int qt = 0; qt < kQTiles; ++qt)
#pragma unroll
            for (int r = 0; r < 16; ++r) o_acc[dt][qt][r] = 0.0f;
    float m_run[kQTiles], l_run[kQTiles];  // l_run: this lane's half of the row sum
#pragma unroll
    for (int qt = 0; qt < kQTiles; ++qt) {
        m_run[qt] = kFold ? 0.0f : -INFINITY;
        l_run[qt] = 0.0f;
    }
    // kFold: scores are computed relative to a per-row REFERENCE m_run that is at most kFoldSlack below the
    // row's running maximum, and the subtraction happens inside the matrix pipe: the accumulators of
    // S^T = K . Q'^T start from -m_run (a lane's accumulators all belong to one query row) instead of
    // from zero.  The reference moves only when a block's row maximum exceeds it by more than the slack
    // (or when the row sees its first key), which after the first blocks is rare, so the steady state has
    // no subtraction, no rescale factor and no rescaling of the output.  Probabilities are then at most
    // 2^kFoldSlack instead of at most 1; the final division by the row sum cancels the reference.
    constexpr float kFoldSlack = 8.0f;
    float16_t c_init[kQTiles];     // -m_run in all 16 registers
    float fold_limit[kQTiles];     // -inf until the row has seen a key, kFoldSlack afterwards
#pragma unroll
    for (int qt = 0; qt < kQTiles; ++qt) {
        fold_limit[qt] = -INFINITY;
#pragma unroll
        for (int r = 0; r < 16; ++r) c_init[qt][r] = 0.0f;
    }

#ifdef NT_ATTN_STAMPS
    asm volatile("" ::"v"(qf[0][0]));  // (the queries have arrived)
    const unsigned long long real_loop = __builtin_amdgcn_s_memrealtime();
    const unsigned long long tick_loop = __builtin_amdgcn_s_memtime();
#endif
    // S^T = K . Q'^T for the block held in a K stage
    auto scores = [&](auto stage_tag, float16_t (&s_acc)[KT][kQTiles]) __attribute__((always_inline)) {
        const NT_LDS unsigned char *sk = stage_k(stage_tag);
        if constexpr (!kFold) {
#pragma unroll
            for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                for (int qt = 0; qt < kQTiles; ++qt)
#pragma unroll
                    for (int r = 0; r < 16; ++r) s_acc[kt][qt][r] = 0.0f;
        }
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            vec8 kf[KT];
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) kf[kt] = *(const NT_LDS vec8 *)(sk + k_off[ks] + kt * (32 * D * 2));
#pragma unroll
            for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                for (int qt = 0; qt < kQTiles; ++qt) {
                    if (kFold && ks == 0) s_acc[kt][qt] = E::mfma32(kf[kt], qf[qt][ks], c_init[qt]);
                    else s_acc[kt][qt] = E::mfma32(kf[kt], qf[qt][ks], s_acc[kt][qt]);
                }
        }
    };

    // masks of block `blk`: keys past the end of the sequence, and (causal) keys
    // after the query.  Few blocks need them (the last one, the ones on the
    // diagonal), so the callers branch on needs_masks (uniform over the wave) to a
    // copy of the block's code with or without the masking arithmetic.
    auto needs_masks = [&](int blk) __attribute__((always_inline)) -> bool {
        const int kv0 = blk * BN;
        const bool mask_tail = kv0 + BN > p.seq_k || blk > last_block;
        const bool mask_causal = p.causal && (kv0 + BN - 1 > q0 + wave * kQTiles * 32);
        return mask_tail || mask_causal;
    };
    auto apply_masks = [&](float16_t (&s_acc)[KT][kQTiles], int blk) __attribute__((always_inline)) {
        const int kv0 = blk * BN;
        const int limit = blk > last_block ? 0 : p.seq_k;
#pragma unroll
        for (int qt = 0; qt < kQTiles; ++qt) {
            // the last key this lane's row may see, relative to the first key of the lane's registers: one
            // comparison with a constant per element
            const int last_key = (p.causal ? min(limit - 1, q_row[qt]) : limit - 1) - kv0 - 4 * g;
#pragma unroll
            for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                for (int r = 0; r < 16; ++r)
                    if (kt * 32 + 8 * (r >> 2) + (r & 3) > last_key) s_acc[kt][qt][r] = -INFINITY;
        }
    };

    // online softmax: turns (masked) S^T into P^T operand fragments, updates the
    // running maximum / sum, returns the factor the output has to be rescaled by
    // (per q tile; 1 when the maximum did not move)
    // kFold, in three pieces so that the pipelined loop can place matrix instructions between them:
    // the row maxima of a block (relative to the reference) ...
    auto row_max = [&](const float16_t (&s_acc)[KT][kQTiles], float (&mx)[kQTiles]) __attribute__((always_inline)) {
#pragma unroll
        for (int qt = 0; qt < kQTiles; ++qt) {
            float top = -INFINITY;
#pragma unroll
            for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                for (int r = 0; r < 16; ++r) top = fmaxf(top, s_acc[kt][qt][r]);
            const unsigned bits = __builtin_bit_cast(unsigned, top);
            auto halves = __builtin_amdgcn_permlane32_swap(bits, bits, false, false);  // exchange with lane ^ 32 in registers
            mx[qt] = fmaxf(__builtin_bit_cast(float, (unsigned)halves[0]), __builtin_bit_cast(float, (unsigned)halves[1]));
        }
    };
    // ... the move of the reference when some row of the wave needs it (wave-uniform branch, rare after
    // the first blocks): the block's scores, the row sums and the accumulator start values follow the
    // new reference; alpha is the factor for the output accumulators ...
    auto rebase = [&](float16_t (&s_acc)[KT][kQTiles], const float (&mx)[kQTiles], float (&alpha)[kQTiles]) __attribute__((always_inline)) {
#pragma unroll
        for (int qt = 0; qt < kQTiles; ++qt) {
            alpha[qt] = 1.0f;
            const bool move = mx[qt] > fold_limit[qt];  // (both lanes of a row hold the same maximum and limit)
            if (__builtin_amdgcn_ballot_w64(move) != 0) {
                const float delta = move ? mx[qt] : 0.0f;
                // a row without keys so far has nothing accumulated: its factor stays 1 (2^-delta may overflow)
                alpha[qt] = fold_limit[qt] == -INFINITY ? 1.0f : __builtin_amdgcn_exp2f(-delta);
                m_run[qt] += delta;
                l_run[qt] *= alpha[qt];
#pragma unroll
                for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                    for (int r = 0; r < 16; ++r) s_acc[kt][qt][r] -= delta;
#pragma unroll
                for (int r = 0; r < 16; ++r) c_init[qt][r] = -m_run[qt];
            }
            if (mx[qt] > -INFINITY) fold_limit[qt] = kFoldSlack;
        }
    };
    // ... and the probabilities with their row sums
    auto exponentials = [&](float16_t (&s_acc)[KT][kQTiles], vec8 (&pf)[PS][kQTiles]) __attribute__((always_inline)) {
#pragma unroll
        for (int qt = 0; qt < kQTiles; ++qt) {
            // four independent partial sums: a single chain would tie every addition to
            // the exponential right before it
            float sum[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const float pv = __builtin_amdgcn_exp2f(s_acc[kt][qt][r]);
                    s_acc[kt][qt][r] = pv;
                    sum[r & 3] += pv;
                }
            l_run[qt] += (sum[0] + sum[1]) + (sum[2] + sum[3]);
        }
#pragma unroll
        for (int ps = 0; ps < PS; ++ps)
#pragma unroll
            for (int qt = 0; qt < kQTiles; ++qt)
#pragma unroll
                for (int e = 0; e < 8; ++e) pf[ps][qt][e] = E::from_float(s_acc[ps / 2][qt][8 * (ps & 1) + e]);
    };

    auto softmax = [&](float16_t (&s_acc)[KT][kQTiles], vec8 (&pf)[PS][kQTiles], float (&alpha)[kQTiles]) __attribute__((always_inline)) {
        if constexpr (kFold) {
            float mx[kQTiles];
            row_max(s_acc, mx);
            rebase(s_acc, mx, alpha);
            exponentials(s_acc, pf);
            return;
        }
#pragma unroll
        for (int qt = 0; qt < kQTiles; ++qt) {
            float mx = -INFINITY;
#pragma unroll
            for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s_acc[kt][qt][r]);
            {   // exchange with lane ^ 32 in registers (no LDS round trip)
                const unsigned bits = __builtin_bit_cast(unsigned, mx);
                auto halves = __builtin_amdgcn_permlane32_swap(bits, bits, false, false);
                mx = fmaxf(__builtin_bit_cast(float, (unsigned)halves[0]), __builtin_bit_cast(float, (unsigned)halves[1]));
            }
            const float m_new = fmaxf(m_run[qt], mx);
            const float m_use = m_new == -INFINITY ? 0.0f : m_new;  // fully masked so far
            alpha[qt] = __builtin_amdgcn_exp2f(m_run[qt] - m_use);
            m_run[qt] = m_new;
            // four independent partial sums: a single chain would tie every addition to
            // the exponential right before it
            float sum[4] = {0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
            for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const float pv = __builtin_amdgcn_exp2f(s_acc[kt][qt][r] - m_use);
                    s_acc[kt][qt][r] = pv;
                    sum[r & 3] += pv;
                }
            l_run[qt] = l_run[qt] * alpha[qt] + ((sum[0] + sum[1]) + (sum[2] + sum[3]));
        }
#pragma unroll
        for (int ps = 0; ps < PS; ++ps)
#pragma unroll
            for (int qt = 0; qt < kQTiles; ++qt)
#pragma unroll
                for (int e = 0; e < 8; ++e) pf[ps][qt][e] = E::from_float(s_acc[ps / 2][qt][8 * (ps & 1) + e]);
    };

    // the running maximum settles after a few blocks; skip the rescale of the
    // output accumulators when no row of this wave's tile moved (wave-uniform)
    auto rescale = [&](const float (&alpha)[kQTiles]) __attribute__((always_inline)) {
#pragma unroll
        for (int qt = 0; qt < kQTiles; ++qt) {
            if (__builtin_amdgcn_ballot_w64(alpha[qt] != 1.0f) != 0) {
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                    for (int r = 0; r < 16; ++r) o_acc[dt][qt][r] *= alpha[qt];
            }
        }
    };

    // O^T += V^T . P^T for the block held in a V stage
    auto accumulate = [&](auto stage_tag, const vec8 (&pf)[PS][kQTiles], auto first_tag, auto last_tag) __attribute__((always_inline)) {
        const NT_LDS unsigned char *sv = stage_v(stage_tag);
#pragma unroll
        for (int ps = decltype(first_tag)::value; ps < decltype(last_tag)::value; ++ps) {
            vec8 vf[DT];
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                short4_t lo = lds_read_tr16_b64(sv + v_off[dt] + (ps * 16) * (D * 2));
                short4_t hi = lds_read_tr16_b64(sv + v_off[dt] + (ps * 16 + 8) * (D * 2));
                short8_t both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                vf[dt] = __builtin_bit_cast(vec8, both);
            }
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int qt = 0; qt < kQTiles; ++qt) o_acc[dt][qt] = E::mfma32(vf[dt], pf[ps][qt], o_acc[dt][qt]);
        }
    };

    typedef std::integral_constant<int, 0> Stage0;
    typedef std::integral_constant<int, 1> Stage1;
    typedef std::integral_constant<int, 0> PsBegin;
    typedef std::integral_constant<int, PS> PsEnd;
    if constexpr (!kPipelined) {
        // two LDS stages, loop unrolled by two; an odd block count runs one fully
        // masked extra block, whose loads re-fetch the last block
        auto block = [&](auto stage_tag, int blk) __attribute__((always_inline)) {
            float16_t s_acc[KT][kQTiles];
            vec8 pf[PS][kQTiles];
            float alpha[kQTiles];
            scores(stage_tag, s_acc);
            if (needs_masks(blk)) apply_masks(s_acc, blk);
            softmax(s_acc, pf, alpha);
            rescale(alpha);
            accumulate(stage_tag, pf, PsBegin(), PsEnd());
        };
        if (num_blocks > first_block) {
            issue_k(Stage0(), first_block);
            issue_v(Stage0(), first_block);
            scale_queries();
            for (int blk = first_block; blk < num_blocks; blk += 2) {
                wait_vmcnt<0>();
                lds_barrier();
                issue_k(Stage1(), min(blk + 1, last_block));
                issue_v(Stage1(), min(blk + 1, last_block));
                block(Stage0(), blk);
                wait_vmcnt<0>();
                lds_barrier();
                issue_k(Stage0(), min(blk + 2, last_block));
                issue_v(Stage0(), min(blk + 2, last_block));
                block(Stage1(), blk + 1);
            }
            wait_vmcnt<0>();  // nothing may still be writing LDS when the workgroup ends
        }
    } else {
        // Software pipeline over key blocks.  Step j holds S(j) from the previous
        // step and runs three mutually independent pieces that the instruction
        // scheduler can interleave: the softmax of block j (VALU), the MFMAs of
        // P(j-1) . V(j-1), and the MFMAs of K(j+1) . Q.  K(j+1) and V(j-1) sit in
        // the stage opposite to the step's parity; K(j+2) and V(j) are requested
        // into the step's own stage.  Past the end the last K block is fetched and
        // multiplied again (its scores are never used), which keeps the steps uniform.
        if (num_blocks > 0) {
            // S(j) and P(j) live in the buffers of j's parity, so nothing is copied
            float16_t s_buf[2][KT][kQTiles];
            vec8 p_buf[2][PS][kQTiles];
            float alpha[kQTiles];
            issue_k(Stage0(), 0);
            issue_k(Stage1(), min(1, last_block));
            scale_queries();
            wait_vmcnt<kInstr>();
            lds_barrier();
            scores(Stage0(), s_buf[0]);
            // step 0: nothing to accumulate yet
            wait_vmcnt<0>();
            lds_barrier();
            issue_k(Stage0(), min(2, last_block));
            issue_v(Stage0(), 0);
            if (needs_masks(0)) apply_masks(s_buf[0], 0);
            softmax(s_buf[0], p_buf[0], alpha);
            scores(Stage1(), s_buf[1]);

            auto step_body = [&](auto parity_tag, auto masked_tag, auto scores_tag, int j) __attribute__((always_inline)) {
                constexpr bool kScores = decltype(scores_tag)::value;  // false in a wave's last step: no block follows
                constexpr int kParity = decltype(parity_tag)::value;
                typedef std::integral_constant<int, kParity> Own;
                typedef std::integral_constant<int, 1 - kParity> Other;
                wait_vmcnt<0>();
                lds_barrier();
                __builtin_amdgcn_sched_barrier(0);  // nothing of this step moves above the barrier
                issue_k(Own(), min(j + 2, last_block));
                issue_v(Own(), j);
                if constexpr (decltype(masked_tag)::value) apply_masks(s_buf[kParity], j);
                if constexpr (kFold) {
                    // Two scheduling regions with the (rare) move of the reference between them: the row
                    // maxima run under the first MFMAs of P(j-1) . V(j-1); the exponentials, row sums and
                    // conversions under the rest of them and under K(j+1) . Q, whose accumulators start
                    // from the reference as it stands after the move.
#ifndef NT_FOLD_SPLIT
#define NT_FOLD_SPLIT 2
#endif
                    typedef std::integral_constant<int, (NT_FOLD_SPLIT < PS ? NT_FOLD_SPLIT : PS)> PsSplit;
                    float mx[kQTiles];
                    row_max(s_buf[kParity], mx);
                    accumulate(Other(), p_buf[1 - kParity], PsBegin(), PsSplit());
                    {
                        constexpr int kMfma = PsSplit::value * DT * kQTiles;
                        constexpr int kReads = PsSplit::value * DT * 2;
                        __builtin_amdgcn_sched_group_barrier(0x100, 6, 0);
                        __builtin_amdgcn_sched_group_barrier(0x020, 2 * kInstr, 0);
                        __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);
                        static_for<0, kMfma>([&](auto i_tag) __attribute__((always_inline)) {
                            constexpr int i = decltype(i_tag)::value;
                            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                            if constexpr (6 + 2 * i < kReads) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
                            __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);
                        });
                    }
                    rebase(s_buf[kParity], mx, alpha);
                    exponentials(s_buf[kParity], p_buf[kParity]);
                    accumulate(Other(), p_buf[1 - kParity], PsSplit(), PsEnd());
                    if constexpr (kScores) scores(Other(), s_buf[1 - kParity]);
                    {
                        constexpr int kMfma = ((PS - PsSplit::value) * DT + (kScores ? KS * KT : 0)) * kQTiles;
                        constexpr int kReads = (PS - PsSplit::value) * DT * 2 + (kScores ? KS * KT : 0);
                        __builtin_amdgcn_sched_group_barrier(0x100, 6, 0);
                        __builtin_amdgcn_sched_group_barrier(0x400, 2, 0);
                        static_for<0, kMfma>([&](auto i_tag) __attribute__((always_inline)) {
                            constexpr int i = decltype(i_tag)::value;
                            __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                            if constexpr (6 + 2 * i < kReads) __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
                            __builtin_amdgcn_sched_group_barrier(0x400, (i % 3 == 0) ? 2 : 1, 0);
                            __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);
                        });
                    }
                } else {
                softmax(s_buf[kParity], p_buf[kParity], alpha);
                accumulate(Other(), p_buf[1 - kParity], PsBegin(), PsEnd());
                if constexpr (kScores) scores(Other(), s_buf[1 - kParity]);
                // desired issue order inside this region: one MFMA, then the LDS reads
                // and softmax arithmetic that fit under it
#ifndef NT_ATTN_SCHEDULE
#define NT_ATTN_SCHEDULE 1
#endif
#if NT_ATTN_SCHEDULE
                // Issue order asked of the scheduler: LDS reads run three MFMAs ahead; every
                // MFMA (32 cycles in the matrix pipe) is followed by the operand reads of a
                // later one and by at most 28 cycles of softmax arithmetic (4 per VALU
                // instruction, 8 per exponential).  The first MFMAs overlap the running-max
                // chain, the exponentials start once the maximum is known.
                constexpr int kMfmaPerStep = (PS * DT + (kScores ? KS * KT : 0)) * kQTiles;
#ifndef NT_ATTN_HEAD_VALU
#define NT_ATTN_HEAD_VALU 12
#endif
                // first the operand reads of the first MFMAs, then the refills of this
                // step's own stage and the head of the running-max chain while those reads
                // are in flight
                __builtin_amdgcn_sched_group_barrier(0x100, 6, 0);
                __builtin_amdgcn_sched_group_barrier(0x020, 2 * kInstr, 0);
                __builtin_amdgcn_sched_group_barrier(0x002, NT_ATTN_HEAD_VALU, 0);
                static_for<0, kMfmaPerStep>([&](auto i_tag) __attribute__((always_inline)) {
                    constexpr int i = decltype(i_tag)::value;
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
                    if constexpr (i < kMfmaPerStep / 8) {
                        __builtin_amdgcn_sched_group_barrier(0x002, 5, 0);
                    } else {
                        __builtin_amdgcn_sched_group_barrier(0x400, (i % 4 == 0) ? 2 : 1, 0);
                        __builtin_amdgcn_sched_group_barrier(0x002, 3, 0);
                    }
                });
#endif
                }
                // P(j) and the row sums are only consumed in later steps; pin them here so
                // that their arithmetic stays in this step, next to the MFMAs it overlaps with
#pragma unroll
                for (int ps = 0; ps < PS; ++ps)
#pragma unroll
                    for (int qt = 0; qt < kQTiles; ++qt) asm volatile("" : "+v"(p_buf[kParity][ps][qt]));
#pragma unroll
                for (int qt = 0; qt < kQTiles; ++qt) asm volatile("" : "+v"(l_run[qt]));
                rescale(alpha);
            };
            // A wave needs the key blocks up to the one that holds the key of its last query row (causal; all of
            // them otherwise): `mine` of the workgroup's num_blocks.  Its
            // step `mine` only multiplies P(mine - 1) by V(mine - 1), and later steps only take part in the loads
            // and barriers of the workgroup -- on the diagonal of a causal problem this spares the waves with the
            // upper query rows the blocks that the masks would zero entirely.
            int mine = num_blocks;
            if (p.causal) mine = min(mine, (q0 + wave * kQTiles * 32 + kQTiles * 32 - 1) / BN + 1);
            auto product_step = [&](auto parity_tag, int j) __attribute__((always_inline)) {
                constexpr int kParity = decltype(parity_tag)::value;
                wait_vmcnt<0>();
                lds_barrier();
                __builtin_amdgcn_sched_barrier(0);
                issue_k(std::integral_constant<int, kParity>(), min(j + 2, last_block));
                issue_v(std::integral_constant<int, kParity>(), j);
                accumulate(std::integral_constant<int, 1 - kParity>(), p_buf[1 - kParity], PsBegin(), PsEnd());
            };
            auto idle_step = [&](auto parity_tag, int j) __attribute__((always_inline)) {
                constexpr int kParity = decltype(parity_tag)::value;
                wait_vmcnt<0>();
                lds_barrier();
                issue_k(std::integral_constant<int, kParity>(), min(j + 2, last_block));
                issue_v(std::integral_constant<int, kParity>(), j);
            };
            // The blocks that need masks are the last ones.  A first loop runs the pairs
            // of steps that lie entirely before them without the masking arithmetic, a
            // second one the rest with it (masking a block that does not need it changes
            // nothing).  The split differs between the waves of a workgroup; the number of
            // steps, and with it the number of barriers, does not.
            int unmasked = p.seq_k / BN;
            if (p.causal) unmasked = min(unmasked, (q0 + wave * kQTiles * 32 + 1) / BN);
            int j = 1;
            for (; j + 1 < unmasked; j += 2) {
                step_body(Stage1(), std::false_type(), std::true_type(), j);
                step_body(Stage0(), std::false_type(), std::true_type(), j + 1);
            }
            for (; j + 1 < mine; j += 2) {
                step_body(Stage1(), std::true_type(), std::true_type(), j);
                step_body(Stage0(), std::true_type(), std::true_type(), j + 1);
            }
            if (j < mine) {
                step_body(Stage1(), std::true_type(), std::true_type(), j);
                ++j;
            }
            // (j == mine; the scores of block `mine`, computed in the step before, are never used)
            for (; j < num_blocks; ++j) {
                if (j == mine) {
                    if (j & 1) product_step(Stage1(), j);
                    else product_step(Stage0(), j);
                } else {
                    if (j & 1) idle_step(Stage1(), j);
                    else idle_step(Stage0(), j);
                }
            }
            // drain: P(last) . V(last); V(last) was requested into the stage of its parity
            wait_vmcnt<0>();
            lds_barrier();
            if (mine == num_blocks) {
                if ((num_blocks - 1) & 1)
                    accumulate(Stage1(), p_buf[1], PsBegin(), PsEnd());
                else
                    accumulate(Stage0(), p_buf[0], PsBegin(), PsEnd());
            }
        }
    }

#ifdef NT_ATTN_STAMPS
    const unsigned long long real_epilogue = __builtin_amdgcn_s_memrealtime();
    const unsigned long long tick_epilogue = __builtin_amdgcn_s_memtime();
#endif
    // ---- epilogue: O[q, d] = O^T[d, q] / l ----
    if constexpr (kSplitKV) {
#pragma unroll
        for (int qt = 0; qt < kQTiles; ++qt) {
            const float l_total = l_run[qt] + __shfl_xor(l_run[qt], 32, 64);
            const float inv = l_total > 0.0f ? 1.0f / l_total : 0.0f;  // a part without keys contributes nothing
            if (q_row[qt] < p.seq_q) {
                const int64_t row = ((int64_t)part * p.batch * p.heads + bh) * p.seq_q + q_row[qt];
                float *dst = p.part_o + row * D;
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                    for (int r4 = 0; r4 < 4; ++r4) {
                        typedef float float4_t __attribute__((ext_vector_type(4)));
                        float4_t out;
#pragma unroll
                        for (int e = 0; e < 4; ++e) out[e] = o_acc[dt][qt][r4 * 4 + e] * inv;
                        *(float4_t *)(dst + dt * 32 + 8 * r4 + 4 * g) = out;
                    }
                if (g == 0) p.part_lse[row] = l_total > 0.0f ? m_run[qt] + __builtin_amdgcn_logf(l_total) : -INFINITY;
            }
        }
        return;
    }
    // A lane holds four consecutive columns of one query row at a time, so stores straight from the registers put
    // 8 bytes into each of 32 rows per instruction.  Where the workgroup's K / V stages have room for one 32-row
    // tile of O per wave (BN >= 32 always holds one or more whole tiles per stage), the tile goes through them instead (16-byte chunks of a row exchanged by the row number,
    // so that neither side meets bank conflicts) and leaves in whole rows: 16 bytes per lane, 64 lanes on
    // consecutive addresses.
    constexpr int kChunks = D / 8;
    constexpr bool kStagedStore = !kPadded && std::is_same<TIO, T>::value && (kChunks & (kChunks - 1)) == 0 && kChunks <= 64 &&
                                  kWaves * 32 * D * 2 <= 4 * kTileBytes;
    if constexpr (kStagedStore) {
        typedef TIO vec4 __attribute__((ext_vector_type(4)));
        typedef unsigned uint4_t __attribute__((ext_vector_type(4)));
        constexpr int kSwizzle = (kChunks < 16 ? kChunks : 16) - 1;
        constexpr int kRowsPerStore = 64 / kChunks;
        lds_barrier();  // every wave has read its last V block
        // the addresses of this exchange are derived from copies of the lane and wave numbers that the compiler
        // cannot trace back, or it computes them before the loop and the loop pays for the registers they hold
        int late_lane = lane, late_wave = wave;
        asm volatile("" : "+v"(late_lane), "+s"(late_wave));
        const int late_l32 = late_lane & 31, late_g = late_lane >> 5;
        // (the four stages stay separate arrays: the compiler orders a read of one stage behind the fills of
        // another only if it cannot tell them apart)
        constexpr int kTilesPerStage = kTileBytes / (32 * D * 2);
        const int stage = late_wave / kTilesPerStage;
        NT_LDS unsigned char *tile = (NT_LDS unsigned char *)(stage == 0 ? lds_k0 : stage == 1 ? lds_v0 : stage == 2 ? lds_k1 : lds_v1) +
                                     (late_wave % kTilesPerStage) * (32 * D * 2);
        NT_LDS unsigned char *put = tile + late_l32 * (D * 2) + late_g * 8;
        const int get_row = late_lane / kChunks, get_chunk = late_lane % kChunks;
#pragma unroll
        for (int qt = 0; qt < kQTiles; ++qt) {
            const float l_total = l_run[qt] + __shfl_xor(l_run[qt], 32, 64);
            const float inv = 1.0f / l_total;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int r4 = 0; r4 < 4; ++r4) {
                    vec4 out;
#pragma unroll
                    for (int e = 0; e < 4; ++e) out[e] = E::from_float(o_acc[dt][qt][r4 * 4 + e] * inv);
                    *(NT_LDS vec4 *)(put + (((dt * 4 + r4) ^ (late_l32 & kSwizzle)) * 16)) = out;
                }
            // (the LDS serves a wave's requests in order; the fence only keeps the compiler from moving them)
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
            __builtin_amdgcn_wave_barrier();
            const int tile_row0 = q0 + (late_wave * kQTiles + qt) * 32;
#pragma unroll
            for (int i = 0; i < 32 / kRowsPerStore; ++i) {
                const int row = i * kRowsPerStore + get_row;
                const uint4_t chunk = *(NT_LDS const uint4_t *)(tile + row * (D * 2) + ((get_chunk ^ (row & kSwizzle)) * 16));
                if (tile_row0 + row < p.seq_q) *(uint4_t *)(O + (int64_t)(tile_row0 + row) * p.o_strides[2] + get_chunk * 8) = chunk;
            }
            __builtin_amdgcn_fence(__ATOMIC_ACQ_REL, "wavefront");
            __builtin_amdgcn_wave_barrier();
        }
    } else
#pragma unroll
    for (int qt = 0; qt < kQTiles; ++qt) {
        const float l_total = l_run[qt] + __shfl_xor(l_run[qt], 32, 64);
        const float inv = 1.0f / l_total;
        if (q_row[qt] < p.seq_q) {
            TIO *dst = O + (int64_t)q_row[qt] * p.o_strides[2];
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int r4 = 0; r4 < 4; ++r4) {
                    typedef TIO vec4 __attribute__((ext_vector_type(4)));
                    vec4 out;
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const float value = o_acc[dt][qt][r4 * 4 + e] * inv;
                        if constexpr (std::is_same<TIO, float>::value) out[e] = value;
                        else out[e] = E::from_float(value);
                    }
                    if (kPadded && dt * 32 + 8 * r4 + 4 * g >= p.head_dim) continue;
                    *(vec4 *)(dst + dt * 32 + 8 * r4 + 4 * g) = out;
                }
        }
    }
#ifdef NT_ATTN_STAMPS
    if (p.stamps && lane == 0) {
        unsigned long long *dst = p.stamps + ((size_t)blockIdx.x * kWaves + wave) * 4;
        dst[0] = real_loop - real_entry;
        dst[1] = real_epilogue - real_loop;
        dst[2] = __builtin_amdgcn_s_memrealtime() - real_epilogue;
        dst[3] = tick_epilogue - tick_loop;
    }
#endif
#endif
}

// merges the parts of a split key range: O = sum_s w_s O_s / sum_s w_s with w_s = 2^(lse_s - max lse);
// one thread per row and four consecutive columns
template <typename TIO, int D>
__global__ __launch_bounds__(256) void attention_merge_kernel(AttentionParams p) {
    typedef float float4_t __attribute__((ext_vector_type(4)));
    constexpr int kGroups = D / 4;
    const int64_t rows = (int64_t)p.batch * p.heads * p.seq_q;
    const int64_t index = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (index >= rows * kGroups) return;
    const int64_t row = index / kGroups;
    const int col = (int)(index - row * kGroups) * 4;
    if (col >= p.head_dim) return;
    float top = -INFINITY;
    for (int s = 0; s < p.parts; ++s) top = fmaxf(top, p.part_lse[s * rows + row]);
    float4_t sum = {0.0f, 0.0f, 0.0f, 0.0f};
    float weights = 0.0f;
    for (int s = 0; s < p.parts; ++s) {
        const float lse = p.part_lse[s * rows + row];
        if (lse == -INFINITY) continue;
        const float w = __builtin_amdgcn_exp2f(lse - top);
        weights += w;
        sum += w * *(const float4_t *)(p.part_o + (s * rows + row) * D + col);
    }
    const float inv = 1.0f / weights;
    const int64_t q_in_head = row % p.seq_q;
    const int64_t bh = row / p.seq_q;
    TIO *dst = (TIO *)p.o + (bh / p.heads) * p.o_strides[0] + (bh % p.heads) * p.o_strides[1] + q_in_head * p.o_strides[2] + col;
    typedef TIO out4_t __attribute__((ext_vector_type(4)));
    out4_t out;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        if constexpr (std::is_same<TIO, float>::value) out[e] = sum[e] * inv;
        else out[e] = Elem<TIO>::from_float(sum[e] * inv);
    }
    *(out4_t *)dst = out;
}

// Few (batch, head, query block) workgroups and a long key sequence (decoding): the key range is split
// so that about 512 workgroups run.  The number of parts for a problem, 0 when it runs in one pass.
constexpr int kSplitKeysBM = kAttnWaves * 32, kSplitKeysBN = 64;
inline int64_t split_key_parts(const AttentionParams &p) {
    const int64_t groups = (int64_t)p.batch * p.heads * ceil_div(p.seq_q, kSplitKeysBM);
    const int key_blocks = ceil_div(p.seq_k, kSplitKeysBN);
    if (groups == 0 || groups >= 128 || key_blocks < 8) return 0;
    const int64_t parts = std::min<int64_t>((512 + groups - 1) / groups, key_blocks / 4);  // at least four key blocks each
    return parts < 2 ? 0 : parts;
}

// returns NINETOOTHED_NO_KERNEL when the problem is not split
template <typename T, int D>
int launch_split_keys(AttentionParams &p, hipStream_t stream) {
    constexpr int BM = kSplitKeysBM, BN = kSplitKeysBN;
    p.q_blocks = ceil_div(p.seq_q, BM);
    const int64_t groups = (int64_t)p.batch * p.heads * p.q_blocks;
    const int key_blocks = ceil_div(p.seq_k, BN);
    const int64_t parts = split_key_parts(p);
    if (parts == 0) return NINETOOTHED_NO_KERNEL;
    p.blocks_per_part = ceil_div(key_blocks, (int)parts);
    p.parts = ceil_div(key_blocks, p.blocks_per_part);
    const int64_t rows = (int64_t)p.batch * p.heads * p.seq_q;
    const size_t bytes = (size_t)p.parts * rows * (D + 1) * sizeof(float);
    if (bytes > (size_t(256) << 20)) return NINETOOTHED_NO_KERNEL;
    WorkspaceLease lease(stream);
    float *scratch = (float *)lease.get(kWorkspaceAttentionParts, bytes);
    if (scratch == nullptr) return NINETOOTHED_NO_KERNEL;  // (graph capture without a buffer, out of memory): one pass
    p.part_o = scratch;
    p.part_lse = scratch + (size_t)p.parts * rows * D;
    note_launch(kLaunchAttention, (int)p.parts, "split key range (this many parts), plain loop, then attention_merge_kernel");
    attention_fwd_kernel<T, D, 1, BN, 2, false, T, kAttnWaves, false, true><<<dim3((unsigned)(groups * p.parts)), dim3(kAttnWaves * 64), 0, stream>>>(p);
    hipError_t err = hipGetLastError();
    if (err != hipSuccess) return (int)err;
    attention_merge_kernel<T, D><<<dim3((unsigned)((rows * (D / 4) + 255) / 256)), dim3(256), 0, stream>>>(p);
    return (int)hipGetLastError();
}

template <typename T, int D, int kQTiles, int BN, int kOcc, bool kPipelined, typename TIO = T, int kWaves = kAttnWaves, bool kPadded = false, bool kFold = true>
hipError_t launch_attention(AttentionParams &p, hipStream_t stream) {
    constexpr int BM = kWaves * 32 * kQTiles;
    p.q_blocks = ceil_div(p.seq_q, BM);
    const int64_t grid = (int64_t)p.batch * p.heads * p.q_blocks;
    if (grid == 0) return hipSuccess;
    attention_fwd_kernel<T, D, kQTiles, BN, kOcc, kPipelined, TIO, kWaves, kPadded, false, kFold><<<dim3((unsigned)grid), dim3(kWaves * 64), 0, stream>>>(p);
    return hipGetLastError();
}

// Head dimensions other than 32, 64 and 128: 256 as it is (one workgroup of four waves per CU: its
// accumulators and Q fragments take most of the register file), other multiples of 8 on the next of
// these sizes with the missing columns read as zeros.
template <typename T, typename TIO>
int launch_other_head_dim(AttentionParams &p, int head_dim, hipStream_t stream) {
    if (head_dim <= 0 || head_dim > 256 || head_dim % 8) return NINETOOTHED_NO_KERNEL;
    if (head_dim == 256) return (int)launch_attention<T, 256, 1, 64, 1, false, TIO>(p, stream);
    // padded rows are fetched through offsets that must lie behind the K / V descriptors
    if ((((int64_t)p.seq_k + 64) * std::max(p.k_strides[2], p.v_strides[2]) + head_dim) * 2 >= (int64_t(1) << 31)) return NINETOOTHED_NO_KERNEL;
    if (head_dim > 128) return (int)launch_attention<T, 256, 1, 64, 1, false, TIO, kAttnWaves, true>(p, stream);
    if (head_dim > 64) return (int)launch_attention<T, 128, 1, 64, 2, false, TIO, kAttnWaves, true>(p, stream);
    if (head_dim > 32) return (int)launch_attention<T, 64, 1, 64, 2, false, TIO, kAttnWaves, true>(p, stream);
    return (int)launch_attention<T, 32, 1, 64, 2, false, TIO, kAttnWaves, true>(p, stream);
}

// fp32 tensors: K and V become contiguous [batch, heads, seq, D] half-precision copies
__global__ __launch_bounds__(256) void attention_narrow_kernel(const float *src, half_t *dst, int64_t total, int heads, int seq, int dim, int64_t s0,
                                                               int64_t s1, int64_t s2, int64_t s3) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < total; i += (int64_t)gridDim.x * 256) {
        const int d = (int)(i % dim);
        int64_t rest = i / dim;
        const int s = (int)(rest % seq);
        rest /= seq;
        const int h = (int)(rest % heads);
        const int64_t b = rest / heads;
        dst[i] = (half_t)src[b * s0 + h * s1 + s * s2 + d * s3];
    }
}

// fp32 tensors as they are, for head dimensions 32, 64 and 128: every product and sum in fp32 on the 32x32x2 fp32
// MFMA (a sixteenth of the fp16 rate), nothing narrowed.  One wave per 32 query rows, four waves per workgroup, no
// LDS and no barriers: operands go from global memory straight into MFMA registers.  Same transposed formulation
// as the fp16 kernel -- S^T[kv, q] = K[kv, :] . Q'[q, :], O^T[d, q] += V^T[d, kv] . P^T[kv, q] -- with 32-key blocks.
// The two contraction slots of an MFMA belong to lane halves g = 0, 1: for S^T they are d = g * D/2 + step (a lane
// reads half a row of K, contiguous), for O^T the keys that the lane's S^T accumulator `r` holds for g = 0 and 1.
template <int D>
__global__ __launch_bounds__(256) void attention_f32_kernel(AttentionParams p) {
#if defined(__HIP_DEVICE_COMPILE__)
    constexpr int BM = 128, BN = 32, DT = D / 32, kHalf = D / 2;
    typedef float float4_t __attribute__((ext_vector_type(4)));
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int g = lane >> 5, l32 = lane & 31;
    const int q_blocks = p.q_blocks;
    // causal: long query blocks first
    const int qb = p.causal ? q_blocks - 1 - (int)(blockIdx.x % q_blocks) : (int)(blockIdx.x % q_blocks);
    const int bh = blockIdx.x / q_blocks;
    const int head = bh % p.heads, batch = bh / p.heads;
    const int q0 = qb * BM + wave * 32;
    if (q0 >= p.seq_q) return;  // (no barriers in this kernel)
    const int q_row = q0 + l32;
    const float *Q = (const float *)p.q + batch * p.q_strides[0] + head * p.q_strides[1];
    const float *K = (const float *)p.k + batch * p.k_strides[0] + head * p.k_strides[1];
    const float *V = (const float *)p.v + batch * p.v_strides[0] + head * p.v_strides[1];
    float *O = (float *)p.o + batch * p.o_strides[0] + head * p.o_strides[1];

    float qf[kHalf];
    {
        const float *src = Q + (int64_t)min(q_row, p.seq_q - 1) * p.q_strides[2] + g * kHalf;
#pragma unroll
        for (int c = 0; c < kHalf / 4; ++c) {
            const float4_t v = *(const float4_t *)(src + 4 * c);
#pragma unroll
            for (int e = 0; e < 4; ++e) qf[4 * c + e] = v[e] * p.q_scale;
        }
    }
    float16_t o_acc[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt)
#pragma unroll
        for (int r = 0; r < 16; ++r) o_acc[dt][r] = 0.0f;
    float m_run = -INFINITY, l_run = 0.0f;  // l_run: this lane's half of the row sum

    const int kv_end = p.causal ? min(p.seq_k, q0 + 32) : p.seq_k;  // keys beyond the wave's last row are masked for all of its rows
    for (int kv0 = 0; kv0 < kv_end; kv0 += BN) {
        float16_t s_acc;
#pragma unroll
        for (int r = 0; r < 16; ++r) s_acc[r] = 0.0f;
        {
            const float *src = K + (int64_t)min(kv0 + l32, p.seq_k - 1) * p.k_strides[2] + g * kHalf;
#pragma unroll
            for (int c = 0; c < kHalf / 4; ++c) {
                typedef float4_t unaligned_float4_t __attribute__((aligned(4)));  // (rows of K may start anywhere: global accesses need the element's alignment only)
                const float4_t v = *(const unaligned_float4_t *)(src + 4 * c);
#pragma unroll
                for (int e = 0; e < 4; ++e) s_acc = __builtin_amdgcn_mfma_f32_32x32x2f32(v[e], qf[4 * c + e], s_acc, 0, 0, 0);
            }
        }
        const bool tail = kv0 + BN > p.seq_k;
        if (tail || (p.causal && kv0 + BN - 1 > q0)) {  // (uniform over the wave)
            const int last_key = (p.causal ? min(p.seq_k - 1, q_row) : p.seq_k - 1) - kv0 - 4 * g;
#pragma unroll
            for (int r = 0; r < 16; ++r)
                if (8 * (r >> 2) + (r & 3) > last_key) s_acc[r] = -INFINITY;
        }
        float mx = -INFINITY;
#pragma unroll
        for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s_acc[r]);
        mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
        const float m_new = fmaxf(m_run, mx);
        const float m_use = m_new == -INFINITY ? 0.0f : m_new;  // fully masked so far
        const float alpha = __builtin_amdgcn_exp2f(m_run - m_use);
        m_run = m_new;
        float sum = 0.0f;
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            s_acc[r] = __builtin_amdgcn_exp2f(s_acc[r] - m_use);
            sum += s_acc[r];
        }
        l_run = l_run * alpha + sum;
        if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int r = 0; r < 16; ++r) o_acc[dt][r] *= alpha;
        }
#pragma unroll
        for (int r = 0; r < 16; ++r) {
            const int kv = kv0 + 8 * (r >> 2) + 4 * g + (r & 3);
            const float *src = V + (int64_t)min(kv, p.seq_k - 1) * p.v_strides[2] + l32;
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                float value = src[dt * 32];
                if (tail && kv >= p.seq_k) value = 0.0f;  // (its probability is 0; the row read instead may hold anything)
                o_acc[dt] = __builtin_amdgcn_mfma_f32_32x32x2f32(value, s_acc[r], o_acc[dt], 0, 0, 0);
            }
        }
    }
    const float l_total = l_run + __shfl_xor(l_run, 32, 64);
    const float inv = 1.0f / l_total;
    if (q_row < p.seq_q) {
        float *dst = O + (int64_t)q_row * p.o_strides[2];
#pragma unroll
        for (int dt = 0; dt < DT; ++dt)
#pragma unroll
            for (int r4 = 0; r4 < 4; ++r4) {
                float4_t out;
#pragma unroll
                for (int e = 0; e < 4; ++e) out[e] = o_acc[dt][r4 * 4 + e] * inv;
                *(float4_t *)(dst + dt * 32 + 8 * r4 + 4 * g) = out;
            }
    }
#endif
}

template <int D>
int launch_attention_f32(AttentionParams &p, hipStream_t stream) {
    p.q_blocks = ceil_div(p.seq_q, 128);
    const int64_t grid = (int64_t)p.batch * p.heads * p.q_blocks;
    if (grid == 0) return 0;
    if (grid > 0x7fffffffll) return NINETOOTHED_NO_KERNEL;
    note_launch(kLaunchAttention, 0, "attention_f32_kernel, fp32 MFMA throughout");
    attention_f32_kernel<D><<<dim3((unsigned)grid), dim3(256), 0, stream>>>(p);
    return (int)hipGetLastError();
}

// fp32 tensors.  Head dimensions 32, 64 and 128 without block-size hints: the fp32 kernel above.  Other head
// dimensions, and calls with a hint (the fast way: sixteen times the MFMA rate): the 16-bit kernels on fp16 copies
// of K and V (values beyond the fp16 range overflow there).
int attention_float32(AttentionParams p, int head_dim, const NineToothedTensor &k, const NineToothedTensor &v, bool exact, hipStream_t stream) {
    if (exact && k.strides[3] == 1 && v.strides[3] == 1) {
        if (head_dim == 128) return launch_attention_f32<128>(p, stream);
        if (head_dim == 64) return launch_attention_f32<64>(p, stream);
        if (head_dim == 32) return launch_attention_f32<32>(p, stream);
    }
    const int64_t total = (int64_t)p.batch * p.heads * p.seq_k * head_dim;
    WorkspaceLease lease(stream);
    half_t *narrow = (half_t *)lease.get(kWorkspaceAttentionNarrow, (size_t)total * 2 * sizeof(half_t));
    if (narrow == nullptr) return (int)hipErrorOutOfMemory;
    const unsigned blocks = (unsigned)((total + 255) / 256 < 256 * 16 ? (total + 255) / 256 : 256 * 16);
    attention_narrow_kernel<<<dim3(blocks), dim3(256), 0, stream>>>((const float *)k.data, narrow, total, p.heads, p.seq_k, head_dim, k.strides[0],
                                                                  k.strides[1], k.strides[2], k.strides[3]);
    attention_narrow_kernel<<<dim3(blocks), dim3(256), 0, stream>>>((const float *)v.data, narrow + total, total, p.heads, p.seq_k, head_dim,
                                                                  v.strides[0], v.strides[1], v.strides[2], v.strides[3]);
    note_launch(kLaunchAttention, 0, "fp32 tensors on fp16 copies of K and V: attention_narrow_kernel twice, then the 16-bit kernel");
    p.k = narrow;
    p.v = narrow + total;
    const int64_t contiguous[3] = {(int64_t)p.heads * p.seq_k * head_dim, (int64_t)p.seq_k * head_dim, head_dim};
    for (int d = 0; d < 3; ++d) p.k_strides[d] = p.v_strides[d] = contiguous[d];
    int result = NINETOOTHED_NO_KERNEL;
    if (head_dim == 128) result = (int)launch_attention<half_t, 128, 1, 64, 2, false, float>(p, stream);
    else if (head_dim == 64) result = (int)launch_attention<half_t, 64, 1, 64, 2, false, float>(p, stream);
    else if (head_dim == 32) result = (int)launch_attention<half_t, 32, 1, 64, 2, false, float>(p, stream);
    else result = launch_other_head_dim<half_t, float>(p, head_dim, stream);
    return result;
}

// variant: 0 = 128 query rows per workgroup, 64-key blocks, two workgroups per CU
//          1 = 256 query rows per workgroup, 64-key blocks, one workgroup per CU
//          2 = 128 query rows per workgroup, 32-key blocks, three workgroups per CU
//          3 = variant 0 with the software-pipelined main loop
//          4 = variant 3 with eight waves (256 query rows) per workgroup, one workgroup per CU
constexpr int kAttentionVariants = 5;
const char *const kAttentionVariantNames[kAttentionVariants] = {
    "plain loop, 64-key blocks, four waves (128 query rows), two workgroups per CU",
    "plain loop, 64-key blocks, 256 query rows per four-wave workgroup, one workgroup per CU",
    "plain loop, 32-key blocks, four waves, three workgroups per CU",
    "software-pipelined loop, 64-key blocks, four waves (128 query rows), two workgroups per CU",
    "software-pipelined loop, 64-key blocks, eight waves (256 query rows), one workgroup per CU",
};

bool attention_choice_known(int index, const int *, int) { return index >= 0 && index < kAttentionVariants; }
const bool g_attention_check_registered = tune_register_check(kTuneAttention, attention_choice_known);

template <typename T>
int dispatch_attention(AttentionParams &p, int head_dim, int variant, hipStream_t stream) {
    if (head_dim == 32) note_launch(kLaunchAttention, 0, "plain loop, 64-key blocks, head dimension 32");
    else if (head_dim != 128 && head_dim != 64) note_launch(kLaunchAttention, 0, "head dimension padded to the next kernel size");
    else note_launch(kLaunchAttention, variant, variant >= 0 && variant < kAttentionVariants ? kAttentionVariantNames[variant] : "measurement variant");
    if (head_dim == 128) {
        if (variant == 4) return (int)launch_attention<T, 128, 1, 64, 2, true, T, 8>(p, stream);
#ifdef NT_MEASUREMENT_AIDS
        if (variant == 5) return (int)launch_attention<T, 128, 1, 64, 2, false, T, 8>(p, stream);
        // 10 + v: variant v with the subtraction of the running maximum done per element (no folding)
        if (variant == 14) return (int)launch_attention<T, 128, 1, 64, 2, true, T, 8, false, false>(p, stream);
        if (variant == 13) return (int)launch_attention<T, 128, 1, 64, 2, true, T, kAttnWaves, false, false>(p, stream);
        if (variant == 11) return (int)launch_attention<T, 128, 2, 64, 1, false, T, kAttnWaves, false, false>(p, stream);
        if (variant == 10) return (int)launch_attention<T, 128, 1, 64, 2, false, T, kAttnWaves, false, false>(p, stream);
#endif
        if (variant == 3) return (int)launch_attention<T, 128, 1, 64, 2, true>(p, stream);
        if (variant == 1) return (int)launch_attention<T, 128, 2, 64, 1, false>(p, stream);
        if (variant == 2) return (int)launch_attention<T, 128, 1, 32, 3, false>(p, stream);
        return (int)launch_attention<T, 128, 1, 64, 2, false>(p, stream);
    }
    if (head_dim == 64) {
        if (variant == 4) return (int)launch_attention<T, 64, 1, 64, 2, true, T, 8>(p, stream);
        if (variant == 3) return (int)launch_attention<T, 64, 1, 64, 2, true>(p, stream);
        if (variant == 1) return (int)launch_attention<T, 64, 2, 64, 1, false>(p, stream);
        if (variant == 2) return (int)launch_attention<T, 64, 1, 32, 3, false>(p, stream);
        return (int)launch_attention<T, 64, 1, 64, 2, false>(p, stream);
    }
    if (head_dim == 32) return (int)launch_attention<T, 32, 1, 64, 2, false>(p, stream);
    return launch_other_head_dim<T, T>(p, head_dim, stream);
}

}  // namespace
}  // namespace nt

using namespace nt;

namespace nt {
namespace {

// validates the call and fills the parameters; returns 0, an error, or -1 when there is nothing to compute
int attention_setup(AttentionParams &p, const NineToothedTensor &q, const NineToothedTensor &k, const NineToothedTensor &v,
                    const NineToothedTensor &is_causal, const NineToothedTensor &scale, const NineToothedTensor &o, int dtype) {
    if (dtype != NINETOOTHED_FLOAT16 && dtype != NINETOOTHED_BFLOAT16 && dtype != NINETOOTHED_FLOAT32) return NINETOOTHED_NO_KERNEL;
    const bool float32 = dtype == NINETOOTHED_FLOAT32;
    const NineToothedTensor *ts[4] = {&q, &k, &v, &o};
    for (const NineToothedTensor *t : ts)
        if (!t->shape || !t->strides) return hipErrorInvalidValue;
    p.parts = 1;
    p.blocks_per_part = 0;
    p.part_o = p.part_lse = nullptr;
    p.batch = (int)q.shape[0];
    p.heads = (int)q.shape[1];
    p.seq_q = (int)q.shape[2];
    p.seq_k = (int)k.shape[2];
    const int64_t head_dim = (int64_t)q.shape[3];
    for (const NineToothedTensor *t : ts) {
        if (t->shape[0] != q.shape[0] || t->shape[1] != q.shape[1] || (int64_t)t->shape[3] != head_dim) return hipErrorInvalidValue;
        if (head_dim % 8 != 0) return NINETOOTHED_NO_KERNEL;  // (launch_nt_attention runs such tensors on padded copies)
        if (float32 && (t == &k || t == &v)) continue;  // converted copies: any strides
        if (t->strides[3] != 1 && head_dim > 1) return NINETOOTHED_NO_KERNEL;
        const int lanes = float32 ? 4 : 8;  // elements per 16 bytes
        if (((uintptr_t)t->data & 15) || t->strides[0] % lanes || t->strides[1] % lanes || t->strides[2] % lanes) return NINETOOTHED_NO_KERNEL;
    }
    if (v.shape[2] != k.shape[2] || o.shape[2] != q.shape[2]) return hipErrorInvalidValue;
    if (q.shape[2] > 0x7fffffffull || k.shape[2] > 0x7fffffffull) return NINETOOTHED_NO_KERNEL;
    // K and V of one (batch, head) are read through 32-bit buffer offsets
    for (const NineToothedTensor *t : {&k, &v}) {
        if (float32) break;
        if (t->strides[2] < 0) return NINETOOTHED_NO_KERNEL;
        if (((int64_t)t->shape[2] + 64) * t->strides[2] * 2 + 2 * head_dim > 0xffffffffll) return NINETOOTHED_NO_KERNEL;
    }
    if (p.batch == 0 || p.heads == 0 || p.seq_q == 0) return -1;
    if (p.seq_k == 0) return NINETOOTHED_NO_KERNEL;  // softmax over nothing
    for (int d = 0; d < 3; ++d) {
        p.q_strides[d] = q.strides[d];
        p.k_strides[d] = k.strides[d];
        p.v_strides[d] = v.strides[d];
        p.o_strides[d] = o.strides[d];
    }
    p.head_dim = (int)head_dim;
    p.q = q.data;
    p.k = k.data;
    p.v = v.data;
    p.o = o.data;
    // Q' = (Q * factor).to(element type).  Without a `scale` argument the factor is the literal of the
    // reference program, `q * 1.44269504089` (tests/test_attention.py:46): a tile times a Python literal is
    // computed in the tile's type with the literal rounded to that type first, and the fp32 product of two
    // 16-bit floats is exact, so rounding it once is that multiplication.  A run-time `scale` is an fp32
    // scalar: `q * (scale * 1.44269504089)` is an fp32 product rounded once.
    if (scale.data) p.q_scale = (float)Scalar0d::as_double(scale) * 1.44269504089f;
    else p.q_scale = dtype == NINETOOTHED_FLOAT16 ? 1.4423828125f : (dtype == NINETOOTHED_BFLOAT16 ? 1.4453125f : 1.44269504089f);
    p.causal = is_causal.data ? (Scalar0d::as_int64(is_causal) != 0) : 0;
#ifdef NT_ATTN_STAMPS
    p.stamps = g_attn_stamps;
#endif
    return 0;
}

void attention_tune_values(const AttentionParams &p, int dtype, int (&values)[7]) {
    const int v[7] = {dtype, p.batch, p.heads, p.seq_q, p.seq_k, p.head_dim, p.causal};
    for (int i = 0; i < 7; ++i) values[i] = v[i];
}

// whether the variants are alternatives for this problem (they exist for head dimensions 64 and 128)
bool attention_tunable(const AttentionParams &p, int dtype) { return dtype != NINETOOTHED_FLOAT32 && (p.head_dim == 128 || p.head_dim == 64); }

// the key range is split instead (decoding-like shapes); returns NINETOOTHED_NO_KERNEL when that does not apply
int attention_split(AttentionParams &p, int dtype, hipStream_t stream) {
    if (p.head_dim != 128 && p.head_dim != 64) return NINETOOTHED_NO_KERNEL;
    if (dtype == NINETOOTHED_FLOAT16) return p.head_dim == 128 ? launch_split_keys<half_t, 128>(p, stream) : launch_split_keys<half_t, 64>(p, stream);
    if (dtype == NINETOOTHED_BFLOAT16) return p.head_dim == 128 ? launch_split_keys<bf16_t, 128>(p, stream) : launch_split_keys<bf16_t, 64>(p, stream);
    return NINETOOTHED_NO_KERNEL;
}

// the variant a call without hints runs before anything is tuned: the pipelined loop, with eight waves for
// non-causal problems that have enough 256-row query blocks to fill the chip twice
int attention_untuned_variant(const AttentionParams &p) {
    return !p.causal && p.head_dim >= 64 && (int64_t)p.batch * p.heads * ceil_div(p.seq_q, 256) >= 512 ? 4 : 3;
}

bool attention_would_split(const AttentionParams &p) { return (p.head_dim == 128 || p.head_dim == 64) && split_key_parts(p) > 0; }

}  // namespace
}  // namespace nt

namespace nt {
namespace {

// ---- tensors the kernels cannot read in place: a head dimension that is no multiple of 8 (the reference pads it
// to a power of two inside its kernel and masks), rows that do not start on 16-byte boundaries, a strided last
// dimension.  Q, K and V are copied into dense [B, H, S, D8] buffers of the stream's scratch memory, D8 = D rounded
// up to 8 with zeros (zero columns add nothing to Q K^T, and the columns of O they produce are dropped), the
// attention runs on the copies, and O is copied back.
template <typename E>
__global__ __launch_bounds__(256) void attention_pad_kernel(const E *src, E *dst, int64_t rows, int heads, int seq, int d, int d8, int64_t s0, int64_t s1,
                                                            int64_t s2, int64_t s3, int back) {
    // back == 0: dst[row][0 .. d8) = src row, zero padded; back != 0: the first d columns of the dense `src` rows go to `dst`.
    // One thread per 8 columns of a row: one load and one store of 8 elements where the strided side is contiguous
    // (global accesses need the element's alignment only), element by element otherwise.
    typedef E vec8 __attribute__((ext_vector_type(8)));
    typedef vec8 unaligned_vec8 __attribute__((aligned(sizeof(E))));
    const int chunks = d8 / 8;
    const int64_t total = rows * chunks;
    for (int64_t index = (int64_t)blockIdx.x * 256 + threadIdx.x; index < total; index += (int64_t)gridDim.x * 256) {
        const int64_t row = index / chunks;
        const int col = (int)(index - row * chunks) * 8;
        const int64_t bh = row / seq;
        const int64_t strided = (bh / heads) * s0 + (bh % heads) * s1 + (row % seq) * s2 + (int64_t)col * s3;
        const bool whole = s3 == 1 && col + 8 <= d;
        if (back) {
            const vec8 values = *(const vec8 *)(src + row * d8 + col);
            if (whole) {
                *(unaligned_vec8 *)(dst + strided) = values;
            } else {
#pragma unroll
                for (int c = 0; c < 8; ++c)
                    if (col + c < d) dst[strided + c * s3] = values[c];
            }
        } else {
            vec8 values;
            if (whole) {
                values = *(const unaligned_vec8 *)(src + strided);
            } else {
#pragma unroll
                for (int c = 0; c < 8; ++c) values[c] = col + c < d ? src[strided + c * s3] : (E)0;
            }
            *(vec8 *)(dst + row * d8 + col) = values;
        }
    }
}

template <typename E>
hipError_t attention_pad(hipStream_t stream, const NineToothedTensor &t, void *dense, int d8, bool back) {
    const int64_t rows = (int64_t)t.shape[0] * t.shape[1] * t.shape[2];
    const int64_t work = rows * (d8 / 8);
    if (work == 0) return hipSuccess;
    const unsigned blocks = (unsigned)std::min<int64_t>((work + 255) / 256, 256 * 64);
    if (back)
        attention_pad_kernel<E><<<dim3(blocks), dim3(256), 0, stream>>>((const E *)dense, (E *)t.data, rows, (int)t.shape[1], (int)t.shape[2], (int)t.shape[3], d8,
                                                                           t.strides[0], t.strides[1], t.strides[2], t.strides[3], 1);
    else
        attention_pad_kernel<E><<<dim3(blocks), dim3(256), 0, stream>>>((const E *)t.data, (E *)dense, rows, (int)t.shape[1], (int)t.shape[2], (int)t.shape[3], d8,
                                                                           t.strides[0], t.strides[1], t.strides[2], t.strides[3], 0);
    return hipGetLastError();
}

int launch_attention(hipStream_t stream, const NineToothedTensor &q, const NineToothedTensor &k, const NineToothedTensor &v, const NineToothedTensor &is_causal,
                     const NineToothedTensor &scale, const NineToothedTensor &o, int dtype, int block_size_m, int block_size_n, bool may_copy);

// 0 / an error when the attention ran on copies, NINETOOTHED_NO_KERNEL when this way does not apply either
int attention_on_padded_copies(hipStream_t stream, const NineToothedTensor &q, const NineToothedTensor &k, const NineToothedTensor &v,
                               const NineToothedTensor &is_causal, const NineToothedTensor &scale, const NineToothedTensor &o, int dtype,
                               int block_size_m, int block_size_n) {
    if (dtype != NINETOOTHED_FLOAT16 && dtype != NINETOOTHED_BFLOAT16 && dtype != NINETOOTHED_FLOAT32) return NINETOOTHED_NO_KERNEL;
    const NineToothedTensor *ts[4] = {&q, &k, &v, &o};
    for (const NineToothedTensor *t : ts)
        if (!t->shape || !t->strides) return NINETOOTHED_NO_KERNEL;
    const uint64_t d = q.shape[3];
    if (d == 0 || d > 256) return NINETOOTHED_NO_KERNEL;
    for (const NineToothedTensor *t : ts)
        if (t->shape[0] != q.shape[0] || t->shape[1] != q.shape[1] || t->shape[3] != d) return NINETOOTHED_NO_KERNEL;
    if (v.shape[2] != k.shape[2] || o.shape[2] != q.shape[2] || k.shape[2] == 0) return NINETOOTHED_NO_KERNEL;
    const int d8 = (int)((d + 7) / 8 * 8);
    const size_t size = dtype == NINETOOTHED_FLOAT32 ? 4 : 2;
    WorkspaceLease lease(stream);  // held until the copy back is enqueued
    const WorkspacePurpose purposes[4] = {kWorkspaceAttentionPaddedQ, kWorkspaceAttentionPaddedK, kWorkspaceAttentionPaddedV, kWorkspaceAttentionPaddedO};
    void *dense[4];
    uint64_t shapes[4][4];
    int64_t strides[4][4];
    NineToothedTensor copies[4];
    for (int i = 0; i < 4; ++i) {
        const NineToothedTensor &t = *ts[i];
        const uint64_t rows = t.shape[0] * t.shape[1] * t.shape[2];
        if (rows * (uint64_t)d8 > 0x7fffffffull * 8) return NINETOOTHED_NO_KERNEL;
        dense[i] = lease.get(purposes[i], (size_t)rows * d8 * size + 256);
        if (dense[i] == nullptr) return NINETOOTHED_NO_KERNEL;
        for (int a = 0; a < 3; ++a) shapes[i][a] = t.shape[a];
        shapes[i][3] = (uint64_t)d8;
        strides[i][3] = 1;
        strides[i][2] = d8;
        strides[i][1] = (int64_t)t.shape[2] * d8;
        strides[i][0] = (int64_t)t.shape[1] * strides[i][1];
        copies[i] = NineToothedTensor{dense[i], shapes[i], strides[i]};
    }
    for (int i = 0; i < 3; ++i) {
        const hipError_t err = size == 4 ? attention_pad<float>(stream, *ts[i], dense[i], d8, false) : attention_pad<uint16_t>(stream, *ts[i], dense[i], d8, false);
        if (err != hipSuccess) return (int)err;
    }
    const int result = launch_attention(stream, copies[0], copies[1], copies[2], is_causal, scale, copies[3], dtype, block_size_m, block_size_n, false);
    if (result != 0) return result;
    return (int)(size == 4 ? attention_pad<float>(stream, o, dense[3], d8, true) : attention_pad<uint16_t>(stream, o, dense[3], d8, true));
}

int launch_attention(hipStream_t stream, const NineToothedTensor &q, const NineToothedTensor &k, const NineToothedTensor &v, const NineToothedTensor &is_causal,
                     const NineToothedTensor &scale, const NineToothedTensor &o, int dtype, int block_size_m, int block_size_n, bool may_copy) {
    AttentionParams p;
    const int status = attention_setup(p, q, k, v, is_causal, scale, o, dtype);
    if (status == NINETOOTHED_NO_KERNEL && may_copy) return attention_on_padded_copies(stream, q, k, v, is_causal, scale, o, dtype, block_size_m, block_size_n);
    if (status != 0) return status < 0 ? 0 : status;
    const int head_dim = p.head_dim;
    if (dtype == NINETOOTHED_FLOAT32) return attention_float32(p, head_dim, k, v, block_size_m == 0 && block_size_n == 0, (hipStream_t)stream);
    // block sizes are hints: 256 query rows select the one-workgroup-per-CU variant, 32-key blocks the
    // three-workgroups-per-CU variant, 64-key blocks the plain loop.  Without a hint the choice is the one
    // tuned for this problem (nt_tune_attention), else the pipelined loop (measured at [4, 32, 4096, 128]:
    // 1.12 against 1.08 PFLOP/s for the plain loop, causal 1.01 against 0.98); non-causal problems with enough
    // 256-row blocks to fill the chip twice run it with eight waves per workgroup, which loads every K / V
    // block once for 256 query rows (1.16 PFLOP/s; causal 0.99, below the four-wave form).
    int variant = block_size_m >= 256 ? 1 : (block_size_n > 0 && block_size_n <= 32 ? 2 : (block_size_n >= 64 ? 0 : 3));
    if (variant == 3 && block_size_m == 0) variant = attention_untuned_variant(p);
#ifdef NT_MEASUREMENT_AIDS
    if (block_size_n >= 1000) variant = block_size_n - 1000;  // explicit variant, for timing harnesses only
#endif
    if (block_size_m == 0 && block_size_n == 0) {  // no hints
        const int result = attention_split(p, dtype, (hipStream_t)stream);  // decoding-like shapes split the keys
        if (result != NINETOOTHED_NO_KERNEL) return result;
        if (attention_tunable(p, dtype)) {
            int values[7];
            attention_tune_values(p, dtype, values);
            const int tuned = tune_lookup(kTuneAttention, values, 7);
            if (tuned >= 0 && tuned < kAttentionVariants) variant = tuned;
        }
    }
    int result;
    if (dtype == NINETOOTHED_FLOAT16) result = dispatch_attention<half_t>(p, head_dim, variant, (hipStream_t)stream);
    else result = dispatch_attention<bf16_t>(p, head_dim, variant, (hipStream_t)stream);
    return result;
}

}  // namespace
}  // namespace nt

extern "C" NineToothedResult launch_nt_attention(NineToothedStream stream, NineToothedTensor q, NineToothedTensor k,
                                                 NineToothedTensor v, NineToothedTensor is_causal,
                                                 NineToothedTensor scale, NineToothedTensor o, int dtype,
                                                 int block_size_m, int block_size_n) {
    return launch_attention((hipStream_t)stream, q, k, v, is_causal, scale, o, dtype, block_size_m, block_size_n, true);
}

// Times the loop variants of launch_nt_attention on this problem and records the fastest for later launches
// without block-size hints.  *best_variant = -1 when nothing was timed (a stream under graph capture), -2 when
// the problem has no alternatives (fp32 tensors, head dimensions other than 64 and 128, shapes that split the keys).
extern "C" NineToothedResult nt_tune_attention(NineToothedStream stream, NineToothedTensor q, NineToothedTensor k, NineToothedTensor v,
                                               NineToothedTensor is_causal, NineToothedTensor scale, NineToothedTensor o, int dtype,
                                               int iters, int *best_variant, float *best_ms) {
    if (best_variant) *best_variant = -2;
    if (best_ms) *best_ms = 0.0f;
    AttentionParams p;
    const int status = attention_setup(p, q, k, v, is_causal, scale, o, dtype);
    if (status == NINETOOTHED_NO_KERNEL) return 0;  // (tensors that launch_nt_attention runs on padded copies: no alternatives)
    if (status != 0) return status < 0 ? 0 : status;
    if (!attention_tunable(p, dtype) || attention_would_split(p)) return 0;
    int best = -1;
    float best_time = 0.0f;
    // the untuned rule's variant comes first and stays unless another one is more than 2 % faster: the pipelined
    // variants lie within a few per cent of each other, and the choice should not change from process to process
    // for nothing
    const int preferred = attention_untuned_variant(p);
    auto variant_of = [&](int i) { return i == 0 ? preferred : (i - 1 < preferred ? i - 1 : i); };
    const int result = tune_time((hipStream_t)stream, kAttentionVariants, iters, [&](int i) -> int {
        AttentionParams copy = p;
        if (dtype == NINETOOTHED_FLOAT16) return dispatch_attention<half_t>(copy, p.head_dim, variant_of(i), (hipStream_t)stream);
        return dispatch_attention<bf16_t>(copy, p.head_dim, variant_of(i), (hipStream_t)stream);
    }, &best, &best_time, 0.02f);
    if (result != 0) return result;
    if (best >= 0) best = variant_of(best);
    if (best_variant) *best_variant = best;
    if (best < 0) return 0;
    int values[7];
    attention_tune_values(p, dtype, values);
    tune_record(kTuneAttention, values, 7, best);
    if (best_ms) *best_ms = best_time;
    return 0;
}

#ifdef NT_ATTN_STAMPS
extern "C" void nt_debug_attention_stamps(void *buffer) { nt::g_attn_stamps = (unsigned long long *)buffer; }
#endif
