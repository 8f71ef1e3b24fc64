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

#include "gemm_fast.h"  // swizzle helpers, static_for, lds_barrier

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
};

constexpr int kAttnWaves = 4;

// BN: key/value rows per block; kOcc: waves per SIMD the register budget is held to
template <typename T, int D, int kQTiles, int BN, int kOcc>
__global__ __launch_bounds__(kAttnWaves * 64, kOcc) void attention_fwd_kernel(AttentionParams p) {
#if defined(__HIP_DEVICE_COMPILE__)
    typedef Elem<T> E;
    typedef typename E::vec8 vec8;
    constexpr int BM = kAttnWaves * 32 * kQTiles;
    constexpr int KT = BN / 32;          // kv tiles of S^T per block
    constexpr int DT = D / 32;           // d tiles of O^T
    constexpr int KS = D / 16;           // contraction steps of S^T
    constexpr int PS = BN / 16;          // contraction steps of O^T
    constexpr int kTileBytes = BN * D * 2;
    constexpr int kChunksPerRow = D / 8;
    constexpr int kRowsPerInstr = 64 / kChunksPerRow;
    constexpr int kInstr = kTileBytes / (kAttnWaves * 1024);
    static_assert(D % 32 == 0 && D >= 32 && D <= 256, "head dim");
    static_assert(kTileBytes % (kAttnWaves * 1024) == 0, "tile/wave mismatch");

    __shared__ __attribute__((aligned(1024))) unsigned char lds_k0[kTileBytes];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_v0[kTileBytes];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_k1[kTileBytes];
    __shared__ __attribute__((aligned(1024))) unsigned char lds_v1[kTileBytes];
    auto stage_k = [&](auto tag) -> NT_LDS unsigned char * {
        if constexpr (decltype(tag)::value == 0) return (NT_LDS unsigned char *)lds_k0;
        else return (NT_LDS unsigned char *)lds_k1;
    };
    auto stage_v = [&](auto tag) -> NT_LDS unsigned char * {
        if constexpr (decltype(tag)::value == 0) return (NT_LDS unsigned char *)lds_v0;
        else return (NT_LDS unsigned char *)lds_v1;
    };

    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int g = lane >> 5;
    const int l32 = lane & 31;

    // workgroup -> (batch, head, query block).  Non-causal: consecutive ids are
    // the query blocks of one (batch, head) and share its K/V in L2.  Causal: the
    // work of a query block grows with its index, so ids walk the (batch, head)
    // pairs first and the query blocks from last (longest) to first; every CU then
    // gets the same mix of long and short blocks.
    int qb, bh;
    if (p.causal) {
        const int pairs = p.batch * p.heads;
        qb = p.q_blocks - 1 - blockIdx.x / pairs;
        bh = blockIdx.x % pairs;
    } else {
        qb = blockIdx.x % p.q_blocks;
        bh = blockIdx.x / p.q_blocks;
    }
    const int head = bh % p.heads;
    const int batch = bh / p.heads;
    const int q0 = qb * BM;

    const T *Q = (const T *)p.q + batch * p.q_strides[0] + head * p.q_strides[1];
    const T *K = (const T *)p.k + batch * p.k_strides[0] + head * p.k_strides[1];
    const T *V = (const T *)p.v + batch * p.v_strides[0] + head * p.v_strides[1];
    T *O = (T *)p.o + batch * p.o_strides[0] + head * p.o_strides[1];

    // ---- Q' fragments (B operand of S^T): lane holds row l32 of its q tile, 8 d's per step ----
    vec8 qf[kQTiles][KS];
    int q_row[kQTiles];
#pragma unroll
    for (int qt = 0; qt < kQTiles; ++qt) {
        q_row[qt] = q0 + (wave * kQTiles + qt) * 32 + l32;
        const int row = min(q_row[qt], p.seq_q - 1);
        const T *src = Q + (int64_t)row * p.q_strides[2];
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            vec8 raw = *(const vec8 *)(src + ks * 16 + 8 * g);
#pragma unroll
            for (int e = 0; e < 8; ++e) raw[e] = E::from_float(E::to_float(raw[e]) * p.q_scale);
            qf[qt][ks] = raw;
        }
    }

    // ---- number of kv blocks this query block needs ----
    int kv_end = p.seq_k;
    if (p.causal) kv_end = min(kv_end, q0 + BM);  // keys beyond the last query row are masked for all rows
    const int num_blocks = ceil_div(kv_end, BN);
    const int last_block = num_blocks - 1;

    // ---- global -> LDS assignment ----
    int ld_row[kInstr];
    unsigned ld_k_col[kInstr], ld_v_col[kInstr];
#pragma unroll
    for (int j = 0; j < kInstr; ++j) {
        const int row = (j * kAttnWaves + wave) * kRowsPerInstr + lane / kChunksPerRow;
        const int phys = lane % kChunksPerRow;
        ld_row[j] = row;
        ld_k_col[j] = a_phys_chunk<D>(row, phys) * 8;
        ld_v_col[j] = b_phys_chunk<D>(row, phys) * 8;
    }
    auto issue_loads = [&](auto stage_tag, int blk) {
        NT_LDS unsigned char *sk = stage_k(stage_tag);
        NT_LDS unsigned char *sv = stage_v(stage_tag);
#pragma unroll
        for (int j = 0; j < kInstr; ++j) {
            const int row = min(blk * BN + ld_row[j], p.seq_k - 1);  // rows past the end are masked later
            global_to_lds_16(K + (int64_t)row * p.k_strides[2] + ld_k_col[j], sk + (j * kAttnWaves + wave) * 1024);
            global_to_lds_16(V + (int64_t)row * p.v_strides[2] + ld_v_col[j], sv + (j * kAttnWaves + wave) * 1024);
        }
    };

    // ---- LDS read offsets ----
    int k_row_off[KT], k_row_sw[KT];
#pragma unroll
    for (int kt = 0; kt < KT; ++kt) {
        const int row = kt * 32 + l32;
        k_row_off[kt] = row * (D * 2);
        k_row_sw[kt] = a_phys_chunk<D>(row, 0);
    }
    const int i16 = lane & 15;
    const int v_row = 4 * g + (i16 >> 2);  // + 16 * step (+ 8 for the upper slots)
    int v_col_chunk[DT], v_col_in[DT];
#pragma unroll
    for (int dt = 0; dt < DT; ++dt) {
        const int col = dt * 32 + 16 * ((lane >> 4) & 1) + 4 * (i16 & 3);
        v_col_chunk[dt] = col >> 3;
        v_col_in[dt] = (col & 7) * 2;
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
        m_run[qt] = -INFINITY;
        l_run[qt] = 0.0f;
    }

    auto process_block = [&](auto stage_tag, int blk) {
        const NT_LDS unsigned char *sk = stage_k(stage_tag);
        const NT_LDS unsigned char *sv = stage_v(stage_tag);

        // S^T = K . Q'^T
        float16_t s_acc[KT][kQTiles];
#pragma unroll
        for (int kt = 0; kt < KT; ++kt)
#pragma unroll
            for (int qt = 0; qt < kQTiles; ++qt)
#pragma unroll
                for (int r = 0; r < 16; ++r) s_acc[kt][qt][r] = 0.0f;
#pragma unroll
        for (int ks = 0; ks < KS; ++ks) {
            vec8 kf[KT];
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) {
                const int chunk = (ks * 2 + g) ^ k_row_sw[kt];
                kf[kt] = *(const NT_LDS vec8 *)(sk + k_row_off[kt] + chunk * 16);
            }
#pragma unroll
            for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                for (int qt = 0; qt < kQTiles; ++qt) s_acc[kt][qt] = E::mfma32(kf[kt], qf[qt][ks], s_acc[kt][qt]);
        }

        // masks: keys past the end of the sequence, and (causal) keys after the query
        const int kv0 = blk * BN;
        const bool mask_tail = kv0 + BN > p.seq_k || blk > last_block;
        const bool mask_causal = p.causal && (kv0 + BN - 1 > q0 + wave * kQTiles * 32);
        if (mask_tail || mask_causal) {
            const int limit = blk > last_block ? 0 : p.seq_k;
#pragma unroll
            for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                for (int qt = 0; qt < kQTiles; ++qt)
#pragma unroll
                    for (int r = 0; r < 16; ++r) {
                        const int kv = kv0 + kt * 32 + 8 * (r >> 2) + 4 * g + (r & 3);
                        const bool keep = kv < limit && (!p.causal || q_row[qt] >= kv);
                        if (!keep) s_acc[kt][qt][r] = -INFINITY;
                    }
        }

        // online softmax per query row (= per lane and q tile)
#pragma unroll
        for (int qt = 0; qt < kQTiles; ++qt) {
            float mx = -INFINITY;
#pragma unroll
            for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                for (int r = 0; r < 16; ++r) mx = fmaxf(mx, s_acc[kt][qt][r]);
            mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
            const float m_new = fmaxf(m_run[qt], mx);
            const float m_use = m_new == -INFINITY ? 0.0f : m_new;  // fully masked so far
            const float alpha = __builtin_amdgcn_exp2f(m_run[qt] - m_use);
            m_run[qt] = m_new;
            float sum = 0.0f;
#pragma unroll
            for (int kt = 0; kt < KT; ++kt)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const float pv = __builtin_amdgcn_exp2f(s_acc[kt][qt][r] - m_use);
                    s_acc[kt][qt][r] = pv;
                    sum += pv;
                }
            l_run[qt] = l_run[qt] * alpha + sum;
            // the running maximum settles after a few blocks; skip the rescale of the
            // output accumulators when no row of this wave's tile moved (wave-uniform)
            if (__builtin_amdgcn_ballot_w64(alpha != 1.0f) != 0) {
#pragma unroll
                for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                    for (int r = 0; r < 16; ++r) o_acc[dt][qt][r] *= alpha;
            }
        }

        // O^T += V^T . P^T
#pragma unroll
        for (int ps = 0; ps < PS; ++ps) {
            vec8 pf[kQTiles];
#pragma unroll
            for (int qt = 0; qt < kQTiles; ++qt)
#pragma unroll
                for (int e = 0; e < 8; ++e) pf[qt][e] = E::from_float(s_acc[ps / 2][qt][8 * (ps & 1) + e]);
            vec8 vf[DT];
#pragma unroll
            for (int dt = 0; dt < DT; ++dt) {
                const int r_lo = ps * 16 + v_row;
                const int r_hi = r_lo + 8;
                const int c_lo = b_phys_chunk<D>(r_lo, v_col_chunk[dt]);
                const int c_hi = b_phys_chunk<D>(r_hi, v_col_chunk[dt]);
                short4_t lo = lds_read_tr16_b64(sv + r_lo * (D * 2) + c_lo * 16 + v_col_in[dt]);
                short4_t hi = lds_read_tr16_b64(sv + r_hi * (D * 2) + c_hi * 16 + v_col_in[dt]);
                short8_t both = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
                vf[dt] = __builtin_bit_cast(vec8, both);
            }
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int qt = 0; qt < kQTiles; ++qt) o_acc[dt][qt] = E::mfma32(vf[dt], pf[qt], o_acc[dt][qt]);
        }
    };

    // two LDS stages, loop unrolled by two; an odd block count runs one fully
    // masked extra block, whose loads re-fetch the last block
    typedef std::integral_constant<int, 0> Stage0;
    typedef std::integral_constant<int, 1> Stage1;
    if (num_blocks > 0) {
        issue_loads(Stage0(), 0);
        for (int blk = 0; blk < num_blocks; blk += 2) {
            wait_vmcnt<0>();
            lds_barrier();
            issue_loads(Stage1(), min(blk + 1, last_block));
            process_block(Stage0(), blk);
            wait_vmcnt<0>();
            lds_barrier();
            issue_loads(Stage0(), min(blk + 2, last_block));
            process_block(Stage1(), blk + 1);
        }
        wait_vmcnt<0>();  // nothing may still be writing LDS when the workgroup ends
    }

    // ---- epilogue: O[q, d] = O^T[d, q] / l ----
#pragma unroll
    for (int qt = 0; qt < kQTiles; ++qt) {
        const float l_total = l_run[qt] + __shfl_xor(l_run[qt], 32, 64);
        const float inv = 1.0f / l_total;
        if (q_row[qt] < p.seq_q) {
            T *dst = O + (int64_t)q_row[qt] * p.o_strides[2];
#pragma unroll
            for (int dt = 0; dt < DT; ++dt)
#pragma unroll
                for (int r4 = 0; r4 < 4; ++r4) {
                    typedef T vec4 __attribute__((ext_vector_type(4)));
                    vec4 out;
#pragma unroll
                    for (int e = 0; e < 4; ++e) out[e] = E::from_float(o_acc[dt][qt][r4 * 4 + e] * inv);
                    *(vec4 *)(dst + dt * 32 + 8 * r4 + 4 * g) = out;
                }
        }
    }
#endif
}

template <typename T, int D, int kQTiles, int BN, int kOcc>
hipError_t launch_attention(AttentionParams &p, hipStream_t stream) {
    constexpr int BM = kAttnWaves * 32 * kQTiles;
    p.q_blocks = ceil_div(p.seq_q, BM);
    const int64_t grid = (int64_t)p.batch * p.heads * p.q_blocks;
    if (grid == 0) return hipSuccess;
    attention_fwd_kernel<T, D, kQTiles, BN, kOcc><<<dim3((unsigned)grid), dim3(kAttnWaves * 64), 0, stream>>>(p);
    return hipGetLastError();
}

// variant: 0 = 128 query rows per workgroup, 64-key blocks, two workgroups per CU (default)
//          1 = 256 query rows per workgroup, 64-key blocks, one workgroup per CU
//          2 = 128 query rows per workgroup, 32-key blocks, three workgroups per CU
template <typename T>
int dispatch_attention(AttentionParams &p, int head_dim, int variant, hipStream_t stream) {
    if (head_dim == 128) {
        if (variant == 1) return (int)launch_attention<T, 128, 2, 64, 1>(p, stream);
        if (variant == 2) return (int)launch_attention<T, 128, 1, 32, 3>(p, stream);
        return (int)launch_attention<T, 128, 1, 64, 2>(p, stream);
    }
    if (head_dim == 64) {
        if (variant == 1) return (int)launch_attention<T, 64, 2, 64, 1>(p, stream);
        if (variant == 2) return (int)launch_attention<T, 64, 1, 32, 3>(p, stream);
        return (int)launch_attention<T, 64, 1, 64, 2>(p, stream);
    }
    if (head_dim == 32) return (int)launch_attention<T, 32, 1, 64, 2>(p, stream);
    return NINETOOTHED_NO_KERNEL;
}

}  // namespace
}  // namespace nt

using namespace nt;

extern "C" NineToothedResult launch_nt_attention(NineToothedStream stream, NineToothedTensor q, NineToothedTensor k,
                                                 NineToothedTensor v, NineToothedTensor is_causal,
                                                 NineToothedTensor scale, NineToothedTensor o, int dtype,
                                                 int block_size_m, int block_size_n) {
    if (dtype != NINETOOTHED_FLOAT16 && dtype != NINETOOTHED_BFLOAT16) return NINETOOTHED_NO_KERNEL;
    const NineToothedTensor *ts[4] = {&q, &k, &v, &o};
    for (const NineToothedTensor *t : ts)
        if (!t->shape || !t->strides) return hipErrorInvalidValue;
    AttentionParams p;
    p.batch = (int)q.shape[0];
    p.heads = (int)q.shape[1];
    p.seq_q = (int)q.shape[2];
    p.seq_k = (int)k.shape[2];
    const int64_t head_dim = (int64_t)q.shape[3];
    for (const NineToothedTensor *t : ts) {
        if (t->shape[0] != q.shape[0] || t->shape[1] != q.shape[1] || (int64_t)t->shape[3] != head_dim) return hipErrorInvalidValue;
        if (t->strides[3] != 1 && head_dim > 1) return NINETOOTHED_NO_KERNEL;
        if (((uintptr_t)t->data & 15) || t->strides[0] % 8 || t->strides[1] % 8 || t->strides[2] % 8) return NINETOOTHED_NO_KERNEL;
    }
    if (v.shape[2] != k.shape[2] || o.shape[2] != q.shape[2]) return hipErrorInvalidValue;
    if (q.shape[2] > 0x7fffffffull || k.shape[2] > 0x7fffffffull) return NINETOOTHED_NO_KERNEL;
    if (p.batch == 0 || p.heads == 0 || p.seq_q == 0) return 0;
    if (p.seq_k == 0) return NINETOOTHED_NO_KERNEL;  // softmax over nothing
    for (int d = 0; d < 3; ++d) {
        p.q_strides[d] = q.strides[d];
        p.k_strides[d] = k.strides[d];
        p.v_strides[d] = v.strides[d];
        p.o_strides[d] = o.strides[d];
    }
    p.q = q.data;
    p.k = k.data;
    p.v = v.data;
    p.o = o.data;
    const double scale_value = scale.data ? Scalar0d::as_double(scale) : 1.0;
    p.q_scale = (float)(scale_value * 1.4426950408889634);
    p.causal = is_causal.data ? (Scalar0d::as_int64(is_causal) != 0) : 0;
    // block sizes are hints: 256 query rows select the one-workgroup-per-CU
    // variant, 32-key blocks the three-workgroups-per-CU variant
    const int variant = block_size_m >= 256 ? 1 : (block_size_n > 0 && block_size_n <= 32 ? 2 : 0);
    if (dtype == NINETOOTHED_FLOAT16) return dispatch_attention<half_t>(p, (int)head_dim, variant, (hipStream_t)stream);
    return dispatch_attention<bf16_t>(p, (int)head_dim, variant, (hipStream_t)stream);
}
