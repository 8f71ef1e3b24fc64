// Measurement kernel: the rate at which this GPU issues 32x32x16 fp16 MFMAs when nothing else happens --
// operands in registers, no LDS, no memory traffic inside the loop -- on operand values taken from caller
// tensors.  It bounds what any fp16 GEMM or attention kernel can reach on the same data: with random operands
// the chip lowers its clock under the matrix pipe's power draw, so the bound is below the 2.5 PFLOP/s that
// 1024 FLOP per clock and SIMD give at 2.4 GHz.  The results are meaningless as numbers.
#include <algorithm>

#include "nt_common.h"

namespace nt {
namespace {

__global__ __launch_bounds__(512, 2) void mfma_rate_kernel(const half_t *a, const half_t *b, int64_t elements, int loops, float *sink) {
#if defined(__HIP_DEVICE_COMPILE__)
    // every lane takes 4 + 2 fragments of 8 consecutive values from the operands (a different place per lane, wave
    // and workgroup), as a wave of the GEMM kernel holds them for one k step of its 128 x 64 tile
    const int64_t lane_id = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    half8_t af[4], bf[2];
#pragma unroll
    for (int i = 0; i < 4; ++i) af[i] = *(const half8_t *)(a + ((lane_id * 4 + i) * 8) % (elements - 8));
#pragma unroll
    for (int i = 0; i < 2; ++i) bf[i] = *(const half8_t *)(b + ((lane_id * 2 + i) * 8) % (elements - 8));
    float16_t acc[4][2];
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[i][j][r] = 0.0f;
    for (int it = 0; it < loops; ++it) {
#pragma unroll
        for (int i = 0; i < 4; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x16_f16(bf[j], af[i], acc[i][j], 0, 0, 0);
        // keep the compiler from collapsing the loop; costs no instruction
#pragma unroll
        for (int i = 0; i < 4; ++i) asm volatile("" : "+v"(af[i]));
    }
    float total = 0.0f;
#pragma unroll
    for (int i = 0; i < 4; ++i)
#pragma unroll
        for (int j = 0; j < 2; ++j)
#pragma unroll
            for (int r = 0; r < 16; ++r) total += acc[i][j][r];
    if (total == 12345.678f) sink[0] = total;  // (never true in practice: the accumulators must stay live)
#endif
}

// The same with 16x16x32 MFMAs (half the FLOP of a 32x32x16 one in half the time): 8 + 4 fragments, as a wave of the
// fast GEMM kernel holds them for its 128 x 64 tile.  On random operands this form sustains a higher rate at the
// part's power limit: per FLOP it moves half as many accumulator values.
__global__ __launch_bounds__(512, 2) void mfma_rate_16x16x32_kernel(const half_t *a, const half_t *b, int64_t elements, int loops, float *sink) {
#if defined(__HIP_DEVICE_COMPILE__)
    const int64_t lane_id = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    half8_t af[8], bf[4];
#pragma unroll
    for (int i = 0; i < 8; ++i) af[i] = *(const half8_t *)(a + ((lane_id * 8 + i) * 8) % (elements - 8));
#pragma unroll
    for (int i = 0; i < 4; ++i) bf[i] = *(const half8_t *)(b + ((lane_id * 4 + i) * 8) % (elements - 8));
    float4_t acc[8][4];
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) acc[i][j] = float4_t{0.0f, 0.0f, 0.0f, 0.0f};
    for (int it = 0; it < loops; ++it) {
#pragma unroll
        for (int i = 0; i < 8; ++i)
#pragma unroll
            for (int j = 0; j < 4; ++j) acc[i][j] = __builtin_amdgcn_mfma_f32_16x16x32_f16(bf[j], af[i], acc[i][j], 0, 0, 0);
#pragma unroll
        for (int i = 0; i < 8; ++i) asm volatile("" : "+v"(af[i]));
    }
    float total = 0.0f;
#pragma unroll
    for (int i = 0; i < 8; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j)
#pragma unroll
            for (int r = 0; r < 4; ++r) total += acc[i][j][r];
    if (total == 12345.678f) sink[0] = total;
#endif
}

// validates the operands of a probe launch; returns the element count both may be read over, or 0
int64_t probe_elements(const NineToothedTensor &a, const NineToothedTensor &b) {
    if (!a.shape || !b.shape || !a.strides || !b.strides || a.data == nullptr || b.data == nullptr) return 0;
    // the kernels read the first shape[0] * shape[1] elements behind each pointer: dense row-major matrices only
    if (a.strides[1] != 1 || b.strides[1] != 1 || a.strides[0] != (int64_t)a.shape[1] || b.strides[0] != (int64_t)b.shape[1]) return 0;
    const int64_t elements = std::min<int64_t>((int64_t)a.shape[0] * (int64_t)a.shape[1], (int64_t)b.shape[0] * (int64_t)b.shape[1]);
    return elements < 4096 ? 0 : elements;
}

int probe_units() {
    int device = 0, units = 0;
    if (hipGetDevice(&device) != hipSuccess || hipDeviceGetAttribute(&units, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess) return 0;
    return units;
}

}  // namespace
}  // namespace nt

// Launches one workgroup of eight waves per compute unit and lets every wave issue loops x 8 MFMAs on fragments
// read from `a` and `b` (FLOAT16 tensors of at least 4096 elements; only their values matter).  *mfma_count
// receives the number of MFMAs issued in total (each 2 x 32 x 32 x 16 FLOP).  Asynchronous on `stream`.
extern "C" NineToothedResult nt_probe_mfma_rate(NineToothedStream stream, NineToothedTensor a, NineToothedTensor b, int loops, float *sink,
                                                int64_t *mfma_count) {
    if (sink == nullptr || loops <= 0) return hipErrorInvalidValue;
    const int64_t elements = nt::probe_elements(a, b);
    if (elements == 0) return hipErrorInvalidValue;
    const int units = nt::probe_units();
    if (units <= 0) return hipErrorInvalidDevice;
    nt::mfma_rate_kernel<<<dim3((unsigned)units), dim3(512), 0, (hipStream_t)stream>>>((const nt::half_t *)a.data, (const nt::half_t *)b.data, elements, loops, sink);
    if (mfma_count) *mfma_count = (int64_t)units * 8 * loops * 8;
    return (int)hipGetLastError();
}

// The same with 16x16x32 MFMAs (2 x 16 x 16 x 32 FLOP each): loops x 32 per wave.
extern "C" NineToothedResult nt_probe_mfma_rate_16x16x32(NineToothedStream stream, NineToothedTensor a, NineToothedTensor b, int loops, float *sink,
                                                         int64_t *mfma_count) {
    if (sink == nullptr || loops <= 0) return hipErrorInvalidValue;
    const int64_t elements = nt::probe_elements(a, b);
    if (elements == 0) return hipErrorInvalidValue;
    const int units = nt::probe_units();
    if (units <= 0) return hipErrorInvalidDevice;
    nt::mfma_rate_16x16x32_kernel<<<dim3((unsigned)units), dim3(512), 0, (hipStream_t)stream>>>((const nt::half_t *)a.data, (const nt::half_t *)b.data, elements, loops, sink);
    if (mfma_count) *mfma_count = (int64_t)units * 8 * loops * 32;
    return (int)hipGetLastError();
}
