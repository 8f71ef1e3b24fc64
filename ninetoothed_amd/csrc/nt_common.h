// Shared definitions for the gfx950 kernels of libnt_hip.so.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

#include "../../include/ninetoothed_hip.h"

namespace nt {

typedef _Float16 half_t;
typedef __bf16 bf16_t;

typedef _Float16 half8_t __attribute__((ext_vector_type(8)));
typedef _Float16 half4_t __attribute__((ext_vector_type(4)));
typedef _Float16 half2_t __attribute__((ext_vector_type(2)));
typedef __bf16 bf16x8_t __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x4_t __attribute__((ext_vector_type(4)));
typedef short short4_t __attribute__((ext_vector_type(4)));
typedef short short8_t __attribute__((ext_vector_type(8)));
typedef float float16_t __attribute__((ext_vector_type(16)));
typedef float float4_t __attribute__((ext_vector_type(4)));
typedef float float2_t __attribute__((ext_vector_type(2)));
typedef int int4_t __attribute__((ext_vector_type(4)));
typedef int int2_t __attribute__((ext_vector_type(2)));

#define NT_LDS __attribute__((address_space(3)))
#define NT_GLOBAL __attribute__((address_space(1)))

#define NT_DEVICE __device__ __forceinline__
#define NT_HOST_DEVICE __host__ __device__ __forceinline__

constexpr int kWaveSize = 64;

// Element traits: storage type, 8-wide vector and the 32x32x16 / 16x16x32 MFMA.
template <typename T>
struct Elem;

template <>
struct Elem<half_t> {
    typedef half8_t vec8;
    static constexpr int kDataType = NINETOOTHED_FLOAT16;
    static NT_DEVICE float16_t mfma32(vec8 a, vec8 b, float16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
    }
    static NT_DEVICE float4_t mfma16(vec8 a, vec8 b, float4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
    }
    static NT_DEVICE float to_float(half_t x) { return (float)x; }
    static NT_DEVICE half_t from_float(float x) { return (half_t)x; }
};

template <>
struct Elem<bf16_t> {
    typedef bf16x8_t vec8;
    static constexpr int kDataType = NINETOOTHED_BFLOAT16;
    static NT_DEVICE float16_t mfma32(vec8 a, vec8 b, float16_t c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
    }
    static NT_DEVICE float4_t mfma16(vec8 a, vec8 b, float4_t c) {
        return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
    }
    static NT_DEVICE float to_float(bf16_t x) { return (float)x; }
    static NT_DEVICE bf16_t from_float(float x) { return (bf16_t)x; }
};

// fp32 operands: the matrix pipe multiplies them as they are (32x32x2, one k value per lane and
// instruction); a lane's 8 k values go through 8 chained instructions.  No 16x16 form.
template <>
struct Elem<float> {
    typedef float vec8 __attribute__((ext_vector_type(8)));
    static constexpr int kDataType = NINETOOTHED_FLOAT32;
    static NT_DEVICE float16_t mfma32(vec8 a, vec8 b, float16_t c) {
#pragma unroll
        for (int i = 0; i < 8; ++i) c = __builtin_amdgcn_mfma_f32_32x32x2f32(a[i], b[i], c, 0, 0, 0);
        return c;
    }
    static NT_DEVICE float to_float(float x) { return x; }
    static NT_DEVICE float from_float(float x) { return x; }
};

template <typename T>
NT_DEVICE T from_float(float x) {
    return (T)x;
}

// 16-byte global -> LDS copy without passing through registers.  The LDS
// destination is wave-uniform `lds_base`; lane i lands at lds_base + 16 * i.
NT_DEVICE void global_to_lds_16(const void *global_ptr, NT_LDS void *lds_base) {
    __builtin_amdgcn_global_load_lds((const NT_GLOBAL void *)global_ptr, lds_base, 16, 0, 0);
}

// LDS transpose read: the 16 lanes of a group each address 4 consecutive
// 16-bit elements of one row; lane i of the group receives element (i % 16) of
// the 16-element row segment formed by the four lanes of each row, for the
// group's 4 rows.  With lane i addressing row i / 4, column 4 * (i % 4) of a
// [4 rows][16 columns] block, lane i gets column i of rows 0..3.
NT_DEVICE short4_t lds_read_tr16_b64(const NT_LDS void *p) {
    return __builtin_amdgcn_ds_read_tr16_b64_v4i16((NT_LDS short4_t *)p);
}

template <int N>
NT_DEVICE void wait_vmcnt() {
    static_assert(N >= 0 && N < 64, "vmcnt out of range");
    // gfx9 encoding: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt_hi[15:14]
    __builtin_amdgcn_s_waitcnt((N & 0xF) | (0x7 << 4) | (0xF << 8) | (((N >> 4) & 0x3) << 14));
}

template <int N>
NT_DEVICE void wait_lgkmcnt() {
    static_assert(N >= 0 && N < 16, "lgkmcnt out of range");
    __builtin_amdgcn_s_waitcnt(0xF | (0x7 << 4) | (N << 8) | (0x3 << 14));
}

NT_HOST_DEVICE constexpr int ceil_div(int a, int b) { return (a + b - 1) / b; }

// True while `stream` records into a graph (or when that cannot be told): the caller then
// must not synchronise, time, allocate, or load code, all of which break a capture.
inline bool stream_is_capturing(hipStream_t stream) {
    hipStreamCaptureStatus status = hipStreamCaptureStatusNone;
    if (hipStreamIsCapturing(stream, &status) != hipSuccess) {
        (void)hipGetLastError();
        return true;
    }
    return status != hipStreamCaptureStatusNone;
}

// Compute units of the current device (looked up once per device; 0 when it cannot be told).
inline int compute_units() {
    static int cached[64] = {};  // (written with the same value by whoever comes first: no lock needed)
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess || device < 0 || device >= 64) return 0;
    int units = __atomic_load_n(&cached[device], __ATOMIC_RELAXED);
    if (units == 0) {
        if (hipDeviceGetAttribute(&units, hipDeviceAttributeMultiprocessorCount, device) != hipSuccess || units <= 0) units = -1;
        __atomic_store_n(&cached[device], units, __ATOMIC_RELAXED);
    }
    return units > 0 ? units : 0;
}

struct Scalar0d {
    static double as_double(const NineToothedTensor &t) { return *(const double *)t.data; }
    static int64_t as_int64(const NineToothedTensor &t) { return *(const int64_t *)t.data; }
};

}  // namespace nt
