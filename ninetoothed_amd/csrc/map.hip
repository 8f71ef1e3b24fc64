// Interpreter kernel for element-wise / reducing tile programs (gfx950).
//
// The host lowers an arrangement's index maps and an application's dataflow
// graph into two stack programs (see the NineToothedMapProgram comment in the
// header); each lane walks output elements with a grid stride, evaluates the
// index code of every operand it touches and the value code of the expression,
// and stores one element.  Consecutive lanes take consecutive values of the last
// output variable, which the host orders so that it is the innermost source
// dimension: loads and stores of contiguous tensors coalesce.  The programs are
// HBM-bound byte work; the interpreter's integer arithmetic hides behind the
// memory latency as long as enough waves are resident (256 lanes per
// workgroup, 8 workgroups per CU).
//
// launch_nt_map first tries a kernel specialised for the program: the two stack
// programs are translated to straight-line HIP source (index constants, extents
// and element types as literals, call-time scalars and pointers as arguments),
// compiled once per distinct program with hipRTC and cached per device.  The
// interpreter kernel below runs when hipRTC is not available (libhiprtc.so is
// loaded on first use, not linked) or when NT_MAP_INTERPRET=1 is set; both
// execute the same operations in the same order.
#include <dlfcn.h>
#include <hip/hip_runtime.h>
#include <hip/hiprtc.h>

#include <cstdio>
#include <cstdlib>
#include <algorithm>
#include <cstring>
#include <map>
#include <mutex>
#include <sstream>
#include <string>
#include <unordered_map>
#include <vector>

#include "nt_common.h"
#include "tune.h"

namespace nt {
namespace {

constexpr int kMapThreads = 256;
constexpr int kIndexStack = 8;
constexpr int kValueStack = 16;

__device__ __forceinline__ int64_t floor_div(int64_t a, int64_t b) {
    int64_t q = a / b;
    if ((a % b != 0) && ((a < 0) != (b < 0))) --q;
    return q;
}

// runs one index segment: returns the offset, clears `valid` when a check fails
__device__ __forceinline__ int64_t run_index(const NineToothedMapProgram &p, int segment, const int64_t *vars, bool &valid) {
    int64_t stack[kIndexStack];
    int top = -1;
    for (int pc = p.segment_begin[segment];; ++pc) {
        const int word = p.index_code[pc];
        const int op = word & 0xff;
        const int arg = word >> 8;
        switch (op) {
            case NT_MAP_I_END: return top >= 0 ? stack[top] : 0;
            case NT_MAP_I_CONST: stack[++top] = p.index_constants[arg]; break;
            case NT_MAP_I_VAR: stack[++top] = vars[arg]; break;
            case NT_MAP_I_MULC: stack[top] *= p.index_constants[arg]; break;
            case NT_MAP_I_ADD: stack[top - 1] += stack[top]; --top; break;
            case NT_MAP_I_DIVC: stack[top] = floor_div(stack[top], p.index_constants[arg]); break;
            case NT_MAP_I_MODC: {
                const int64_t c = p.index_constants[arg];
                stack[top] -= floor_div(stack[top], c) * c;
                break;
            }
            case NT_MAP_I_CHECK: {
                const int64_t v = stack[top--];
                valid = valid && v >= 0 && v < p.index_constants[arg];
                break;
            }
            default: return 0;
        }
    }
}

__device__ __forceinline__ double load_element(const void *data, int dtype, int64_t offset) {
    switch (dtype) {
        case NINETOOTHED_INT8: return (double)((const int8_t *)data)[offset];
        case NINETOOTHED_INT16: return (double)((const int16_t *)data)[offset];
        case NINETOOTHED_INT32: return (double)((const int32_t *)data)[offset];
        case NINETOOTHED_INT64: return (double)((const int64_t *)data)[offset];
        case NINETOOTHED_UINT8: return (double)((const uint8_t *)data)[offset];
        case NINETOOTHED_UINT16: return (double)((const uint16_t *)data)[offset];
        case NINETOOTHED_UINT32: return (double)((const uint32_t *)data)[offset];
        case NINETOOTHED_UINT64: return (double)((const uint64_t *)data)[offset];
        case NINETOOTHED_FLOAT16: return (double)(float)((const half_t *)data)[offset];
        case NINETOOTHED_BFLOAT16: return (double)(float)((const bf16_t *)data)[offset];
        case NINETOOTHED_FLOAT32: return (double)((const float *)data)[offset];
        default: return ((const double *)data)[offset];
    }
}

__device__ __forceinline__ void store_element(void *data, int dtype, int64_t offset, double v) {
    switch (dtype) {
        case NINETOOTHED_INT8: ((int8_t *)data)[offset] = (int8_t)(int64_t)v; break;
        case NINETOOTHED_INT16: ((int16_t *)data)[offset] = (int16_t)(int64_t)v; break;
        case NINETOOTHED_INT32: ((int32_t *)data)[offset] = (int32_t)(int64_t)v; break;
        case NINETOOTHED_INT64: ((int64_t *)data)[offset] = (int64_t)v; break;
        case NINETOOTHED_UINT8: ((uint8_t *)data)[offset] = (uint8_t)(int64_t)v; break;
        case NINETOOTHED_UINT16: ((uint16_t *)data)[offset] = (uint16_t)(int64_t)v; break;
        case NINETOOTHED_UINT32: ((uint32_t *)data)[offset] = (uint32_t)(int64_t)v; break;
        case NINETOOTHED_UINT64: ((uint64_t *)data)[offset] = (uint64_t)v; break;
        case NINETOOTHED_FLOAT16: ((half_t *)data)[offset] = (half_t)(float)v; break;
        case NINETOOTHED_BFLOAT16: ((bf16_t *)data)[offset] = (bf16_t)(float)v; break;
        case NINETOOTHED_FLOAT32: ((float *)data)[offset] = (float)v; break;
        default: ((double *)data)[offset] = v; break;
    }
}

__device__ __forceinline__ void atomic_add_element(void *data, int dtype, int64_t offset, double v) {
    switch (dtype) {
        case NINETOOTHED_INT32: atomicAdd((int *)data + offset, (int)(int64_t)v); break;
        case NINETOOTHED_UINT32: atomicAdd((unsigned int *)data + offset, (unsigned int)(int64_t)v); break;
        case NINETOOTHED_INT64: atomicAdd((unsigned long long *)data + offset, (unsigned long long)(int64_t)v); break;
        case NINETOOTHED_UINT64: atomicAdd((unsigned long long *)data + offset, (unsigned long long)v); break;
        case NINETOOTHED_FLOAT32: atomicAdd((float *)data + offset, (float)v); break;
        case NINETOOTHED_FLOAT64: atomicAdd((double *)data + offset, v); break;
        default: break;
    }
}

// the value as the reference would hold it in a tile of type `dtype`
__device__ __forceinline__ double round_to(double v, int dtype) {
    switch (dtype) {
        case NINETOOTHED_FLOAT16: return (double)(float)(half_t)(float)v;
        case NINETOOTHED_BFLOAT16: return (double)(float)(bf16_t)(float)v;
        case NINETOOTHED_FLOAT32: return (double)(float)v;
        case NINETOOTHED_FLOAT64: return v;
        case NINETOOTHED_INT8: return (double)(int8_t)(int64_t)v;
        case NINETOOTHED_INT16: return (double)(int16_t)(int64_t)v;
        case NINETOOTHED_INT32: return (double)(int32_t)(int64_t)v;
        case NINETOOTHED_UINT8: return (double)(uint8_t)(int64_t)v;
        case NINETOOTHED_UINT16: return (double)(uint16_t)(int64_t)v;
        case NINETOOTHED_UINT32: return (double)(uint32_t)(int64_t)v;
        case NINETOOTHED_UINT64: return (double)(uint64_t)v;
        default: return (double)(int64_t)v;
    }
}

// Philox-4x32 with 10 rounds, counter (offset_lo, offset_hi, 0, 0), key = the two
// halves of the seed; the first output word becomes a float in [0, 1): negative
// values (as int32) are mirrored, then scaled by 2^-31.
__device__ __forceinline__ double philox_uniform(uint64_t seed, uint64_t offset) {
    uint32_t c0 = (uint32_t)offset, c1 = (uint32_t)(offset >> 32), c2 = 0, c3 = 0;
    uint32_t k0 = (uint32_t)seed, k1 = (uint32_t)(seed >> 32);
    for (int round = 0; round < 10; ++round) {
        const uint32_t a = 0xD2511F53u, b = 0xCD9E8D57u;
        const uint32_t p0 = c0, p2 = c2;
        c0 = __umulhi(b, p2) ^ c1 ^ k0;
        c2 = __umulhi(a, p0) ^ c3 ^ k1;
        c1 = b * p2;
        c3 = a * p0;
        k0 += 0x9E3779B9u;
        k1 += 0xBB67AE85u;
    }
    int32_t x = (int32_t)c0;
    if (x < 0) x = -x - 1;
    return (double)((float)x * 4.6566127342e-10f);
}

// runs value_code[begin, end) on a stack that starts as `initial` (when `seeded`)
__device__ __forceinline__ double run_value(const NineToothedMapProgram &p, int begin, int end, int64_t *vars, bool seeded,
                                             double initial, const double *reduced = nullptr) {
    double stack[kValueStack];
    int top = -1;
    if (seeded) stack[++top] = initial;
    for (int pc = begin; pc < end; ++pc) {
        const int word = p.value_code[pc];
        const int op = word & 0xff;
        const int arg = word >> 8;
        switch (op) {
            case NT_MAP_V_LOAD: {
                const NineToothedMapOperand &operand = p.operands[arg];
                bool valid = true;
                const int64_t offset = run_index(p, operand.segment, vars, valid);
                stack[++top] = valid ? load_element(operand.data, operand.dtype, offset) : operand.other;
                break;
            }
            case NT_MAP_V_CONST: stack[++top] = p.value_constants[arg]; break;
            case NT_MAP_V_OFFSET: {
                bool valid = true;
                stack[++top] = (double)run_index(p, arg, vars, valid);
                break;
            }
#define NT_BINARY(OP, EXPR)                          \
    case OP: {                                       \
        const double b = stack[top--];               \
        const double a = stack[top];                 \
        stack[top] = (EXPR);                         \
        break;                                       \
    }
            NT_BINARY(NT_MAP_V_ADD, a + b)
            NT_BINARY(NT_MAP_V_SUB, a - b)
            NT_BINARY(NT_MAP_V_MUL, a * b)
            NT_BINARY(NT_MAP_V_DIV, a / b)
            NT_BINARY(NT_MAP_V_FLOORDIV, floor(a / b))
            NT_BINARY(NT_MAP_V_MOD, a - floor(a / b) * b)
            NT_BINARY(NT_MAP_V_POW, (double)powf((float)a, (float)b))
            NT_BINARY(NT_MAP_V_MAX, (a != a || b != b) ? (a + b) : (a > b ? a : b))
            NT_BINARY(NT_MAP_V_MIN, (a != a || b != b) ? (a + b) : (a < b ? a : b))
            NT_BINARY(NT_MAP_V_LT, a < b ? 1.0 : 0.0)
            NT_BINARY(NT_MAP_V_LE, a <= b ? 1.0 : 0.0)
            NT_BINARY(NT_MAP_V_GT, a > b ? 1.0 : 0.0)
            NT_BINARY(NT_MAP_V_GE, a >= b ? 1.0 : 0.0)
            NT_BINARY(NT_MAP_V_EQ, a == b ? 1.0 : 0.0)
            NT_BINARY(NT_MAP_V_NE, a != b ? 1.0 : 0.0)
            NT_BINARY(NT_MAP_V_AND, (a != 0.0 && b != 0.0) ? 1.0 : 0.0)
            NT_BINARY(NT_MAP_V_OR, (a != 0.0 || b != 0.0) ? 1.0 : 0.0)
#undef NT_BINARY
#define NT_UNARY(OP, EXPR)            \
    case OP: {                        \
        const double a = stack[top];  \
        stack[top] = (EXPR);          \
        break;                        \
    }
            NT_UNARY(NT_MAP_V_NEG, -a)
            NT_UNARY(NT_MAP_V_NOT, a == 0.0 ? 1.0 : 0.0)
            NT_UNARY(NT_MAP_V_ABS, fabs(a))
            NT_UNARY(NT_MAP_V_EXP, (double)expf((float)a))
            NT_UNARY(NT_MAP_V_EXP2, (double)exp2f((float)a))
            NT_UNARY(NT_MAP_V_LOG, (double)logf((float)a))
            NT_UNARY(NT_MAP_V_LOG2, (double)log2f((float)a))
            NT_UNARY(NT_MAP_V_SQRT, sqrt(a))
            NT_UNARY(NT_MAP_V_RSQRT, (double)(1.0f / sqrtf((float)a)))
            NT_UNARY(NT_MAP_V_SIGMOID, (double)(1.0f / (1.0f + expf(-(float)a))))
            NT_UNARY(NT_MAP_V_TANH, (double)tanhf((float)a))
            NT_UNARY(NT_MAP_V_SIN, (double)sinf((float)a))
            NT_UNARY(NT_MAP_V_COS, (double)cosf((float)a))
            NT_UNARY(NT_MAP_V_FLOOR, floor(a))
            NT_UNARY(NT_MAP_V_CEIL, ceil(a))
#undef NT_UNARY
            case NT_MAP_V_WHERE: {
                const double b = stack[top--];
                const double a = stack[top--];
                stack[top] = stack[top] != 0.0 ? a : b;
                break;
            }
            case NT_MAP_V_ROUND: stack[top] = round_to(stack[top], arg); break;
            case NT_MAP_V_RAND: {
                const double offset = stack[top--];
                stack[top] = philox_uniform((uint64_t)(int64_t)stack[top], (uint64_t)(int64_t)offset);
                break;
            }
            case NT_MAP_V_SETVAR: vars[arg] = (int64_t)stack[top--]; break;
            case NT_MAP_V_REDUCED: stack[++top] = reduced[arg]; break;
            default: break;
        }
    }
    return top >= 0 ? stack[top] : 0.0;
}

__global__ __launch_bounds__(kMapThreads) void map_kernel(const NineToothedMapProgram p, int64_t total_out, int64_t total_reduced) {
    const int num_out = p.num_vars - p.num_reduced;
    const int64_t stride = (int64_t)gridDim.x * kMapThreads;
    for (int64_t element = (int64_t)blockIdx.x * kMapThreads + threadIdx.x; element < total_out; element += stride) {
        int64_t vars[NT_MAP_MAX_VARS];
        for (int v = p.num_vars; v < p.num_vars + p.num_dynamic; ++v) vars[v] = 0;
        int64_t rest = element;
        for (int v = num_out - 1; v >= 0; --v) {
            const int64_t extent = p.extents[v];
            vars[v] = rest % extent;
            rest /= extent;
        }
        double value;
        if (p.reduce_op == NT_MAP_REDUCE_NONE) {
            value = run_value(p, 0, p.value_code_length, vars, false, 0.0);
        } else {
            double acc = p.reduce_op == NT_MAP_REDUCE_SUM ? 0.0 : (p.reduce_op == NT_MAP_REDUCE_MAX ? -INFINITY : INFINITY);
            for (int64_t position = 0; position < total_reduced; ++position) {
                int64_t inner = position;
                for (int v = p.num_vars - 1; v >= num_out; --v) {
                    const int64_t extent = p.extents[v];
                    vars[v] = inner % extent;
                    inner /= extent;
                }
                const double term = run_value(p, 0, p.reduce_split, vars, false, 0.0);
                if (p.reduce_op == NT_MAP_REDUCE_SUM) {
                    acc = round_to(acc + term, p.reduce_dtype);
                } else if (term != term || acc != acc) {
                    acc = acc + term;  // NaN propagates
                } else if (p.reduce_op == NT_MAP_REDUCE_MAX) {
                    acc = term > acc ? term : acc;
                } else {
                    acc = term < acc ? term : acc;
                }
            }
            value = run_value(p, p.reduce_split, p.value_code_length, vars, true, acc);
        }
        const NineToothedMapOperand &out = p.operands[p.output];
        bool valid = true;
        const int64_t offset = run_index(p, out.segment, vars, valid);
        if (valid) {
            if (p.store_op == NT_MAP_STORE_ATOMIC_ADD) atomic_add_element(out.data, out.dtype, offset, value);
            else store_element(out.data, out.dtype, offset, value);
        }
    }
}

// acc (op) term with the rounding / NaN rules of the element kernel's reductions
__device__ __forceinline__ double reduce_combine(int op, int dtype, double acc, double term) {
    if (op == NT_MAP_REDUCE_SUM) return round_to(acc + term, dtype);
    if (term != term || acc != acc) return acc + term;  // NaN propagates
    if (op == NT_MAP_REDUCE_MAX) return term > acc ? term : acc;
    return term < acc ? term : acc;
}

__device__ __forceinline__ double reduce_identity(int op) {
    return op == NT_MAP_REDUCE_SUM ? 0.0 : (op == NT_MAP_REDUCE_MAX ? -INFINITY : INFINITY);
}

// all threads of the workgroup get the combination of everybody's `value`
__device__ __forceinline__ double block_reduce(int op, int dtype, double value, double *scratch) {
    for (int offset = 32; offset > 0; offset >>= 1) value = reduce_combine(op, dtype, value, __shfl_xor(value, offset, 64));
    constexpr int kWaves = kMapThreads / 64;
    __syncthreads();  // scratch may still be read from the previous phase
    if ((threadIdx.x & 63) == 0) scratch[threadIdx.x >> 6] = value;
    __syncthreads();
    value = scratch[0];
    for (int w = 1; w < kWaves; ++w) value = reduce_combine(op, dtype, value, scratch[w]);
    return value;
}

// Tile mode: one workgroup per tile; phases of whole-tile reductions, then the stored expression.
__global__ __launch_bounds__(kMapThreads) void map_tile_kernel(const NineToothedMapProgram p, int64_t tiles, int64_t tile_elements) {
    __shared__ double scratch[kMapThreads / 64];
    for (int64_t tile = blockIdx.x; tile < tiles; tile += gridDim.x) {
        int64_t vars[NT_MAP_MAX_VARS];
        int64_t rest = tile;
        for (int v = p.num_grid - 1; v >= 0; --v) {
            const int64_t extent = p.extents[v];
            vars[v] = rest % extent;
            rest /= extent;
        }
        auto decode = [&](int64_t element) {
            for (int v = p.num_vars - 1; v >= p.num_grid; --v) {
                const int64_t extent = p.extents[v];
                vars[v] = element % extent;
                element /= extent;
            }
        };
        double reduced[NT_MAP_MAX_PHASES];
        int begin = 0;
        for (int k = 0; k < p.num_phases; ++k) {
            double acc = reduce_identity(p.phase_op[k]);
            for (int64_t element = threadIdx.x; element < tile_elements; element += kMapThreads) {
                decode(element);
                acc = reduce_combine(p.phase_op[k], p.phase_dtype[k], acc, run_value(p, begin, p.phase_end[k], vars, false, 0.0, reduced));
            }
            reduced[k] = block_reduce(p.phase_op[k], p.phase_dtype[k], acc, scratch);
            begin = p.phase_end[k];
        }
        const NineToothedMapOperand &out = p.operands[p.output];
        for (int64_t element = threadIdx.x; element < tile_elements; element += kMapThreads) {
            decode(element);
            const double value = run_value(p, begin, p.value_code_length, vars, false, 0.0, reduced);
            bool valid = true;
            const int64_t offset = run_index(p, out.segment, vars, valid);
            if (valid) store_element(out.data, out.dtype, offset, value);
        }
    }
}

bool well_formed(const NineToothedMapProgram &p) {
    if (p.num_vars < 0 || p.num_vars > NT_MAP_MAX_VARS || p.num_reduced < 0 || p.num_reduced > p.num_vars) return false;
    if (p.num_dynamic < 0 || p.num_vars + p.num_dynamic > NT_MAP_MAX_VARS) return false;
    if (p.num_operands < 1 || p.num_operands > NT_MAP_MAX_OPERANDS || p.output < 0 || p.output >= p.num_operands) return false;
    if (p.store_op != NT_MAP_STORE_ASSIGN && p.store_op != NT_MAP_STORE_ATOMIC_ADD) return false;
    if (p.store_op == NT_MAP_STORE_ATOMIC_ADD) {
        const int dtype = p.operands[p.output].dtype;
        if (dtype != NINETOOTHED_INT32 && dtype != NINETOOTHED_UINT32 && dtype != NINETOOTHED_INT64 && dtype != NINETOOTHED_UINT64 &&
            dtype != NINETOOTHED_FLOAT32 && dtype != NINETOOTHED_FLOAT64)
            return false;
    }
    if (p.num_segments < 1 || p.num_segments > NT_MAP_MAX_SEGMENTS) return false;
    if (p.value_code_length < 0 || p.value_code_length > NT_MAP_MAX_VALUE_CODE) return false;
    if (p.reduce_split < 0 || p.reduce_split > p.value_code_length) return false;
    if (p.reduce_op < NT_MAP_REDUCE_NONE || p.reduce_op > NT_MAP_REDUCE_SUM) return false;
    if ((p.reduce_op == NT_MAP_REDUCE_NONE) != (p.num_reduced == 0 && p.reduce_split == p.value_code_length)) return false;
    for (int i = 0; i < p.num_operands; ++i) {
        const NineToothedMapOperand &operand = p.operands[i];
        if (operand.dtype < NINETOOTHED_INT8 || operand.dtype > NINETOOTHED_FLOAT64) return false;
        if (operand.segment < 0 || operand.segment >= p.num_segments) return false;
    }
    // every segment must end inside the code array, use known opcodes, in-range
    // arguments, and keep the stack within its bounds
    for (int s = 0; s < p.num_segments; ++s) {
        int pc = p.segment_begin[s];
        if (pc < 0) return false;
        int depth = 0;
        for (;; ++pc) {
            if (pc >= NT_MAP_MAX_INDEX_CODE) return false;
            const int op = p.index_code[pc] & 0xff, arg = p.index_code[pc] >> 8;
            if (op == NT_MAP_I_END) break;
            if (op == NT_MAP_I_VAR) {
                if (arg < 0 || arg >= p.num_vars + p.num_dynamic) return false;
                ++depth;
            } else if (op == NT_MAP_I_ADD) {
                if (depth < 2) return false;
                --depth;
            } else if (op == NT_MAP_I_CONST || op == NT_MAP_I_MULC || op == NT_MAP_I_DIVC || op == NT_MAP_I_MODC || op == NT_MAP_I_CHECK) {
                if (arg < 0 || arg >= NT_MAP_MAX_INDEX_CONSTANTS) return false;
                if ((op == NT_MAP_I_DIVC || op == NT_MAP_I_MODC) && p.index_constants[arg] == 0) return false;
                if (op == NT_MAP_I_CONST) ++depth;
                else if (depth < 1) return false;
                if (op == NT_MAP_I_CHECK) --depth;
            } else {
                return false;
            }
            if (depth > kIndexStack) return false;
        }
    }
    if (p.num_phases < 0 || p.num_phases > NT_MAP_MAX_PHASES) return false;
    if (p.num_phases > 0) {
        if (p.reduce_op != NT_MAP_REDUCE_NONE || p.num_dynamic != 0 || p.store_op != NT_MAP_STORE_ASSIGN) return false;
        if (p.num_grid < 0 || p.num_grid > p.num_vars) return false;
        int previous = 0;
        for (int k = 0; k < p.num_phases; ++k) {
            if (p.phase_end[k] <= previous || p.phase_end[k] >= p.value_code_length) return false;
            if (p.phase_op[k] < NT_MAP_REDUCE_MAX || p.phase_op[k] > NT_MAP_REDUCE_SUM) return false;
            if (p.phase_dtype[k] < NINETOOTHED_INT8 || p.phase_dtype[k] > NINETOOTHED_FLOAT64) return false;
            previous = p.phase_end[k];
        }
    }
    int depth = 0;
    int phase = 0;  // the phase the code at `pc` belongs to (num_phases: the stored expression)
    for (int pc = 0; pc < p.value_code_length; ++pc) {
        if (phase < p.num_phases && pc == p.phase_end[phase]) {
            if (depth != 1) return false;  // a phase leaves exactly its term
            depth = 0;
            ++phase;
        }
        if (pc == p.reduce_split && p.reduce_op != NT_MAP_REDUCE_NONE) {
            if (depth != 1) return false;  // the per-position code leaves exactly the term
        }
        const int op = p.value_code[pc] & 0xff, arg = p.value_code[pc] >> 8;
        if (op == NT_MAP_V_LOAD) {
            if (arg < 0 || arg >= p.num_operands) return false;
            ++depth;
        } else if (op == NT_MAP_V_CONST) {
            if (arg < 0 || arg >= NT_MAP_MAX_VALUE_CONSTANTS) return false;
            ++depth;
        } else if (op == NT_MAP_V_OFFSET) {
            if (arg < 0 || arg >= p.num_segments) return false;
            ++depth;
        } else if (op >= NT_MAP_V_ADD && op <= NT_MAP_V_OR) {
            if (depth < 2) return false;
            --depth;
        } else if (op >= NT_MAP_V_NEG && op <= NT_MAP_V_CEIL) {
            if (depth < 1) return false;
        } else if (op == NT_MAP_V_WHERE) {
            if (depth < 3) return false;
            depth -= 2;
        } else if (op == NT_MAP_V_ROUND) {
            if (depth < 1 || arg < NINETOOTHED_INT8 || arg > NINETOOTHED_FLOAT64) return false;
        } else if (op == NT_MAP_V_RAND) {
            if (depth < 2) return false;
            --depth;
        } else if (op == NT_MAP_V_SETVAR) {
            if (depth < 1 || arg < p.num_vars || arg >= p.num_vars + p.num_dynamic) return false;
            --depth;
        } else if (op == NT_MAP_V_REDUCED) {
            if (arg < 0 || arg >= phase) return false;
            ++depth;
        } else {
            return false;
        }
        if (depth > kValueStack) return false;
    }
    if (p.reduce_op != NT_MAP_REDUCE_NONE && p.reduce_split == p.value_code_length && depth != 1) return false;
    return depth == 1;
}


// ---- specialised kernels through hipRTC ----------------------------------------------

struct MapJitArgs {
    void *data[NT_MAP_MAX_OPERANDS];
    double other[NT_MAP_MAX_OPERANDS];
    double constants[NT_MAP_MAX_VALUE_CONSTANTS];
    long long total_out;
};

const char *c_type(int dtype) {
    switch (dtype) {
        case NINETOOTHED_INT8: return "signed char";
        case NINETOOTHED_INT16: return "short";
        case NINETOOTHED_INT32: return "int";
        case NINETOOTHED_INT64: return "long long";
        case NINETOOTHED_UINT8: return "unsigned char";
        case NINETOOTHED_UINT16: return "unsigned short";
        case NINETOOTHED_UINT32: return "unsigned int";
        case NINETOOTHED_UINT64: return "unsigned long long";
        case NINETOOTHED_FLOAT16: return "_Float16";
        case NINETOOTHED_BFLOAT16: return "__bf16";
        case NINETOOTHED_FLOAT32: return "float";
        default: return "double";
    }
}

std::string round_expr(const std::string &v, int dtype) {
    switch (dtype) {
        case NINETOOTHED_FLOAT16: return "(double)(float)(_Float16)(float)(" + v + ")";
        case NINETOOTHED_BFLOAT16: return "(double)(float)(__bf16)(float)(" + v + ")";
        case NINETOOTHED_FLOAT32: return "(double)(float)(" + v + ")";
        case NINETOOTHED_FLOAT64: return v;
        case NINETOOTHED_UINT64: return "(double)(unsigned long long)(" + v + ")";
        case NINETOOTHED_INT64: return "(double)(long long)(" + v + ")";
        default: return std::string("(double)(") + c_type(dtype) + ")(long long)(" + v + ")";
    }
}

std::string load_expr(const std::string &pointer, int dtype, const std::string &offset) {
    const std::string element = std::string("((const ") + c_type(dtype) + " *)" + pointer + ")[" + offset + "]";
    if (dtype == NINETOOTHED_FLOAT16 || dtype == NINETOOTHED_BFLOAT16) return "(double)(float)" + element;
    return "(double)" + element;
}

// Stores are non-temporal: the output of a streaming kernel is not read again by it, and the hint lets
// the stores of a wave leave as whole lines (2^26-element add: fp32 5.65 -> 5.85 TB/s, fp16 3.98 -> 6.66;
// row normalisations 5-18 % faster).  Loads stay plain: non-temporal loads cost 7-20 % in the softmax kernel.
std::string store_stmt(const std::string &pointer, int dtype, const std::string &offset, const std::string &v) {
    const std::string target = std::string("((") + c_type(dtype) + " *)" + pointer + ")[" + offset + "]";
    std::string value;
    switch (dtype) {
        case NINETOOTHED_FLOAT16:
        case NINETOOTHED_BFLOAT16: value = std::string("(") + c_type(dtype) + ")(float)(" + v + ")"; break;
        case NINETOOTHED_FLOAT32:
        case NINETOOTHED_FLOAT64:
        case NINETOOTHED_INT64:
        case NINETOOTHED_UINT64: value = std::string("(") + c_type(dtype) + ")(" + v + ")"; break;
        default: value = std::string("(") + c_type(dtype) + ")(long long)(" + v + ")"; break;
    }
    return "__builtin_nontemporal_store(" + value + ", &" + target + ");";
}

std::string atomic_add_stmt(const std::string &pointer, int dtype, const std::string &offset, const std::string &v) {
    const char *type = dtype == NINETOOTHED_INT32 ? "int" : dtype == NINETOOTHED_UINT32 ? "unsigned int" : dtype == NINETOOTHED_FLOAT32 ? "float"
                       : dtype == NINETOOTHED_FLOAT64 ? "double" : "unsigned long long";
    const bool integer = dtype != NINETOOTHED_FLOAT32 && dtype != NINETOOTHED_FLOAT64 && dtype != NINETOOTHED_UINT64;
    return std::string("atomicAdd((") + type + " *)" + pointer + " + " + offset + ", (" + type + ")" + (integer ? "(long long)" : "") + "(" + v + "));";
}

// Translates the programs into HIP source.  `counter` numbers temporaries.
// value of an index segment at one point of the variables (checks ignored)
long long segment_offset_at(const NineToothedMapProgram &q, int segment, const long long *vars) {
    std::vector<long long> stack;
    for (int pc = q.segment_begin[segment];; ++pc) {
        const int op = q.index_code[pc] & 0xff, arg = q.index_code[pc] >> 8;
        if (op == NT_MAP_I_END) break;
        switch (op) {
            case NT_MAP_I_CONST: stack.push_back((long long)q.index_constants[arg]); break;
            case NT_MAP_I_VAR: stack.push_back(vars[arg]); break;
            case NT_MAP_I_MULC: stack.back() *= (long long)q.index_constants[arg]; break;
            case NT_MAP_I_ADD: {
                const long long b = stack.back();
                stack.pop_back();
                stack.back() += b;
                break;
            }
            case NT_MAP_I_DIVC:
            case NT_MAP_I_MODC: {
                const long long c = (long long)q.index_constants[arg], a = stack.back();
                if (c == 0) return 0;
                long long quotient = a / c;
                if ((a % c != 0) && ((a < 0) != (c < 0))) --quotient;
                stack.back() = op == NT_MAP_I_DIVC ? quotient : a - quotient * c;
                break;
            }
            case NT_MAP_I_CHECK: stack.pop_back(); break;
            default: return 0;
        }
    }
    return stack.empty() ? 0 : stack.back();
}

// Reductions whose reduced positions lie closer together in memory than the outputs do (row sums of a
// row-major matrix) run with one wave per output element: the lanes stride the reduced positions, so
// a wave reads consecutive elements, and combine their partial results with shuffles.  With one thread
// per output the lanes of a wave would read a row each.  Returns the lanes per output element: 1, 64, or -- few outputs over long ranges -- the whole workgroup.
int cooperative_lanes(const NineToothedMapProgram &q);

// Threads of a workgroup.  In tile mode (one workgroup per tile) a tile of up to 16384 elements gets enough
// threads that each holds at most 16 elements, preferably 8, which the generated code then keeps in registers
// (layer norm over 4096 rows of fp32, 256 threads -> this choice: 4096 wide 38 -> 27 us, 8192 wide 83 -> 54,
// 16384 wide 168 -> 119; 1024 threads on 8192 columns: the same for the norms, softmax 64 us against 46).
int workgroup_threads(const NineToothedMapProgram &q) {
    if (q.num_phases == 0) return kMapThreads;
    long long tile_elements = 1;
    for (int v = q.num_grid; v < q.num_vars; ++v) tile_elements *= (long long)q.extents[v];
    if (tile_elements > 2048 && tile_elements <= 8192) return 512;
    if (tile_elements > 8192 && tile_elements <= 16384) return 1024;
    return kMapThreads;
}

// Threads that share a tile in tile mode: a wave for tiles of up to 512 elements (a workgroup then holds four
// tiles and the reductions need no LDS exchange and no barrier), else the whole workgroup.
int tile_group(const NineToothedMapProgram &q) {
    long long tile_elements = 1;
    for (int v = q.num_grid; v < q.num_vars; ++v) tile_elements *= (long long)q.extents[v];
    return q.num_phases > 0 && tile_elements <= 512 ? 64 : workgroup_threads(q);
}

int cooperative_lanes(const NineToothedMapProgram &q) {
    const int num_out = q.num_vars - q.num_reduced;
    if (q.num_phases != 0 || q.reduce_op == NT_MAP_REDUCE_NONE || q.num_dynamic != 0 || q.num_reduced == 0 || q.store_op != NT_MAP_STORE_ASSIGN) return 1;
    long long reduced = 1;
    for (int v = num_out; v < q.num_vars; ++v) reduced *= q.extents[v];
    if (reduced < 128) return 1;
    int operand = -1;  // the first tensor the reduced term loads
    for (int pc = 0; pc < q.reduce_split && operand < 0; ++pc)
        if ((q.value_code[pc] & 0xff) == NT_MAP_V_LOAD) operand = q.value_code[pc] >> 8;
    if (operand < 0 || operand >= q.num_operands) return 1;
    const int segment = q.operands[operand].segment;
    long long vars[NT_MAP_MAX_VARS] = {0};
    const long long base = segment_offset_at(q, segment, vars);
    const int inner_reduced = q.num_vars - 1;
    if (q.extents[inner_reduced] < 2) return 1;
    vars[inner_reduced] = 1;
    const long long step_reduced = std::llabs(segment_offset_at(q, segment, vars) - base);
    vars[inner_reduced] = 0;
    long long step_out = 0;
    for (int v = num_out - 1; v >= 0 && step_out == 0; --v) {  // the fastest output variable that moves this tensor
        if (q.extents[v] < 2) continue;
        vars[v] = 1;
        step_out = std::llabs(segment_offset_at(q, segment, vars) - base);
        vars[v] = 0;
    }
    if (!(step_reduced != 0 && (step_out == 0 || step_reduced < step_out))) return 1;
    // few outputs over long ranges (64 rows of a million elements): a wave per output would leave most of the chip
    // idle, so the whole workgroup shares an output and its waves exchange their partial results through LDS
    long long outputs = 1;
    for (int v = 0; v < num_out; ++v) outputs *= q.extents[v];
    return outputs <= 2048 && reduced >= 16384 ? kMapThreads : 64;
}

struct MapCodegen {
    const NineToothedMapProgram &p;
    std::ostringstream out;
    int counter = 0;
    std::string indent = "        ";

    bool narrow;  // index arithmetic in 32 bits: every index value provably fits
    int lanes;    // lanes per output element (cooperative_lanes)
    int threads;  // of a workgroup (workgroup_threads)
    int group;    // threads that share a tile in tile mode (tile_group)
    // Tile mode with small tiles: a thread's elements stay in registers between the phases.
    // `kept` lists the operands whose loaded values an earlier phase left in `ld<slot>[e]`,
    // `in_body` maps operands already loaded in the loop body being emitted to their temporaries.
    bool keep_loads = false;
    int tile_width = 0;  // tile mode over 16-bit tensors: elements per group of consecutive ones that a thread handles (0: one by one)
    // a masked element takes the operand's `other`, which the host rounds to the element type: a float holds both
    bool kept_as_float(int slot) const {
        const int dtype = p.operands[slot].dtype;
        return dtype == NINETOOTHED_FLOAT16 || dtype == NINETOOTHED_BFLOAT16 || dtype == NINETOOTHED_FLOAT32;
    }
    std::vector<bool> kept = std::vector<bool>(NT_MAP_MAX_OPERANDS, false);
    std::map<int, std::string> in_body;

    explicit MapCodegen(const NineToothedMapProgram &program) : p(program), narrow(fits_int32(program)), lanes(cooperative_lanes(program)), threads(workgroup_threads(program)), group(tile_group(program)) {}

    std::string fresh(const char *prefix) { return prefix + std::to_string(counter++); }

    const char *idx() const { return narrow ? "int" : "long long"; }
    std::string lit(long long value) const { return std::to_string(value) + (narrow ? "" : "LL"); }
    std::string ulit(long long value) const { return std::to_string(value) + (narrow ? "u" : "ULL"); }

    // Interval evaluation of the index programs over the variables' ranges: true when the element
    // count, every constant and every intermediate value stay within 31 bits (then `int` arithmetic
    // computes the same offsets with a fraction of the instructions of 64-bit arithmetic).
    static bool fits_int32(const NineToothedMapProgram &q) {
        typedef __int128 wide;
        const wide limit = (wide)1 << 31;
        if (q.num_dynamic != 0) return false;
        wide total = 1;
        for (int v = 0; v < q.num_vars; ++v) {
            if (q.extents[v] < 0 || (wide)q.extents[v] >= limit) return false;
            if (v < q.num_vars - q.num_reduced) total *= q.extents[v] > 0 ? q.extents[v] : 1;
            if (total >= ((wide)1 << 30)) return false;  // leaves room for the loop increment
        }
        for (int segment = 0; segment < q.num_segments; ++segment) {
            std::vector<std::pair<wide, wide>> stack;
            for (int pc = q.segment_begin[segment];; ++pc) {
                const int op = q.index_code[pc] & 0xff, arg = q.index_code[pc] >> 8;
                if (op == NT_MAP_I_END) break;
                const wide c = op == NT_MAP_I_VAR ? 0 : (wide)q.index_constants[arg];
                if (op != NT_MAP_I_VAR && op != NT_MAP_I_ADD && (c >= limit || c < -limit)) return false;
                switch (op) {
                    case NT_MAP_I_CONST: stack.push_back({c, c}); break;
                    case NT_MAP_I_VAR: stack.push_back({0, q.extents[arg] > 0 ? (wide)q.extents[arg] - 1 : 0}); break;
                    case NT_MAP_I_MULC: {
                        const wide a = stack.back().first * c, b = stack.back().second * c;
                        stack.back() = {a < b ? a : b, a < b ? b : a};
                        break;
                    }
                    case NT_MAP_I_ADD: {
                        const std::pair<wide, wide> b = stack.back();
                        stack.pop_back();
                        stack.back().first += b.first;
                        stack.back().second += b.second;
                        break;
                    }
                    case NT_MAP_I_DIVC:
                    case NT_MAP_I_MODC: {  // never larger in magnitude than the operand (and the divisor)
                        wide bound = stack.back().first < 0 ? -stack.back().first : stack.back().first;
                        const wide other = stack.back().second < 0 ? -stack.back().second : stack.back().second;
                        if (other > bound) bound = other;
                        stack.back() = {-bound - 1, bound + 1};
                        break;
                    }
                    case NT_MAP_I_CHECK: stack.pop_back(); break;
                    default: return false;
                }
                if (!stack.empty() && (stack.back().first < -limit || stack.back().second >= limit)) return false;
            }
        }
        return true;
    }

    // emits the statements of one index segment; returns the offset expression and
    // and-s the checks into `valid` (a declared bool variable) when it is not empty
    std::string index_segment(int segment, const std::string &valid) {
        std::vector<std::string> stack;
        for (int pc = p.segment_begin[segment];; ++pc) {
            const int op = p.index_code[pc] & 0xff, arg = p.index_code[pc] >> 8;
            if (op == NT_MAP_I_END) break;
            switch (op) {
                case NT_MAP_I_CONST: stack.push_back(lit((long long)p.index_constants[arg])); break;
                case NT_MAP_I_VAR: stack.push_back("v" + std::to_string(arg)); break;
                case NT_MAP_I_MULC: stack.back() = "(" + stack.back() + " * " + lit((long long)p.index_constants[arg]) + ")"; break;
                case NT_MAP_I_ADD: {
                    const std::string b = stack.back();
                    stack.pop_back();
                    stack.back() = "(" + stack.back() + " + " + b + ")";
                    break;
                }
                case NT_MAP_I_DIVC:
                case NT_MAP_I_MODC: {
                    const std::string name = fresh("i");
                    const std::string c = lit((long long)p.index_constants[arg]);
                    out << indent << "const " << idx() << " " << name << " = " << (op == NT_MAP_I_DIVC ? "nt_floor_div(" : "nt_floor_mod(") << stack.back() << ", " << c << ");\n";
                    stack.back() = name;
                    break;
                }
                case NT_MAP_I_CHECK: {
                    const std::string name = fresh("i");
                    out << indent << "const " << idx() << " " << name << " = " << stack.back() << ";\n";
                    out << indent << valid << " = " << valid << " && " << name << " >= 0 && " << name << " < " << lit((long long)p.index_constants[arg]) << ";\n";
                    stack.pop_back();
                    break;
                }
            }
        }
        const std::string name = fresh("i");
        out << indent << "const " << idx() << " " << name << " = " << (stack.empty() ? lit(0) : stack.back()) << ";\n";
        return name;
    }

    // emits value_code[begin, end); `seed` (if not empty) is the initial stack entry
    std::string value_range(int begin, int end, const std::string &seed) {
        std::vector<std::string> stack;
        if (!seed.empty()) stack.push_back(seed);
        auto define = [&](const std::string &expr) {
            const std::string name = fresh("t");
            out << indent << "const double " << name << " = " << expr << ";\n";
            return name;
        };
        std::map<std::string, std::string> integer_of;  // temporaries that are an index converted to fp64
        for (int pc = begin; pc < end; ++pc) {
            const int op = p.value_code[pc] & 0xff, arg = p.value_code[pc] >> 8;
            if (op == NT_MAP_V_LOAD && keep_loads && kept[arg]) {
                stack.push_back(kept_as_float(arg) ? "(double)ld" + std::to_string(arg) + "[e]" : "ld" + std::to_string(arg) + "[e]");
            } else if (op == NT_MAP_V_LOAD && keep_loads && in_body.count(arg)) {
                stack.push_back(in_body[arg]);
            } else if (op == NT_MAP_V_LOAD) {
                const NineToothedMapOperand &operand = p.operands[arg];
                const std::string valid = fresh("ok");
                out << indent << "bool " << valid << " = true;\n";
                const std::string offset = index_segment(operand.segment, valid);
                const std::string pointer = "a.data[" + std::to_string(arg) + "]";
                stack.push_back(define(valid + " ? " + load_expr(pointer, operand.dtype, offset) + " : a.other[" + std::to_string(arg) + "]"));
                if (keep_loads) {
                    out << indent << "ld" << arg << "[e] = " << (kept_as_float(arg) ? "(float)" : "") << stack.back() << ";\n";
                    in_body[arg] = stack.back();
                }
            } else if (op == NT_MAP_V_CONST) {
                stack.push_back("a.constants[" + std::to_string(arg) + "]");
            } else if (op == NT_MAP_V_OFFSET) {
                const std::string valid = fresh("ok");
                out << indent << "bool " << valid << " = true;\n";
                const std::string index = index_segment(arg, valid);
                stack.push_back(define("(double)" + index));
                integer_of[stack.back()] = index;
            } else if (op >= NT_MAP_V_ADD && op <= NT_MAP_V_OR) {
                const std::string b = stack.back();
                stack.pop_back();
                const std::string a = stack.back();
                std::string e;
                switch (op) {
                    case NT_MAP_V_ADD: e = a + " + " + b; break;
                    case NT_MAP_V_SUB: e = a + " - " + b; break;
                    case NT_MAP_V_MUL: e = a + " * " + b; break;
                    case NT_MAP_V_DIV: e = a + " / " + b; break;
                    case NT_MAP_V_FLOORDIV: e = "floor(" + a + " / " + b + ")"; break;
                    case NT_MAP_V_MOD: e = a + " - floor(" + a + " / " + b + ") * " + b; break;
                    case NT_MAP_V_POW: e = "(double)powf((float)" + a + ", (float)" + b + ")"; break;
                    case NT_MAP_V_MAX: e = "(" + a + " != " + a + " || " + b + " != " + b + ") ? (" + a + " + " + b + ") : (" + a + " > " + b + " ? " + a + " : " + b + ")"; break;
                    case NT_MAP_V_MIN: e = "(" + a + " != " + a + " || " + b + " != " + b + ") ? (" + a + " + " + b + ") : (" + a + " < " + b + " ? " + a + " : " + b + ")"; break;
                    case NT_MAP_V_LT: e = a + " < " + b + " ? 1.0 : 0.0"; break;
                    case NT_MAP_V_LE: e = a + " <= " + b + " ? 1.0 : 0.0"; break;
                    case NT_MAP_V_GT: e = a + " > " + b + " ? 1.0 : 0.0"; break;
                    case NT_MAP_V_GE: e = a + " >= " + b + " ? 1.0 : 0.0"; break;
                    case NT_MAP_V_EQ: e = a + " == " + b + " ? 1.0 : 0.0"; break;
                    case NT_MAP_V_NE: e = a + " != " + b + " ? 1.0 : 0.0"; break;
                    case NT_MAP_V_AND: e = "(" + a + " != 0.0 && " + b + " != 0.0) ? 1.0 : 0.0"; break;
                    default: e = "(" + a + " != 0.0 || " + b + " != 0.0) ? 1.0 : 0.0"; break;
                }
                stack.back() = define(e);
            } else if (op >= NT_MAP_V_NEG && op <= NT_MAP_V_CEIL) {
                const std::string a = stack.back();
                std::string e;
                switch (op) {
                    case NT_MAP_V_NEG: e = "-" + a; break;
                    case NT_MAP_V_NOT: e = a + " == 0.0 ? 1.0 : 0.0"; break;
                    case NT_MAP_V_ABS: e = "fabs(" + a + ")"; break;
                    // exponentials and the sigmoid through the hardware's 2^x, as Triton's `tl.exp` / `tl.sigmoid` do
                    case NT_MAP_V_EXP: e = "(double)__expf((float)" + a + ")"; break;
                    case NT_MAP_V_EXP2: e = "(double)exp2f((float)" + a + ")"; break;
                    case NT_MAP_V_LOG: e = "(double)logf((float)" + a + ")"; break;
                    case NT_MAP_V_LOG2: e = "(double)log2f((float)" + a + ")"; break;
                    case NT_MAP_V_SQRT: e = "sqrt(" + a + ")"; break;
                    case NT_MAP_V_RSQRT: e = "(double)(1.0f / sqrtf((float)" + a + "))"; break;
                    case NT_MAP_V_SIGMOID: e = "(double)__fdividef(1.0f, 1.0f + __expf(-(float)" + a + "))"; break;
                    case NT_MAP_V_TANH: e = "(double)tanhf((float)" + a + ")"; break;
                    case NT_MAP_V_SIN: e = "(double)sinf((float)" + a + ")"; break;
                    case NT_MAP_V_COS: e = "(double)cosf((float)" + a + ")"; break;
                    case NT_MAP_V_FLOOR: e = "floor(" + a + ")"; break;
                    default: e = "ceil(" + a + ")"; break;
                }
                stack.back() = define(e);
            } else if (op == NT_MAP_V_WHERE) {
                const std::string b = stack.back();
                stack.pop_back();
                const std::string a = stack.back();
                stack.pop_back();
                stack.back() = define(stack.back() + " != 0.0 ? " + a + " : " + b);
            } else if (op == NT_MAP_V_ROUND) {
                stack.back() = define(round_expr(stack.back(), arg));
            } else if (op == NT_MAP_V_RAND) {
                const std::string offset = stack.back();
                stack.pop_back();
                // (an offset that is an index as it stands skips the detour through fp64)
                const std::string counter = integer_of.count(offset) ? integer_of[offset] : offset;
                stack.back() = define("nt_philox_uniform((unsigned long long)(long long)" + stack.back() + ", (unsigned long long)(long long)" + counter + ")");
            } else if (op == NT_MAP_V_SETVAR) {
                out << indent << "v" << arg << " = (nt_idx)(" << stack.back() << ");\n";
                stack.pop_back();
            } else if (op == NT_MAP_V_REDUCED) {
                stack.push_back("r" + std::to_string(arg));
            }
        }
        return stack.empty() ? std::string("0.0") : stack.back();
    }

    std::string combine_expr(int op, int dtype, const std::string &acc, const std::string &term) {
        if (op == NT_MAP_REDUCE_SUM) return round_expr(acc + " + " + term, dtype);
        const char *cmp = op == NT_MAP_REDUCE_MAX ? ">" : "<";
        return "(" + term + " != " + term + " || " + acc + " != " + acc + ") ? " + acc + " + " + term + " : (" + term + " " + cmp + " " + acc + " ? " + term + " : " + acc + ")";
    }

    void decode_tile_variables() {
        out << indent << "nt_uidx rest = (nt_uidx)element;\n";
        for (int v = p.num_vars - 1; v >= p.num_grid; --v)
            out << indent << "const nt_idx v" << v << " = (nt_idx)(rest % " << ulit((long long)p.extents[v]) << "); rest /= " << ulit((long long)p.extents[v]) << ";\n";
    }

    // opens the loop over a thread's elements of the tile; `keep_loads` unrolls it over a constant count
    void open_element_loop(long long tile_elements, int per_thread, const char *pad) {
        if (keep_loads) {
            out << pad << "#pragma unroll\n"
                << pad << "for (int e = 0; e < " << per_thread << "; ++e) {\n";
            if (tile_width > 0)  // a thread's elements come in groups of `tile_width` consecutive ones
                out << pad << "    const nt_idx element = (member + (e / " << tile_width << ") * " << group << ") * " << tile_width << " + e % " << tile_width << ";\n";
            else
                out << pad << "    const nt_idx element = member + e * " << group << ";\n";
            out << pad << "    if (element >= " << lit(tile_elements) << ") break;\n";
        } else {
            out << pad << "for (nt_idx element = member; element < " << lit(tile_elements) << "; element += " << group << ") {\n";
        }
        in_body.clear();
    }

    void close_element_loop(const char *pad) {
        out << pad << "}\n";
        for (const auto &entry : in_body) kept[entry.first] = true;
        in_body.clear();
    }

    // Tile mode over 16-bit tensors whose elements a thread keeps in registers: groups of 8 consecutive elements per
    // thread (one 16-byte access per tensor and group) when every tensor advances by one element or not at all along
    // the tile's last variable.  0: element by element (fp32 tensors alone are as fast that way).
    int tile_vector_width(long long tile_elements) const {
        if (p.num_dynamic != 0 || p.store_op == NT_MAP_STORE_ATOMIC_ADD || p.num_vars <= p.num_grid) return 0;
        std::vector<int> used(1, p.output);
        for (int pc = 0; pc < p.value_code_length; ++pc) {
            const int op = p.value_code[pc] & 0xff;
            if (op == NT_MAP_V_LOAD) used.push_back(p.value_code[pc] >> 8);
            if (op == NT_MAP_V_SETVAR) return 0;
        }
        bool narrow_type = false;
        for (int slot : used) {
            if (!kept_as_float(slot)) return 0;
            if (p.operands[slot].dtype != NINETOOTHED_FLOAT32) narrow_type = true;
        }
        const int width = 8, last = p.num_vars - 1;
        if (!narrow_type || p.extents[last] <= 0 || p.extents[last] % width != 0 || tile_elements % width != 0) return 0;
        if (group_step(p.operands[p.output].segment, last, width) != 1) return 0;
        for (int slot : used)
            if (group_step(p.operands[slot].segment, last, width) < 0) return 0;
        return width;
    }

    static std::string vector_type(int dtype) {  // (declared by vector_typedefs; global accesses need the element's alignment only)
        return std::string("nt_vec_") + (dtype == NINETOOTHED_FLOAT32 ? "f32" : dtype == NINETOOTHED_FLOAT16 ? "f16" : "bf16");
    }

    void vector_typedefs(int width, const char *pad) {
        out << pad << "typedef float nt_vec_f32 __attribute__((ext_vector_type(" << width << "), aligned(4)));\n"
            << pad << "typedef _Float16 nt_vec_f16 __attribute__((ext_vector_type(" << width << "), aligned(2)));\n"
            << pad << "typedef __bf16 nt_vec_bf16 __attribute__((ext_vector_type(" << width << "), aligned(2)));\n";
    }

    // `width` values of operand `slot` from the element the variables stand at into ld<slot>[first .. first + width)
    void load_group(int slot, int width, const std::string &first) {
        const int last = p.num_vars - 1;
        const NineToothedMapOperand &operand = p.operands[slot];
        const std::string valid = fresh("ok");
        out << indent << "bool " << valid << " = true;\n";
        const std::string offset = index_segment(operand.segment, valid);
        const std::string pointer = std::string("((const ") + c_type(operand.dtype) + " *)a.data[" + std::to_string(slot) + "] + " + offset + ")";
        if (group_step(operand.segment, last, width) == 1) {
            out << indent << "if (" << valid << ") {\n"
                << indent << "    const " << vector_type(operand.dtype) << " loaded = *(const " << vector_type(operand.dtype) << " *)" << pointer << ";\n"
                << indent << "    _Pragma(\"unroll\") for (int j = 0; j < " << width << "; ++j) ld" << slot << "[" << first << " + j] = (float)loaded[j];\n"
                << indent << "} else {\n"
                << indent << "    _Pragma(\"unroll\") for (int j = 0; j < " << width << "; ++j) ld" << slot << "[" << first << " + j] = (float)a.other[" << slot << "];\n"
                << indent << "}\n";
        } else {
            out << indent << "{\n"
                << indent << "    const float shared = " << valid << " ? (float)*" << pointer << " : (float)a.other[" << slot << "];\n"
                << indent << "    _Pragma(\"unroll\") for (int j = 0; j < " << width << "; ++j) ld" << slot << "[" << first << " + j] = shared;\n"
                << indent << "}\n";
        }
    }

    // tile mode in groups: every operand's values of the thread's groups, loaded once before the phases
    void preload_groups(long long tile_elements, int per_thread) {
        vector_typedefs(tile_width, "        ");
        out << "        #pragma unroll\n"
            << "        for (int g = 0; g < " << per_thread / tile_width << "; ++g) {\n"
            << "            const nt_idx element = (member + g * " << group << ") * " << tile_width << ";\n"
            << "            if (element >= " << lit(tile_elements) << ") break;\n";
        indent = "            ";
        decode_tile_variables();
        for (int pc = 0; pc < p.value_code_length; ++pc) {
            if ((p.value_code[pc] & 0xff) != NT_MAP_V_LOAD) continue;
            const int slot = p.value_code[pc] >> 8;
            if (kept[slot]) continue;
            kept[slot] = true;
            load_group(slot, tile_width, "g * " + std::to_string(tile_width));
        }
        out << "        }\n";
    }

    // tile mode in groups: the stored expression, a group's values in one store
    void store_groups(long long tile_elements, int per_thread, int begin) {
        const int last = p.num_vars - 1;
        const NineToothedMapOperand &target = p.operands[p.output];
        out << "        #pragma unroll\n"
            << "        for (int g = 0; g < " << per_thread / tile_width << "; ++g) {\n"
            << "            const nt_idx element = (member + g * " << group << ") * " << tile_width << ";\n"
            << "            if (element >= " << lit(tile_elements) << ") break;\n";
        indent = "            ";
        decode_tile_variables();
        out << indent << "bool store_ok = true;\n";
        const std::string offset = index_segment(target.segment, "store_ok");
        out << indent << "const nt_idx nt_first = v" << last << ";\n"
            << indent << vector_type(target.dtype) << " result;\n"
            << indent << "#pragma unroll\n"
            << indent << "for (int j = 0; j < " << tile_width << "; ++j) {\n";
        indent += "    ";
        out << indent << "const nt_idx v" << last << " = nt_first + j;\n"
            << indent << "const int e = g * " << tile_width << " + j;\n";
        const std::string value = value_range(begin, p.value_code_length, "");
        out << indent << "result[j] = (" << c_type(target.dtype) << ")(float)(" << value << ");\n";
        indent.resize(indent.size() - 4);
        out << indent << "}\n"
            << indent << "if (store_ok) __builtin_nontemporal_store(result, (" << vector_type(target.dtype) << " *)((" << c_type(target.dtype) << " *)a.data[" << p.output << "] + " << offset
            << "));\n"
            << "        }\n";
    }

    // one workgroup per tile: reduction phases, then the stored expression (see the tile mode of the header)
    std::string generate_tile() {
        long long tiles = 1, tile_elements = 1;
        for (int v = 0; v < p.num_vars; ++v) (v < p.num_grid ? tiles : tile_elements) *= (long long)p.extents[v];
        // up to 16 elements per thread: every operand is read from memory once and kept in registers
        // (4096 rows of fp32: softmax(2x) 1024 wide 13 us against 16, 2048 wide 20 against 27, 4096 wide 33
        // against 42; 32 per thread spills: 8192 wide rms norm 97 us against 62; longer rows get more threads)
        int per_thread = (int)((tile_elements + group - 1) / group);
        keep_loads = tile_elements <= (long long)group * 16;
        // (measured on 4096 rows of fp16, element by element -> groups: one reduction -- rms norm -- 4096 wide 18.9 -> 14.5 us,
        // 8192 wide 40.7 -> 31.9, 16384 wide 73.3 -> 39.8; two reductions -- softmax, layer norm -- 16384 wide 109 -> 87 and
        // 97 -> 48 us, but 8192 wide 39.7 -> 62.4 and 36.7 -> 43.1, 4096 wide 24.2 -> 29.8 and 19.6 -> 17.4: those stay
        // element by element)
        tile_width = keep_loads && (p.num_phases == 1 || tile_elements >= 16384) ? tile_vector_width(tile_elements) : 0;
        if (tile_width > 0) per_thread = (int)((tile_elements / tile_width + group - 1) / group) * tile_width;
        const bool wave_tiles = group == 64 && threads > 64;  // a wave per tile: no exchange through LDS
        if (wave_tiles)
            out << "    const nt_idx member = threadIdx.x & 63;\n"
                << "    for (nt_idx tile = (nt_idx)blockIdx.x * " << threads / 64 << " + (threadIdx.x >> 6); tile < " << lit(tiles) << "; tile += (nt_idx)gridDim.x * " << threads / 64 << ") {\n";
        else
            out << "    __shared__ double scratch[" << threads / 64 << "];\n"
                << "    const nt_idx member = threadIdx.x;\n"
                << "    for (nt_idx tile = (nt_idx)blockIdx.x; tile < " << lit(tiles) << "; tile += (nt_idx)gridDim.x) {\n";
        out
            << "        nt_uidx tile_rest = (nt_uidx)tile;\n";
        for (int v = p.num_grid - 1; v >= 0; --v)
            out << "        const nt_idx v" << v << " = (nt_idx)(tile_rest % " << ulit((long long)p.extents[v]) << "); tile_rest /= " << ulit((long long)p.extents[v]) << ";\n";
        if (keep_loads) {
            std::fill(kept.begin(), kept.end(), false);
            // (values of 16- and 32-bit floating-point tensors are kept as floats: half the registers)
            for (int slot = 0; slot < p.num_operands; ++slot) out << "        " << (kept_as_float(slot) ? "float" : "double") << " ld" << slot << "[" << per_thread << "];\n";
        }
        if (tile_width > 0) preload_groups(tile_elements, per_thread);
        int begin = 0;
        for (int k = 0; k < p.num_phases; ++k) {
            const int op = p.phase_op[k], dtype = p.phase_dtype[k];
            const char *init = op == NT_MAP_REDUCE_SUM ? "0.0" : (op == NT_MAP_REDUCE_MAX ? "-__builtin_inf()" : "__builtin_inf()");
            // a reduction of fp32 values (terms rounded to a 16- or 32-bit floating-point type, sums rounded to one after
            // every addition) is carried in a float: the same values, half the shuffles and no fp64 instructions
            const int last_op = p.phase_end[k] > begin ? p.value_code[p.phase_end[k] - 1] : 0;
            const auto single_type = [](int t) { return t == NINETOOTHED_FLOAT32 || t == NINETOOTHED_FLOAT16 || t == NINETOOTHED_BFLOAT16; };
            const bool single = single_type(dtype) && (((last_op & 0xff) == NT_MAP_V_ROUND && single_type(last_op >> 8)) ||
                                                       ((last_op & 0xff) == NT_MAP_V_LOAD && kept_as_float(last_op >> 8)));
            const char *carried = single ? "float" : "double";
            out << "        " << carried << " r" << k << ";\n        {\n            " << carried << " acc = " << init << ";\n";
            open_element_loop(tile_elements, per_thread, "            ");
            indent = "                ";
            decode_tile_variables();
            const std::string term = value_range(begin, p.phase_end[k], "");
            out << indent << "acc = " << combine_expr(op, dtype, "acc", term) << ";\n";
            close_element_loop("            ");
            out << "            for (int offset = 32; offset > 0; offset >>= 1) { const " << carried << " other = __shfl_xor(acc, offset, 64); acc = "
                << combine_expr(op, dtype, "acc", "other") << "; }\n";
            if (wave_tiles) {
                out << "            r" << k << " = acc;\n        }\n";
                begin = p.phase_end[k];
                continue;
            }
            out << "            __syncthreads();\n            if ((threadIdx.x & 63) == 0) scratch[threadIdx.x >> 6] = acc;\n            __syncthreads();\n"
                << "            acc = scratch[0];\n"
                << "            for (int w = 1; w < " << threads / 64 << "; ++w) { const " << carried << " other = scratch[w]; acc = " << combine_expr(op, dtype, "acc", "other")
                << "; }\n            r" << k << " = acc;\n        }\n";
            begin = p.phase_end[k];
        }
        const NineToothedMapOperand &target = p.operands[p.output];
        if (tile_width > 0) {
            store_groups(tile_elements, per_thread, begin);
            out << "    }\n}\n";
            keep_loads = false;
            tile_width = 0;
            return out.str();
        }
        open_element_loop(tile_elements, per_thread, "        ");
        indent = "            ";
        decode_tile_variables();
        const std::string result = value_range(begin, p.value_code_length, "");
        out << indent << "bool store_ok = true;\n";
        const std::string offset = index_segment(target.segment, "store_ok");
        out << indent << "if (store_ok) " << store_stmt("a.data[" + std::to_string(p.output) + "]", target.dtype, offset, result) << "\n";
        close_element_loop("        ");
        out << "    }\n}\n";
        keep_loads = false;
        return out.str();
    }

    // ---- element-wise maps, several consecutive elements per thread ----
    //
    // How an index segment depends on the last output variable when that variable moves through an aligned group of
    // `width` values: 0 = not at all (the group shares one element), 1 = it advances by one element per value and the
    // segment's checks hold for the whole group or for none of it, -1 = anything else.  Abstract interpretation of
    // the index program: a value is invariant, or `rest + k * last` with `rest` known to be a multiple of `width` or
    // not; a division or remainder of such a sum by a multiple of `width` keeps the group together.
    int group_step(int segment, int last, long long width) const {
        struct Shape {
            bool moves;
            long long k;
            bool multiple;  // the value at last = 0 is a multiple of `width`
        };
        std::vector<Shape> stack;
        for (int pc = p.segment_begin[segment];; ++pc) {
            const int op = p.index_code[pc] & 0xff, arg = p.index_code[pc] >> 8;
            if (op == NT_MAP_I_END) break;
            const long long c = op == NT_MAP_I_VAR || op == NT_MAP_I_ADD ? 0 : (long long)p.index_constants[arg];
            switch (op) {
                case NT_MAP_I_CONST: stack.push_back({false, 0, c % width == 0}); break;
                case NT_MAP_I_VAR: stack.push_back(arg == last ? Shape{true, 1, true} : Shape{false, 0, false}); break;
                case NT_MAP_I_MULC:
                    stack.back().k *= c;
                    stack.back().multiple = stack.back().multiple || c % width == 0;
                    if (stack.back().moves && stack.back().k == 0) stack.back().moves = false;
                    break;
                case NT_MAP_I_ADD: {
                    const Shape b = stack.back();
                    stack.pop_back();
                    Shape &a = stack.back();
                    a = {a.moves || b.moves, a.k + b.k, a.multiple && b.multiple};
                    if (a.moves && a.k == 0) return -1;  // (cancelling terms: not worth following)
                    break;
                }
                case NT_MAP_I_DIVC:
                case NT_MAP_I_MODC: {
                    Shape &a = stack.back();
                    if (c <= 0) return -1;
                    if (!a.moves) {
                        a = {false, 0, false};
                    } else {
                        if (a.k != 1 || !a.multiple || c % width != 0) return -1;
                        a = op == NT_MAP_I_DIVC ? Shape{false, 0, false} : Shape{true, 1, true};
                    }
                    break;
                }
                case NT_MAP_I_CHECK: {
                    const Shape a = stack.back();
                    stack.pop_back();
                    if (a.moves && (a.k != 1 || !a.multiple || c % width != 0)) return -1;
                    break;
                }
                default: return -1;
            }
        }
        if (stack.empty() || !stack.back().moves) return 0;
        return stack.back().k == 1 ? 1 : -1;
    }

    // Elements per thread for a plain element-wise map (no reduction, no data-dependent index) over 16- and 32-bit
    // floating-point tensors whose output and operands are contiguous along the last variable (or do not depend on
    // it): 8 when a 16-bit tensor takes part (16 bytes of it per access).  0: one element per thread.
    int vector_width() const {
        if (p.num_phases > 0 || p.reduce_op != NT_MAP_REDUCE_NONE || p.num_reduced != 0 || p.num_dynamic != 0 || lanes != 1) return 0;
        if (p.store_op == NT_MAP_STORE_ATOMIC_ADD || p.num_vars < 1) return 0;
        std::vector<int> used(1, p.output);
        bool random = false;
        for (int pc = 0; pc < p.value_code_length; ++pc) {
            const int op = p.value_code[pc] & 0xff;
            if (op == NT_MAP_V_LOAD) used.push_back(p.value_code[pc] >> 8);
            if (op == NT_MAP_V_RAND) random = true;
            if (op == NT_MAP_V_SETVAR || op == NT_MAP_V_REDUCED) return 0;
        }
        // (measured on 2^26 elements, one per thread -> groups: fp16 copy 50 -> 39 us, fp16 add 59.5 -> 58; fp32 add
        // 137 -> 151 with groups of 4 and 160 with groups of 2, so maps over fp32 tensors alone keep one element per
        // thread -- unless they draw random numbers, whose rounds then run four chains deep: dropout 196 -> 160)
        int width = random ? 4 : 0;
        for (int slot : used) {
            if (!kept_as_float(slot)) return 0;
            if (p.operands[slot].dtype != NINETOOTHED_FLOAT32) width = 8;
        }
        if (width == 0) return 0;
        const int last = p.num_vars - 1;
        if (p.extents[last] <= 0 || p.extents[last] % width != 0) return 0;
        if (group_step(p.operands[p.output].segment, last, width) != 1) return 0;
        for (int slot : used)
            if (group_step(p.operands[slot].segment, last, width) < 0) return 0;
        return width;
    }

    std::string generate_vector(int width) {
        const int last = p.num_vars - 1;
        vector_typedefs(width, "    ");
        out << "    const nt_idx groups = total_out / " << width << ";\n"
            << "    for (nt_idx group = (nt_idx)blockIdx.x * " << kMapThreads << " + threadIdx.x; group < groups; group += stride) {\n"
            << "        nt_uidx rest = (nt_uidx)group * " << width << "u;\n";
        for (int v = last; v >= 0; --v)
            out << "        const nt_idx v" << v << " = (nt_idx)(rest % " << ulit((long long)p.extents[v]) << "); rest /= " << ulit((long long)p.extents[v]) << ";\n";
        // the operands' values of the group, as floats
        std::fill(kept.begin(), kept.end(), false);
        for (int pc = 0; pc < p.value_code_length; ++pc) {
            if ((p.value_code[pc] & 0xff) != NT_MAP_V_LOAD) continue;
            const int slot = p.value_code[pc] >> 8;
            if (kept[slot]) continue;
            kept[slot] = true;
            out << indent << "float ld" << slot << "[" << width << "];\n";
            load_group(slot, width, "0");
        }
        const NineToothedMapOperand &target = p.operands[p.output];
        out << indent << "bool store_ok = true;\n";
        const std::string target_offset = index_segment(target.segment, "store_ok");
        out << indent << "const nt_idx nt_first = v" << last << ";\n"
            << indent << vector_type(target.dtype) << " result;\n"
            << indent << "#pragma unroll\n"
            << indent << "for (int e = 0; e < " << width << "; ++e) {\n";
        indent += "    ";
        out << indent << "const nt_idx v" << last << " = nt_first + e;\n";
        keep_loads = true;
        const std::string value = value_range(0, p.value_code_length, "");
        keep_loads = false;
        out << indent << "result[e] = (" << c_type(target.dtype) << ")(float)(" << value << ");\n";
        indent.resize(indent.size() - 4);
        out << indent << "}\n"
            << indent << "if (store_ok) __builtin_nontemporal_store(result, (" << vector_type(target.dtype) << " *)((" << c_type(target.dtype) << " *)a.data[" << p.output << "] + "
            << target_offset << "));\n"
            << "    }\n}\n";
        return out.str();
    }

    std::string generate() {
        const int num_out = p.num_vars - p.num_reduced;
        out << "struct MapJitArgs { void *data[" << NT_MAP_MAX_OPERANDS << "]; double other[" << NT_MAP_MAX_OPERANDS << "]; double constants["
            << NT_MAP_MAX_VALUE_CONSTANTS << "]; long long total_out; };\n"
            << "typedef " << idx() << " nt_idx;\n"
            << "typedef unsigned " << idx() << " nt_uidx;  // element numbers are decoded unsigned: no sign fix-ups in the divisions\n"
            << "__device__ inline nt_idx nt_floor_div(nt_idx a, nt_idx b) { nt_idx q = a / b; if ((a % b != 0) && ((a < 0) != (b < 0))) --q; return q; }\n"
            << "__device__ inline nt_idx nt_floor_mod(nt_idx a, nt_idx b) { return a - nt_floor_div(a, b) * b; }\n"
            << "__device__ inline double nt_philox_uniform(unsigned long long seed, unsigned long long offset) {\n"
            << "    unsigned int c0 = (unsigned int)offset, c1 = (unsigned int)(offset >> 32), c2 = 0, c3 = 0;\n"
            << "    unsigned int k0 = (unsigned int)seed, k1 = (unsigned int)(seed >> 32);\n"
            << "    for (int round = 0; round < 10; ++round) {\n"
            << "        const unsigned long long a0 = 0xD2511F53ull * c0, b2 = 0xCD9E8D57ull * c2;  // (one 32 x 32 -> 64 bit multiplication each)\n"
            << "        c0 = (unsigned int)(b2 >> 32) ^ c1 ^ k0; c2 = (unsigned int)(a0 >> 32) ^ c3 ^ k1; c1 = (unsigned int)b2; c3 = (unsigned int)a0;\n"
            << "        k0 += 0x9E3779B9u; k1 += 0xBB67AE85u;\n"
            << "    }\n"
            << "    int x = (int)c0; if (x < 0) x = -x - 1;\n"
            << "    return (double)((float)x * 4.6566127342e-10f);\n"
            << "}\n"
            << "extern \"C\" __global__ __launch_bounds__(" << threads << ") void nt_map_specialised(const MapJitArgs a) {\n"
            << "    const nt_idx stride = (nt_idx)gridDim.x * " << kMapThreads << ";\n"
            << "    const nt_idx total_out = (nt_idx)a.total_out;\n";
        if (p.num_phases > 0) return generate_tile();
        if (const int width = vector_width()) return generate_vector(width);
        if (lanes > 64) out << "    __shared__ double nt_partial[" << lanes / 64 << "];\n";
        if (lanes > 1)
            out << "    const nt_idx lane = threadIdx.x & " << lanes - 1 << ";\n"
                << "    for (nt_idx element = ((nt_idx)blockIdx.x * " << kMapThreads << " + threadIdx.x) / " << lanes << "; element < total_out; element += stride / " << lanes << ") {\n"
                << "        nt_uidx rest = (nt_uidx)element;\n";
        else
        out << "    for (nt_idx element = (nt_idx)blockIdx.x * " << kMapThreads << " + threadIdx.x; element < total_out; element += stride) {\n"
            << "        nt_uidx rest = (nt_uidx)element;\n";
        for (int v = num_out - 1; v >= 0; --v)
            out << "        const nt_idx v" << v << " = (nt_idx)(rest % " << ulit((long long)p.extents[v]) << "); rest /= " << ulit((long long)p.extents[v]) << ";\n";
        for (int v = p.num_vars; v < p.num_vars + p.num_dynamic; ++v) out << "        nt_idx v" << v << " = 0;\n";
        std::string result;
        if (p.reduce_op == NT_MAP_REDUCE_NONE) {
            result = value_range(0, p.value_code_length, "");
        } else {
            const char *init = p.reduce_op == NT_MAP_REDUCE_SUM ? "0.0" : (p.reduce_op == NT_MAP_REDUCE_MAX ? "-__builtin_inf()" : "__builtin_inf()");
            // (a reduction of fp32 values is carried in a float, as in tile mode)
            const int last_op = p.reduce_split > 0 ? p.value_code[p.reduce_split - 1] : 0;
            const auto single_type = [](int t) { return t == NINETOOTHED_FLOAT32 || t == NINETOOTHED_FLOAT16 || t == NINETOOTHED_BFLOAT16; };
            const bool single = single_type(p.reduce_dtype) && (((last_op & 0xff) == NT_MAP_V_ROUND && single_type(last_op >> 8)) ||
                                                                ((last_op & 0xff) == NT_MAP_V_LOAD && kept_as_float(last_op >> 8)));
            const char *carried = single ? "float" : "double";
            out << "        " << carried << " acc = " << init << ";\n";
            long long reduced_total = 1;
            for (int v = num_out; v < p.num_vars; ++v) reduced_total *= p.extents[v];
            if (lanes > 1) {  // the lanes of a wave stride the reduced positions
                // (few waves per output: the loads of several iterations have to be in flight at once)
                if (lanes > 64) out << indent << "#pragma unroll 8\n";
                out << indent << "for (nt_idx position = lane; position < " << lit(reduced_total) << "; position += " << lanes << ") {\n";
                indent += "    ";
                out << indent << "nt_uidx inner = (nt_uidx)position;\n";
                for (int v = p.num_vars - 1; v >= num_out; --v)
                    out << indent << "const nt_idx v" << v << " = (nt_idx)(inner % " << ulit((long long)p.extents[v]) << "); inner /= " << ulit((long long)p.extents[v]) << ";\n";
            } else
            for (int v = num_out; v < p.num_vars; ++v) {
                out << indent << "for (nt_idx v" << v << " = 0; v" << v << " < " << lit((long long)p.extents[v]) << "; ++v" << v << ") {\n";
                indent += "    ";
            }
            const std::string term = value_range(0, p.reduce_split, "");
            if (p.reduce_op == NT_MAP_REDUCE_SUM) {
                out << indent << "acc = " << round_expr("acc + " + term, p.reduce_dtype) << ";\n";
            } else {
                const char *cmp = p.reduce_op == NT_MAP_REDUCE_MAX ? ">" : "<";
                out << indent << "acc = (" << term << " != " << term << " || acc != acc) ? acc + " << term << " : (" << term << " " << cmp << " acc ? " << term << " : acc);\n";
            }
            if (lanes > 1) {
                indent.resize(indent.size() - 4);
                out << indent << "}\n";
                for (int offset = 32; offset > 0; offset >>= 1)
                    out << indent << "{ const " << carried << " other = __shfl_xor(acc, " << offset << ", 64); acc = " << combine_expr(p.reduce_op, p.reduce_dtype, "acc", "other") << "; }\n";
                if (lanes > 64) {  // the waves of the workgroup (all of them work on this element: the loop is uniform)
                    out << indent << "if ((threadIdx.x & 63) == 0) nt_partial[threadIdx.x >> 6] = acc;\n"
                        << indent << "__syncthreads();\n"
                        << indent << "acc = nt_partial[0];\n";
                    for (int w = 1; w < lanes / 64; ++w)
                        out << indent << "{ const " << carried << " other = nt_partial[" << w << "]; acc = " << combine_expr(p.reduce_op, p.reduce_dtype, "acc", "other") << "; }\n";
                    out << indent << "__syncthreads();\n";
                }
            } else
            for (int v = num_out; v < p.num_vars; ++v) {
                indent.resize(indent.size() - 4);
                out << indent << "}\n";
            }
            result = value_range(p.reduce_split, p.value_code_length, "acc");
        }
        const NineToothedMapOperand &target = p.operands[p.output];
        out << indent << "bool store_ok = true;\n";
        const std::string offset = index_segment(target.segment, "store_ok");
        const std::string pointer = "a.data[" + std::to_string(p.output) + "]";
        out << indent << (lanes > 1 ? "if (store_ok && lane == 0) " : "if (store_ok) ")
            << (p.store_op == NT_MAP_STORE_ATOMIC_ADD ? atomic_add_stmt(pointer, target.dtype, offset, result) : store_stmt(pointer, target.dtype, offset, result))
            << "\n";
        out << "    }\n}\n";
        return out.str();
    }
};

// hipRTC entry points, resolved at first use so that the library loads without it
struct Hiprtc {
    void *handle = nullptr;
    hiprtcResult (*create)(hiprtcProgram *, const char *, const char *, int, const char **, const char **) = nullptr;
    hiprtcResult (*compile)(hiprtcProgram, int, const char **) = nullptr;
    hiprtcResult (*code_size)(hiprtcProgram, size_t *) = nullptr;
    hiprtcResult (*code)(hiprtcProgram, char *) = nullptr;
    hiprtcResult (*log_size)(hiprtcProgram, size_t *) = nullptr;
    hiprtcResult (*log)(hiprtcProgram, char *) = nullptr;
    hiprtcResult (*destroy)(hiprtcProgram *) = nullptr;
    bool ok = false;

    Hiprtc() {
        for (const char *name : {"libhiprtc.so", "libhiprtc.so.7", "/opt/rocm/lib/libhiprtc.so"}) {
            handle = dlopen(name, RTLD_NOW | RTLD_LOCAL);
            if (handle) break;
        }
        if (!handle) return;
        create = (decltype(create))dlsym(handle, "hiprtcCreateProgram");
        compile = (decltype(compile))dlsym(handle, "hiprtcCompileProgram");
        code_size = (decltype(code_size))dlsym(handle, "hiprtcGetCodeSize");
        code = (decltype(code))dlsym(handle, "hiprtcGetCode");
        log_size = (decltype(log_size))dlsym(handle, "hiprtcGetProgramLogSize");
        log = (decltype(log))dlsym(handle, "hiprtcGetProgramLog");
        destroy = (decltype(destroy))dlsym(handle, "hiprtcDestroyProgram");
        ok = create && compile && code_size && code && log_size && log && destroy;
    }
};

std::mutex g_jit_mutex;
std::unordered_map<std::string, hipFunction_t> g_jit_cache;  // a null function = "do not try again"

// `may_compile` false (the stream is being captured into a graph: compiling and loading code would break
// the capture): only a kernel specialised earlier is returned, and a miss is not remembered
hipFunction_t specialised_kernel(const NineToothedMapProgram &p, bool may_compile) {
    static Hiprtc rtc;
    if (!rtc.ok) return nullptr;
    int device = 0;
    if (hipGetDevice(&device) != hipSuccess) return nullptr;
    // the key is everything the source depends on: all of the program but pointers,
    // `other` values and value constants (those are kernel arguments)
    NineToothedMapProgram shape = p;
    for (int i = 0; i < NT_MAP_MAX_OPERANDS; ++i) {
        shape.operands[i].data = nullptr;
        shape.operands[i].other = 0.0;
        if (i >= p.num_operands) shape.operands[i].dtype = shape.operands[i].segment = 0;
    }
    memset(shape.value_constants, 0, sizeof(shape.value_constants));
    for (int v = p.num_vars; v < NT_MAP_MAX_VARS; ++v) shape.extents[v] = 0;
    for (int i = p.num_segments; i < NT_MAP_MAX_SEGMENTS; ++i) shape.segment_begin[i] = 0;
    for (int i = p.value_code_length; i < NT_MAP_MAX_VALUE_CODE; ++i) shape.value_code[i] = 0;
    for (int k = p.num_phases; k < NT_MAP_MAX_PHASES; ++k) shape.phase_end[k] = shape.phase_op[k] = shape.phase_dtype[k] = 0;
    if (p.num_phases == 0) shape.num_grid = 0;
    std::string key((const char *)&shape, sizeof(shape));
    key.push_back((char)device);
    std::lock_guard<std::mutex> lock(g_jit_mutex);
    auto found = g_jit_cache.find(key);
    if (found != g_jit_cache.end()) return found->second;
    if (!may_compile) return nullptr;
    MapCodegen generator(p);
    const std::string source = generator.generate();
    hipFunction_t function = nullptr;
    hiprtcProgram program = nullptr;
    if (rtc.create(&program, source.c_str(), "nt_map_specialised.hip", 0, nullptr, nullptr) == HIPRTC_SUCCESS) {
        // same code generation switches as the rest of the library: gfx950, packed FP32 off
        // and no contraction: every operation is rounded on its own, as the value program says
        const char *options[] = {"--offload-arch=gfx950", "-O3", "-ffp-contract=off", "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"};
        const hiprtcResult compiled = rtc.compile(program, 7, options);
        if (compiled == HIPRTC_SUCCESS) {
            size_t size = 0;
            if (rtc.code_size(program, &size) == HIPRTC_SUCCESS && size > 0) {
                std::vector<char> binary(size);
                hipModule_t module = nullptr;
                if (rtc.code(program, binary.data()) == HIPRTC_SUCCESS && hipModuleLoadData(&module, binary.data()) == hipSuccess) {
                    if (hipModuleGetFunction(&function, module, "nt_map_specialised") != hipSuccess) function = nullptr;
                }
            }
        } else if (getenv("NT_MAP_VERBOSE")) {
            size_t size = 0;
            rtc.log_size(program, &size);
            std::vector<char> text(size + 1, 0);
            rtc.log(program, text.data());
            fprintf(stderr, "nt_hip: specialising a tile map failed:\n%s\n%s\n", text.data(), source.c_str());
        }
        rtc.destroy(&program);
    }
    g_jit_cache.emplace(key, function);
    return function;
}

}  // namespace
}  // namespace nt

using namespace nt;

extern "C" NineToothedResult launch_nt_map(NineToothedStream stream, const NineToothedMapProgram *program) {
    if (program == nullptr) return hipErrorInvalidValue;
    const NineToothedMapProgram &p = *program;
    if (!well_formed(p)) return NINETOOTHED_NO_KERNEL;
    int64_t total_out = 1, total_reduced = 1;
    const int num_out = p.num_vars - p.num_reduced;
    for (int v = 0; v < p.num_vars; ++v) {
        if (p.extents[v] < 0) return hipErrorInvalidValue;
        if (v < num_out) total_out *= p.extents[v];
        else total_reduced *= p.extents[v];
        if (total_out > (int64_t)1 << 46 || total_reduced > (int64_t)1 << 46) return NINETOOTHED_NO_KERNEL;
    }
    if (total_out == 0) return 0;  // empty launch is legal
    for (int i = 0; i < p.num_operands; ++i)
        if (p.operands[i].data == nullptr) return hipErrorInvalidValue;
    // enough workgroups for 8 per CU; the grid stride covers the rest
    const int lanes = cooperative_lanes(p);  // (the interpreter kernels below run one thread per element regardless)
    int64_t blocks = (total_out * lanes + kMapThreads - 1) / kMapThreads;
    if (blocks > 256 * 32) blocks = 256 * 32;
    int64_t tiles = 1, tile_elements = 1;
    if (p.num_phases > 0) {  // tile mode: one workgroup per tile
        for (int v = 0; v < p.num_vars; ++v) (v < p.num_grid ? tiles : tile_elements) *= p.extents[v];
        const int64_t tiles_per_block = tile_group(p) == 64 ? workgroup_threads(p) / 64 : 1;  // (only the generated kernel shares a workgroup)
        blocks = (tiles + tiles_per_block - 1) / tiles_per_block;
        if (blocks > 256 * 32) blocks = 256 * 32;
    }
    const char *interpret = getenv("NT_MAP_INTERPRET");
    if (!(interpret && interpret[0] == '1')) {
        if (hipFunction_t function = specialised_kernel(p, !stream_is_capturing((hipStream_t)stream))) {
            MapJitArgs args;
            for (int i = 0; i < NT_MAP_MAX_OPERANDS; ++i) {
                args.data[i] = i < p.num_operands ? p.operands[i].data : nullptr;
                args.other[i] = i < p.num_operands ? p.operands[i].other : 0.0;
            }
            memcpy(args.constants, p.value_constants, sizeof(args.constants));
            args.total_out = total_out;
            size_t size = sizeof(args);
            void *config[] = {HIP_LAUNCH_PARAM_BUFFER_POINTER, &args, HIP_LAUNCH_PARAM_BUFFER_SIZE, &size, HIP_LAUNCH_PARAM_END};
            nt::note_launch(nt::kLaunchMap, 0, "kernel generated for the program and compiled with hipRTC");
            return (int)hipModuleLaunchKernel(function, (unsigned)blocks, 1, 1, (unsigned)workgroup_threads(p), 1, 1, 0, (hipStream_t)stream, nullptr, config);
        }
    }
    nt::note_launch(nt::kLaunchMap, 1, "interpreter kernel");
    if (p.num_phases > 0)
        map_tile_kernel<<<dim3((unsigned)blocks), dim3(kMapThreads), 0, (hipStream_t)stream>>>(p, tiles, tile_elements);
    else
        map_kernel<<<dim3((unsigned)blocks), dim3(kMapThreads), 0, (hipStream_t)stream>>>(p, total_out, total_reduced);
    return (int)hipGetLastError();
}

extern "C" NineToothedResult nt_map_source(const NineToothedMapProgram *program, char *buffer, int size) {
    if (program == nullptr || buffer == nullptr || size <= 0) return hipErrorInvalidValue;
    if (!well_formed(*program)) return NINETOOTHED_NO_KERNEL;
    MapCodegen generator(*program);
    const std::string source = generator.generate();
    if ((int)source.size() + 1 > size) return hipErrorInvalidValue;
    memcpy(buffer, source.c_str(), source.size() + 1);
    return 0;
}
